"""Batched-GEMM tile tuner (mirror of python/gtl/compiler/autotuner/bmm_tuner.py:29-122)."""
from .tuner_base import AutoTunerBase


class BMMTuner(AutoTunerBase):
    table = "best_config_bmm"

    def key(self) -> str:
        return f"{self.L}_" + super().key()
