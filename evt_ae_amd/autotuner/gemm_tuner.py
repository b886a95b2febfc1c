"""GEMM tile tuner (mirror of python/gtl/compiler/autotuner/gemm_tuner.py:27-153)."""
from .tuner_base import AutoTunerBase


class MMTuner(AutoTunerBase):
    table = "best_config_mm"
