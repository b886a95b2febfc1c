"""Writes tests/golden/configs_small.npz: seeded inputs of the five headline
subgraphs at the fixture shapes (patterns.GOLDEN_SHAPES) and the outputs of PyTorch's fp32 eager
evaluation of each subgraph on CPU (the specified oracle for this path; the
reference itself ships no numeric vectors and cannot run here because its
CUTLASS dependency is an empty submodule).

Run from the repository root:  python tests/golden/make_golden.py
"""
import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))

from tests import patterns as W   # noqa: E402
from oracle import evt_oracle           # noqa: E402


def main():
    arrays = {}
    for cfg in (1, 2, 3, 4, 5):
        inputs = W.make_inputs(cfg, W.GOLDEN_SHAPES[cfg])
        outs = evt_oracle.eval_fp32(W.CONFIGS[cfg].module(), inputs)
        for i, t in enumerate(inputs):
            arrays[f"c{cfg}_in{i}"] = t.numpy()
        for i, t in enumerate(outs):
            arrays[f"c{cfg}_out{i}"] = t.numpy().astype(np.float32)
    out = Path(__file__).parent / "configs_small.npz"
    np.savez_compressed(out, **arrays)
    print("wrote", out, out.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
