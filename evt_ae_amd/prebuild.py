"""Ahead-of-time build of every kernel module the smoke check and the benchmark
use, so that nothing has to be compiled on the GPU box (tests/prebuild_tests.py
does the same for the modules of the tests).

Each workload is traced on meta tensors (no data, no GPU) exactly as it will be
at run time, which registers its kernel module; the modules are then compiled
in parallel with hipcc for gfx950.  The reference has no counterpart: it JITs
through nvcc on first use and keeps cubins in compiled_cache.db.
"""
from __future__ import annotations

import sys
import time
from concurrent.futures import ThreadPoolExecutor
from typing import List

import torch

from . import jit, workloads as W


def _meta(inputs):
    return [torch.empty(t.shape, dtype=t.dtype, device="meta") for t in inputs]


def _shapes_of(cfg: int, shapes: dict):
    """Input shapes/dtypes without materialising full-size random data."""
    import inspect
    fn = W.CONFIGS[cfg].make_inputs
    sig = inspect.signature(fn)
    kw = {k: v.default for k, v in list(sig.parameters.items())[1:]}
    kw.update(shapes or {})

    class _G:   # shape-only stand-in for torch.Generator
        pass
    shapes_only = {
        1: lambda M, N, K: [((M, K), torch.half), ((K, N), torch.half), ((N,), torch.half)],
        2: lambda L, S, D: [((L, S, D), torch.half), ((L, S, D), torch.half)],
        3: lambda M, N, K: [((M, K), torch.half), ((K, N), torch.half), ((N,), torch.half), ((M, N), torch.half)],
        4: lambda M, N, K: [((M, K), torch.half), ((N, K), torch.half), ((M, N), torch.half)],
        5: lambda M, N, K: [((M, K), torch.half), ((K, N), torch.half), ((M,), torch.int32)],
    }[cfg](**kw)
    return [torch.empty(s, dtype=d, device="meta") for s, d in shapes_only]


def register_all() -> List[jit.LazyModule]:
    """Trace what the benchmark and the smoke check run, which registers their kernel modules."""
    for cfg in W.CONFIGS:
        gm = W.fuse(W.CONFIGS[cfg].module(), _shapes_of(cfg, None))
        op = W.fused_nodes(gm)[0].target
        jit.load_module(op.ir, op.spec, clock_probe=True)      # the benchmark's --clock-probe builds
        W.fuse(W.CONFIGS[cfg].module(), _shapes_of(cfg, W.SMALL_SHAPES[cfg]))
    for name, (cls, shapes, _) in W.ROW_BENCH.items():
        W.fuse(cls(), [torch.empty(sh, dtype=dt, device="meta") for sh, dt in shapes])
    from .aot_helper import aot_capture
    # traced on the meta device: its dtype rules are the GPU's (fp32 layer norm statistics for fp16 inputs), so the
    # modules registered here are the ones a GPU run asks for
    aot_capture(*W.encoder_layer(device="meta", **W.ENCODER_BENCH))      # bench.py's training-step leg
    return jit.registered_modules()


def build_all(jobs: int = 8, force: bool = False, verbose: bool = True, register=None) -> List[jit.LazyModule]:
    """`register`: further tracing to do before the build (a callable; it registers modules as a side effect)."""
    mods = register_all()
    if register is not None:
        register()
        mods = jit.registered_modules()
    todo = [m for m in mods if force or not m.path.exists()]
    t0 = time.time()
    if verbose:
        print(f"[prebuild] {len(mods)} modules registered, {len(todo)} to compile", flush=True)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        for m, _ in zip(todo, pool.map(lambda mod: mod.build(force=force), todo)):
            if verbose:
                print(f"[prebuild] built {m.name} -> {m.path.name}", flush=True)
    if verbose:
        print(f"[prebuild] done in {time.time() - t0:.1f}s", flush=True)
    return mods


if __name__ == "__main__":
    build_all(force="--force" in sys.argv)
