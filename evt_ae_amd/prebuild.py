"""Ahead-of-time build of every kernel module the smoke check and the benchmark
use, so that nothing has to be compiled on the GPU box (`--with-tests` adds the
modules of the repository's tests, which tests/prebuild_tests.py lists).

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


def _register_tests():
    """The test catalogue's tracing step, when the repository's tests/ tree is there (a checkout); an installed
    package has none, and only the benchmark's modules are built then."""
    try:
        from tests import prebuild_tests
    except ImportError:
        return None
    return prebuild_tests.register_tests


def prune_stale(mods, verbose: bool = True) -> int:
    """Remove the files of modules that nothing registered any more: after a change of the kernel headers or the
    ABI every module has a new hash, and the old binaries would still be picked up by whoever lists the folder."""
    keep = {m.path.stem for m in mods}
    removed = 0
    for f in jit.KERNEL_DIR.glob("evt_*"):
        if f.suffix in (".so", ".hip") and f.stem not in keep:
            f.unlink()
            removed += 1
    if verbose and removed:
        print(f"[prebuild] removed {removed} files of modules no longer registered", flush=True)
    return removed


def build_all(jobs: int = 8, force: bool = False, verbose: bool = True, register=None,
              with_tests: bool = False, prune: bool = False) -> List[jit.LazyModule]:
    """`register`: further tracing to do before the build (a callable; it registers modules as a side effect).
    `with_tests` (command line: --with-tests): the modules of the repository's tests as well, if tests/ is there.
    `prune` (--prune): afterwards delete the binaries and sources of modules that were not registered."""
    mods = register_all()
    if with_tests and register is None:
        register = _register_tests()
        if register is None and verbose:
            print("[prebuild] no tests/ tree beside the package: building the benchmark's modules only", flush=True)
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
    if prune:
        prune_stale(mods, verbose)
    return mods


if __name__ == "__main__":
    build_all(force="--force" in sys.argv, with_tests="--with-tests" in sys.argv, prune="--prune" in sys.argv)
