"""Tune the tile configuration of the headline workloads and record the winners
in the tuner cache (the counterpart of the `tuner_cache.db` files the reference
ships next to its benchmarks, e.g. benchmark/bert/tuner_cache.db).

    python -m evt_ae_amd.autotuner.tune_workloads --build-only   # compile every candidate (no GPU needed)
    python -m evt_ae_amd.autotuner.tune_workloads [--cache FILE]  # time them on the GPU, store the best
"""
from __future__ import annotations

import argparse
import os
import sys
from concurrent.futures import ThreadPoolExecutor

import torch


def _tuners():
    from .. import prebuild, workloads as W
    from ..autotuner.bmm_tuner import BMMTuner
    from ..autotuner.gemm_tuner import MMTuner
    from ..evt_fuser import FusedBMM
    out = []
    for cfg in W.CONFIGS:
        gm = W.fuse(W.CONFIGS[cfg].module(), prebuild._shapes_of(cfg, None))
        (node,) = W.fused_nodes(gm)
        op = node.target
        cls = BMMTuner if isinstance(op, FusedBMM) else MMTuner
        out.append((cfg, cls(op.problem, op.a_kc, op.b_kc, op.spec.bf16, op.tile.dma, op.ir)))
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--build-only", action="store_true")
    ap.add_argument("--cache", default=None, help="tuner cache file to write (default: the package's)")
    ap.add_argument("--jobs", type=int, default=min(8, os.cpu_count() or 1))
    args = ap.parse_args()
    # candidates must be enumerated without consulting an existing cache
    os.environ["EVT_TUNER_CACHE"] = "/nonexistent/tuner_cache.db"
    tuners = _tuners()
    from .. import jit
    from ..codegen import KernelSpec
    mods = []
    for cfg, t in tuners:
        for tile in t.candidates():
            mods.append(jit.load_module(t.ir, KernelSpec(t.a_kc, t.b_kc, t.bf16, tile)))
    todo = [m for m in mods if not m.path.exists()]
    print(f"[tune] {len(mods)} candidate modules, {len(todo)} to compile", flush=True)
    with ThreadPoolExecutor(args.jobs) as pool:
        list(pool.map(lambda m: m.build(), todo))
    if args.build_only:
        return
    if not torch.cuda.is_available():
        sys.exit("tuning needs a HIP device")
    from .tuner_base import default_cache_file
    if args.cache:
        os.environ["EVT_TUNER_CACHE"] = args.cache
    else:
        os.environ.pop("EVT_TUNER_CACHE")
    for cfg, t in tuners:
        t.cache_file = default_cache_file()
        results = []
        for tile in t.candidates():
            try:
                us = t.profile(tile)
            except RuntimeError as exc:
                print(f"[tune] config {cfg} {tile.tag()}: {exc}", flush=True)
                continue
            results.append((us, tile))
            print(f"[tune] config {cfg} {tile.tag():40s} {us:9.2f} us", flush=True)
        us, best = min(results, key=lambda r: r[0])
        t.store(best, us)
        print(f"[tune] config {cfg} best {best.tag()} {us:.2f} us -> {t.cache_file}", flush=True)


if __name__ == "__main__":
    main()
