"""Tune the tile configuration of the headline workloads and record the winners
in the tuner cache (the counterpart of the `tuner_cache.db` files the reference
ships next to its benchmarks, e.g. benchmark/bert/tuner_cache.db).

    python -m evt_ae_amd.autotuner.tune_workloads --build-only   # compile every candidate (no GPU needed)
    python -m evt_ae_amd.autotuner.tune_workloads [--cache FILE]  # time them on the GPU, store the best
    ... --encoder [--short-list] [--dims d,heads,ffn,batch,seq]   # the GEMMs / batched products of an encoder
                                                                  # layer's training step (default: BERT-large)
    ... --reference-keys [SUBSTRING ...] [--short-list]           # the problems of the reference's own tuner caches
                                                                  # (tests/golden/reference_tuner_keys.json; needs the
                                                                  # repository's tests/ tree), all or those matching
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


def _encoder_tuners(dims=None):
    """One tuner per distinct fused GEMM / BMM of the encoder layer's training
    step at the benchmark's size, or at `dims` = (d, heads, ffn, batch, seq)
    with separate Q / K / V projections (traced on the meta device: the GPU's
    dtypes)."""
    from .. import workloads as W
    from ..aot_helper import aot_capture
    from ..autotuner.bmm_tuner import BMMTuner
    from ..autotuner.gemm_tuner import MMTuner
    from ..evt_fuser import FusedBMM, FusedGEMM
    kw = W.ENCODER_BENCH if dims is None else dict(zip(("d", "heads", "ffn", "batch", "seq"), dims), fused_qkv=False)
    box = aot_capture(*W.encoder_layer(device="meta", **kw))
    out, seen = [], set()
    for node in W.fused_nodes(box["joint"]):
        op = node.target
        if not isinstance(op, (FusedGEMM, FusedBMM)):
            continue
        cls = BMMTuner if isinstance(op, FusedBMM) else MMTuner
        t = cls(op.problem, op.a_kc, op.b_kc, op.spec.bf16, op.tile.dma, op.ir)
        if t.key() not in seen:
            seen.add(t.key())
            out.append((f"encoder {op.problem}", t))
    return out


def _reference_key_tuners(only=None):
    """One tuner per GEMM / BMM key of the reference's tuner caches, with the synthetic epilogue of the key's
    node counts (tests/patterns.py: the cache key holds the counts, not the expression)."""
    from tests import patterns as P
    from ..autotuner.bmm_tuner import BMMTuner
    from ..autotuner.gemm_tuner import MMTuner
    from ..evt_fuser import FusedBMM
    out, seen = [], set()
    for _table, key, case in P.reference_key_cases():
        if only and not any(o in key for o in only):
            continue
        gm = P.fuse(*P.counted_epilogue(case))
        (node,) = P.fused_nodes(gm)
        op = node.target
        cls = BMMTuner if isinstance(op, FusedBMM) else MMTuner
        M, N, K, L = op.problem
        t = cls((M, N, getattr(op, "kernel_k", K), L), op.a_kc, op.b_kc, op.spec.bf16, op.tile.dma, op.ir)
        if t.key() not in seen:
            seen.add(t.key())
            out.append((key, t))
    return out


# the tiles that have won somewhere so far: a short list keeps the compile time of a new model's problems bounded
SHORT_LIST = [(256, 256, 64, 4, 2, 2, 2), (256, 256, 64, 2, 4, 2, 3), (256, 256, 64, 2, 4, 2, 6), (256, 256, 64, 4, 2, 2, 0),
              (256, 128, 64, 4, 2, 3, 3), (256, 128, 64, 4, 2, 3, 10), (256, 128, 64, 4, 2, 3, 2),
              (128, 256, 64, 2, 4, 3, 3), (128, 256, 64, 2, 4, 3, 10), (128, 256, 64, 2, 4, 3, 2), (128, 128, 64, 2, 4, 4, 2),
              (128, 128, 64, 4, 2, 2, 2), (128, 128, 64, 2, 4, 2, 3), (128, 128, 64, 2, 2, 2, 0), (64, 64, 64, 2, 2, 2, 0),
              (128, 128, 64, 2, 2, 3, 12), (128, 128, 64, 2, 2, 4, 12),
              (256, 256, 64, 2, 4, 2, 7), (256, 256, 64, 4, 2, 2, 7), (256, 128, 64, 4, 2, 3, 5), (128, 128, 64, 2, 2, 2, 12),
              (128, 64, 64, 4, 1, 2, 0), (128, 64, 64, 2, 2, 2, 0), (256, 64, 64, 4, 2, 2, 0), (64, 128, 64, 1, 4, 2, 0),
              (128, 512, 64, 4, 2, 2, 0)]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--build-only", action="store_true")
    ap.add_argument("--encoder", action="store_true", help="tune the encoder layer's problems instead of the five configs")
    ap.add_argument("--dims", default=None, help="with --encoder: d,heads,ffn,batch,seq of the layer (default: the benchmark's)")
    ap.add_argument("--reference-keys", nargs="*", metavar="SUBSTRING", default=None,
                    help="tune the problems of the reference's tuner caches (all, or those whose key contains one of "
                         "the substrings) instead of the five configs")
    ap.add_argument("--short-list", action="store_true",
                    help="only the tiles of SHORT_LIST (with their single-stage forms where K fits one tile, and walking "
                         "forms where the candidates have them)")
    ap.add_argument("--cache", default=None, help="tuner cache file to write (default: the package's)")
    ap.add_argument("--resume", action="store_true", help="skip problems the cache file already has a row for")
    ap.add_argument("--jobs", type=int, default=min(8, os.cpu_count() or 1))
    ap.add_argument("--sigma", default=None, help="standard deviations of the timing operands, 'sigma_A,sigma_B' "
                                                    "(default: 1.0,0.02, activations against weights)")
    args = ap.parse_args()
    # candidates must be enumerated without consulting an existing cache
    os.environ["EVT_TUNER_CACHE"] = "/nonexistent/tuner_cache.db"
    dims = tuple(int(x) for x in args.dims.split(",")) if args.dims else None
    if args.reference_keys is not None:
        tuners = _reference_key_tuners(args.reference_keys or None)
    else:
        tuners = _encoder_tuners(dims) if args.encoder else _tuners()
    if args.short_list:
        for _, t in tuners:
            full = t.candidates()
            short = [c for c in full
                     if (c.bm, c.bn, c.bk, c.wm, c.wn, c.stages, c.pipe) in SHORT_LIST
                     or (c.stages == 1 and (c.bm, c.bn, c.bk, c.wm, c.wn, 2, c.pipe) in SHORT_LIST)]
            t.candidates = (lambda s=short: s)
    from .. import jit
    from ..codegen import KernelSpec
    mods = []
    for cfg, t in tuners:
        for tile in t.candidates():
            mods.append(jit.load_module(t.ir, KernelSpec.for_problem(t.K, t.a_kc, t.b_kc, t.bf16, tile, t.M, t.N)))
    mods = list({str(m.path): m for m in mods}.values())       # problems with one epilogue structure share modules
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
    if args.sigma:
        sigma = tuple(float(x) for x in args.sigma.split(","))
    for cfg, t in tuners:
        t.cache_file = default_cache_file()
        if args.sigma:
            t.operand_sigma = sigma
        if args.resume and t.fetch_cached() is not None:
            print(f"[tune] config {cfg}: already in {t.cache_file}", flush=True)
            continue

        def report(tile, us, note, cfg=cfg):
            if us is None:
                print(f"[tune] config {cfg} {tile.tag():40s} FAILED: {note.splitlines()[0][:200]}", flush=True)
            else:
                print(f"[tune] config {cfg} {tile.tag():40s} {us:9.2f} us" + (f"  ({note})" if note else ""), flush=True)
        results = t.sweep(report)
        if not results:
            print(f"[tune] config {cfg}: no candidate could be timed", flush=True)
            continue
        us, best = t.second_stage(results, report)
        t.store(best, us)
        print(f"[tune] config {cfg} best {best.tag()} {us:.2f} us -> {t.cache_file} "
              f"(operands N(0, {t.operand_sigma[0]}) x N(0, {t.operand_sigma[1]}), {len(t.failed)} candidates failed)", flush=True)


if __name__ == "__main__":
    main()
