"""Tune the tile configuration of the headline workloads and record the winners
in the tuner cache (the counterpart of the `tuner_cache.db` files the reference
ships next to its benchmarks, e.g. benchmark/bert/tuner_cache.db).

    python -m evt_ae_amd.autotuner.tune_workloads --build-only   # compile every candidate (no GPU needed)
    python -m evt_ae_amd.autotuner.tune_workloads [--cache FILE]  # time them on the GPU, store the best
    ... --encoder [--short-list] [--dims d,heads,ffn,batch,seq]   # the GEMMs / batched products of an encoder
                                                                  # layer's training step (default: BERT-large)
    ... --encoder --in-step 3                                     # then time each problem's best three tiles inside
                                                                  # the layer's training step and keep what the step
                                                                  # prefers
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


class _StepTimer:
    """The encoder layer's training step, compiled with the tiles a cache file holds, and compared kernel by kernel
    with another such step: durations come from torch.profiler's device events, so host gaps do not count, and only
    the kernels that differ between the two steps (and the kernel behind each, which reads what they wrote) enter
    the comparison; the rest of the step would only add its scatter."""

    def __init__(self, kw, iters=10, regions=3):
        self.kw, self.iters, self.regions = kw, iters, regions

    def build(self, cache_file):
        """step() of a freshly traced layer: tiles are chosen at trace time, from `cache_file`."""
        from .. import workloads as W
        from ..aot_helper import aot_optimize
        os.environ["EVT_TUNER_CACHE"] = str(cache_file)
        torch.manual_seed(0)
        model, (x, target) = W.encoder_layer(device="cuda", **self.kw)
        fused = aot_optimize(model)
        params = list(model.parameters())

        def step():
            for p in params:
                p.grad = None
            fused(x, target).backward()
        for _ in range(3):
            step()
        torch.cuda.synchronize()
        return step

    def kernels(self, step):
        """[(kernel name, mean duration in us)] by position in the step."""
        from torch.profiler import ProfilerActivity, profile
        with profile(activities=[ProfilerActivity.CUDA]) as prof:
            for _ in range(self.iters):
                step()
            torch.cuda.synchronize()
        evs = sorted((e for e in prof.events() if e.device_type == torch.autograd.DeviceType.CUDA),
                     key=lambda e: e.time_range.start)
        n = len(evs) // self.iters
        if n == 0 or n * self.iters != len(evs):
            raise RuntimeError(f"{len(evs)} device events over {self.iters} steps: the steps do not repeat")
        return [(evs[i].name, sum(evs[i + k * n].device_time for k in range(self.iters)) / self.iters) for i in range(n)]

    def compare(self, step_a, step_b):
        """(us of a, us of b, us per whole step of a, of b): medians over regions taken in turns; the first pair
        sums the kernels that differ between the steps and their successors."""
        runs_a, runs_b = [], []
        for _ in range(self.regions):
            runs_a.append(self.kernels(step_a))
            runs_b.append(self.kernels(step_b))
        med = lambda v: sorted(v)[len(v) // 2]
        tot_a, tot_b = med([sum(d for _, d in r) for r in runs_a]), med([sum(d for _, d in r) for r in runs_b])
        if len(runs_a[0]) != len(runs_b[0]):        # another number of launches (a split that needs a second kernel)
            return tot_a, tot_b, tot_a, tot_b
        pos = {i for i, (x, y) in enumerate(zip(runs_a[0], runs_b[0])) if x[0] != y[0]}
        pos |= {i + 1 for i in pos if i + 1 < len(runs_a[0])}
        return (med([sum(r[i][1] for i in pos) for r in runs_a]), med([sum(r[i][1] for i in pos) for r in runs_b]),
                tot_a, tot_b)


def _in_step_stage(kw, ranked, top, gain=0.01, timer=None):
    """Third stage of a model's cache.  The sweep times a problem alone, its operands rotating through HBM; inside
    the step the previous kernel has just written them, the clock is what the neighbouring kernels left, and the
    ranking of close candidates can turn round.  Problem by problem, the sweep's best `top` tiles are put into the
    cache in turn, the step is traced again and compared with the step of the rows kept so far; a row changes
    only if the kernels it touches get faster by more than `gain`.  `timer` (build(cache file) -> step,
    compare(step, step) -> the four times of _StepTimer.compare) stands in for the GPU in tests."""
    from .tuner_base import default_cache_file
    timer = timer or _StepTimer(kw)
    cache = default_cache_file()
    kept = timer.build(cache)
    for name, t, results in ranked:
        current = t.fetch_cached()
        cur_us = next((us for us, tile in results if tile == current), None)
        for us, tile in sorted(results, key=lambda r: r[0])[:top]:
            if tile == current:
                continue
            t.store(tile, us)
            trial = timer.build(cache)
            us_kept, us_trial, step_kept, step_trial = timer.compare(kept, trial)
            better = us_trial < us_kept * (1.0 - gain)
            print(f"[tune] in step: {name} {tile.tag():40s} {us_trial:8.1f} us against {us_kept:8.1f} with {current.tag()} "
                  f"(kernels of the step: {step_trial:.1f} against {step_kept:.1f} us): {'taken' if better else 'not taken'}",
                  flush=True)
            if better:
                kept, current, cur_us = trial, tile, us
            else:
                t.store(current, cur_us if cur_us is not None else us)
            del trial
            if torch.cuda.is_available():
                torch.cuda.empty_cache()


# the tiles that have won somewhere so far: a short list keeps the compile time of a new model's problems bounded
SHORT_LIST = [(256, 256, 64, 4, 2, 2, 2), (256, 256, 64, 2, 4, 2, 3), (256, 256, 64, 2, 4, 2, 6), (256, 256, 64, 4, 2, 2, 0),
              (256, 128, 64, 4, 2, 3, 3), (256, 128, 64, 4, 2, 3, 10), (256, 128, 64, 4, 2, 3, 2),
              (128, 256, 64, 2, 4, 3, 3), (128, 256, 64, 2, 4, 3, 10), (128, 256, 64, 2, 4, 3, 2), (128, 128, 64, 2, 4, 4, 2),
              (128, 128, 64, 4, 2, 2, 2), (128, 128, 64, 2, 4, 2, 3), (128, 128, 64, 2, 2, 2, 0), (64, 64, 64, 2, 2, 2, 0),
              (128, 128, 64, 2, 2, 3, 12), (128, 128, 64, 2, 2, 4, 12),
              (256, 256, 64, 2, 4, 2, 7), (256, 256, 64, 4, 2, 2, 7), (256, 128, 64, 4, 2, 3, 5), (128, 128, 64, 2, 2, 2, 12),
              (128, 64, 64, 4, 1, 2, 0), (128, 64, 64, 2, 2, 2, 0), (256, 64, 64, 4, 2, 2, 0), (64, 128, 64, 1, 4, 2, 0),
              (128, 512, 64, 4, 2, 2, 0), (128, 256, 64, 2, 4, 3, 27), (128, 256, 64, 2, 4, 3, 21), (256, 128, 64, 4, 2, 3, 21)]


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
    ap.add_argument("--in-step", type=int, default=0, metavar="N",
                    help="with --encoder: after the sweep, time each problem's best N tiles inside the layer's training "
                         "step and keep a tile only if the step as a whole gets faster")
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
    ranked = []
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
        ranked.append((cfg, t, results))
        print(f"[tune] config {cfg} best {best.tag()} {us:.2f} us -> {t.cache_file} "
              f"(operands N(0, {t.operand_sigma[0]}) x N(0, {t.operand_sigma[1]}), {len(t.failed)} candidates failed)", flush=True)
    if args.in_step > 0 and args.encoder and ranked:
        from .. import workloads as W
        kw = W.ENCODER_BENCH if dims is None else dict(zip(("d", "heads", "ffn", "batch", "seq"), dims), fused_qkv=False)
        _in_step_stage(kw, ranked, args.in_step)


if __name__ == "__main__":
    main()
