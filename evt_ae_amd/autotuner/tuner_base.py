"""Tile autotuner base: candidate enumeration, sqlite result cache, timing.

Mirror of python/gtl/compiler/autotuner/tuner_base.py:28-289 of the reference
(`AutoTunerBase`: sqlite `tuner_cache.db`, key = problem + dtypes + layouts + the
seven epilogue-node counts :107-152, `get_best_config` :263-270).  The search
space is this backend's (workgroup tile, wave grid, LDS stages, k-depth,
raster group) instead of CUTLASS tile descriptions x swizzling functors, and
timing uses HIP events on the current stream instead of a torch.profiler sum.

Tuning runs only when EVT_AUTOTUNE=1 and a GPU is present; otherwise a cached
row or the analytic heuristic is used, so tracing never needs a device.
"""
from __future__ import annotations

import json
import logging
import os
import sqlite3
from contextlib import contextmanager
from dataclasses import asdict, fields, replace
from pathlib import Path
from typing import List, Optional, Sequence, Tuple

import torch

from ..codegen import KernelSpec, TileConfig, reduction_lds_bytes
from ..ir import EpilogueIR

NUM_CUS = 256
ROTATE_BYTES = 320 << 20
LDS_LIMIT = 160 * 1024

DTYPE_BY_NAME = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32, "bool": torch.bool,
                 "i32": torch.int32, "i64": torch.int64, "u8": torch.uint8}


def default_cache_file() -> Path:
    return Path(os.environ.get("EVT_TUNER_CACHE", Path(__file__).resolve().parent / "tuner_cache.db"))


_FORCED_TILE: Optional[TileConfig] = None


@contextmanager
def force_tile(tile: TileConfig):
    """Every fast-path (DMA) problem traced inside the block uses `tile` instead
    of the cached / heuristic choice (tests of one pipeline variant, experiments)."""
    global _FORCED_TILE
    prev, _FORCED_TILE = _FORCED_TILE, tile
    try:
        yield
    finally:
        _FORCED_TILE = prev


log = logging.getLogger("evt_ae_amd.tuner")


def default_operand_sigma() -> Tuple[float, float]:
    """Standard deviations the tuner draws its A and B operands with.  The clock the part holds, and with it the
    ranking of tiles, depends on the bit activity of the operands, so candidates are timed on data distributed like
    the workload's: activations against weights, N(0, 1) x N(0, 0.02), unless EVT_TUNE_SIGMA="sa,sb" says otherwise
    (the fuser knows shapes, not distributions)."""
    env = os.environ.get("EVT_TUNE_SIGMA")
    if env:
        sa, sb = (float(x) for x in env.split(","))
        return sa, sb
    return 1.0, 0.02


class AutoTunerBase:
    table = "best_config"
    warmup_iterations = 10
    profile_iterations = 50
    # second stage (reference: gemm_tuner.py:102-137, the best tiles timed again with the epilogue in place): the
    # `second_stage_tiles` fastest candidates of the sweep are timed again, in turns, `second_stage_rounds` times
    second_stage_tiles = 3
    second_stage_rounds = 3

    def __init__(self, problem: Tuple[int, int, int, int], a_kc: bool, b_kc: bool, bf16: bool, dma: bool,
                 ir: EpilogueIR) -> None:
        self.M, self.N, self.K, self.L = problem
        self.a_kc, self.b_kc, self.bf16, self.dma, self.ir = a_kc, b_kc, bf16, dma, ir
        self.cache_file = default_cache_file()
        self.operand_sigma = default_operand_sigma()      # (sigma_A, sigma_B) of the timing operands
        self.failed: List[Tuple[TileConfig, str]] = []    # candidates that did not build or launch, and why

    # -- key (reference: tuner_base.py:107-152, gemm_tuner.py:95-100) -----------
    def epilogue_key(self) -> str:
        return "_".join(str(c) for c in self.ir.epilogue_counts())

    def key(self) -> str:
        e = "bf16" if self.bf16 else "f16"
        la = "R" if self.a_kc else "C"
        lb = "C" if self.b_kc else "R"
        align = "a8" if self.dma else "a1"
        return f"{self.M}_{self.N}_{self.K}_{e}_{e}_{la}_{lb}_{align}_{self.epilogue_key()}"

    # -- cache -------------------------------------------------------------------
    def _connect(self) -> sqlite3.Connection:
        con = sqlite3.connect(str(self.cache_file), timeout=30)
        con.execute(f"CREATE TABLE IF NOT EXISTS {self.table}(key TEXT PRIMARY KEY, config TEXT, us REAL)")
        return con

    def fetch_cached(self) -> Optional[TileConfig]:
        if not self.cache_file.exists():
            return None
        try:
            con = self._connect()
            row = con.execute(f"SELECT config FROM {self.table} WHERE key=?", (self.key(),)).fetchone()
            con.close()
        except sqlite3.Error:
            return None
        if row is None:
            return None
        cfg = json.loads(row[0])
        known = {f.name for f in fields(TileConfig)}
        if any(k not in known and v for k, v in cfg.items()):
            return None      # uses an option this version does not have: ignore the row
        tile = TileConfig(**{k: v for k, v in cfg.items() if k in known})
        # the key holds the epilogue's node counts, not its reduction states: a row tuned for another epilogue
        # with the same counts may be too small for this one's exchange area
        return tile if self.fits(tile) else None

    def store(self, tile: TileConfig, us: float) -> None:
        con = self._connect()
        with con:
            con.execute(f"INSERT OR REPLACE INTO {self.table} VALUES (?,?,?)",
                        (self.key(), json.dumps(asdict(tile), sort_keys=True), us))
        con.close()

    # -- search space --------------------------------------------------------------
    def candidates(self) -> List[TileConfig]:
        out = []
        if self.dma:
            # (bm, bn, bk, wave grid, LDS stages, pipeline): plain ring (0), look-ahead ring (1),
            # ping-pong with two barriers (2) or one barrier (3) per k-tile
            shapes = [(256, 256, 64, 4, 2, 2, 0), (256, 256, 64, 2, 4, 2, 0), (256, 256, 32, 4, 2, 4, 1),
                      (256, 256, 32, 2, 4, 4, 1), (256, 256, 32, 4, 2, 5, 1), (256, 256, 32, 2, 4, 5, 1),
                      (256, 128, 64, 4, 2, 2, 0), (256, 128, 64, 4, 2, 3, 1), (256, 128, 32, 4, 2, 4, 1),
                      (256, 128, 32, 4, 2, 6, 1),
                      (128, 256, 64, 2, 4, 2, 0), (128, 256, 64, 2, 4, 3, 1), (128, 256, 32, 2, 4, 4, 1),
                      (128, 256, 32, 2, 4, 6, 1),
                      (128, 128, 64, 2, 2, 2, 0), (128, 128, 64, 2, 2, 4, 1), (128, 128, 32, 2, 2, 4, 1),
                      (64, 64, 64, 2, 2, 2, 0), (64, 64, 32, 2, 2, 2, 0)]
            for pipe in (2, 3):
                shapes += [(256, 256, 64, 4, 2, 2, pipe), (256, 256, 64, 2, 4, 2, pipe), (256, 256, 32, 2, 4, 4, pipe),
                           (256, 256, 32, 4, 2, 4, pipe), (256, 128, 64, 4, 2, 3, pipe), (128, 256, 64, 2, 4, 3, pipe),
                           (128, 256, 32, 2, 4, 4, pipe), (128, 128, 64, 2, 4, 4, pipe),
                           # two stages: 64 KB of LDS, so two such workgroups share a CU and one's epilogue runs
                           # under the other's main loop (measured 12-17 % faster than four stages on 128 x 128)
                           (128, 128, 64, 4, 2, 2, pipe), (128, 128, 64, 2, 4, 2, pipe)]
            # options of the one-barrier ping-pong loop (pipe 4 + flags, see TileConfig.pipe)
            for pipe in (5, 6, 7):
                shapes += [(256, 256, 64, 4, 2, 2, pipe), (256, 256, 64, 2, 4, 2, pipe)]
            for pipe in (5, 6, 7, 8, 10):
                shapes += [(256, 128, 64, 4, 2, 3, pipe), (128, 256, 64, 2, 4, 3, pipe)]
            # the same loops with every k-tile split between the two wave groups (pipe 16 + p): 128 x 64 / 64 x 128
            # wave tiles in the loop, a quarter fewer LDS reads per MFMA, one exchange of accumulators through LDS
            # behind it (measured 2.5-4.4 % faster than the best unsplit loop on 8192 x 1024 x 4096 with row
            # statistics, level on the same product with per-column sums)
            for pipe in (21, 26, 27):
                shapes += [(256, 128, 64, 4, 2, 3, pipe), (128, 256, 64, 2, 4, 3, pipe)]
            # one wave per SIMD (pipe 12): 64 x 64 wave tiles on 128 x 128 (measured 8-19 % faster than eight
            # waves on the 4096 x 1024 and 1024 x 4096 products of an encoder layer), 64 x 128 on the larger ones
            shapes += [(128, 128, 64, 2, 2, 3, 12), (128, 128, 64, 2, 2, 4, 12), (256, 128, 64, 2, 2, 3, 12),
                       (128, 256, 64, 2, 2, 3, 12),
                       # at most 80 KB of LDS and 256 registers: two such workgroups share a CU, one's epilogue runs
                       # under the other's main loop (measured 1.36 x over one per CU on the classifier problem,
                       # where the ping-pong tiles that walk still win)
                       (128, 256, 32, 2, 2, 3, 12), (256, 128, 32, 4, 1, 3, 12), (128, 128, 64, 2, 2, 2, 12)]
            # narrow outputs (GCN's 736389 x 64 products): a tile wider than the problem leaves every tile partial,
            # which costs the epilogue its check-free path and the main loop half its MFMAs; measured on
            # 736389 x 64 x 64 with two residual loads 459 us on 256 x 128 tiles, 61 us on 128 x 64
            if self.N <= 64 or self.N % 128 == 64 or self.K <= 64:
                shapes += [(128, 64, 64, 4, 1, 2, 0), (128, 64, 64, 2, 2, 2, 0), (256, 64, 64, 4, 1, 2, 0),
                           (256, 64, 64, 4, 2, 2, 0)]
            if self.M <= 64 or self.M % 128 == 64 or self.K <= 64:
                shapes += [(64, 128, 64, 1, 4, 2, 0), (64, 128, 64, 2, 2, 2, 0), (64, 256, 64, 1, 4, 2, 0),
                           (64, 256, 64, 2, 4, 2, 0)]
            if self.N == 512:     # one tile spans the rows: row statistics complete inside the workgroup
                shapes += [(128, 512, 64, 2, 4, 2, 0), (64, 512, 64, 1, 8, 2, 0),
                           # 32 x 256 wave tiles: 8 columns per lane halve the cross-lane steps per element of a
                           # per-row reduction
                           (128, 512, 64, 4, 2, 2, 0)]
        else:
            shapes = [(128, 128, 32, 2, 2, 2, 0), (64, 64, 32, 2, 2, 2, 0)]
        if self.dma and self.K <= 64:
            # the whole K extent fits one tile: a single LDS stage leaves room for more workgroups per CU
            bk = 64 if self.K > 32 else 32
            shapes += [(bm, bn, bk, wm, wn, 1, 0) for (bm, bn, _, wm, wn, st, pipe) in shapes if pipe == 0 and st == 2]
        for bm, bn, bk, wm, wn, st, pipe in shapes:
            t = TileConfig(bm, bn, bk, wm, wn, st, self.dma, 4, pipe)
            if self.fits(t) and t not in out:
                out.append(t)
        # many more tiles than CUs: workgroups that walk over 2, 4 or 8 tiles of a row block (ping-pong tiles
        # with two or three stages; fits() knows the other conditions), as long as every CU still gets one
        for t in list(out):
            tiles_n = -(-self.N // t.bn)
            tiles = -(-self.M // t.bm) * tiles_n * self.L
            if t.pipe in (2, 3) and t.stages <= 3 and tiles >= 4 * NUM_CUS:
                for walk in (2, 4, 8):
                    tw = replace(t, walk=walk)
                    if walk <= tiles_n and tiles // walk >= NUM_CUS and self.fits(tw) and tw not in out:
                        out.append(tw)
        return out

    def fits(self, t: TileConfig) -> bool:
        """The tile's stages fit the LDS and hold this epilogue's reduction exchange area."""
        need = reduction_lds_bytes(t, self.ir.row_state, self.ir.col_state)
        if t.walk > 1:
            # the epilogue's exchange area is the one stage the ring leaves free between tiles; the running row
            # states sit behind the stages
            return (2 <= t.pipe <= 11 and not self.ir.col_state and need <= t.stage_bytes()
                    and self.K % t.bk == 0 and self.K // t.bk >= t.stages
                    and t.lds_bytes() + t.bm * max(1, self.ir.row_state) * 4 <= LDS_LIMIT)
        return need <= t.lds_bytes() <= LDS_LIMIT

    def heuristic(self) -> TileConfig:
        """Pick the candidate with the lowest modelled time: number of
        workgroup rounds on 256 CUs x work per tile / efficiency of the tile."""
        eff = {(256, 256): 1.0, (256, 128): 0.85, (128, 256): 0.85, (128, 128): 0.7, (64, 64): 0.3,
               (128, 64): 0.5, (64, 128): 0.5, (256, 64): 0.45, (64, 256): 0.45}
        # K fits one k-tile: nothing to pipeline and next to no arithmetic, the launch streams its operands in and its
        # output out.  What counts is the area the tiles cover (the edge tiles of a 264 x 264 batch cost a whole
        # workgroup each) and how many workgroups a CU holds; measured on the reference's batched K = 64 problems,
        # single-stage 128 x 64 tiles with 4 x 1 waves lead or tie everywhere (1536 x 264 x 264 x 64: 128 us
        # against 155 on 128 x 128 and 178 on 64 x 64; 512 x 512 x 512 x 64: 59.7 against 72.4 and 68.2 on the
        # ping-pong 256 x 256)
        one_k_tile = self.dma and self.K <= 64
        eff_stream = {(128, 64): 1.0, (256, 64): 0.95, (64, 128): 0.95, (128, 512): 0.95, (256, 128): 0.9,
                      (128, 256): 0.9, (128, 128): 0.85, (256, 256): 0.8, (64, 64): 0.7}
        best, best_cost = None, None
        for t in self.candidates():
            tiles = -(-self.M // t.bm) * -(-self.N // t.bn) * self.L
            if one_k_tile:
                if t.stages != 1 or t.pipe != 0 or t.walk > 1:
                    continue
                cost = tiles * t.bm * t.bn / eff_stream.get((t.bm, t.bn), 0.6)
                if t.bn > self.N or t.bm > self.M:
                    cost *= 2.0
                if self.ir.row_state and t.bn >= self.N:
                    cost *= 0.6         # the whole row in one tile: its statistics finish inside the workgroup
                cost *= 1.0 + (0.002 if t.wm < t.wn else 0.0)
                if best_cost is None or cost < best_cost:
                    best, best_cost = t, cost
                continue
            # untuned default: a ping-pong tile or the plain double-buffered ring, or, for one round of 128 x 128
            # tiles with a CU each, the one-wave-per-SIMD loop (measured 8-19 % faster there than eight waves)
            solo = t.pipe == 12 and (t.bm, t.bn, t.stages) == (128, 128, 3) and tiles <= NUM_CUS and self.K >= 4 * t.bk
            # the one-barrier ping-pong loops with the options that won the sweeps of the reference's large
            # products: 256 x 256 with 2 x 4 waves and pipe 7 (within 1 % of the best on every one of twelve
            # shapes and layouts, 5-20 % ahead of 4 x 2 waves with two barriers), pipe 5 / 10 on the half tiles
            tuned = (t.pipe, t.bm, t.bn, t.stages) in ((7, 256, 256, 2), (5, 256, 128, 3), (10, 128, 256, 3))
            if (t.pipe not in (0, 2) and not solo and not tuned) or t.stages == 1 or t.walk > 1:
                continue
            wg_per_cu = max(1, min(2, LDS_LIMIT // t.lds_bytes())) if t.bm * t.bn <= 128 * 128 else 1
            if tiles <= NUM_CUS:
                wg_per_cu = 1       # one workgroup per CU at most: nothing shares a CU's throughput
            rounds = -(-tiles // (NUM_CUS * wg_per_cu))
            loop = 1.3 if solo else 1.2 if tuned else 1.15 if t.pipe == 2 else 1.0
            cost = rounds * wg_per_cu * t.bm * t.bn / (eff.get((t.bm, t.bn), 0.5) * loop)
            if t.bn > self.N or t.bm > self.M:
                cost *= 2.0         # no tile is whole: every epilogue access is checked (measured 3-7 x on narrow outputs)
            # few tiles, a long K and a small output: the kernel splits K over several workgroups per tile (the
            # rule of the generated host code); the exchange of partial tiles eats about half of the gain, and
            # more than four splits are not rewarded here
            kt = -(-self.K // t.bk)
            if t.stages > 1 and tiles * 2 <= NUM_CUS and kt >= 8 and self.M * self.N * self.L <= (1 << 20):
                cost /= 0.5 * max(2, min(4, NUM_CUS // tiles, kt // 4))
            # ties: deeper k-tiles first; fewer stages when several workgroups share a CU (they hide each other's
            # latency and epilogue, and two 2-stage workgroups fit where one 4-stage one does), more stages when a
            # workgroup has its CU to itself (measured both ways on 128 x 128 tiles)
            stage_pref = 0.005 * (t.stages - 2) if tiles > NUM_CUS else -0.005 * (t.stages - 2)
            # 256 x 256: 2 x 4 waves (128 x 64 wave tiles) ahead of 4 x 2 in every layout measured
            wave_pref = (-0.03 if t.wm < t.wn else 0.0) if (t.bm, t.bn) == (256, 256) else (0.002 if t.wm < t.wn else 0.0)
            cost *= 1.0 + 0.01 * (64 // t.bk - 1) + stage_pref + wave_pref
            if best_cost is None or cost < best_cost:
                best, best_cost = t, cost
        if best is None and one_k_tile:      # no single-stage tile holds this epilogue: the general model
            one_k_tile_was, self_k = True, self.K
            try:
                self.K = 65
                return self.heuristic()
            finally:
                self.K = self_k
        return best

    # -- timing ----------------------------------------------------------------------
    def make_arguments(self):
        """Synthetic operands and epilogue tensors for profiling."""
        from .. import jit
        dev = "cuda"
        dt = torch.bfloat16 if self.bf16 else torch.float16
        M, N, K, L = self.M, self.N, self.K, self.L
        sa, sb = self.operand_sigma
        # rows padded to the transfer path's 8 elements where an extent is no multiple of 8 (what the fused op's
        # padded copies look like, FusedGEMM.pad)
        r8 = (lambda v: (v + 7) & ~7) if self.dma else (lambda v: v)
        lda, ldb = r8(K if self.a_kc else M), r8(K if self.b_kc else N)
        A = (torch.randn((L, M, lda) if self.a_kc else (L, K, lda), device=dev, dtype=torch.float32) * sa).to(dt)
        B = (torch.randn((L, N, ldb) if self.b_kc else (L, K, ldb), device=dev, dtype=torch.float32) * sb).to(dt)
        a = jit.EvtArgs()
        a.M, a.N, a.K, a.L = M, N, K, L
        a.A, a.lda, a.batch_stride_A = A.data_ptr(), lda, A.shape[1] * lda
        a.B, a.ldb, a.batch_stride_B = B.data_ptr(), ldb, B.shape[1] * ldb
        a.num_tensors, a.num_scalars = len(self.ir.slots), len(self.ir.scalars)
        keep = [A, B]
        nbytes = (A.numel() + B.numel()) * 2
        for k, s in enumerate(self.ir.slots):
            st = s.strides
            span = ((L - 1) // st.l_div) * st.stride_l + (st.l_div - 1) * st.stride_l2 + (M - 1) * st.stride_m + (N - 1) * st.stride_n + 1
            dtype = DTYPE_BY_NAME[s.dtype]
            if dtype.is_floating_point:
                t = torch.randn(span, device=dev, dtype=torch.float32).to(dtype)
            else:
                t = torch.zeros(span, device=dev, dtype=dtype)
            keep.append(t)
            nbytes += t.numel() * t.element_size()
            ta = a.tensors[k]
            ta.ptr, ta.stride_l, ta.stride_m, ta.stride_n, ta.l_div = t.data_ptr(), st.stride_l, st.stride_m, st.stride_n, st.l_div
            ta.l_mod, ta.stride_l2 = st.l_mod, st.stride_l2
        for i, v in enumerate(self.ir.scalars):
            a.scalars[i] = v
        return a, keep, nbytes

    def argument_sets(self):
        """Enough independent buffer sets (> 256 MB together) that a launch never
        finds its operands in the Infinity Cache, as in a real pipeline."""
        if getattr(self, "_sets", None) is None:
            first = self.make_arguments()
            n = max(2, -(-ROTATE_BYTES // max(first[2], 1)))
            self._sets = [first] + [self.make_arguments() for _ in range(min(n, 12) - 1)]
        return self._sets

    def profile(self, tile: TileConfig) -> float:
        from .. import jit
        module = jit.load_module(self.ir, KernelSpec.for_problem(self.K, self.a_kc, self.b_kc, self.bf16, tile, self.M, self.N))
        sets = self.argument_sets()
        stream = torch.cuda.current_stream().cuda_stream
        nbytes = module.workspace_bytes(sets[0][0])
        ws = torch.empty(max(nbytes, 4), dtype=torch.uint8, device="cuda")
        module.workspace_init(ws.data_ptr(), nbytes, stream)
        for i in range(self.warmup_iterations):
            module.launch(sets[i % len(sets)][0], ws.data_ptr(), nbytes, stream)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(self.profile_iterations):
            module.launch(sets[i % len(sets)][0], ws.data_ptr(), nbytes, stream)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / self.profile_iterations

    def sweep(self, report=None) -> List[Tuple[float, TileConfig]]:
        """Time every candidate once; a candidate that fails to build or to launch is recorded in `self.failed`
        and logged, never dropped silently.  `report(tile, us or None, error or None)` is called per candidate."""
        results = []
        self.failed = []
        for tile in self.candidates():
            try:
                us = self.profile(tile)
            except RuntimeError as exc:
                self.failed.append((tile, str(exc)))
                log.warning("tuner: candidate %s of %s failed: %s", tile.tag(), self.key(), str(exc).splitlines()[0][:300])
                if report is not None:
                    report(tile, None, str(exc))
                continue
            results.append((us, tile))
            if report is not None:
                report(tile, us, None)
        return results

    def second_stage(self, results: List[Tuple[float, TileConfig]], report=None) -> Tuple[float, TileConfig]:
        """The fastest few tiles of the sweep timed again, in turns (so that clock drift and neighbours on the
        machine hit all of them alike); the winner is the tile with the lowest median."""
        top = sorted(results, key=lambda r: r[0])[:max(1, self.second_stage_tiles)]
        if len(top) == 1 or self.second_stage_rounds <= 0:
            return top[0]
        samples = {tile: [us] for us, tile in top}
        for _ in range(self.second_stage_rounds):
            for _, tile in top:
                try:
                    samples[tile].append(self.profile(tile))
                except RuntimeError as exc:
                    self.failed.append((tile, str(exc)))
                    log.warning("tuner: candidate %s of %s failed in the second stage: %s", tile.tag(), self.key(),
                                str(exc).splitlines()[0][:300])
        med = {tile: sorted(v)[len(v) // 2] for tile, v in samples.items()}
        best = min(med, key=med.get)
        if report is not None:
            for tile, us in med.items():
                report(tile, us, "second stage")
        return med[best], best

    def tune(self) -> TileConfig:
        results = self.sweep()
        if not results:
            log.warning("tuner: no candidate of %s could be timed (%d failed); using the modelled tile", self.key(), len(self.failed))
            return self.heuristic()
        best_us, best = self.second_stage(results)
        self.store(best, best_us)
        return best

    def get_best_config(self) -> TileConfig:
        if _FORCED_TILE is not None and self.dma:
            return _FORCED_TILE
        cached = self.fetch_cached()
        if cached is not None:
            return cached
        if os.environ.get("EVT_AUTOTUNE", "0") == "1" and torch.cuda.is_available():
            return self.tune()
        return self.heuristic()
