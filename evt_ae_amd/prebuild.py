"""Ahead-of-time build of every kernel module the tests, the smoke check and the
benchmark use, so that nothing has to be compiled on the GPU box.

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
    for cfg in W.CONFIGS:
        for shapes in (None, W.SMALL_SHAPES[cfg], W.RAGGED_SHAPES[cfg], W.UNALIGNED_SHAPES[cfg], W.GOLDEN_SHAPES[cfg]):
            gm = W.fuse(W.CONFIGS[cfg].module(), _shapes_of(cfg, shapes))
            if shapes is None:   # the benchmark's --clock-probe builds of the headline kernels
                op = W.fused_nodes(gm)[0].target
                jit.load_module(op.ir, op.spec, clock_probe=True)
    # shapes of single tests: the determinism test's classifier, bf16 operands
    W.fuse(W.CONFIGS[5].module(), _shapes_of(5, dict(M=256, N=8192, K=256)))
    W.fuse(W.CONFIGS[1].module(), [torch.empty(t.shape, dtype=torch.bfloat16 if t.dtype == torch.float16 else t.dtype,
                                               device="meta") for t in _shapes_of(1, W.SMALL_SHAPES[1])])
    for name, (cls, _) in W.RANDOM_PATTERNS.items():
        W.fuse(cls(), _meta(W.pattern_inputs(name)))
    W.fuse(W.FoldConsecutiveBatches(), _meta(W.fold_consecutive_inputs()))
    for name, (cls, _) in W.MULTI_ANCHOR_PATTERNS.items():
        W.fuse(cls(), _meta(W.pattern_inputs(name)))
    for name, (cls, _) in W.ROW_ANCHOR_PATTERNS.items():
        W.fuse(cls(), _meta(W.pattern_inputs(name)))
    for anchor in ("softmax", "softmax_backward", "layernorm", "layernorm_backward"):
        for n in W.ROW_EDGE_LENGTHS:
            for dt in W.ROW_EDGE_DTYPES:
                mod, ins = W.row_edge_case(anchor, n, dt)
                W.fuse(mod, _meta(ins))
    from .passes import pass_decomposition, pass_fusion
    for n in W.AFFINE_LN_LENGTHS:
        mod, ins = W.affine_layer_norm(n)
        W.fuse(mod, _meta(ins), passes=[pass_decomposition, pass_fusion])
    from .evt_fuser import EVTFuser
    for swap in (True, False):          # column-major outputs: operands exchanged, and the strided stores without
        EVTFuser.allow_transpose = swap
        try:
            for transposed in (False, True):
                mod, ins = W.head_merge_bias_grad(transposed=transposed)
                W.fuse(mod, _meta(ins))
                mod, ins = W.head_merge_bias_grad(transposed=transposed, **W.HEAD_MERGE_MANY_PARTIALS)
                W.fuse(mod, _meta(ins))
            for batched in (False, True):
                for dtype in (torch.float16, torch.bfloat16):
                    mod, ins = W.column_major_store(batched, dtype=dtype)
                    W.fuse(mod, _meta(ins))
        finally:
            EVTFuser.allow_transpose = True
    for anchor in W.RANDOM_EPILOGUE_ANCHORS:
        for seed in W.RANDOM_EPILOGUE_SEEDS[:12 if anchor == "mm" else 6]:
            mod, ins = W.random_epilogue(seed, anchor)
            W.fuse(mod, _meta(ins))
            if anchor in ("mm", "bmm") and seed < 6:
                mod, ins = W.random_epilogue(seed, anchor, column_major=True)
                W.fuse(mod, _meta(ins))
    for anchor, n, dt in W.ROW_LONG_CASES:
        mod, ins = W.row_edge_case(anchor, n, dt)
        W.fuse(mod, _meta(ins))
    for name, (cls, shapes, _) in W.ROW_BENCH.items():
        W.fuse(cls(), [torch.empty(sh, dtype=dt, device="meta") for sh, dt in shapes])
    from .aot_helper import aot_capture, evt_backend
    # traced on the meta device: its dtype rules are the GPU's (fp32 layer norm statistics for fp16 inputs), so the
    # modules registered here are the ones a GPU run asks for
    aot_capture(*W.mlp_classifier(device="meta"))
    aot_capture(*W.mlp_classifier())
    aot_capture(*W.encoder_layer(device="meta"))
    aot_capture(*W.encoder_layer(device="meta", fused_qkv=False))
    aot_capture(*W.dropout_block(device="meta"))
    aot_capture(*W.decoder_block(device="meta"))
    aot_capture(*W.decoder_block(device="meta", dtype=torch.bfloat16))
    aot_capture(*W.encoder_layer(device="meta", **W.ENCODER_BENCH))      # bench.py's training-step leg
    # the same step through torch.compile: Dynamo's graph differs slightly, so
    # its kernels are registered as well (tracing stops at the first launch
    # when there is no GPU)
    model, inputs = W.mlp_classifier()
    try:
        torch.compile(model, backend=evt_backend)(*inputs)
    except RuntimeError as e:
        if "HIP device only" not in str(e):
            raise
    from .passes import pass_decomposition, pass_fusion
    W.fuse(W.Dropout1Undecomposed(), _meta(W.pattern_inputs("dropout1")), passes=[pass_decomposition, pass_fusion])
    from .autotuner.tuner_base import force_tile
    from .codegen import TileConfig
    for cfg, shapes in W.SPLIT_K_SHAPES.items():
        W.fuse(W.CONFIGS[cfg].module(), _shapes_of(cfg, shapes))
        for tile in W.SPLIT_K_TILES:
            with force_tile(TileConfig(*tile)):
                W.fuse(W.CONFIGS[cfg].module(), _shapes_of(cfg, shapes))
    for tile in W.pipeline_tiles():
        with force_tile(tile):
            for cfg in W.CONFIGS:
                W.fuse(W.CONFIGS[cfg].module(), _shapes_of(cfg, W.PIPELINE_SHAPES[cfg]))
    for cfg, shapes, tile in W.walk_cases():
        with force_tile(tile):
            W.fuse(W.CONFIGS[cfg].module(), _shapes_of(cfg, shapes))
    from .codegen import TileConfig
    with force_tile(TileConfig(*W.NO_ALLOC_TILE)):
        for cfg, cases in W.NO_ALLOC_SHAPES.items():
            for shapes in cases:
                W.fuse(W.CONFIGS[cfg].module(), _shapes_of(cfg, shapes))
    cfg, shapes, tile = W.NO_ALLOC_TOO_BIG
    with force_tile(TileConfig(*tile)):
        W.fuse(W.CONFIGS[cfg].module(), _shapes_of(cfg, shapes))
    for name, (cls, _) in W.REFERENCE_PATTERNS.items():
        g = torch.Generator(device="cpu").manual_seed(0)
        # shapes only: generate on CPU lazily is costly for the big patterns, so
        # take shapes from a meta run of the generator functions
        with torch.device("meta"):
            pass
        ins = W.pattern_inputs(name) if name not in ("mm10", "mm11") else None
        if ins is None:
            shapes = {"mm10": [(16384, 1024), (1024, 4096)], "mm11": [(33792, 768), (33792, 768)]}[name]
            metas = [torch.empty(s, dtype=torch.half, device="meta") for s in shapes]
        else:
            metas = _meta(ins)
        W.fuse(cls(), metas)
    return jit.registered_modules()


def build_all(jobs: int = 8, force: bool = False, verbose: bool = True) -> List[jit.LazyModule]:
    mods = register_all()
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
