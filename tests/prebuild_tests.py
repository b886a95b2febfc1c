"""Ahead-of-time build of the kernel modules the tests use, so that nothing has to
be compiled on the GPU box: every case of the test catalogue (tests/patterns.py)
is traced on meta tensors exactly as the test will trace it, which registers its
kernel module; evt_ae_amd.prebuild compiles what is registered.

    python -m tests.prebuild_tests [--force]      # from the repository root
"""
from __future__ import annotations

import sys

import torch

from evt_ae_amd import prebuild
from evt_ae_amd.prebuild import _meta, _shapes_of
from tests import patterns as W


def register_tests() -> None:
    for cfg in W.CONFIGS:
        for shapes in (W.RAGGED_SHAPES[cfg], W.UNALIGNED_SHAPES[cfg], W.GOLDEN_SHAPES[cfg]):
            W.fuse(W.CONFIGS[cfg].module(), _shapes_of(cfg, shapes))
    # shapes of single tests: the determinism test's classifier, bf16 operands
    W.fuse(W.CONFIGS[5].module(), _shapes_of(5, dict(M=256, N=8192, K=256)))
    W.fuse(W.CONFIGS[1].module(), [torch.empty(t.shape, dtype=torch.bfloat16 if t.dtype == torch.float16 else t.dtype,
                                               device="meta") for t in _shapes_of(1, W.SMALL_SHAPES[1])])
    for name, (cls, _) in W.RANDOM_PATTERNS.items():
        W.fuse(cls(), _meta(W.pattern_inputs(name)))
    for dims in W.MaskedScores.GPU_DIMS:
        W.fuse(W.MaskedScores(dims), _meta(W.MaskedScores.inputs(dims=dims)))
    W.fuse(W.TwoMaskedLayers(), _meta(W.TwoMaskedLayers.inputs()))
    W.fuse(W.TwoMaskedLayers(), _meta(W.TwoMaskedLayers.inputs(m=1000, n=520)))
    W.fuse(W.FoldConsecutiveBatches(), _meta(W.fold_consecutive_inputs()))
    W.fuse(W.FoldedLogSumExp(), _meta(W.fold_consecutive_inputs()))
    W.fuse(W.FoldedModuloVariance(), _meta(W.fold_consecutive_inputs()))
    for name, (cls, _) in W.MULTI_ANCHOR_PATTERNS.items():
        W.fuse(cls(), _meta(W.pattern_inputs(name)))
    for name, (cls, _) in W.ROW_ANCHOR_PATTERNS.items():
        W.fuse(cls(), _meta(W.pattern_inputs(name)))
    for anchor in ("softmax", "softmax_backward", "layernorm", "layernorm_backward"):
        for n in W.ROW_EDGE_LENGTHS:
            for dt in W.ROW_EDGE_DTYPES:
                mod, ins = W.row_edge_case(anchor, n, dt)
                W.fuse(mod, _meta(ins))
    from evt_ae_amd.passes import pass_decomposition, pass_fusion
    for n in W.AFFINE_LN_LENGTHS:
        mod, ins = W.affine_layer_norm(n)
        W.fuse(mod, _meta(ins), passes=[pass_decomposition, pass_fusion])
    from evt_ae_amd.evt_fuser import EVTFuser
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
    from evt_ae_amd.aot_helper import aot_capture, evt_backend
    # traced on the meta device: its dtype rules are the GPU's (fp32 layer norm statistics for fp16 inputs), so the
    # modules registered here are the ones a GPU run asks for
    aot_capture(*W.mlp_classifier(device="meta"))
    aot_capture(*W.mlp_classifier())
    aot_capture(*W.encoder_layer(device="meta"))
    aot_capture(*W.encoder_layer(device="meta", fused_qkv=False))
    aot_capture(*W.dropout_block(device="meta"))
    aot_capture(*W.decoder_block(device="meta"))
    aot_capture(*W.decoder_block(device="meta", dtype=torch.bfloat16))
    # the same step through torch.compile: Dynamo's graph differs slightly, so its kernels are registered as well
    # (tracing stops at the first launch when there is no GPU)
    model, inputs = W.mlp_classifier()
    try:
        torch.compile(model, backend=evt_backend)(*inputs)
    except RuntimeError as e:
        if "HIP device only" not in str(e):
            raise
    W.fuse(W.Dropout1Undecomposed(), _meta(W.pattern_inputs("dropout1")), passes=[pass_decomposition, pass_fusion])
    from evt_ae_amd.autotuner.tuner_base import force_tile
    from evt_ae_amd.codegen import TileConfig
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
    with force_tile(TileConfig(*W.NO_ALLOC_TILE)):
        for cfg, cases in W.NO_ALLOC_SHAPES.items():
            for shapes in cases:
                W.fuse(W.CONFIGS[cfg].module(), _shapes_of(cfg, shapes))
    cfg, shapes, tile = W.NO_ALLOC_TOO_BIG
    with force_tile(TileConfig(*tile)):
        W.fuse(W.CONFIGS[cfg].module(), _shapes_of(cfg, shapes))
    # the reference's tuner-cache keys (tests/golden/reference_tuner_keys.json): one synthetic epilogue per key
    for _table, _key, case in W.reference_key_cases():
        W.fuse(*W.counted_epilogue(case))
    for _key, _anchor, _rows, _cols, mod, metas in W.reference_row_key_cases():
        W.fuse(mod, metas)
    from evt_ae_amd.evt_fuser import FusedGEMM
    floor = FusedGEMM.pad_min_flops
    try:
        for FusedGEMM.pad_min_flops in (0.0, float("inf")):      # padded operands, and the element-wise path
            for i in range(len(W.PADDED_GEMM_CASES)):
                W.fuse(*W.counted_epilogue(W.padded_gemm_case(i)))
    finally:
        FusedGEMM.pad_min_flops = floor
    for name, (cls, _) in W.REFERENCE_PATTERNS.items():
        if name in ("mm10", "mm11"):      # shapes only: their inputs are large
            shapes = {"mm10": [(16384, 1024), (1024, 4096)], "mm11": [(33792, 768), (33792, 768)]}[name]
            metas = [torch.empty(s, dtype=torch.half, device="meta") for s in shapes]
        else:
            metas = _meta(W.pattern_inputs(name))
        W.fuse(cls(), metas)


def build_all(jobs: int = 8, force: bool = False, verbose: bool = True):
    """The benchmark's and the tests' modules together."""
    return prebuild.build_all(jobs=jobs, force=force, verbose=verbose, register=register_tests)


if __name__ == "__main__":
    build_all(force="--force" in sys.argv)
