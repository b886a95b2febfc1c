"""The test catalogue: everything the tests run beyond the benchmark's own
workloads (evt_ae_amd.workloads, whose names are visible here as well, so a test
imports this module alone).  The graph patterns of the reference's fuser tests
(unittest/evt_fuser/mm.py:30-236, bmm.py:29-94, dropout.py, softmax.py,
layernorm*.py) restated as ATen-level modules with seeded inputs, shapes that
reach the kernels' edges (ragged, unaligned, split-K, pipeline variants, walking
workgroups), seeded random epilogue trees, multi-anchor graphs and small models
for the training-step tests."""
from __future__ import annotations

import math
import operator
from typing import List

import torch

from evt_ae_amd.workloads import *          # noqa: F401,F403
from evt_ae_amd.workloads import _randn     # noqa: F401

aten = torch.ops.aten

RAGGED_SHAPES = {
    1: dict(M=100, N=72, K=40),
    2: dict(L=2, S=77, D=24),
    3: dict(M=33, N=136, K=72),
    4: dict(M=130, N=56, K=88),
    5: dict(M=37, N=1000, K=64),
}
# shapes of the committed golden fixtures (tests/golden)
GOLDEN_SHAPES = {
    1: dict(M=64, N=96, K=64),
    2: dict(L=2, S=64, D=32),
    3: dict(M=64, N=128, K=64),
    4: dict(M=96, N=64, K=64),
    5: dict(M=32, N=512, K=64),
}
# several workgroup tiles in M and N, several k-tiles with a K tail: the shapes
# the main-loop pipeline variants (PIPELINE_TILES) are checked on
# few output tiles and a long K: the kernels split K over several workgroups per tile (K tail included)
SPLIT_K_SHAPES = {
    1: dict(M=264, N=200, K=2120),
    3: dict(M=136, N=520, K=4168),
    4: dict(M=520, N=136, K=3080),
    5: dict(M=72, N=1032, K=2056),
}

# tiles the split-K shapes are also run with (besides the tuner's own choice): a ping-pong loop and the
# one-wave-per-SIMD loop, (bm, bn, bk, wm, wn, stages, dma, group_m, pipe)
SPLIT_K_TILES = ((128, 256, 64, 2, 4, 3, True, 4, 10), (128, 128, 64, 2, 2, 3, True, 4, 12))

PIPELINE_SHAPES = {
    1: dict(M=300, N=264, K=200),
    2: dict(L=2, S=200, D=72),
    3: dict(M=264, N=520, K=328),
    4: dict(M=520, N=264, K=136),
    5: dict(M=136, N=1032, K=264),
}
# no dimension a multiple of 8: operands are not 16-byte aligned row by row, so
# these run the element-wise (safe) operand path
UNALIGNED_SHAPES = {
    1: dict(M=33, N=17, K=41),
    2: dict(L=2, S=45, D=19),
    3: dict(M=70, N=129, K=33),
    4: dict(M=65, N=31, K=50),
    5: dict(M=19, N=333, K=27),
}


# evt_launch_static against evt_launch: (config, first problem, a smaller second one) through one module; the
# classifier's 6 MiB of partial results exceed the static array
NO_ALLOC_TILE = (128, 128, 64, 2, 4, 2, True, 4, 2)
NO_ALLOC_SHAPES = {3: (dict(M=1024, N=512, K=256), dict(M=384, N=256, K=128)),
                   4: (dict(M=1024, N=512, K=256), dict(M=384, N=256, K=128))}
NO_ALLOC_TOO_BIG = (5, dict(M=1024, N=131072, K=64), (256, 256, 64, 4, 2, 2, True, 4, 2))


def pipeline_tiles():
    """Ping-pong main-loop variants (pipe 2: two barriers per k-tile, pipe 3:
    one), the one-wave-per-SIMD loop (pipe 12) and the ping-pong loops with split
    k-tiles (pipe 16 + p) on every stage count / k-depth / wave grid they are
    instantiated with."""
    from evt_ae_amd.codegen import TileConfig
    return [TileConfig(256, 256, 64, 4, 2, 2, True, 4, 2), TileConfig(128, 256, 64, 2, 4, 3, True, 4, 2),
            TileConfig(256, 256, 32, 2, 4, 4, True, 4, 2), TileConfig(256, 128, 64, 4, 2, 3, True, 4, 3),
            TileConfig(128, 256, 64, 2, 4, 3, True, 4, 3), TileConfig(256, 256, 64, 2, 4, 2, True, 4, 3),
            # options of the one-barrier loop: transfers issued among the LDS reads (both groups), barrier inside
            # group 0's MFMA phase
            TileConfig(128, 256, 64, 2, 4, 3, True, 4, 10), TileConfig(256, 128, 64, 4, 2, 3, True, 4, 11),
            TileConfig(256, 256, 64, 2, 4, 2, True, 4, 7),
            # one wave per SIMD: three and four stages, square and oblong wave tiles, two stages
            TileConfig(128, 128, 64, 2, 2, 3, True, 4, 12), TileConfig(128, 128, 64, 2, 2, 4, True, 4, 12),
            TileConfig(256, 128, 64, 2, 2, 3, True, 4, 12), TileConfig(128, 256, 64, 2, 2, 2, True, 4, 12),
            # k-tiles split between the wave groups (pipe 16 + p): loop wave tiles 128 x 64 and 64 x 128, epilogue
            # wave tiles of two row blocks and of one, three stages and two
            TileConfig(128, 256, 64, 2, 4, 3, True, 4, 21), TileConfig(128, 256, 64, 4, 2, 3, True, 4, 26),
            TileConfig(256, 128, 64, 4, 2, 3, True, 4, 27), TileConfig(128, 128, 64, 4, 2, 2, True, 4, 19)]


# Workgroups that walk over several tiles of a row block (TileConfig.walk): (config, shapes, tile).  K is a
# multiple of bk throughout (the walk's condition); N leaves a partial last tile and a last workgroup with fewer
# tiles than the others; M leaves a partial row block.
def walk_cases():
    from evt_ae_amd.codegen import TileConfig
    return [
        # per-row reductions only, 10 tiles along N in runs of 4 (4 + 4 + 2) and of 8 (8 + 2)
        (5, dict(M=300, N=2504, K=192), TileConfig(256, 256, 64, 4, 2, 2, True, 4, 2, 4)),
        (5, dict(M=300, N=2504, K=192), TileConfig(256, 256, 64, 4, 2, 2, True, 4, 3, 8)),
        # tile loads and stores + Welford statistics, three stages, 5 tiles in runs of 2
        (3, dict(M=200, N=1096, K=256), TileConfig(128, 256, 64, 2, 4, 3, True, 4, 3, 2)),
        # two k-tiles cannot prime three stages: the module falls back to a workgroup per tile
        (3, dict(M=200, N=1096, K=128), TileConfig(128, 256, 64, 2, 4, 3, True, 4, 3, 2)),
        # stores only, k-row B tile (columns regrouped after the main loop), transfers issued among the LDS reads
        (1, dict(M=300, N=1800, K=128), TileConfig(256, 256, 64, 2, 4, 2, True, 4, 6, 3)),
        # batched, softmax statistics + store
        (2, dict(L=3, S=520, D=128), TileConfig(128, 128, 64, 2, 4, 2, True, 4, 2, 2)),
    ]


# ---------------------------------------------------------------------------
# graph patterns of the reference's fuser tests
# ---------------------------------------------------------------------------

class MMPartition1(torch.nn.Module):   # mm.py:30-50  bias + GELU, two stores through views
    def forward(self, primals_1, view_11, primals_2):
        permute_24 = aten.permute(primals_1, [1, 0])
        mm_37 = aten.mm(view_11, permute_24)
        add_21 = aten.add(mm_37, primals_2)
        view_12 = aten.view(add_21, [512, 2, 4096])
        gelu = aten.gelu(view_12, approximate="tanh")
        view_13 = aten.view(gelu, [1024, 4096])
        return view_13, view_12


class MMPartition2(torch.nn.Module):   # mm.py:52-70  tiny M, bias + tanh
    def forward(self, select, primals_5, primals_6):
        permute_32 = aten.permute(primals_5, [1, 0])
        mm_45 = aten.mm(select, permute_32)
        add_29 = aten.add(mm_45, primals_6)
        tanh = aten.tanh(add_29)
        return tanh


class MMPartition3(torch.nn.Module):   # mm.py:72-91  view before the bias add
    def forward(self, view_93, primals_10, primals_11):
        permute_112 = aten.permute(primals_10, [1, 0])
        mm = aten.mm(view_93, permute_112)
        view = aten.view(mm, [512, 2, 1024])
        add = aten.add(view, primals_11)
        view_3 = aten.view(add, [512, 32, 64])
        return view_3


class MMPartition4(torch.nn.Module):   # mm.py:93-111  N = 2
    def forward(self, tanh, primals_41, primals_42):
        permute_123 = aten.permute(primals_41, [1, 0])
        mm_47 = aten.mm(tanh, permute_123)
        add = aten.add(mm_47, primals_42)
        view_39 = aten.view(add, [2, 2])
        return view_39


class MMPartition5(torch.nn.Module):   # mm.py:113-127  tanh_backward + column sum, K = 2
    def forward(self, A, B, tanh):
        mm = aten.mm(A, B)
        out = aten.tanh_backward(mm, tanh)
        sum = aten.sum(out, [0], True)
        return out, sum


class MMPartition6(torch.nn.Module):   # mm.py:129-146  residual adds, permuted output
    def forward(self, view_295, primals_12, add_17, view_299):
        mm_33 = aten.mm(view_295, primals_12)
        view_298 = aten.view(mm_33, [512, 4, 1024])
        add_18 = aten.add(view_298, add_17)
        add_19 = aten.add(add_18, view_299)
        permute_183 = aten.permute(add_19, [1, 0, 2])
        return permute_183


class MMPartition7(torch.nn.Module):   # mm.py:148-165  four outputs
    def forward(self, view_295, primals_12, add_17, view_299):
        mm_33 = aten.mm(view_295, primals_12)
        view_298 = aten.view(mm_33, [512, 4, 1024])
        add_18 = aten.add(view_298, add_17)
        add_19 = aten.add(add_18, view_299)
        view_183 = aten.view(add_19, [2048, 1024])
        return view_298, add_18, add_19, view_183


class MMPartition9(torch.nn.Module):   # mm.py:167-186  bias used twice
    def forward(self, select, primals_5, primals_6):
        permute_32 = aten.permute(primals_5, [1, 0])
        mm_45 = aten.mm(select, permute_32)
        add_29 = aten.add(mm_45, primals_6)
        tanh = aten.tanh(add_29)
        add_30 = aten.add(tanh, primals_6)
        return add_30


class MMPartition10(torch.nn.Module):  # mm.py:188-200  store + column sum, large M
    def forward(self, view_237, primals_34):
        mm_12 = aten.mm(view_237, primals_34)
        sum_6 = aten.sum(mm_12, [0], True)
        return mm_12, sum_6


class MMPartition11(torch.nn.Module):  # mm.py:202-214  weight gradient A^T B
    def forward(self, view_206, view_160):
        permute_142 = aten.permute(view_206, [1, 0])
        mm_9 = aten.mm(permute_142, view_160)
        return mm_9


class BMMPartition1(torch.nn.Module):  # bmm.py:29-46  permuted B, permuted + reshaped store
    def forward(self, view_5, view_7):
        permute_127 = aten.permute(view_5, [1, 0, 2])
        bmm_1 = aten.bmm(view_7, permute_127)
        permute_132 = aten.permute(bmm_1, [1, 0, 2])
        clone_3 = aten.clone(permute_132, memory_format=torch.contiguous_format)
        view_8 = aten.view(clone_3, [512, 2, 1024])
        view_9 = aten.view(view_8, [1024, 1024])
        return view_9


class BMMPartition3(torch.nn.Module):  # bmm.py:69-94  QK^T * scale + additive mask (mask output kept outside)
    def forward(self, view_3, view_4, primals_44, const_scalar0, const_scalar1, inv_const_scalar2):
        unsqueeze = aten.unsqueeze(primals_44, 1)
        unsqueeze_1 = aten.unsqueeze(unsqueeze, 2)
        mul_40 = aten.mul(unsqueeze_1, -1.0)
        add_37 = aten.add(mul_40, const_scalar0)
        mul_1 = aten.mul(add_37, const_scalar1)
        permute_125 = aten.permute(view_3, [1, 0, 2])
        permute_126 = aten.permute(view_4, [1, 2, 0])
        bmm = aten.bmm(permute_125, permute_126)
        view_6 = aten.view(bmm, [2, 16, 512, 512])
        mul = aten.mul(view_6, inv_const_scalar2)
        add_3 = aten.add(mul, mul_1)
        return add_3, mul_1


def _h(g, shape, scale=1.0):
    return _randn(g, shape, scale)


class BMMPartition2(torch.nn.Module):
    """unittest/evt_fuser/bmm.py:48-67.  Its sum runs over the sequence axis (N)
    and over half of the batch axis (l = b*16 + h, summed over b): a per-row
    reduction that folds the batches which agree modulo 16."""
    def forward(self, view_3, view_83):
        permute_128 = aten.permute(view_3, [1, 2, 0])
        bmm_10 = aten.bmm(permute_128, view_83)
        permute_177 = aten.permute(bmm_10, [2, 0, 1])
        view_84 = aten.view(permute_177, [512, 2, 1024])
        sum_15 = aten.sum(view_84, [0, 1], True)
        clone_11 = aten.clone(view_84, memory_format=torch.contiguous_format)
        view_101 = aten.view(clone_11, [1024, 1024])
        div = aten.div(sum_15, 20)
        return view_101, div


class FoldConsecutiveBatches(torch.nn.Module):
    """Not a reference test: a BMM whose per-row sum also runs over pairs of
    consecutive batches (the other way batches can fold into one result)."""
    def forward(self, a, b, r):
        bmm = aten.bmm(a, b)
        y = aten.add(bmm, r)
        v = aten.view(y, [3, 2, 40, 72])
        s = aten.sum(v, [1, 3])
        return y, aten.mul(s, 0.5)


class FoldedLogSumExp(torch.nn.Module):
    """Not a reference test: log-sum-exp and (biased) variance / mean of a BMM result along its rows and over
    pairs of consecutive batches -- reductions with a two- and a three-word state that fold batches."""
    def forward(self, a, b, r):
        bmm = aten.bmm(a, b)
        y = aten.add(bmm, r)
        v = aten._to_copy(aten.view(y, [3, 2, 40, 72]), dtype=torch.float32)
        lse = aten.logsumexp(v, [1, 3])
        vm = aten.var_mean(v, [1, 3], correction=0, keepdim=False)
        return y, lse, operator.getitem(vm, 0), operator.getitem(vm, 1)


class FoldedModuloVariance(torch.nn.Module):
    """The same statistics over the batches that agree modulo 3 (batch l = i * 3 + j, reduced over i)."""
    def forward(self, a, b, r):
        bmm = aten.bmm(a, b)
        y = aten.add(bmm, r)
        v = aten._to_copy(aten.view(y, [2, 3, 40, 72]), dtype=torch.float32)
        vm = aten.var_mean(v, [0, 3], correction=0, keepdim=False)
        lse = aten.logsumexp(v, [0, 3])
        return y, operator.getitem(vm, 0), operator.getitem(vm, 1), lse


def fold_consecutive_inputs():
    g = torch.Generator(device="cpu").manual_seed(17)
    return [_h(g, (6, 40, 24), 0.3), _h(g, (6, 24, 72), 0.3), _h(g, (6, 40, 72), 0.3)]


class MMPartition12(torch.nn.Module):
    """unittest/evt_fuser/mm.py:216-236: relu, its `ne` mask, and a dropout
    (rand_like / ge / mul) whose mask is returned too."""
    def forward(self, primals_7, cat, primals_8):
        permute_11 = aten.permute(primals_7, [1, 0])
        mm_4 = aten.mm(cat, permute_11)
        add = aten.add(mm_4, primals_8)
        relu_3 = aten.relu(add)
        ne = aten.ne(relu_3, 0)
        rand_like = torch.rand_like(relu_3)
        ge = aten.ge(rand_like, 1e-19)
        mul_1 = aten.mul(relu_3, ge)
        mul_2 = aten.mul(mul_1, 1.0)
        return ne, ge, mul_2


class Dropout1(torch.nn.Module):
    """unittest/evt_fuser/dropout.py:33-46 after the reference's decomposition of
    native_dropout(x, 0.7, True) into ge(rand_like(x), p), two muls
    (pass_decomposition.py:359-369)."""
    def forward(self, view_9, primals_16, primals_17, permute_104):
        permute_115 = aten.permute(primals_16, [1, 0])
        mm_36 = aten.mm(view_9, permute_115)
        add_20 = aten.add(mm_36, primals_17)
        view_10 = aten.view(add_20, [512, 2, 1024])
        mask = aten.ge(torch.rand_like(view_10), 0.7)
        output = aten.mul(view_10, mask)
        scaled_output = aten.mul(output, 1. / (1 - 0.7))
        add_4 = aten.add(scaled_output, permute_104)
        return add_4, mask


class Dropout1Undecomposed(torch.nn.Module):
    """unittest/evt_fuser/dropout.py:33-46 verbatim: native_dropout, decomposed by
    pass_decomposition before pass_fusion as in the reference's test."""
    def forward(self, view_9, primals_16, primals_17, permute_104):
        permute_115 = aten.permute(primals_16, [1, 0])
        mm_36 = aten.mm(view_9, permute_115)
        add_20 = aten.add(mm_36, primals_17)
        view_10 = aten.view(add_20, [512, 2, 1024])
        dropout = aten.native_dropout(view_10, 0.7, True)
        getitem_2 = operator.getitem(dropout, 0)
        getitem_3 = operator.getitem(dropout, 1)
        add_4 = aten.add(getitem_2, permute_104)
        return add_4, getitem_3


class SoftmaxDropout(torch.nn.Module):
    """Attention-probability dropout: softmax over masked scores, then the
    decomposed native_dropout (pass_decomposition.py:359-369) on the
    probabilities; both the mask and the dropped probabilities leave the kernel."""
    P = 0.1

    def forward(self, scores, causal):
        masked = aten.where(causal, -65504.0, scores)
        probs = aten._softmax(masked, -1, False)
        mask = aten.ge(torch.rand_like(probs), self.P)
        out = aten.mul(aten.mul(probs, mask), 1. / (1 - self.P))
        return out, mask, probs


def _causal(s):
    return torch.ones(s, s, dtype=torch.bool).triu(1)


# patterns that draw random numbers in the epilogue: checked with the generator's stream replayed on the CPU
RANDOM_PATTERNS = {
    "softmax_dropout": (SoftmaxDropout, lambda g: [_h(g, (3, 4, 136, 136)), _causal(136)]),
    "mm12": (MMPartition12, lambda g: [_h(g, (512, 24576), 0.01), _h(g, (1024, 24576)), _h(g, (512,))]),
    "dropout1": (Dropout1, lambda g: [_h(g, (1024, 1024)), _h(g, (1024, 1024), 0.03), _h(g, (1024,)),
                                      _h(g, (512, 2, 1024))]),
}

# name -> (module class, input generator(generator) -> CPU tensors, allclose criteria of the reference test)
REFERENCE_PATTERNS = {
    "mm1": (MMPartition1, lambda g: [_h(g, (4096, 1024), 0.03), _h(g, (1024, 1024)), _h(g, (4096,))]),
    "mm2": (MMPartition2, lambda g: [_h(g, (4, 1024)), _h(g, (1024, 1024), 0.018), _h(g, (1024,), 0.018)]),
    "mm3": (MMPartition3, lambda g: [_h(g, (1024, 1024)), _h(g, (1024, 1024), 0.03), _h(g, (1024,))]),
    "mm4": (MMPartition4, lambda g: [_h(g, (2, 1024)), _h(g, (2, 1024), 0.03), _h(g, (2,))]),
    "mm5": (MMPartition5, lambda g: [_h(g, (4, 2)), _h(g, (2, 1024)), torch.tanh(_h(g, (4, 1024)).float()).half()]),
    "mm6": (MMPartition6, lambda g: [_h(g, (2048, 1024)), _h(g, (1024, 1024), 0.03), _h(g, (512, 4, 1024)),
                                     _h(g, (512, 4, 1024))]),
    "mm7": (MMPartition7, lambda g: [_h(g, (2048, 1024)), _h(g, (1024, 1024), 0.03), _h(g, (512, 4, 1024)),
                                     _h(g, (512, 4, 1024))]),
    "mm9": (MMPartition9, lambda g: [_h(g, (4, 1024)), _h(g, (1024, 1024), 0.018), _h(g, (1024,), 0.018)]),
    "mm10": (MMPartition10, lambda g: [_h(g, (16384, 1024), 0.05), _h(g, (1024, 4096), 0.05)]),
    "mm11": (MMPartition11, lambda g: [_h(g, (33792, 768), 0.01), _h(g, (33792, 768))]),
    "bmm1": (BMMPartition1, lambda g: [_h(g, (512, 32, 64)), _h(g, (32, 512, 512), 0.05)]),
    "bmm2": (BMMPartition2, lambda g: [_h(g, (512, 32, 64), 0.3), _h(g, (32, 512, 512), 0.05)]),
    "bmm3": (BMMPartition3, lambda g: [_h(g, (512, 32, 64)), _h(g, (512, 32, 64), 0.2), _h(g, (2, 512)),
                                       _h(g, (1,)), _h(g, (1,)), _h(g, (1,))]),
}


# ---------------------------------------------------------------------------
# graphs with several anchors: which epilogue takes a shared node is the
# partitioner's decision (reference: the ILP of pass_fusion.py:216-983)
# ---------------------------------------------------------------------------

class TwoAnchorsMixedWidth(torch.nn.Module):
    """z can join either GEMM; joining the second keeps a 32-bit edge on chip,
    joining the first (what graph order suggests) only a 16-bit one.  y1 and t
    are results of the graph as well, so neither can be recomputed inside the
    other GEMM's epilogue: the kernels move 96 M N bits of epilogue tensors
    with z in the second partition and 112 M N with z in the first."""
    def forward(self, a, b, c, d):
        y1 = aten.mm(a, b)
        y2 = aten.mm(c, d)
        y2f = aten._to_copy(y2, dtype=torch.float32)
        t = aten.exp(y2f)
        z = aten.mul(t, y1)
        return y1, t, z


class CrossedAnchors(torch.nn.Module):
    """Each GEMM's epilogue candidate needs the other GEMM's result through an
    op no epilogue can hold: fusing both would make the two kernels wait for
    each other."""
    def forward(self, a, b, c, d):
        y1 = aten.mm(a, b)
        y2 = aten.mm(c, d)
        u1 = aten.flip(y1, [1])
        u2 = aten.flip(y2, [1])
        e1 = aten.mul(y1, u2)
        e2 = aten.mul(y2, u1)
        return e1, e2


class ThreeAnchorsDiamond(torch.nn.Module):
    """Two GEMMs meet in a product that a third GEMM's result scales, followed
    by a column sum of magnitudes.  (Products and magnitudes rather than sums:
    tensors that cross from one kernel to the next are rounded to fp16 on the
    way, and an element-wise relative tolerance is only meaningful where that
    rounding is not amplified by cancellation.)"""
    def forward(self, a, b, c, d, e, f, bias):
        y1 = aten.mm(a, b)
        y2 = aten.mm(c, d)
        y3 = aten.mm(e, f)
        p = aten.add(y1, bias)
        q = aten.gelu(y2, approximate="tanh")
        r = aten.mul(p, q)
        rf = aten._to_copy(r, dtype=torch.float32)
        s = aten.mul(rf, y3)
        sa = aten.abs(s)
        col = aten.sum(sa, [0])
        return r, s, col


_MA = (384, 512, 256)   # M, N, K of every GEMM in the multi-anchor graphs


def _ma_inputs(g, n_gemms: int, bias: bool):
    M, N, K = _MA
    out = []
    for _ in range(n_gemms):
        out += [_h(g, (M, K), 0.25), _h(g, (K, N), 0.25)]
    if bias:
        out.append(_h(g, (N,)))
    return out


MULTI_ANCHOR_PATTERNS = {
    "two_mixed_width": (TwoAnchorsMixedWidth, lambda g: _ma_inputs(g, 2, False)),
    "crossed": (CrossedAnchors, lambda g: _ma_inputs(g, 2, False)),
    "three_diamond": (ThreeAnchorsDiamond, lambda g: _ma_inputs(g, 3, True)),
}


# ---------------------------------------------------------------------------
# a whole training step through AOT autograd: the joint graph holds the
# forward GEMMs (bias + GELU, bias + cast) and the backward ones (data
# gradient with GELU' and the bias gradient, two weight gradients)
# ---------------------------------------------------------------------------

class MLPClassifier(torch.nn.Module):
    """fp16 two-layer classifier with a summed cross-entropy loss, the shape
    of the reference's XML-CNN head (benchmark/subgraphs/xmlcnn/xmlcnn.py)."""
    def __init__(self, d_in: int = 256, hidden: int = 1024, classes: int = 128) -> None:
        super().__init__()
        self.l1 = torch.nn.Linear(d_in, hidden)
        self.l2 = torch.nn.Linear(hidden, classes)

    def forward(self, x, y):
        z = self.l2(torch.nn.functional.gelu(self.l1(x), approximate="tanh"))
        return torch.nn.functional.cross_entropy(z.float(), y, reduction="sum")


MLP_BATCH = 512


def mlp_classifier(seed: int = 0, device: str = "cpu", dtype=torch.float16):
    """(model, (x, labels)) with seeded fp16 parameters and inputs."""
    g = torch.Generator(device="cpu").manual_seed(0xA07 + seed)
    model = MLPClassifier()
    with torch.no_grad():
        for p in model.parameters():
            p.copy_(torch.randn(p.shape, generator=g) * (0.05 if p.dim() == 2 else 0.02))
    model = model.to(dtype).to(device)
    x = torch.randn(MLP_BATCH, model.l1.in_features, generator=g).to(dtype).to(device)
    y = torch.randint(0, model.l2.out_features, (MLP_BATCH,), generator=g).to(device)
    return model, (x, y)


# ---------------------------------------------------------------------------
# row-wise anchors: the patterns of the reference's softmax / layer norm fuser
# tests (unittest/evt_fuser/softmax.py:30-105, softmax_backward.py:30-41,
# layernorm.py:31-78, layernorm_backward.py:31-55)
# ---------------------------------------------------------------------------

class SoftmaxAuxStore(torch.nn.Module):      # softmax.py:30-41
    def forward(self, input):
        _softmax = aten._softmax(input, -1, False)
        return aten.view(_softmax, [16384, 512])


class SoftmaxAuxLoad(torch.nn.Module):       # softmax.py:43-55
    def forward(self, input, aux):
        return aten.add(aten._softmax(input, -1, False), aux)


class SoftmaxRowBroadcast(torch.nn.Module):  # softmax.py:57-69
    def forward(self, input, row):
        return aten.add(aten._softmax(input, -1, False), row)


class SoftmaxScalar(torch.nn.Module):        # softmax.py:71-82
    def forward(self, input):
        return aten.mul(aten._softmax(input, -1, False), 2.)


class SoftmaxColumnBroadcast(torch.nn.Module):   # softmax.py:99-111
    def forward(self, input, col):
        return aten.add(aten._softmax(input, -1, False), col)


class SoftmaxColumnReduce(torch.nn.Module):   # softmax.py:84-97
    def forward(self, input):
        out = aten.mul(aten._softmax(input, -1, False), 2.)
        return out, aten.sum(out, [0], True)


class SoftmaxRagged(torch.nn.Module):
    """Rank 4, a row length that is no multiple of 8, fp32 result of fp16 logits, two results."""
    def forward(self, input, mask):
        s = aten._softmax(input, -1, True)
        return s, aten.mul(s, mask)


class SoftmaxBackward(torch.nn.Module):      # softmax_backward.py:30-41
    def forward(self, grad, out):
        return aten._softmax_backward_data(grad, out, -1, torch.float16)


class LayerNormPattern1(torch.nn.Module):    # layernorm.py:31-52
    def forward(self, add_4, primals_18, primals_19):
        ln = aten.native_layer_norm(add_4, [1024], None, None, 1e-12)
        getitem_46 = operator.getitem(ln, 0)
        getitem_47 = operator.getitem(ln, 1)
        getitem_48 = operator.getitem(ln, 2)
        mul_2 = aten.mul(getitem_46, primals_18)
        add_32 = aten.add(mul_2, primals_19)
        view_11 = aten.view(add_32, [1024, 1024])
        return getitem_47, getitem_48, add_32, view_11


class LayerNormPattern2(torch.nn.Module):    # layernorm.py:54-78  (permuted result)
    def forward(self, add_8, primals_36, primals_37):
        ln = aten.native_layer_norm(add_8, [1024], None, None, 1e-12)
        getitem_55 = operator.getitem(ln, 0)
        getitem_56 = operator.getitem(ln, 1)
        getitem_57 = operator.getitem(ln, 2)
        mul_5 = aten.mul(getitem_55, primals_36)
        add_35 = aten.add(mul_5, primals_37)
        permute_141 = aten.permute(add_35, [1, 0, 2])
        clone_5 = aten.clone(permute_141, memory_format=torch.contiguous_format)
        view_33 = aten.view(clone_5, [1024, 1024])
        return getitem_56, getitem_57, clone_5, view_33


class LayerNormBackwardMasked(torch.nn.Module):   # layernorm_backward.py:31-44 without its column sum
    def forward(self, grad, input, mean, invstd, gamma, beta, ge_1):
        ln = aten.native_layer_norm_backward(grad, input, [1024], mean, invstd, gamma, beta, [True, False, False])
        getitem = operator.getitem(ln, 0)
        mul_42 = aten.mul(getitem, ge_1)
        mul_43 = aten.mul(mul_42, 1.0)
        view_282 = aten.view(mul_43, [2048, 1024])
        return getitem, view_282


class LayerNormBackwardColumnSum(torch.nn.Module):   # layernorm_backward.py:31-44 as written there
    def forward(self, grad, input, mean, invstd, gamma, beta, ge_1):
        ln = aten.native_layer_norm_backward(grad, input, [1024], mean, invstd, gamma, beta, [True, False, False])
        getitem = operator.getitem(ln, 0)
        mul_42 = aten.mul(getitem, ge_1)
        mul_43 = aten.mul(mul_42, 1.0)
        view_282 = aten.view(mul_43, [2048, 1024])
        sum_13 = aten.sum(view_282, [0], True)
        return getitem, view_282, sum_13


class LayerNormBackwardFull(torch.nn.Module):
    """Input, weight and bias gradients of a layer norm in one pass (the
    reference computes the input gradient only, evt_fuser.py:905-970)."""
    def forward(self, grad, input, mean, invstd, gamma, beta, ge_1):
        ln = aten.native_layer_norm_backward(grad, input, [1024], mean, invstd, gamma, beta, [True, True, True])
        dx = aten.mul(operator.getitem(ln, 0), ge_1)
        return dx, operator.getitem(ln, 1), operator.getitem(ln, 2)


def _softmax_out(g, shape):
    return torch.softmax(_h(g, shape).float(), -1).half()


def _ln_backward_inputs(g):
    grad, x = _h(g, (512, 4, 1024)), _h(g, (512, 4, 1024))
    mean = x.float().mean(-1, keepdim=True)
    rstd = torch.rsqrt(x.float().var(-1, unbiased=False, keepdim=True) + 1e-5)
    gamma, beta = _h(g, (1024,)), _h(g, (1024,))
    keep = torch.rand(x.shape, generator=g) >= 0.5
    return [grad, x, mean, rstd, gamma, beta, keep]


ROW_ANCHOR_PATTERNS = {
    "softmax_aux_store": (SoftmaxAuxStore, lambda g: [_h(g, (16384, 512))]),
    "softmax_aux_load": (SoftmaxAuxLoad, lambda g: [_h(g, (16384, 512)), _h(g, (16384, 512))]),
    "softmax_row_broadcast": (SoftmaxRowBroadcast, lambda g: [_h(g, (16384, 512)), _h(g, (512,))]),
    "softmax_scalar": (SoftmaxScalar, lambda g: [_h(g, (16384, 512))]),
    "softmax_column_broadcast": (SoftmaxColumnBroadcast, lambda g: [_h(g, (16384, 512)), _h(g, (16384, 1))]),
    "softmax_column_reduce": (SoftmaxColumnReduce, lambda g: [_h(g, (16, 512))]),
    "softmax_column_reduce_tall": (SoftmaxColumnReduce, lambda g: [_h(g, (40000, 512))]),
    # rows over several waves of a workgroup with a sum over all rows behind them (every lane carries the partials
    # of its own columns): 12288 columns, and a vocabulary-sized row whose length is no multiple of 8
    "softmax_column_reduce_wide": (SoftmaxColumnReduce, lambda g: [_h(g, (300, 12288))]),
    "softmax_column_reduce_vocab": (SoftmaxColumnReduce, lambda g: [_h(g, (70, 30522))]),
    "softmax_ragged": (SoftmaxRagged, lambda g: [_h(g, (3, 5, 37, 203), 3.0), _h(g, (37, 1))]),
    "softmax_backward": (SoftmaxBackward, lambda g: [_h(g, (4, 16, 512, 512)), _softmax_out(g, (4, 16, 512, 512))]),
    "layernorm1": (LayerNormPattern1, lambda g: [_h(g, (512, 2, 1024)) + 1., _h(g, (1024,)), _h(g, (1024,))]),
    "layernorm2": (LayerNormPattern2, lambda g: [_h(g, (512, 2, 1024)) + 1., _h(g, (1024,)), _h(g, (1024,))]),
    "layernorm_backward": (LayerNormBackwardMasked, _ln_backward_inputs),
    "layernorm_backward_column_sum": (LayerNormBackwardColumnSum, _ln_backward_inputs),
    "layernorm_backward_full": (LayerNormBackwardFull, _ln_backward_inputs),
}


# row lengths and element types of the row-wise anchors beyond the reference's patterns: the shortest and the
# longest supported rows, lengths that are no multiple of 8 (generic path), bf16 and fp32 operands

class _BareSoftmax(torch.nn.Module):
    def forward(self, x):
        return aten._softmax(x, -1, False)


class _BareSoftmaxBackward(torch.nn.Module):
    def __init__(self, dtype):
        super().__init__()
        self.dtype = dtype

    def forward(self, g, y):
        return aten._softmax_backward_data(g, y, -1, self.dtype)


class _BareLayerNorm(torch.nn.Module):
    def __init__(self, n):
        super().__init__()
        self.n = n

    def forward(self, x):
        ln = aten.native_layer_norm(x, [self.n], None, None, 1e-5)
        return operator.getitem(ln, 0), operator.getitem(ln, 1), operator.getitem(ln, 2)


class _BareLayerNormBackward(torch.nn.Module):
    def __init__(self, n):
        super().__init__()
        self.n = n

    def forward(self, g, x, mean, rstd):
        ln = aten.native_layer_norm_backward(g, x, [self.n], mean, rstd, None, None, [True, False, False])
        return operator.getitem(ln, 0)


class HeadMergeBiasGrad(torch.nn.Module):
    """What the backward pass of an attention layer does with the gradient of a
    projection's output: a batched product over L = B * H heads whose result is
    merged back into [B * S, H * D] (permute + copy, folded into the store) and
    summed over all rows for the bias gradient -- per column and over the
    batches that agree modulo H.  `transposed`: the product comes out as
    [D, S] per head (the key gradient), so the same sum runs along rows."""
    def __init__(self, B: int, H: int, S: int, D: int, transposed: bool = False) -> None:
        super().__init__()
        self.dims, self.transposed = (B, H, S, D), transposed

    def forward(self, a, b):
        B, H, S, D = self.dims
        out = aten.bmm(a, b)
        if self.transposed:                                      # [L, D, S]
            merged = aten.permute(aten.view(out, [B, H, D, S]), [0, 3, 1, 2])
        else:                                                    # [L, S, D]
            merged = aten.permute(aten.view(out, [B, H, S, D]), [0, 2, 1, 3])
        w = aten.view(aten.clone(merged, memory_format=torch.contiguous_format), [B * S, H * D])
        return w, aten.view(aten.sum(w, [0], True), [H * D])


# more batches per result than the last workgroup of a column block combines itself (64 partials): 24 batches x
# 3 .. 10 row tiles per result, finished by the finalize kernel
HEAD_MERGE_MANY_PARTIALS = dict(B=24, H=2, S=640, D=64, K=32)


def head_merge_bias_grad(B: int = 4, H: int = 6, S: int = 320, D: int = 64, K: int = 96, transposed: bool = False,
                         seed: int = 0):
    g = torch.Generator(device="cpu").manual_seed(0xB1A5 + seed)
    h = lambda *sh: (torch.randn(*sh, generator=g) * 0.3).half()   # noqa: E731
    a = h(B * H, D, K) if transposed else h(B * H, S, K)
    b = h(B * H, K, S) if transposed else h(B * H, K, D)
    return HeadMergeBiasGrad(B, H, S, D, transposed), [a, b]


class ColumnMajorStore(torch.nn.Module):
    """A product whose result leaves the kernel transposed: gelu(a @ b + bias +
    r^T) stored as [N, M] (permute + copy, folded into the store), r read
    through the same permute, with a reduction of the stored values on top --
    the bias-gradient sum over all rows for the GEMM, a maximum along every
    row for the batched product.  The column-major outputs of the reference's
    `transposed` problems (evt_fuser.py:573-596)."""
    def __init__(self, batched: bool) -> None:
        super().__init__()
        self.batched = batched

    def forward(self, a, b, bias, r):
        perm = [0, 2, 1] if self.batched else [1, 0]
        out = aten.bmm(a, b) if self.batched else aten.mm(a, b)
        y = aten.gelu(aten.add(aten.add(out, bias), aten.permute(r, perm)))
        yt = aten.clone(aten.permute(y, perm), memory_format=torch.contiguous_format)
        red = aten.amax(y, [2]) if self.batched else aten.sum(y, [0])
        return yt, red


def column_major_store(batched: bool, seed: int = 0, dtype=torch.float16):
    g = torch.Generator(device="cpu").manual_seed(0xC01A + seed)
    h = lambda *sh: (torch.randn(*sh, generator=g) * 0.3).to(dtype)   # noqa: E731
    lead, (M, N, K) = ((3,), (200, 136, 64)) if batched else ((), (320, 192, 96))
    return ColumnMajorStore(batched), [h(*lead, M, K), h(*lead, K, N), h(N), h(*lead, N, M)]


class RandomEpilogue(torch.nn.Module):
    """A seeded random epilogue tree behind a GEMM: 5 .. 9 element-wise steps
    over the accumulator, a same-shape tensor, a row vector, a column vector
    and immediates, drawn from the fuser's vocabulary; one or two results are
    stored, and a per-row or per-column sum of one of them may come on top.
    Beyond the reference's hand-written patterns: the generator has no idea
    which combinations are easy."""
    UNARY = ("relu", "tanh", "sigmoid", "neg", "abs", "gelu", "exp_small", "sqrt_abs", "rsqrt_abs1")
    BINARY = ("add", "sub", "mul", "maximum", "minimum", "div_abs1", "where_gt")

    def __init__(self, seed: int, anchor: str = "mm", n: int = 0, column_major: bool = False):
        super().__init__()
        import random
        rng = random.Random(0xE71 + seed + 1000 * ("mm", "bmm", "softmax", "layernorm").index(anchor))
        self.anchor, self.n = anchor, n
        # the same-shape tensor is stored [N, M] and read through a permute, and the full-size results leave
        # through permute + copy: every full-tensor access of the epilogue is column-major (products only)
        self.column_major = column_major
        self.steps = []
        n_vals = 4                       # accum, aux, row, col
        # the first operand of every step comes from the accumulator's side (value 0 or an earlier step), so the
        # whole tree belongs to the epilogue: a side expression run eagerly would hand over an fp16-rounded
        # tensor, and a later subtraction can blow that rounding up beyond any fixed tolerance
        from_acc = lambda: rng.choice([0] + list(range(4, n_vals)))   # noqa: E731
        for _ in range(rng.randint(5, 9)):
            if rng.random() < 0.45:
                self.steps.append((rng.choice(self.UNARY), from_acc(), None))
            else:
                a = from_acc()
                op = rng.choice(self.BINARY)
                tensor_only = op in ("maximum", "minimum")         # aten.maximum / minimum take no immediates
                b = rng.randrange(n_vals) if tensor_only or rng.random() < 0.75 else ("imm", rng.choice((0.5, -1.25, 2.0, 0.1)))
                self.steps.append((op, a, b))
            n_vals += 1
        # results: the last value and possibly an earlier full-size one; the last always depends on the accumulator
        self.extra = rng.randrange(4, n_vals - 1) if rng.random() < 0.6 else None      # an earlier step's value
        self.reduce = rng.choice((None, None, 0, 1))
        if anchor in ("softmax", "layernorm") and self.reduce == 1:
            self.reduce = 0              # behind a row-wise anchor only sums over the rows are fused

    def forward(self, A, B, aux, row, col):
        if self.anchor == "mm":
            acc = aten.mm(A, B)
        elif self.anchor == "bmm":
            acc = aten.bmm(A, B)
        elif self.anchor == "softmax":
            acc = aten._softmax(A, -1, False)
        else:
            acc = operator.getitem(aten.native_layer_norm(A, [self.n], None, None, 1e-5), 0)
        perm = [0, 2, 1] if self.anchor == "bmm" else [1, 0]
        if self.column_major:
            aux = aten.permute(aux, perm)
        vals = [acc, aux, row, col]
        for op, a, b in self.steps:
            x = vals[a]
            imm = isinstance(b, tuple)
            y = None if b is None else (b[1] if imm else vals[b])
            if op == "exp_small":
                r = aten.exp(aten.mul(x, 0.125))
            elif op == "sqrt_abs":
                r = aten.sqrt(aten.abs(x))
            elif op == "rsqrt_abs1":
                r = aten.rsqrt(aten.add(aten.abs(x), 1.0))
            elif op == "gelu":
                r = aten.gelu(x, approximate="tanh")
            elif op == "div_abs1":
                d = abs(y) + 1.0 if imm else aten.add(aten.abs(y), 1.0)
                r = aten.div(x, d)
            elif op == "where_gt":
                other = aten.mul(x, y) if imm else y
                r = aten.where(aten.gt(x, other), x, aten.mul(other, 0.5))
            elif b is None:
                r = getattr(aten, op)(x)
            else:
                r = getattr(aten, op)(x, y)
            vals.append(r)
        last = aten.add(vals[-1], aten.mul(acc, 0.25))          # full size, accumulator inside
        outs = [last]
        if self.extra is not None:
            outs.append(aten.add(vals[self.extra], aux))           # full size whatever the value's own shape
        if self.column_major:
            outs = [aten.clone(aten.permute(o, perm), memory_format=torch.contiguous_format) for o in outs]
        if self.reduce is not None:
            outs.append(aten.sum(aten.abs(last), [self.reduce + (1 if self.anchor == "bmm" else 0)], True))
        return tuple(outs)


RANDOM_EPILOGUE_SEEDS = tuple(range(12))


RANDOM_EPILOGUE_ANCHORS = ("mm", "bmm", "softmax", "layernorm")


def random_epilogue(seed: int, anchor: str = "mm", M: int = 320, N: int = 192, K: int = 96, L: int = 3,
                    column_major: bool = False):
    """(module, CPU inputs) of the seeded random epilogue behind `anchor`; M, N, K are no multiples of the
    large tiles.  The row-wise anchors take A alone ([M, N]); B is an unused input there.  `column_major`
    (products only): see RandomEpilogue."""
    g = torch.Generator(device="cpu").manual_seed(0xE71 + seed)
    h = lambda *sh: (torch.randn(*sh, generator=g) * 0.5).half()   # noqa: E731
    full = (N, M) if column_major else (M, N)
    if anchor == "mm":
        ins = [h(M, K), h(K, N), h(*full), h(N), h(M, 1)]
    elif anchor == "bmm":
        ins = [h(L, M, K), h(L, K, N), h(L, *full), h(N), h(M, 1)]
    else:
        ins = [h(M, N) * 4, h(1), h(M, N), h(N), h(M, 1)]
    return RandomEpilogue(seed, anchor, N, column_major), ins


class AffineLayerNorm(torch.nn.Module):
    """Layer norm with weight and bias over rows of any length (GPT-3's hidden size 12288 goes over two waves)."""
    def __init__(self, n):
        super().__init__()
        self.n = n

    def forward(self, x, w, b):
        ln = aten.native_layer_norm(x, [self.n], w, b, 1e-5)
        return operator.getitem(ln, 0), operator.getitem(ln, 1), operator.getitem(ln, 2)


def affine_layer_norm(n: int, dtype=torch.float16, rows: int = 40, seed: int = 0):
    g = torch.Generator(device="cpu").manual_seed(0xAF1 + n + seed)
    x = (torch.randn(rows, n, generator=g) * 1.5 + 0.25).to(dtype)
    w = (1.0 + 0.2 * torch.randn(n, generator=g)).to(dtype)
    b = (0.1 * torch.randn(n, generator=g)).to(dtype)
    return AffineLayerNorm(n), [x, w, b]


AFFINE_LN_LENGTHS = (8192, 12288, 20480)
ROW_EDGE_LENGTHS = (8, 24, 1000, 8192)
ROW_EDGE_DTYPES = (torch.float16, torch.bfloat16, torch.float32)
# rows spread over the waves of a workgroup (longer than 8192): vocabulary-sized rows, the longest each anchor
# takes, lengths that are no multiple of 8
ROW_LONG_CASES = (
    ("softmax", 8200, torch.float16), ("softmax", 30522, torch.float16), ("softmax", 50257, torch.bfloat16),
    ("softmax", 65536, torch.float16), ("softmax", 30522, torch.float32),
    ("softmax_backward", 8200, torch.float16), ("softmax_backward", 30522, torch.float16),
    ("softmax_backward", 32768, torch.bfloat16), ("softmax_backward", 16384, torch.float32),
    ("layernorm", 12288, torch.float16), ("layernorm", 65536, torch.bfloat16),
    ("layernorm_backward", 12288, torch.float16), ("layernorm_backward", 24000, torch.bfloat16),
)


def row_edge_case(anchor: str, n: int, dtype, seed: int = 0):
    """(module, CPU inputs) for a bare anchor on 3 x 7 rows of length n."""
    g = torch.Generator(device="cpu").manual_seed(0xED6E + 31 * n + seed)
    shape = (3, 7, n)
    x = (torch.randn(shape, generator=g) * 2 + 0.5).to(dtype)
    if anchor == "softmax":
        return _BareSoftmax(), [x]
    if anchor == "softmax_backward":
        y = torch.softmax(torch.randn(shape, generator=g), -1).to(dtype)
        return _BareSoftmaxBackward(dtype), [x, y]
    if anchor == "layernorm":
        return _BareLayerNorm(n), [x]
    grad = torch.randn(shape, generator=g).to(dtype)
    xf = x.float()
    mean = xf.mean(-1, keepdim=True)
    rstd = torch.rsqrt(xf.var(-1, unbiased=False, keepdim=True) + 1e-5)
    return _BareLayerNormBackward(n), [grad, x, mean, rstd]


class DropoutBlock(torch.nn.Module):
    """Feed-forward block with two dropouts and a post layer norm, in training
    mode: `native_dropout` is decomposed to rand_like / ge / mul and the masks
    are drawn inside the GEMM epilogues (reference: pass_decomposition.py:350-379,
    unittest/evt_fuser/dropout.py)."""
    P = 0.1

    def __init__(self, d: int = 256, ffn: int = 512) -> None:
        super().__init__()
        self.l1 = torch.nn.Linear(d, ffn)
        self.l2 = torch.nn.Linear(ffn, d)
        self.ln = torch.nn.LayerNorm(d)

    def forward(self, x, target):
        F = torch.nn.functional
        h = F.dropout(F.gelu(self.l1(x), approximate="tanh"), self.P, True)
        y = self.ln(x + F.dropout(self.l2(h), self.P, True))
        return ((y.float() - target) ** 2).sum()

    def forward_with_masks(self, x, target, m1, m2):
        """The same computation with the two keep masks given."""
        F = torch.nn.functional
        h = F.gelu(self.l1(x), approximate="tanh") * m1 / (1 - self.P)
        y = self.ln(x + self.l2(h) * m2 / (1 - self.P))
        return ((y.float() - target) ** 2).sum()


def dropout_block(seed: int = 0, device: str = "cpu", dtype=torch.float16):
    g = torch.Generator(device="cpu").manual_seed(0xD40 + seed)
    model = DropoutBlock()
    with torch.no_grad():
        for name, p in model.named_parameters():
            if p.dim() == 2:
                p.copy_(torch.randn(p.shape, generator=g) * 0.05)
            elif name == "ln.weight":
                p.copy_(1.0 + 0.1 * torch.randn(p.shape, generator=g))
            else:
                p.copy_(0.02 * torch.randn(p.shape, generator=g))
    model = model.to(dtype).to(device)
    x = torch.randn(512, 256, generator=g).to(dtype).to(device)
    target = torch.randn(512, 256, generator=g).to(device)
    return model, (x, target)


class DecoderBlock(torch.nn.Module):
    """Pre-layer-norm decoder block in training mode: causal `masked_fill` on the
    scores (decomposed to `where`, fused behind the Q K^T BMM), softmax with the
    attention-probability dropout drawn behind it in the same row kernel, GELU
    feed-forward, residuals.  Not one of the reference's models: it exercises
    rand_like behind a row-wise anchor and a layer norm backward whose input
    gradient is the only one some consumers need."""
    P = 0.1

    def __init__(self, d: int = 256, heads: int = 4) -> None:
        super().__init__()
        self.h = heads
        self.ln1 = torch.nn.LayerNorm(d)
        self.ln2 = torch.nn.LayerNorm(d)
        self.qkv = torch.nn.Linear(d, 3 * d)
        self.o = torch.nn.Linear(d, d)
        self.f1 = torch.nn.Linear(d, 4 * d)
        self.f2 = torch.nn.Linear(4 * d, d)

    def _block(self, x, target, drop):
        F = torch.nn.functional
        B, S, D = x.shape
        H, dh = self.h, D // self.h
        q, k, v = self.qkv(self.ln1(x)).view(B, S, 3, H, dh).permute(2, 0, 3, 1, 4)
        att = (q @ k.transpose(-1, -2)) / math.sqrt(dh)
        keep = torch.ones(S, S, dtype=torch.bool, device=x.device).tril()
        att = drop(torch.softmax(att.masked_fill(~keep, float("-inf")), -1))
        x = x + self.o((att @ v).permute(0, 2, 1, 3).reshape(B, S, D))
        x = x + self.f2(F.gelu(self.f1(self.ln2(x)), approximate="tanh"))
        return ((x.float() - target) ** 2).sum()

    def forward(self, x, target):
        return self._block(x, target, lambda p: torch.nn.functional.dropout(p, self.P, True))

    def forward_with_masks(self, x, target, m):
        """The same computation with the attention keep mask given."""
        return self._block(x, target, lambda p: p * m / (1 - self.P))


def decoder_block(seed: int = 0, device: str = "cpu", dtype=torch.float16, batch: int = 4, seq: int = 128):
    g = torch.Generator(device="cpu").manual_seed(0xDEC + seed)
    model = DecoderBlock()
    with torch.no_grad():
        for name, p in model.named_parameters():
            if p.dim() == 2:
                p.copy_(torch.randn(p.shape, generator=g) * 0.05)
            elif name.endswith("ln1.weight") or name.endswith("ln2.weight"):
                p.copy_(1.0 + 0.1 * torch.randn(p.shape, generator=g))
            else:
                p.copy_(0.02 * torch.randn(p.shape, generator=g))
    model = model.to(dtype).to(device)
    x = torch.randn(batch, seq, 256, generator=g).to(dtype).to(device)
    target = torch.randn(batch, seq, 256, generator=g).to(device)
    return model, (x, target)


def pattern_inputs(name: str, seed: int = 0) -> List[torch.Tensor]:
    g = torch.Generator(device="cpu").manual_seed(0x5EED + seed)
    return (REFERENCE_PATTERNS.get(name) or RANDOM_PATTERNS.get(name) or MULTI_ANCHOR_PATTERNS.get(name)
            or ROW_ANCHOR_PATTERNS[name])[1](g)


# ---------------------------------------------------------------------------
# A per-column vector computed in an epilogue and read by other kernels (the reference's row store,
# visitor_store.hpp:46-145): BERT turns its attention mask into (1 - mask) * -10000 once; the first attention
# product's kernel computes and writes it, the later ones load it.
# ---------------------------------------------------------------------------

class MaskedScores(torch.nn.Module):
    """scores[B*H, S, S] = q k^T / 8 + (1 - mask[B, 1, 1, S]) * -10000; the transformed mask is an output too."""
    DIMS = (2, 3, 40, 16)
    GPU_DIMS = ((2, 3, 40, 16), (2, 2, 264, 64), (3, 2, 512, 64))     # unaligned; several row tiles, ragged; aligned

    def __init__(self, dims=None):
        super().__init__()
        self.B, self.H, self.S, self.D = dims or self.DIMS

    def forward(self, q, k, mask):
        B, H, S = self.B, self.H, self.S
        ext = aten.mul(aten.rsub(mask, 1.0), -10000.0)
        sc = aten.view(aten.bmm(q, aten.permute(k, [0, 2, 1])), [B, H, S, S])
        sc = aten.add(aten.div(sc, 8.0), ext)
        return aten.view(sc, [B * H, S, S]), ext

    @classmethod
    def inputs(cls, seed=0, dims=None):
        g = torch.Generator().manual_seed(seed)
        B, H, S, D = dims or cls.DIMS
        q = torch.randn(B * H, S, D, generator=g).half()
        k = torch.randn(B * H, S, D, generator=g).half()
        mask = (torch.rand(B, 1, 1, S, generator=g) > 0.3).half()
        return [q, k, mask]


class TwoMaskedLayers(torch.nn.Module):
    """Two products that add the same transformed [N] mask: one kernel writes it, the other reads it."""

    def forward(self, x, w1, w2, mask):
        ext = aten.mul(aten.rsub(mask, 1.0), -100.0)
        h = aten.relu(aten.add(aten.mm(x, w1), ext))
        y = aten.add(aten.mm(h, w2), ext)
        return y

    @staticmethod
    def inputs(seed=0, m=72, n=48):
        g = torch.Generator().manual_seed(seed)
        x = torch.randn(m, n, generator=g).half()
        w1 = (torch.randn(n, n, generator=g) * n ** -0.5).half()
        w2 = (torch.randn(n, n, generator=g) * n ** -0.5).half()
        mask = (torch.rand(n, generator=g) > 0.3).half()
        return [x, w1, w2, mask]


# ---------------------------------------------------------------------------
# The reference's tuner caches as a coverage checklist (tests/golden/reference_tuner_keys.json): every GEMM / BMM
# problem key there names a shape, a layout pair and seven epilogue-node counts
# (python/gtl/compiler/autotuner/tuner_base.py:107-152).  `CountedEpilogue` is a synthetic epilogue with exactly
# those counts behind a product of that shape and layout.
# ---------------------------------------------------------------------------

class CountedEpilogue(torch.nn.Module):
    """acc = A B; x = acc + aux_0 + ... + rowvec_0 + ..., times colvec_0 ...;
    stores x, gelu(x), relu(x) ... (aux_store of them), sums over the rows of x,
    x * x ... (row_reduction of them: [N] results, fp32) and sums along the rows
    (column_reduction: [M] results, fp32).  row_store: a value of the [N]
    vectors alone that the epilogue uses and that leaves the kernel as well
    (the reference stores BERT's transformed attention mask that way,
    (1 - mask) * -10000: visitor_store.hpp:46-145): the first row_store row
    vectors enter x in that form, and the transformed vectors are outputs.
    forward(A, B, *aux, *rowvec, *colvec)."""

    def __init__(self, counts, a_row: bool, b_row: bool, batched: bool):
        super().__init__()
        self.counts = tuple(int(c) for c in counts)
        self.a_row, self.b_row, self.batched = a_row, b_row, batched

    @staticmethod
    def with_arity(counts, a_row: bool, b_row: bool, batched: bool) -> "CountedEpilogue":
        """torch.fx traces positional parameters only: a subclass whose forward names every input."""
        n = int(counts[0]) + int(counts[1]) + int(counts[2])
        names = ", ".join(f"e{i}" for i in range(n))
        scope: dict = {}
        exec(f"def forward(self, A, B{', ' + names if n else ''}):\n    return self.body(A, B, [{names}])\n", scope)
        cls = type(f"CountedEpilogue_{'_'.join(str(int(c)) for c in counts)}", (CountedEpilogue,), {"forward": scope["forward"]})
        return cls(counts, a_row, b_row, batched)

    def forward(self, A, B, *extra):
        return self.body(A, B, list(extra))

    def body(self, A, B, extra):
        aux, rowb, colb, stores, rowred, colred, rowstore = self.counts
        swap = [0, 2, 1] if self.batched else [1, 0]
        a = A if self.a_row else aten.permute(A, swap)
        b = B if self.b_row else aten.permute(B, swap)
        x = aten.bmm(a, b) if self.batched else aten.mm(a, b)
        extra = list(extra)
        for _ in range(aux):
            x = aten.add(x, extra.pop(0))
        rows = [extra.pop(0) for _ in range(rowb)]
        masks = [aten.mul(aten.rsub(r, 1.0), -10000.0) for r in rows[:rowstore]]
        for r in masks + rows[len(masks):]:
            x = aten.add(x, r)
        for _ in range(colb):
            x = aten.mul(x, extra.pop(0))
        outs = []
        variants = (lambda t: t, lambda t: aten.gelu(t, approximate="tanh"), aten.relu, aten.tanh)
        for j in range(stores):
            outs.append(variants[j % len(variants)](x))
        if rowred or colred:
            xf = aten._to_copy(x, dtype=torch.float32)
            power = xf
            for j in range(rowred):
                outs.append(aten.sum(power, [-2]))
                power = aten.mul(power, xf)
            power = xf
            for j in range(colred):
                outs.append(aten.sum(power, [-1]))
                power = aten.mul(power, xf)
        outs.extend(masks)
        return tuple(outs)


# products whose extents break the 16-byte rule of the transfer path, run on zero-padded copies of their operands
# (FusedGEMM.pad): (M, N, K, A row-major, B row-major, the seven epilogue counts)
PADDED_GEMM_CASES = [
    (203, 141, 589, True, True, (1, 1, 0, 1, 1, 1, 0)),
    (203, 141, 589, True, False, (0, 1, 1, 2, 0, 1, 0)),
    (203, 141, 589, False, True, (1, 0, 0, 1, 1, 0, 0)),
    (203, 141, 589, False, False, (0, 1, 0, 1, 0, 0, 0)),
    (520, 588, 1028, True, True, (0, 1, 0, 1, 1, 0, 0)),
]


def padded_gemm_case(i):
    M, N, K, a_row, b_row, counts = PADDED_GEMM_CASES[i]
    return dict(L=1, M=M, N=N, K=K, a_row=a_row, b_row=b_row, counts=counts, batched=False)


def parse_reference_key(key: str, batched: bool):
    """`M_N_K_h_h_R_C[_7 counts]` (`L_M_N_K_...` batched) -> dict(L, M, N, K, a_row, b_row, counts), counts None for
    the keys of the reference tuner's first stage (no epilogue: a plain store)."""
    parts = key.split("_")
    nd = 4 if batched else 3
    dims = [int(p) for p in parts[:nd]]
    L = dims.pop(0) if batched else 1
    M, N, K = dims
    assert parts[nd] == parts[nd + 1] == "h", key
    la, lb = parts[nd + 2], parts[nd + 3]
    rest = parts[nd + 4:]
    counts = tuple(int(c) for c in rest) if rest else None
    assert counts is None or len(counts) == 7, key
    return dict(L=L, M=M, N=N, K=K, a_row=la == "R", b_row=lb == "R", counts=counts)


def counted_epilogue_shapes(case):
    """(shape, dtype) of every input of CountedEpilogue for a parsed key."""
    L, M, N, K = case["L"], case["M"], case["N"], case["K"]
    counts = case["counts"] or (0, 0, 0, 1, 0, 0, 0)
    lead = (L,) if case["L"] > 1 or case.get("batched") else ()
    shapes = [(lead + ((M, K) if case["a_row"] else (K, M)), torch.half),
              (lead + ((K, N) if case["b_row"] else (N, K)), torch.half)]
    shapes += [(lead + (M, N), torch.half)] * counts[0]
    shapes += [((N,), torch.half)] * counts[1]
    shapes += [(lead + (M, 1), torch.half)] * counts[2]
    return shapes


def counted_epilogue(case):
    """-> (module, meta inputs) for a parsed reference key."""
    counts = case["counts"] or (0, 0, 0, 1, 0, 0, 0)
    batched = bool(case.get("batched"))
    mod = CountedEpilogue.with_arity(counts, case["a_row"], case["b_row"], batched)
    metas = [torch.empty(s, dtype=d, device="meta") for s, d in counted_epilogue_shapes(case)]
    return mod, metas


def reference_key_cases():
    """Every GEMM / BMM key of the committed fixture, parsed: [(table, key, case)]."""
    import json
    from pathlib import Path
    doc = json.loads((Path(__file__).resolve().parent / "golden" / "reference_tuner_keys.json").read_text())
    out = []
    for table, batched in (("best_config_mm", False), ("best_config_bmm", True)):
        for key in doc["tables"][table]:
            case = parse_reference_key(key, batched)
            case["batched"] = batched
            out.append((table, key, case))
    return out


def reference_row_key_cases():
    """The distinct (anchor, rows, columns) of the fixture's softmax / layer norm keys, each with the bare anchor
    as a module and its meta inputs: [(key, anchor, rows, cols, module, metas)]."""
    import json
    from pathlib import Path
    doc = json.loads((Path(__file__).resolve().parent / "golden" / "reference_tuner_keys.json").read_text())
    half, f32 = torch.float16, torch.float32
    seen, out = set(), []
    for table, anchor in (("best_config_softmax", "softmax"), ("best_config_softmax_backward", "softmax_backward"),
                          ("best_config_layernorm", "layernorm"), ("best_config_layernorm_backward", "layernorm_backward")):
        for key in doc["tables"][table]:
            rows, cols = (int(v) for v in key.partition(")")[0].strip("(").split(","))
            if (anchor, rows, cols) in seen:
                continue
            seen.add((anchor, rows, cols))
            x = torch.empty((rows, cols), dtype=half, device="meta")
            stat = torch.empty((rows, 1), dtype=f32, device="meta")
            mod, metas = {"softmax": (_BareSoftmax(), [x]), "softmax_backward": (_BareSoftmaxBackward(half), [x, x]),
                          "layernorm": (_BareLayerNorm(cols), [x]),
                          "layernorm_backward": (_BareLayerNormBackward(cols), [x, x, stat, stat])}[anchor]
            out.append((key, anchor, rows, cols, mod, metas))
    return out
