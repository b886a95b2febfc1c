"""The fused-subgraph workloads this backend is measured and tested on.

`CONFIGS` holds the five headline subgraphs (FFN up-projection + GELU,
attention scores + softmax statistics, output projection + residual +
LayerNorm statistics, FFN backward + bias gradient, classifier + cross
entropy), written as ATen-level modules the way the reference's own fuser
tests are (unittest/evt_fuser/mm.py:30-236, bmm.py:29-94), each with its seeded
input generator, algorithmic flop / byte counts and output roles; besides them the
bandwidth cases of the row-wise anchors (`ROW_BENCH`) and the encoder layer whose
training step the benchmark times and the tuner ships tiles for.  The catalogue of
test patterns lives with the tests (tests/patterns.py).
"""
from __future__ import annotations

import operator
from dataclasses import dataclass
from typing import Callable, Dict, List, Sequence, Tuple

import torch
from torch.fx import GraphModule, symbolic_trace
from torch.fx.passes.shape_prop import ShapeProp

aten = torch.ops.aten


# ---------------------------------------------------------------------------
# the five headline configurations
# ---------------------------------------------------------------------------

class FFNUpGelu(torch.nn.Module):
    """Y = GELU_tanh(X W + b)"""
    def forward(self, x, w, b):
        mm = aten.mm(x, w)
        add = aten.add(mm, b)
        gelu = aten.gelu(add, approximate="tanh")
        return gelu


class AttnScoreSoftmaxStats(torch.nn.Module):
    """S = (Q K^T) / 8 ; per-row max and sum-exp of S"""
    def forward(self, q, k):
        kt = aten.permute(k, [0, 2, 1])
        bmm = aten.bmm(q, kt)
        s = aten.mul(bmm, 0.125)
        sf = aten._to_copy(s, dtype=torch.float32)
        m = aten.amax(sf, [-1], True)
        sub = aten.sub(sf, m)
        e = aten.exp(sub)
        l = aten.sum(e, [-1], True)
        return s, m, l


class OutProjResidualLNStats(torch.nn.Module):
    """O = X W + b + R ; per-row mean and (biased) variance of O"""
    def forward(self, x, w, b, r):
        mm = aten.mm(x, w)
        add = aten.add(mm, b)
        o = aten.add(add, r)
        of = aten._to_copy(o, dtype=torch.float32)
        vm = aten.var_mean(of, [1], correction=0, keepdim=False)
        var = operator.getitem(vm, 0)
        mean = operator.getitem(vm, 1)
        return o, mean, var


class FFNBackwardDBias(torch.nn.Module):
    """dP = (dY W^T) * GELU_tanh'(P) ; dbias = sum_m dP"""
    def forward(self, dy, w, p):
        wt = aten.permute(w, [1, 0])
        mm = aten.mm(dy, wt)
        dp = aten.gelu_backward(mm, p, approximate="tanh")
        dpf = aten._to_copy(dp, dtype=torch.float32)
        db = aten.sum(dpf, [0])
        return dp, db


class ClassifierCrossEntropy(torch.nn.Module):
    """loss_m = logsumexp_n(H W) - (H W)[m, label_m]   (logits never stored)"""
    def forward(self, h, w, labels):
        mm = aten.mm(h, w)
        lf = aten._to_copy(mm, dtype=torch.float32)
        lse = aten.logsumexp(lf, [1])
        idx64 = aten._to_copy(labels, dtype=torch.int64)
        idx = aten.unsqueeze(idx64, 1)
        z = aten.gather(lf, 1, idx)
        zs = aten.squeeze(z, 1)
        loss = aten.sub(lse, zs)
        return loss


def _randn(g, shape, scale=1.0):
    return (torch.randn(shape, generator=g, dtype=torch.float32) * scale).half()


@dataclass
class Workload:
    name: str
    module: Callable[[], torch.nn.Module]
    make_inputs: Callable[[torch.Generator, float], List[torch.Tensor]]   # (generator, size scale) -> CPU tensors
    dims: Tuple[int, int, int, int]          # M, N, K, L at full size
    flops: int
    bytes: int
    reduction_outputs: Tuple[int, ...] = ()  # indices of fp32 reduction outputs (tolerance 1e-3)
    description: str = ""

    def seed(self, cfg_index: int) -> int:
        return 0xE7A0 + cfg_index


def _cfg1(g, M=4096, N=4096, K=1024):
    return [_randn(g, (M, K)), _randn(g, (K, N), 0.02), _randn(g, (N,), 0.02)]


def _cfg2(g, L=64, S=512, D=64):
    return [_randn(g, (L, S, D)), _randn(g, (L, S, D))]


def _cfg3(g, M=8192, N=1024, K=4096):
    return [_randn(g, (M, K)), _randn(g, (K, N), 0.02), _randn(g, (N,), 0.02), _randn(g, (M, N))]


def _cfg4(g, M=8192, N=1024, K=4096):
    return [_randn(g, (M, K), 0.01), _randn(g, (N, K), 0.02), _randn(g, (M, N))]


def _cfg5(g, M=1024, N=131072, K=512):
    h = _randn(g, (M, K))
    w = _randn(g, (K, N), 0.02)
    labels = torch.randint(0, N, (M,), generator=g, dtype=torch.int64).to(torch.int32)
    return [h, w, labels]


CONFIGS: Dict[int, Workload] = {
    1: Workload("ffn_up_gelu", FFNUpGelu, _cfg1, (4096, 4096, 1024, 1), 34_359_738_368, 50_339_840, (),
                "BERT-large FFN up-projection: GELU_tanh(XW+b)"),
    2: Workload("attn_score_softmax_stats", AttnScoreSoftmaxStats, _cfg2, (512, 512, 64, 64), 2_147_483_648,
                42_205_184, (1, 2), "QK^T/8 + per-row max and sum-exp"),
    3: Workload("out_proj_residual_ln_stats", OutProjResidualLNStats, _cfg3, (8192, 1024, 4096, 1),
                68_719_476_736, 109_119_488, (1, 2), "XW+b+R + per-row mean/var"),
    4: Workload("ffn_backward_dbias", FFNBackwardDBias, _cfg4, (8192, 1024, 4096, 1), 68_719_476_736,
                109_056_000, (1,), "(dY W^T) * GELU'(P) + column sum"),
    5: Workload("classifier_cross_entropy", ClassifierCrossEntropy, _cfg5, (1024, 131072, 512, 1),
                137_438_953_472, 135_274_496, (0,), "HW -> per-row CE loss"),
}

# small instances of the same graphs (shape arguments for make_inputs) used by
# parity tests where the CPU oracle must finish in seconds
SMALL_SHAPES = {
    1: dict(M=256, N=384, K=128),
    2: dict(L=3, S=192, D=64),
    3: dict(M=320, N=640, K=256),
    4: dict(M=512, N=320, K=192),
    5: dict(M=128, N=4096, K=128),
}


def make_inputs(cfg: int, shapes: dict = None, seed: int = None) -> List[torch.Tensor]:
    g = torch.Generator(device="cpu").manual_seed(CONFIGS[cfg].seed(cfg) if seed is None else seed)
    fn = CONFIGS[cfg].make_inputs
    return fn(g, **(shapes or {}))


def unfused_eager(cfg: int) -> Callable:
    """The literal unfused GPU sequence (rocBLAS/hipBLASLt GEMM + one eager
    kernel per epilogue op) the fused kernel is compared with."""
    F = torch.nn.functional
    if cfg == 1:
        return lambda x, w, b: F.gelu(torch.mm(x, w) + b, approximate="tanh")
    if cfg == 2:
        def f(q, k):
            s = torch.bmm(q, k.transpose(1, 2)) * 0.125
            sf = s.float()
            m = sf.amax(-1, keepdim=True)
            return s, m, (sf - m).exp().sum(-1, keepdim=True)
        return f
    if cfg == 3:
        def f(x, w, b, r):
            o = torch.mm(x, w) + b + r
            var, mean = torch.var_mean(o.float(), dim=1, correction=0)
            return o, mean, var
        return f
    if cfg == 4:
        def f(dy, w, p):
            dp = aten.gelu_backward(torch.mm(dy, w.t()), p, approximate="tanh")
            return dp, dp.float().sum(0)
        return f
    if cfg == 5:
        def f(h, w, labels):
            lf = torch.mm(h, w).float()
            return torch.logsumexp(lf, 1) - lf.gather(1, labels.long().unsqueeze(1)).squeeze(1)
        return f
    raise KeyError(cfg)


# ---------------------------------------------------------------------------
# tracing helper (symbolic_trace + ShapeProp on meta tensors: no data needed)
# ---------------------------------------------------------------------------

def trace_module(module: torch.nn.Module, example_inputs: Sequence[torch.Tensor]) -> GraphModule:
    gm = symbolic_trace(module)
    metas = [t.to("meta") if isinstance(t, torch.Tensor) else t for t in example_inputs]
    ShapeProp(gm).propagate(*metas)
    return gm


def fused_nodes(gm: GraphModule):
    """The fused-kernel call nodes `EVTFuser.trace` placed in `gm` (meta["evt"])."""
    return [n for n in gm.graph.nodes if n.op == "call_function" and n.meta.get("evt")]


def fuse(module: torch.nn.Module, example_inputs: Sequence[torch.Tensor], passes=None) -> GraphModule:
    """symbolic_trace -> ShapeProp -> pass_fusion -> recompile, as the
    reference's UnitTestBase.util_test does (python/gtl/helper/test_helper.py:78-96)."""
    from .passes import pass_fusion
    gm = trace_module(module, example_inputs)
    for p in (passes or [pass_fusion]):
        p(gm, gm.graph)
    gm.recompile()
    return gm


# bandwidth cases for the row-wise anchors (bench.py): attention probabilities of 256 x 512 x 512 and
# 131072 rows of a 1024-wide layer norm, fp16, sized so that a few rotating buffer sets exceed the 256 MB cache

class RowBenchSoftmax(torch.nn.Module):
    def forward(self, x):
        return aten._softmax(x, -1, False)


class RowBenchSoftmaxBackward(torch.nn.Module):
    def forward(self, g, y):
        return aten._softmax_backward_data(g, y, -1, torch.float16)


class RowBenchLayerNorm(torch.nn.Module):
    def forward(self, x, w, b):
        ln = aten.native_layer_norm(x, [1024], None, None, 1e-5)
        y = aten.add(aten.mul(operator.getitem(ln, 0), w), b)
        return y, operator.getitem(ln, 1), operator.getitem(ln, 2)


class RowBenchLayerNormBackward(torch.nn.Module):
    def forward(self, g, x, mean, rstd, w):
        ln = aten.native_layer_norm_backward(g, x, [1024], mean, rstd, w, None, [True, False, False])
        return operator.getitem(ln, 0)


def _row_bench_shapes():
    sm, ln = (256, 512, 512), (131072, 1024)
    h, f = torch.float16, torch.float32
    return {
        # vocabulary-sized rows (one workgroup of 8 waves per row): BERT's 30522 as it is (no 16-byte accesses:
        # rows start at odd multiples of 4 bytes) and padded to a multiple of 8
        "softmax_vocab_30522": (RowBenchSoftmax, [((4096, 30522), h)], 2 * 2 * 4096 * 30522),
        "softmax_vocab_30528": (RowBenchSoftmax, [((4096, 30528), h)], 2 * 2 * 4096 * 30528),
        # name: (module, [(shape, dtype), ...] inputs, algorithmic bytes per launch)
        "softmax": (RowBenchSoftmax, [(sm, h)], 2 * 2 * 256 * 512 * 512),
        "softmax_backward": (RowBenchSoftmaxBackward, [(sm, h), (sm, h)], 3 * 2 * 256 * 512 * 512),
        "layernorm": (RowBenchLayerNorm, [(ln, h), ((1024,), h), ((1024,), h)], 2 * 2 * 131072 * 1024 + 8 * 131072),
        "layernorm_backward": (RowBenchLayerNormBackward,
                               [(ln, h), (ln, h), ((131072, 1), f), ((131072, 1), f), ((1024,), h)],
                               3 * 2 * 131072 * 1024 + 8 * 131072),
    }


ROW_BENCH = _row_bench_shapes()


class EncoderLayer(torch.nn.Module):
    """fp16 post-LN transformer encoder layer with a squared-error loss: Q, K, V
    projections (three Linear layers as in the reference's BERT, or one fused
    [d, 3d] projection), batched QK^T and PV products, softmax, output
    projection, two layer norms and the GELU feed-forward block (the shape of
    the reference's BERT test, unittest/fx_passes/bert.py, at a small size)."""
    def __init__(self, d: int = 256, heads: int = 4, ffn: int = 1024, fused_qkv: bool = True) -> None:
        super().__init__()
        self.heads = heads
        self.fused_qkv = fused_qkv
        if fused_qkv:
            self.qkv = torch.nn.Linear(d, 3 * d)
        else:
            self.q = torch.nn.Linear(d, d)
            self.k = torch.nn.Linear(d, d)
            self.v = torch.nn.Linear(d, d)
        self.out = torch.nn.Linear(d, d)
        self.ln1 = torch.nn.LayerNorm(d)
        self.ln2 = torch.nn.LayerNorm(d)
        self.ffn1 = torch.nn.Linear(d, ffn)
        self.ffn2 = torch.nn.Linear(ffn, d)

    def forward(self, x, target):
        B, S, D = x.shape
        H = self.heads
        dh = D // H
        if self.fused_qkv:
            qkv = self.qkv(x).view(B, S, 3, H, dh).permute(2, 0, 3, 1, 4)
            q, k, v = qkv[0], qkv[1], qkv[2]
        else:
            split = lambda t: t.view(B, S, H, dh).permute(0, 2, 1, 3)      # noqa: E731
            q, k, v = split(self.q(x)), split(self.k(x)), split(self.v(x))
        att = torch.softmax((q @ k.transpose(-1, -2)) / (dh ** 0.5), -1)
        ctx = (att @ v).permute(0, 2, 1, 3).reshape(B, S, D)
        x = self.ln1(x + self.out(ctx))
        x = self.ln2(x + self.ffn2(torch.nn.functional.gelu(self.ffn1(x), approximate="tanh")))
        return ((x.float() - target) ** 2).sum()


# a BERT-large layer, with separate Q / K / V projections as in the reference's BERT
ENCODER_BENCH = dict(d=1024, heads=16, ffn=4096, batch=8, seq=512, fused_qkv=False)


def encoder_layer(seed: int = 0, device: str = "cpu", dtype=torch.float16, d: int = 256, heads: int = 4,
                  ffn: int = 1024, batch: int = 8, seq: int = 128, fused_qkv: bool = True):
    """(model, (x, target)) with seeded parameters and inputs (default: batch 8, sequence 128, width 256)."""
    g = torch.Generator(device="cpu").manual_seed(0xE9C + seed)
    model = EncoderLayer(d, heads, ffn, fused_qkv)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if p.dim() == 2:
                p.copy_(torch.randn(p.shape, generator=g) * 0.05)
            elif "ln" in name and name.endswith("weight"):
                p.copy_(1.0 + 0.1 * torch.randn(p.shape, generator=g))
            else:
                p.copy_(0.02 * torch.randn(p.shape, generator=g))
    model = model.to(dtype).to(device)
    x = torch.randn(batch, seq, d, generator=g).to(dtype).to(device)
    target = torch.randn(batch, seq, d, generator=g).to(device)
    return model, (x, target)
