"""Pins of the CPU oracle (oracle/evt_oracle.py): each part is checked against
something that does not share its code -- an independent float64 closed form,
a brute-force loop, a mathematical identity, or the committed fixtures -- so a
dropped term, a wrong sign or a transposed operand fails at least one check."""
import math
from pathlib import Path

import numpy as np
import pytest
import torch

from tests import patterns as W
from oracle import evt_oracle as O

aten = torch.ops.aten


@pytest.mark.parametrize("cfg", [1, 2, 3, 4, 5])
@pytest.mark.parametrize("shapes", ["small", "ragged", "unaligned"])
def test_eager_fp32_matches_closed_form(cfg, shapes):
    sh = {"small": W.SMALL_SHAPES, "ragged": W.RAGGED_SHAPES, "unaligned": W.UNALIGNED_SHAPES}[shapes][cfg]
    inputs = W.make_inputs(cfg, sh)
    got = O.eval_fp32(W.CONFIGS[cfg].module(), inputs)
    want = O.closed_form(cfg, inputs)
    assert len(got) == len(want)
    for g, w in zip(got, want):
        assert O.max_rel_err(g.numpy().reshape(w.shape), w) <= 2e-4   # fp32 vs float64 accumulation


def test_gemm_index_conventions_bruteforce():
    g = torch.Generator().manual_seed(7)
    a = torch.randn(5, 7, generator=g).half()
    b = torch.randn(7, 3, generator=g).half()
    ref = O.gemm_bruteforce(a, b)
    assert np.allclose((a.double() @ b.double()).numpy(), ref, atol=1e-12)
    # config 4 uses W^T: (dY W^T)[i][j] = sum_k dY[i][k] W[j][k]
    w = torch.randn(3, 7, generator=g).half()
    p = torch.zeros(5, 3).half()          # GELU'(0) = 0.5
    dp, db = O.closed_form(4, [a, w, p])
    assert np.allclose(dp, 0.5 * O.gemm_bruteforce(a, w.t()), atol=1e-12)
    assert np.allclose(db, dp.sum(0))
    # config 2 contracts the last axis of both operands
    q = torch.randn(2, 4, 6, generator=g).half()
    k = torch.randn(2, 5, 6, generator=g).half()
    s = O.closed_form(2, [q, k])[0]
    for l in range(2):
        assert np.allclose(s[l], 0.125 * O.gemm_bruteforce(q[l], k[l].t()), atol=1e-12)


def test_identity_and_ones_cases():
    n = 16
    eye = torch.eye(n).half()
    w = (torch.arange(n * n).reshape(n, n).float() / 64).half()
    bias = torch.arange(n).half()
    out = O.eval_fp32(W.FFNUpGelu(), [eye, w, bias])[0]
    want = torch.nn.functional.gelu(w.float() + bias.float(), approximate="tanh")   # A = I => D = epi(B)
    assert torch.allclose(out, want, atol=1e-6)
    # bias must broadcast along rows (one value per column)
    out0 = O.eval_fp32(W.FFNUpGelu(), [torch.zeros(n, n).half(), w, bias])[0]
    assert torch.allclose(out0, O_gelu(bias.float()).expand(n, n), atol=1e-6)
    # column sums of an all-ones product are exact integers: sum_m (1 * K) * GELU'(0)
    ones = torch.ones(32, 8).half()
    dp, db = O.eval_fp32(W.FFNBackwardDBias(), [ones, torch.ones(4, 8).half(), torch.zeros(32, 4).half()])
    assert torch.equal(db, torch.full((4,), 32 * 8 * 0.5))


def O_gelu(x):
    return torch.from_numpy(O.gelu_tanh(x.double().numpy())).float()


def test_gelu_definition_and_gradient():
    x = np.linspace(-6, 6, 241)
    t = torch.from_numpy(x)
    assert np.allclose(O.gelu_tanh(x), torch.nn.functional.gelu(t, approximate="tanh").numpy(), atol=1e-12)
    assert O.gelu_tanh(np.array([0.0]))[0] == 0.0
    assert abs(O.gelu_tanh(np.array([30.0]))[0] - 30.0) < 1e-9 and abs(O.gelu_tanh(np.array([-30.0]))[0]) < 1e-9
    assert np.allclose(O.gelu_tanh(x) - O.gelu_tanh(-x), x, atol=1e-12)      # odd-part identity
    h = 1e-6
    fd = (O.gelu_tanh(x + h) - O.gelu_tanh(x - h)) / (2 * h)
    assert np.allclose(O.gelu_tanh_grad(x), fd, atol=1e-8)
    gb = aten.gelu_backward(torch.ones_like(t), t, approximate="tanh").numpy()
    assert np.allclose(O.gelu_tanh_grad(x), gb, atol=1e-12)
    # tanh and erf flavours differ by more than fp16 resolution somewhere: the oracle must not confuse them
    erf = torch.nn.functional.gelu(t).numpy()
    assert np.max(np.abs(erf - O.gelu_tanh(x))) > 1e-4


def test_softmax_stats_identities():
    inputs = W.make_inputs(2, W.SMALL_SHAPES[2])
    s, m, l = O.eval_fp32(W.AttnScoreSoftmaxStats(), inputs)
    assert torch.all(l >= 1.0)
    p = torch.exp(s - m) / l
    assert torch.allclose(p.sum(-1), torch.ones_like(p.sum(-1)), atol=1e-5)
    assert torch.allclose(torch.logsumexp(s, -1, keepdim=True), m + torch.log(l), atol=1e-5)
    # shift invariance: scaling q by 2 doubles s; instead shift via closed form
    s64, m64, l64 = O.closed_form(2, inputs)
    c = 3.25
    m2 = (s64 + c).max(-1, keepdims=True)
    assert np.allclose(m2, m64 + c) and np.allclose(np.exp(s64 + c - m2).sum(-1, keepdims=True), l64)


def test_layernorm_stats_identities():
    inputs = W.make_inputs(3, W.SMALL_SHAPES[3])
    o, mean, var = O.eval_fp32(W.OutProjResidualLNStats(), inputs)
    v2, m2 = torch.var_mean(o.double(), dim=1, correction=0)
    assert torch.allclose(mean.double(), m2, atol=1e-5) and torch.allclose(var.double(), v2, rtol=1e-5)
    # constant rows: zero weights, zero residual -> every row equals the bias ... var over N of the bias
    x, w, b, r = inputs
    o0, mean0, var0 = O.eval_fp32(W.OutProjResidualLNStats(), [x, torch.zeros_like(w), torch.full_like(b, 0.5), torch.zeros_like(r)])
    assert torch.all(var0 == 0) and torch.all(mean0 == 0.5)
    # affine: adding a constant to the residual shifts the mean, keeps the variance
    o1, mean1, var1 = O.eval_fp32(W.OutProjResidualLNStats(), [x, w, b, (r.float() + 2).half()])
    assert torch.allclose(mean1, mean + 2, atol=2e-3) and torch.allclose(var1, var, rtol=5e-3, atol=1e-3)


def test_cross_entropy_identities():
    M, N, K = 8, 64, 16
    h = torch.randn(M, K).half()
    labels = torch.arange(M, dtype=torch.int32)
    (loss,) = O.eval_fp32(W.ClassifierCrossEntropy(), [h, torch.zeros(K, N).half(), labels])
    assert torch.allclose(loss, torch.full((M,), math.log(N)), atol=1e-6)        # uniform logits
    inputs = W.make_inputs(5, W.SMALL_SHAPES[5])
    (loss,) = O.eval_fp32(W.ClassifierCrossEntropy(), inputs)
    logits = inputs[0].float() @ inputs[1].float()
    want = torch.nn.functional.cross_entropy(logits, inputs[2].long(), reduction="none")
    assert torch.allclose(loss, want, atol=1e-5)
    # a dominant label logit gives a loss near zero
    w = torch.zeros(K, N)
    hh = torch.zeros(M, K); hh[:, 0] = 1.0
    w[0, 3] = 50.0
    (l0,) = O.eval_fp32(W.ClassifierCrossEntropy(), [hh.half(), w.half(), torch.full((M,), 3, dtype=torch.int32)])
    assert torch.all(l0.abs() < 1e-6)


def test_combine_operators_are_partition_independent():
    rng = np.random.default_rng(0)
    x = rng.normal(size=257) * 3
    m_ref = x.max(); l_ref = np.exp(x - m_ref).sum()
    n_ref, mean_ref, m2_ref = len(x), x.mean(), ((x - x.mean()) ** 2).sum()
    for trial in range(20):
        cuts = np.sort(rng.choice(np.arange(1, len(x)), size=rng.integers(1, 9), replace=False))
        parts = np.split(x, cuts)
        order = rng.permutation(len(parts))
        ms = (-math.inf, 0.0)
        wf = (0.0, 0.0, 0.0)
        for i in order:
            p = parts[i]
            ms = O.combine_maxsumexp(ms, (p.max(), np.exp(p - p.max()).sum()))
            wf = O.combine_welford(wf, (len(p), p.mean(), ((p - p.mean()) ** 2).sum()))
        assert abs(ms[0] - m_ref) < 1e-12 and abs(ms[1] - l_ref) / l_ref < 1e-12
        assert wf[0] == n_ref and abs(wf[1] - mean_ref) < 1e-12 and abs(wf[2] - m2_ref) / m2_ref < 1e-12


def test_error_metric():
    ref = torch.tensor([1.0, -2.0, 0.0, 4.0])
    assert O.max_rel_err(ref, ref) == 0.0
    assert abs(O.max_rel_err(ref * 1.01, ref) - 0.01) < 1e-6
    rms = math.sqrt((1 + 4 + 16) / 4)
    out = ref.clone(); out[2] = 1e-3                     # error where ref == 0 is measured against tau
    assert abs(O.max_rel_err(out, ref) - 1e-3 / (1e-2 * rms)) < 1e-6
    assert O.max_rel_err(torch.tensor([float("nan")]), torch.tensor([1.0])) == float("inf")


def test_golden_fixtures_match_oracle():
    gold = np.load(Path(__file__).parent / "golden" / "configs_small.npz")
    for cfg in (1, 2, 3, 4, 5):
        inputs = W.make_inputs(cfg, W.GOLDEN_SHAPES[cfg])
        for i, t in enumerate(inputs):
            assert np.array_equal(gold[f"c{cfg}_in{i}"], t.numpy())
        outs = O.eval_fp32(W.CONFIGS[cfg].module(), inputs)
        closed = O.closed_form(cfg, inputs)
        for i, (o, c) in enumerate(zip(outs, closed)):
            g = gold[f"c{cfg}_out{i}"]
            assert O.max_rel_err(o.numpy(), g) <= 1e-6
            assert O.max_rel_err(g.reshape(c.shape), c) <= 2e-4


def test_philox_known_answers():
    """Philox4x32-10 against the known-answer vectors of the Random123
    distribution (kat_vectors: philox4x32 10), and the [0, 1) mapping."""
    import numpy as np
    from oracle import philox
    kat = [([0, 0, 0, 0], (0, 0), [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]),
           ([0xffffffff] * 4, (0xffffffff, 0xffffffff), [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]),
           ([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], (0xa4093822, 0x299f31d0),
            [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1])]
    for ctr, key, want in kat:
        got = philox.philox4x32_10(np.array([ctr], dtype=np.uint32), key)[0]
        assert [int(x) for x in got] == want
    u = philox.uniform(seed=7, offset=3, salt=1, numel=1 << 18)
    assert u.dtype == np.float32 and u.min() >= 0.0 and u.max() < 1.0
    assert abs(float(u.mean()) - 0.5) < 3e-3 and abs(float((u >= 0.7).mean()) - 0.3) < 3e-3
    # element e is word e & 3 of the block with counter (e >> 2, 0, offset, salt) under key = seed
    blk = philox.philox4x32_10(np.array([[5, 0, 3, 1]], dtype=np.uint32), (7, 0))[0]
    assert np.array_equal(u[20:24], (blk >> np.uint32(8)).astype(np.float32) * np.float32(2.0 ** -24))
    # a different offset or salt is a different stream
    assert not np.array_equal(u, philox.uniform(7, 4, 1, 1 << 18))
    assert not np.array_equal(u, philox.uniform(7, 3, 2, 1 << 18))


# ---------------------------------------------------------------------------
# row-wise anchors: the oracle evaluates the ATen ops themselves; what they
# must equal is fixed by calculus (autograd of the forward definition, float64)
# and by closed forms
# ---------------------------------------------------------------------------

def test_row_anchor_oracle_against_definitions():
    g = torch.Generator().manual_seed(11)
    for n in (8, 24, 1000):
        # softmax: closed form; rows sum to one; shift invariance
        mod, (x,) = W.row_edge_case("softmax", n, torch.float16)
        (y,) = O.eval_fp32(mod, [x])
        xd = x.double()
        e = np.exp(xd.numpy() - xd.numpy().max(-1, keepdims=True))
        assert np.allclose(y.numpy(), e / e.sum(-1, keepdims=True), rtol=1e-5, atol=1e-7)
        # softmax backward = vector-Jacobian product of softmax
        mod, (gr, ys) = W.row_edge_case("softmax_backward", n, torch.float16)
        (dx,) = O.eval_fp32(mod, [gr, ys])
        z = torch.randn(3, 7, n, dtype=torch.float64, generator=g).requires_grad_()
        sm = torch.softmax(z, -1)
        (auto,) = torch.autograd.grad(sm, z, gr.double())
        manual = (gr.double() - (gr.double() * sm).sum(-1, keepdim=True)) * sm
        assert torch.allclose(auto, manual.detach(), rtol=1e-9, atol=1e-12)            # the formula itself
        yd = ys.double()
        assert torch.allclose(dx.double(), (gr.double() - (gr.double() * yd).sum(-1, keepdim=True)) * yd, rtol=1e-4, atol=1e-6)
        # layer norm: closed form of y, mean, rstd
        mod, (x,) = W.row_edge_case("layernorm", n, torch.float16)
        yv, mean, rstd = O.eval_fp32(mod, [x])
        xd = x.double().numpy()
        mu, var = xd.mean(-1, keepdims=True), xd.var(-1, keepdims=True)
        assert np.allclose(mean.numpy(), mu, rtol=1e-5, atol=1e-6)
        assert np.allclose(rstd.numpy(), 1 / np.sqrt(var + 1e-5), rtol=1e-5)
        assert np.allclose(yv.numpy(), (xd - mu) / np.sqrt(var + 1e-5), rtol=1e-4, atol=1e-5)
        # layer norm backward = vector-Jacobian product of layer norm (no weight)
        mod, (gr, x, mean, rstd) = W.row_edge_case("layernorm_backward", n, torch.float16)
        (dx,) = O.eval_fp32(mod, [gr, x, mean, rstd])
        z = x.double().clone().requires_grad_()
        out = torch.nn.functional.layer_norm(z, (n,), eps=1e-5)
        (auto,) = torch.autograd.grad(out, z, gr.double())
        assert torch.allclose(dx.double(), auto, rtol=2e-4, atol=2e-5)
