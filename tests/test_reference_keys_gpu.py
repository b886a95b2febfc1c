"""The problems of the reference's tuner caches at their real sizes
(tests/golden/reference_tuner_keys.json), one launch each through the C ABI: every GEMM / BMM key and every
softmax / layer norm problem against the oracle (the tests at the end of this file), and the extreme ones with
checks of their own:

  * `2048_670208_512_h_h_R_C_1_1_0_1_1_0_0`  a 2.75 GB fp16 output and a 2.75 GB residual (byte offsets past
    2^31), a [N] vector, a per-column sum over 8 row tiles;
  * `736389_64_128_h_h_R_C_0_1_0_1_0_0_0`     odd M, 2877 or more row tiles, one narrow column tile;
  * `16384_1024_30528_h_h_R_R_1_0_2_1_2_0_0`  K = 30528, two [M] vectors, two per-column reductions;
  * `64_64_736389_h_h_C_R_0_0_0_1_0_0_0`      one output tile, K = 736389 (odd: a K tail in the last k-tile);
  * `512_512_512_64_h_h_R_R_0_1_0_1_0_0_1`    the batched key with a row store ([N] values the epilogue forms, uses
    and writes from the tiles that hold row 0).

The oracle (PyTorch fp32 on the CPU, oracle/evt_oracle.py) is evaluated on the same inputs restricted to sampled
rows / columns -- first and last tiles, the columns on either side of the 2^31-byte boundary -- where the whole
problem would take minutes, and on everything where it takes seconds; on top, properties that hold for the whole
output: its sum against the closed form sum_k (sum_m A)(sum_n B) + ..., and the reduction outputs against sums of
the stored tensor."""
import pytest
import torch

from evt_ae_amd.workloads import fused_nodes
from oracle import evt_oracle
from tests import patterns as W

pytestmark = pytest.mark.gpu


def _inputs(case, seed):
    """Seeded inputs on the GPU (generated there: the large ones run to gigabytes), scaled so that every value
    of the epilogue is O(1)."""
    g = torch.Generator(device="cuda").manual_seed(seed)
    out = []
    for i, (shape, dt) in enumerate(W.counted_epilogue_shapes(case)):
        t = torch.empty(shape, dtype=dt, device="cuda")
        flat = t.view(-1)
        step = 1 << 28
        is_col = len(shape) >= 2 and shape[-1] == 1 and i >= 2
        for lo in range(0, flat.numel(), step):
            n = min(step, flat.numel() - lo)
            if is_col:       # [M, 1] factors around one
                flat[lo:lo + n] = (torch.rand(n, generator=g, device="cuda") + 0.5).to(dt)
            else:
                scale = case["K"] ** -0.5 if i == 1 else 1.0
                flat[lo:lo + n] = (torch.randn(n, generator=g, device="cuda") * scale).to(dt)
        out.append(t)
    return out


def _fused(case, inputs):
    mod, _ = W.counted_epilogue(case)
    gm = W.fuse(mod, [t.to("meta") for t in inputs])
    (node,) = fused_nodes(gm)
    return mod, gm, node.target


def _restrict(case, inputs, rows=None, cols=None):
    """CPU copies of the inputs restricted to some rows and / or columns of the output."""
    counts = case["counts"]
    lead = 1 if case["batched"] else 0
    out = []
    for i, t in enumerate(inputs):
        if i == 0:      # A: [M, K] or [K, M]
            if rows is not None:
                t = t.index_select(lead + (0 if case["a_row"] else 1), rows)
        elif i == 1:    # B: [K, N] or [N, K]
            if cols is not None:
                t = t.index_select(lead + (1 if case["b_row"] else 0), cols)
        elif i < 2 + counts[0]:                 # aux [M, N]
            if rows is not None:
                t = t.index_select(lead, rows)
            if cols is not None:
                t = t.index_select(lead + 1, cols)
        elif i < 2 + counts[0] + counts[1]:     # [N]
            if cols is not None:
                t = t.index_select(0, cols)
        else:                                   # [M, 1]
            if rows is not None:
                t = t.index_select(lead, rows)
        out.append(t.cpu())
    return out


def _check(name, got, ref, reduction):
    ok, err = evt_oracle.check(got.cpu(), ref, reduction=reduction)
    assert ok, (name, err)


def test_output_and_residual_beyond_two_gigabytes():
    key = "2048_670208_512_h_h_R_C_1_1_0_1_1_0_0"
    case = W.parse_reference_key(key, False); case["batched"] = False
    M, N, K = case["M"], case["N"], case["K"]
    inputs = _inputs(case, 11)
    A, B, aux, rv = inputs
    assert aux.numel() * 2 > (1 << 31)
    mod, gm, op = _fused(case, inputs)
    out, colsum = gm(*inputs)
    torch.cuda.synchronize()
    assert out.shape == (M, N) and colsum.shape == (N,) and colsum.dtype == torch.float32
    # columns: both ends, the last (partial) column tile, and whole columns for the per-column sums
    g = torch.Generator().manual_seed(5)
    cols = torch.cat([torch.arange(0, 8), torch.arange(N - 8, N), torch.randint(0, N, (48,), generator=g)]).cuda()
    ref_out, ref_sum = evt_oracle.eval_fp32(mod, _restrict(case, inputs, cols=cols))
    _check("columns", out.index_select(1, cols), ref_out, False)
    _check("column sums", colsum.index_select(0, cols), ref_sum, True)
    # rows on either side of the 2^31-byte boundary of the output (row 1602 starts past it), first and last
    boundary = (1 << 31) // (2 * N)
    rows = torch.tensor([0, 1, boundary - 1, boundary, boundary + 1, M - 1]).cuda()
    ref_rows, _ = evt_oracle.eval_fp32(mod, _restrict(case, inputs, rows=rows))
    _check("rows", out.index_select(0, rows), ref_rows, False)
    # the whole output: its sum against the closed form, and the per-column sums against the stored tensor
    f64 = torch.float64
    total = float((A.sum(0, dtype=f64) * B.sum(0, dtype=f64)).sum() + aux.sum(dtype=f64) + M * rv.sum(dtype=f64))
    got_total = float(colsum.double().sum())
    scale = float(colsum.double().abs().sum())
    assert abs(got_total - total) <= 1e-5 * scale, (got_total, total, scale)
    stored = torch.zeros(N, dtype=torch.float64, device="cuda")
    for lo in range(0, M, 256):
        stored += out[lo:lo + 256].double().sum(0)
    # the stored tensor is rounded to fp16 (at most 2^-12 of its magnitude per element, signs random): a sum of M of
    # them strays by a few sqrt(M) such steps
    bound = 4.0 * M ** 0.5 * 2.0 ** -12 * float(out.abs().max())
    assert float((stored - colsum.double()).abs().max()) <= bound


def test_odd_row_count_with_thousands_of_row_tiles():
    key = "736389_64_128_h_h_R_C_0_1_0_1_0_0_0"
    case = W.parse_reference_key(key, False); case["batched"] = False
    inputs = _inputs(case, 12)
    mod, gm, op = _fused(case, inputs)
    (out,) = gm(*inputs)
    torch.cuda.synchronize()
    (ref,) = evt_oracle.eval_fp32(mod, [t.cpu() for t in inputs])       # the whole problem: 6 GFLOP
    _check(key, out, ref, False)
    assert -(-case["M"] // op.tile.bm) >= 2877


def test_long_k_with_two_column_vectors_and_two_column_reductions():
    key = "16384_1024_30528_h_h_R_R_1_0_2_1_2_0_0"
    case = W.parse_reference_key(key, False); case["batched"] = False
    M, N, K = case["M"], case["N"], case["K"]
    inputs = _inputs(case, 13)
    mod, gm, op = _fused(case, inputs)
    out, s1, s2 = gm(*inputs)
    torch.cuda.synchronize()
    g = torch.Generator().manual_seed(6)
    cols = torch.cat([torch.arange(0, 4), torch.arange(N - 4, N), torch.randint(0, N, (24,), generator=g)]).cuda()
    ref_out, ref_s1, ref_s2 = evt_oracle.eval_fp32(mod, _restrict(case, inputs, cols=cols))
    _check("columns", out.index_select(1, cols), ref_out, False)
    _check("sum x", s1.index_select(0, cols), ref_s1, True)
    _check("sum x^2", s2.index_select(0, cols), ref_s2, True)
    rows = torch.tensor([0, 255, 256, M - 1]).cuda()
    ref_rows = evt_oracle.eval_fp32(mod, _restrict(case, inputs, rows=rows))[0]
    _check("rows", out.index_select(0, rows), ref_rows, False)
    # the reductions against the stored tensor, every column
    xs = out.double()
    assert float((xs.sum(0) - s1.double()).abs().max()) <= 4.0 * M ** 0.5 * 2.0 ** -12 * float(out.abs().max())
    assert float(((xs * xs).sum(0) - s2.double()).abs().max() / s2.double().abs().max()) <= 2e-3


def test_one_tile_with_an_odd_k_of_736389():
    key = "64_64_736389_h_h_C_R_0_0_0_1_0_0_0"
    case = W.parse_reference_key(key, False); case["batched"] = False
    inputs = _inputs(case, 14)
    mod, gm, op = _fused(case, inputs)
    (out,) = gm(*inputs)
    torch.cuda.synchronize()
    (ref,) = evt_oracle.eval_fp32(mod, [t.cpu() for t in inputs])
    _check(key, out, ref, False)
    (again,) = gm(*inputs)                      # repeated launches give the same bits
    torch.cuda.synchronize()
    assert torch.equal(out, again)


def test_batched_key_with_a_row_store():
    key = "512_512_512_64_h_h_R_R_0_1_0_1_0_0_1"
    case = W.parse_reference_key(key, True); case["batched"] = True
    inputs = _inputs(case, 15)
    mod, gm, op = _fused(case, inputs)
    assert op.ir.epilogue_counts() == case["counts"]
    out, rowvec = gm(*inputs)
    torch.cuda.synchronize()
    ref_out, ref_vec = evt_oracle.eval_fp32(mod, [t.cpu() for t in inputs])
    _check("scores", out, ref_out, False)
    _check("row store", rowvec, ref_vec, False)


# ---------------------------------------------------------------------------
# every GEMM / BMM key of the catalogue at its real size
# ---------------------------------------------------------------------------

_ALL_KEYS = [(table, key) for table, key, _ in W.reference_key_cases()]


def _split_outputs(counts, outs):
    """CountedEpilogue's outputs by kind: ([M, N] stores, [N] sums over the rows, [M] sums along the rows, [N] masks)."""
    outs = list(outs) if isinstance(outs, (tuple, list)) else [outs]
    a, b, c = counts[3], counts[3] + counts[4], counts[3] + counts[4] + counts[5]
    return outs[:a], outs[a:b], outs[b:c], outs[c:]


@pytest.mark.parametrize("table,key", _ALL_KEYS, ids=[k for _, k in _ALL_KEYS])
def test_every_reference_key_at_its_size(table, key):
    """One launch per key of the reference's tuner caches, on the problem size the key names, against the oracle:
    on the whole problem where that is at most 2e10 flop, else on sampled rows (all columns: the stores and the
    sums along the rows) and sampled columns (all rows: the stores and the sums over the rows), first and last
    tiles included."""
    batched = table == "best_config_bmm"
    case = W.parse_reference_key(key, batched); case["batched"] = batched
    counts = case["counts"] or (0, 0, 0, 1, 0, 0, 0)
    L, M, N, K = case["L"], case["M"], case["N"], case["K"]
    lead = 1 if batched else 0
    inputs = _inputs(case, 100 + len(key))
    mod, gm, op = _fused(case, inputs)
    assert op.ir.epilogue_counts() == tuple(counts), key
    outs = gm(*inputs)
    torch.cuda.synchronize()
    stores, over_rows, along_rows, masks = _split_outputs(counts, outs)
    if 2.0 * L * M * N * K <= 2e10:
        refs = _split_outputs(counts, evt_oracle.eval_fp32(mod, [t.cpu() for t in inputs]))
        for kind, got, ref in zip(("store", "sum over rows", "sum along rows", "row store"), (stores, over_rows, along_rows, masks), refs):
            for j, (o, r) in enumerate(zip(got, ref)):
                _check(f"{key} {kind} {j}", o, r, kind.startswith("sum"))
        return
    g = torch.Generator().manual_seed(len(key))
    rows = torch.unique(torch.cat([torch.tensor([0, 1, M - 1]), torch.randint(0, M, (9,), generator=g)])).cuda()
    cols = torch.unique(torch.cat([torch.arange(0, 4), torch.arange(N - 4, N), torch.randint(0, N, (16,), generator=g)])).cuda()
    r_stores, _, r_along, r_masks = _split_outputs(counts, evt_oracle.eval_fp32(mod, _restrict(case, inputs, rows=rows)))
    for j, (o, r) in enumerate(zip(stores, r_stores)):
        _check(f"{key} store {j} rows", o.index_select(lead, rows), r, False)
    for j, (o, r) in enumerate(zip(along_rows, r_along)):
        _check(f"{key} sum along rows {j}", o.index_select(lead, rows), r, True)
    for j, (o, r) in enumerate(zip(masks, r_masks)):
        _check(f"{key} row store {j}", o, r, False)
    c_stores, c_over, _, _ = _split_outputs(counts, evt_oracle.eval_fp32(mod, _restrict(case, inputs, cols=cols)))
    for j, (o, r) in enumerate(zip(stores, c_stores)):
        _check(f"{key} store {j} columns", o.index_select(lead + 1, cols), r, False)
    for j, (o, r) in enumerate(zip(over_rows, c_over)):
        _check(f"{key} sum over rows {j}", o.index_select(lead, cols), r, True)


_ROW_KEYS = W.reference_row_key_cases()


@pytest.mark.parametrize("case", _ROW_KEYS, ids=[f"{c[1]}-{c[2]}x{c[3]}" for c in _ROW_KEYS])
def test_every_reference_row_key_at_its_size(case):
    """The softmax / layer norm problems of the reference's tuner caches (2 columns to 30528, 32 rows to 736392) on
    the row-wise kernels at their real size.  Rows do not interact in these anchors, so the oracle is evaluated
    on the first and last 64 rows and 1000 random ones."""
    key, anchor, rows, cols, mod, metas = case
    g = torch.Generator(device="cuda").manual_seed(rows % 9973 + cols)
    half = torch.float16

    def randn():
        t = torch.empty((rows, cols), dtype=half, device="cuda")
        flat, step = t.view(-1), 1 << 28
        for lo in range(0, flat.numel(), step):
            n = min(step, flat.numel() - lo)
            flat[lo:lo + n] = torch.randn(n, generator=g, device="cuda").to(half)
        return t
    x = randn()
    if anchor == "softmax":
        inputs = [x]
    elif anchor == "softmax_backward":
        inputs = [randn(), torch.softmax(x.float(), -1).to(half)]
    elif anchor == "layernorm":
        inputs = [x]
    else:
        var, mean = torch.var_mean(x.float(), -1, unbiased=False, keepdim=True)
        inputs = [randn(), x, mean, torch.rsqrt(var + 1e-5)]
    gm = W.fuse(mod, [t.to("meta") for t in inputs])
    (node,) = fused_nodes(gm)
    outs = gm(*inputs)
    outs = list(outs) if isinstance(outs, (tuple, list)) else [outs]
    torch.cuda.synchronize()
    pick = torch.Generator().manual_seed(cols)
    idx = torch.unique(torch.cat([torch.arange(0, min(64, rows)), torch.arange(max(rows - 64, 0), rows),
                                  torch.randint(0, rows, (1000,), generator=pick)])).cuda()
    refs = evt_oracle.eval_fp32(mod, [t.index_select(0, idx).cpu() for t in inputs])
    assert len(refs) == len(outs)
    for j, (o, r) in enumerate(zip(outs, refs)):
        got = o.index_select(0, idx).cpu()
        ok, err = evt_oracle.check(got, r, reduction=o.dtype == torch.float32)
        # the probabilities of a vocabulary-sized softmax lie below fp16's normal range (6.1e-5), where the output
        # format's spacing is 2^-24 whatever the value: there the bound is the relative one plus half that spacing
        denormal_ok = o.dtype == half and bool(((got.float() - r).abs() <= 2e-2 * r.abs() + 2.0 ** -25).all())
        assert ok or denormal_ok, (key, anchor, j, err)


@pytest.mark.parametrize("i", range(len(W.PADDED_GEMM_CASES)), ids=lambda i: "_".join(map(str, W.PADDED_GEMM_CASES[i][:5])))
def test_misaligned_extents_run_on_padded_operands(i, monkeypatch):
    """Odd M, N and K in every operand layout: the fused op copies its operands into zero-padded buffers and runs
    the transfer-path kernel (ViT's K = 588 patch embedding takes this route at its real size); outputs, sums over
    the rows and along the rows against the oracle -- the padding must not reach any of them."""
    from evt_ae_amd.evt_fuser import FusedGEMM
    monkeypatch.setattr(FusedGEMM, "pad_min_flops", 0.0)
    case = W.padded_gemm_case(i)
    inputs = _inputs(case, 40 + i)
    mod, gm, op = _fused(case, inputs)
    assert op.pad is not None and op.tile.dma and (op.kernel_k % 8 == 0 or not (op.a_kc or op.b_kc))
    outs = gm(*inputs)
    torch.cuda.synchronize()
    counts = case["counts"]
    got = _split_outputs(counts, outs)
    ref = _split_outputs(counts, evt_oracle.eval_fp32(mod, [t.cpu() for t in inputs]))
    for kind, gs, rs in zip(("store", "sum over rows", "sum along rows", "row store"), got, ref):
        for j, (o, r) in enumerate(zip(gs, rs)):
            assert tuple(o.shape) == tuple(r.shape)
            _check(f"{kind} {j}", o, r, kind.startswith("sum"))
    # the same product on the element-wise path gives the same values up to the order of the K sum
    monkeypatch.setattr(FusedGEMM, "pad_min_flops", float("inf"))
    _, gm2, op2 = _fused(case, inputs)
    assert op2.pad is None and not op2.tile.dma
    outs2 = gm2(*inputs)
    torch.cuda.synchronize()
    for o, o2 in zip(outs if isinstance(outs, (tuple, list)) else [outs], outs2 if isinstance(outs2, (tuple, list)) else [outs2]):
        assert evt_oracle.max_rel_err(o, o2.float().cpu()) <= 2e-2
