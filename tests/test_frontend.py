"""Host logic without a GPU: EVTFuser.trace / pass_fusion lower the headline
subgraphs and the reference's fuser-test patterns (unittest/evt_fuser/mm.py,
bmm.py) to an IR whose CPU interpretation equals PyTorch's fp32 eager
evaluation of the original module."""
import operator

import pytest
import torch

from tests import patterns as W
from evt_ae_amd.evt_fuser import EVTFuser, FusedBMM, FusedGEMM, target_name
from oracle import evt_oracle
from tests.util import fused_nodes, rand_slot, run_emulated

aten = torch.ops.aten


def _check(module_cls, inputs, n_fused=1, tol=2e-5):
    gm = W.fuse(module_cls(), inputs)
    fused = fused_nodes(gm)
    assert len(fused) == n_fused
    for n in fused:
        assert n.meta.get("evt") is True
        assert n.target.__name__ in ("cutlass_gemm_with_visitor", "cutlass_bmm_with_visitor")
    got = run_emulated(gm, inputs)
    ref = evt_oracle.eval_fp32(module_cls(), inputs)
    assert len(got) == len(ref)
    for g, r in zip(got, ref):
        assert tuple(g.shape) == tuple(r.shape)
        if r.dtype == torch.bool:
            assert torch.equal(g.bool(), r)
            continue
        # the emulation rounds each store to the output dtype once
        err = evt_oracle.max_rel_err(g.float(), r)
        lim = 5e-3 if g.dtype in (torch.float16, torch.bfloat16) else tol
        assert err <= lim, err
    return gm


@pytest.mark.parametrize("cfg", [1, 2, 3, 4, 5])
@pytest.mark.parametrize("shapes", ["small", "ragged"])
def test_headline_configs_lower_correctly(cfg, shapes):
    sh = W.SMALL_SHAPES[cfg] if shapes == "small" else W.RAGGED_SHAPES[cfg]
    inputs = W.make_inputs(cfg, sh)
    _check(W.CONFIGS[cfg].module, inputs)


def test_config_classification():
    """Loads and stores are classified as the reference's pass manager names them
    (tuner_base.py:120-152): bias -> RowBroadcast, residual -> AuxLoad,
    labels -> ColumnBroadcast, dbias -> RowReduction ([N]), stats -> ColumnReduction ([M])."""
    kinds = {}
    for cfg in (1, 3, 4, 5):
        inputs = W.make_inputs(cfg, W.SMALL_SHAPES[cfg])
        gm = W.fuse(W.CONFIGS[cfg].module(), [t.to("meta") for t in inputs])
        (n,) = fused_nodes(gm)
        kinds[cfg] = {s.name: (s.role, s.kind, s.domain) for s in n.target.ir.slots}
        assert n.target.ir.epilogue_counts() == {
            1: (0, 1, 0, 1, 0, 0, 0), 3: (1, 1, 0, 1, 0, 2, 0), 4: (1, 0, 0, 1, 1, 0, 0), 5: (0, 0, 1, 0, 0, 1, 0)}[cfg]
    assert kinds[1]["b"] == ("load", "row", "tile")
    assert kinds[3]["r"] == ("load", "aux", "tile")
    assert kinds[5]["labels"] == ("load", "col", "tile")
    assert kinds[4]["sum_1"] == ("store", "row", "col")


def test_operand_layouts_follow_permutes():
    """permute [1, 0] in front of mm selects the column-major operand without a
    copy (evt_fuser.py:548-558); 3-D permutes give BMM strides (bmm.py:36-56)."""
    i4 = W.make_inputs(4, W.SMALL_SHAPES[4])
    (n4,) = fused_nodes(W.fuse(W.CONFIGS[4].module(), i4))
    assert isinstance(n4.target, FusedGEMM) and n4.target.rhs_layout == "ColumnMajor" and n4.target.b_kc
    i2 = W.make_inputs(2, W.SMALL_SHAPES[2])
    (n2,) = fused_nodes(W.fuse(W.CONFIGS[2].module(), i2))
    assert isinstance(n2.target, FusedBMM) and n2.target.b_kc and n2.target.a_kc
    i1 = W.pattern_inputs("bmm1")
    (b1,) = fused_nodes(W.fuse(W.BMMPartition1(), [t.to("meta") for t in i1]))
    assert (b1.target.b_kc, b1.target.ldb, b1.target.bsb) == (False, 2048, 64)


SMALL_PATTERNS = ["mm2", "mm3", "mm4", "mm5", "mm9", "bmm1", "bmm3"]   # (bmm2 has its own test below)


@pytest.mark.parametrize("name", SMALL_PATTERNS)
def test_reference_patterns_lower_correctly(name):
    cls, _ = W.REFERENCE_PATTERNS[name]
    inputs = W.pattern_inputs(name)
    _check(cls, inputs)


def test_batch_folded_row_reductions_lower_correctly():
    """bmm.py:48-67 (sum over the sequence axis and over the batches that agree
    modulo 16) and a sum over pairs of consecutive batches: one fused kernel
    each, the fold recorded in the IR and in the output tensor's batch term."""
    inputs = W.pattern_inputs("bmm2")
    gm = _check(W.BMMPartition2, inputs)
    (n,) = fused_nodes(gm)
    # the product is stored with the row index fastest, so the problem is computed transposed
    # (evt_fuser.py:573-596): the sum over the sequence axis is then one per column
    assert n.target.transposed
    (red,) = n.target.ir.reduces.values()
    assert (red.axis, red.fold, red.fold_step, red.fold_count) == ("col", "mod", 16, 2)
    (st,) = [s.strides for s in n.target.ir.slots if s.domain == "col"]
    assert (st.l_mod, st.l_div, st.stride_l, st.stride_m, st.stride_n) == (16, 1, 64, 0, 1)

    gm = _check(W.FoldConsecutiveBatches, W.fold_consecutive_inputs())
    (n,) = fused_nodes(gm)
    (red,) = n.target.ir.reduces.values()
    assert (red.fold, red.fold_count) == ("div", 2)

    # reductions with a two- and a three-word state fold batches as well: (max, sum-exp) and (count, mean, M2)
    # states of the batches that share a result are merged with their own combine operators
    gm = _check(W.FoldedLogSumExp, W.fold_consecutive_inputs())
    (n,) = fused_nodes(gm)
    assert sorted((r.kind, r.fold, r.fold_count) for r in n.target.ir.reduces.values()) == \
        [("maxsumexp", "div", 2), ("welford", "div", 2)]
    gm = _check(W.FoldedModuloVariance, W.fold_consecutive_inputs())
    (n,) = fused_nodes(gm)
    assert sorted((r.kind, r.fold, r.fold_step, r.fold_count) for r in n.target.ir.reduces.values()) == \
        [("maxsumexp", "mod", 3, 2), ("welford", "mod", 3, 2)]


def test_fit_strides_batch_terms():
    from evt_ae_amd.ir import Coord, accum_coord, fit_strides
    L, M, N = 12, 5, 7
    c = accum_coord(L, M, N, True)
    assert fit_strides(c, L, M, N).l_mod == 0
    per_head = c.reshape((3, 4, M, N)).reduce([0, 3], False)      # l = b*4 + h, reduced over b and n -> [h, m]
    st = fit_strides(per_head, L, M, N)
    assert (st.l_mod, st.l_div, st.stride_l, st.stride_m, st.stride_n) == (4, 1, M, 1, 0)
    per_group = c.reshape((3, 4, M, N)).reduce([1, 3], False)     # reduced over h and n -> [b, m]
    st = fit_strides(per_group, L, M, N)
    assert (st.l_mod, st.l_div, st.stride_l, st.stride_m, st.stride_n) == (0, 4, M, 1, 0)


def test_reference_patterns_shrunk():
    """mm1/mm6/mm7 at reduced sizes (same graphs; the view shapes are fixed by
    the reference so M = 1024 / 2048 stays, K is what the CPU pays for)."""
    g = torch.Generator().manual_seed(3)
    h = lambda *s: (torch.randn(*s, generator=g) * 0.5).half()   # noqa: E731
    _check(W.MMPartition1, [h(4096, 64), h(1024, 64), h(4096)])
    gm = _check(W.MMPartition6, [h(2048, 32), h(32, 1024), h(512, 4, 1024), h(512, 4, 1024)])
    (n,) = fused_nodes(gm)
    assert n.target.post_reshape_permute   # stored un-permuted, returned as a view
    gm = _check(W.MMPartition7, [h(2048, 32), h(32, 1024), h(512, 4, 1024), h(512, 4, 1024)])
    (n,) = fused_nodes(gm)
    # add_19 and its view share one store (the reference's output2store aliasing)
    assert len({v for v in n.target.output2store.values()}) == 3


def test_random_patterns_lower_correctly():
    """rand_like in the epilogue (unittest/evt_fuser/mm.py:216-236 at reduced K,
    dropout.py:33-46 decomposed): the IR draws from the element-indexed Philox
    stream; with that stream replayed in the eager module every output matches,
    masks bit for bit, and successive calls draw different numbers."""
    g = torch.Generator().manual_seed(5)
    h = lambda *s: (torch.randn(*s, generator=g) * 0.5).half()   # noqa: E731
    for cls, inputs in ((W.MMPartition12, [h(512, 64), h(1024, 64), h(512)]),
                        (W.Dropout1, [h(1024, 32), h(1024, 32), h(1024), h(512, 2, 1024)])):
        gm = W.fuse(cls(), inputs)
        (n,) = fused_nodes(gm)
        op = n.target
        op.rand_seed = 0x1234_5678_9ABC
        masks = []
        for call in range(2):
            got = run_emulated(gm, inputs)
            seed, offset = op.last_rand_state
            assert (seed, offset) == (0x1234_5678_9ABC, call)
            ref = evt_oracle.eval_fp32(cls(), inputs, rand=(seed, offset, rand_slot(op)))
            assert len(got) == len(ref)
            for o, r in zip(got, ref):
                assert tuple(o.shape) == tuple(r.shape)
                if r.dtype == torch.bool:
                    assert torch.equal(o.bool(), r)
                else:
                    assert evt_oracle.max_rel_err(o.float(), r) <= 5e-3
            masks.append([o for o in got if o.dtype == torch.bool][-1])
        if cls is W.Dropout1:     # (mm12 keeps with probability 1 - 1e-19: its mask is all ones)
            assert not torch.equal(masks[0], masks[1])
    keep = masks[0].float().mean().item()      # Dropout1: p = 0.7 dropped
    assert abs(keep - 0.3) < 5e-3


class TwoDropoutLayers(torch.nn.Module):
    """Two layers of the reference's dropout pattern (unittest/evt_fuser/dropout.py:33-46) in one graph: two
    fused partitions whose rand_like tensors have the same shape."""
    def forward(self, x, w1, b1, w2, b2):
        h = aten.add(aten.mm(x, aten.permute(w1, [1, 0])), b1)
        m1 = aten.ge(torch.rand_like(h), 0.7)
        h = aten.mul(aten.mul(h, m1), 1. / (1 - 0.7))
        y = aten.add(aten.mm(h, aten.permute(w2, [1, 0])), b2)
        m2 = aten.ge(torch.rand_like(y), 0.7)
        y = aten.mul(aten.mul(y, m2), 1. / (1 - 0.7))
        return y, m1, m2


def test_two_dropout_partitions_draw_unrelated_masks():
    """Two fused ops of one graph whose rand_like tensors have the same shape
    (the hidden dropouts of two layers) must not share a random stream: same
    seed, same offset, same slot index, yet different masks -- every op mixes a
    stream id of its own into the generator's counter.  The id comes from the
    anchor node's name, so tracing the same model again (in the same process,
    whatever was traced in between) gives the same (seed, offset, salt) and
    the same masks, as eager PyTorch does for a fixed seed.  And the seed is
    read when the op is called, so torch.manual_seed after tracing still takes
    effect."""
    g = torch.Generator().manual_seed(7)
    h = lambda *s: (torch.randn(*s, generator=g) * 0.5).half()   # noqa: E731
    inputs = [h(256, 128), h(128, 128), h(128), h(128, 128), h(128)]
    runs = []
    for trace in range(2):
        gm = W.fuse(TwoDropoutLayers(), inputs)
        ops = [n.target for n in fused_nodes(gm)]
        assert len(ops) == 2
        assert ops[0].rand_stream != ops[1].rand_stream
        torch.manual_seed(1234)
        got = run_emulated(gm, inputs)
        assert all(op.last_rand_state == (1234, 0) for op in ops)
        m1, m2 = [o for o in got if o.dtype == torch.bool]
        assert not torch.equal(m1, m2)
        agree = (m1 == m2).float().mean().item()      # independent masks with keep rate 0.3 agree on 58 %
        assert abs(agree - (0.3 * 0.3 + 0.7 * 0.7)) < 2e-2
        runs.append((gm, ops, [op.rand_salt(0) for op in ops], (m1, m2)))
        W.fuse(W.Dropout1(), W.pattern_inputs("dropout1"))     # an unrelated trace in between changes nothing
    assert runs[0][2] == runs[1][2]
    assert torch.equal(runs[0][3][0], runs[1][3][0]) and torch.equal(runs[0][3][1], runs[1][3][1])
    gm, ops = runs[0][0], runs[0][1]
    torch.manual_seed(99)                                      # after tracing: a new seed, new numbers
    again = [o for o in run_emulated(gm, inputs) if o.dtype == torch.bool]
    assert ops[0].last_rand_state == (99, 1)
    assert not torch.equal(again[0], runs[0][3][0])


def test_pass_decomposition_rewrites():
    """The reference's Decomposition replacements this path depends on
    (pass_decomposition.py:280-502): same values after the rewrite, the targeted
    ops gone, and the reference's dropout test graph (native_dropout,
    dropout.py:33-46) becomes one fused kernel that returns the mask."""
    from evt_ae_amd.passes import pass_decomposition, pass_fusion

    class Mixed(torch.nn.Module):
        def forward(self, b, x, w, g):
            y = torch.ops.aten.addmm(b, x, torch.ops.aten.t(w))
            y = torch.ops.aten._unsafe_view(y, [4, 8, 24])
            y = torch.ops.aten.transpose(y, 0, 1)
            r = torch.ops.aten.rsub(y, 1.0)
            tb = torch.ops.aten.threshold_backward(g, r, 0.5)
            return torch.ops.aten.native_dropout_backward(tb, tb > 0, 2.0)
    gen = torch.Generator().manual_seed(11)
    b, x, w = torch.randn(24, generator=gen), torch.randn(32, 16, generator=gen), torch.randn(24, 16, generator=gen)
    g = torch.randn(8, 4, 24, generator=gen)
    gm = W.trace_module(Mixed(), [b, x, w, g])
    want = Mixed()(b, x, w, g)
    pass_decomposition(gm, gm.graph)
    from evt_ae_amd.evt_fuser import target_name
    names = {target_name(n.target) for n in gm.graph.nodes if n.op == "call_function"}
    assert not names & {"addmm", "t", "transpose", "_unsafe_view", "rsub", "threshold_backward",
                        "native_dropout_backward"}
    assert {"mm", "permute", "view", "sub", "gt", "mul"} <= names
    assert torch.allclose(gm(b, x, w, g), want, atol=1e-5)
    assert all("tensor_meta" in n.meta for n in gm.graph.nodes if n.op == "call_function")

    inputs = W.pattern_inputs("dropout1")
    gm = W.fuse(W.Dropout1Undecomposed(), inputs, passes=[pass_decomposition, pass_fusion])
    (n,) = fused_nodes(gm)
    assert not any(target_name(x.target) == "native_dropout" for x in gm.graph.nodes if x.op == "call_function")
    assert any(s.kind == "rand" for s in n.target.ir.slots)
    assert [tuple(v[0]) for v in n.target.store_meta.values()] and len(n.target.outputs) == 2


def test_in_situ_checker():
    """FusedOpBase.reference_base (the reference's MODE=DEBUG self check,
    evt_fuser.py:98-172): the extracted epilogue module fed with the eager anchor
    agrees with the fused result, and a corrupted result is reported with its
    error figures."""
    for cls, inputs in ((W.CONFIGS[3].module, W.make_inputs(3, W.SMALL_SHAPES[3])),
                        (W.BMMPartition1, W.pattern_inputs("bmm1"))):
        gm = W.fuse(cls(), inputs)
        (n,) = fused_nodes(gm)
        op = n.target
        ph = [x for x in gm.graph.nodes if x.op == "placeholder"]
        args = [inputs[ph.index(a)].float() for a in n.args]      # fp32 on the CPU: eager half matmul is slow there
        from tests.util import emulate_fused
        results = [r.float() for r in emulate_fused(op, *[inputs[ph.index(a)] for a in n.args])]
        report = op.reference_base(args, results, verbose=False)
        assert [r["name"] for r in report] == [op.get_output_name(o) for o in op.outputs]
        assert all(r["match"] or r["rtol_pass_rate"] > 0.99 for r in report), report
        bad = [r.clone() for r in results]
        bad[0].view(-1)[::7] += 1.0
        report = op.reference_base(args, bad, verbose=False)
        assert not report[0]["match"] and report[0]["max_abs"] >= 0.9 and report[0]["rtol_pass_rate"] < 0.9


def test_unsupported_ops_raise():
    class Bad(torch.nn.Module):
        def forward(self, a, b):
            mm = torch.ops.aten.mm(a, b)
            return torch.ops.aten.erf(mm)
    a, b = torch.randn(64, 32).half(), torch.randn(32, 64).half()
    gm = W.trace_module(Bad(), [a, b])
    names = [n.name for n in gm.graph.nodes if n.op == "call_function"]
    assert EVTFuser.fusible(names, gm)
    with pytest.raises(NotImplementedError):
        EVTFuser().trace(gm, names)
    # pass_fusion falls back to fusing the anchor alone
    gm2 = W.fuse(Bad(), [a, b])
    assert len(fused_nodes(gm2)) == 1


def test_stubbed_anchors():
    from evt_ae_amd import evt_fuser
    for name in ("FusedConvFprop", "FusedConvDgrad", "FusedSpmm"):
        with pytest.raises(NotImplementedError):
            getattr(evt_fuser, name)(None, None)


# ---------------------------------------------------------------------------
# row-wise anchors (softmax / layer norm, forward and backward)
# ---------------------------------------------------------------------------

ROW_CLASSES = {"softmax": "FusedSoftmax", "softmax_backward": "FusedSoftmaxBackward",
               "layernorm": "FusedLayerNorm", "layernorm_backward": "FusedLayerNormBackward"}


@pytest.mark.parametrize("name", list(W.ROW_ANCHOR_PATTERNS))
def test_row_anchor_patterns_trace(name):
    """Every pattern of the reference's softmax / layer norm fuser tests becomes
    one fused node of the matching class whose module describes a row kernel
    (reference: FusedSoftmax ... FusedLayerNormBackward, evt_fuser.py:700-970)."""
    from evt_ae_amd.codegen import RowSpec
    cls, _ = W.ROW_ANCHOR_PATTERNS[name]
    inputs = W.pattern_inputs(name)
    gm = W.fuse(cls(), [t.to("meta") for t in inputs])
    (node,) = fused_nodes(gm)
    op = node.target
    kind = op.row_spec.op
    assert type(op).__name__ == ROW_CLASSES[kind] and isinstance(op.row_spec, RowSpec)
    M, N, K, L = op.problem
    assert K == 1 and N == inputs[0].shape[-1] and L * M * N == inputs[0].numel()
    assert op.row_spec.max_n >= N and op.row_spec.lpr in (8, 16, 32, 64) and 1 <= op.row_spec.ch <= 16
    spec = op.module.spec
    assert spec["abi"] == 5 and spec["anchor"] == kind and spec["row"]["max_n"] == op.row_spec.max_n
    assert op.num_anchor_inputs == {"softmax": 1, "softmax_backward": 2, "layernorm": 1, "layernorm_backward": 5}[kind]
    if kind == "layernorm":
        # eps travels as a scalar; mean and rstd are per-row stores
        assert op.ir.scalars[spec["anchor_scalars"]] == pytest.approx(1e-12)
        assert sum(1 for s in op.ir.slots if s.role == "store" and s.domain == "row") == 2
    if kind == "layernorm_backward":
        assert [op.ir.slots[k].name for k in spec["anchor_tensors"]] == ["mean", "invstd", "gamma"]
    if name == "layernorm_backward_full":
        assert L == 1 and spec["col_state"] == 2 and "Cfg = evt::RowCfg<3, 2, 64, 0, 2, 8, 1>" in op.module.source
    if "column" in name and "broadcast" not in name and "full" not in name:
        # a sum over every row: one batch of L * M rows, partials per workgroup in the workspace
        assert L == 1 and spec["col_state"] == 1 and "sum" in " ".join(op.partition_names)


def test_row_anchor_limits():
    from evt_ae_amd.codegen import RowSpec
    aten = torch.ops.aten

    class SoftmaxOverRows(torch.nn.Module):
        def forward(self, x):
            return aten._softmax(x, 0, False)

    class LayerNormWithWeight(torch.nn.Module):
        def forward(self, x, w, b):
            return operator.getitem(aten.native_layer_norm(x, [64], w, b, 1e-5), 0)

    class SoftmaxThenRowSum(torch.nn.Module):
        def forward(self, x):
            y = aten.mul(aten._softmax(x, -1, False), 2.)
            return y, aten.sum(y, [1], True)

    x = torch.empty(32, 64, dtype=torch.float16, device="meta")
    for mod, ins in ((SoftmaxOverRows(), [x]), (LayerNormWithWeight(), [x, x[0], x[0]])):
        gm = W.trace_module(mod, ins)
        names = [n.name for n in gm.graph.nodes if n.op == "call_function"]
        with pytest.raises(NotImplementedError):
            EVTFuser().trace(gm, names)
        assert not fused_nodes(W.fuse(mod, ins))                 # pass_fusion leaves such an anchor to eager
    # a second reduction along the row is not fused (the reference leaves it out too, softmax.py:113-123):
    # the partition is cut in front of it
    gm = W.fuse(SoftmaxThenRowSum(), [x])
    (node,) = fused_nodes(gm)
    assert node.target.partition_names == ["_softmax", "mul"]
    assert [target_name(n.target) for n in gm.graph.nodes if n.op == "call_function"].count("sum") == 1
    # row length -> lanes per row and chunks
    assert RowSpec.for_row_length("softmax", 64, "f16") == RowSpec("softmax", 1, 8, "f16")
    assert RowSpec.for_row_length("softmax", 512, "f16") == RowSpec("softmax", 4, 16, "f16")
    assert RowSpec.for_row_length("softmax_backward", 512, "f16") == RowSpec("softmax_backward", 2, 32, "f16")
    assert RowSpec.for_row_length("layernorm", 1024, "f16") == RowSpec("layernorm", 2, 64, "f16")
    assert RowSpec.for_row_length("layernorm", 8192, "bf16") == RowSpec("layernorm", 16, 64, "bf16")
    # longer rows go over several waves of a workgroup, as few as the registers allow
    assert RowSpec.for_row_length("softmax", 8200, "f16") == RowSpec("softmax", 9, 64, "f16", 2)
    assert RowSpec.for_row_length("softmax", 30522, "f16") == RowSpec("softmax", 8, 64, "f16", 8)
    assert RowSpec.for_row_length("softmax", 65536, "bf16") == RowSpec("softmax", 8, 64, "bf16", 16)
    assert RowSpec.for_row_length("softmax_backward", 30522, "f16") == RowSpec("softmax_backward", 4, 64, "f16", 16)
    for op, n, elt in (("softmax", 65537, "f16"), ("layernorm", 50000, "f32"), ("softmax_backward", 32776, "f16")):
        with pytest.raises(NotImplementedError):
            RowSpec.for_row_length(op, n, elt)


def test_rows_too_long_for_the_row_kernel_stay_eager():
    aten = torch.ops.aten

    class WideSoftmax(torch.nn.Module):
        def forward(self, x):
            return aten.mul(aten._softmax(x, -1, False), 2.)

    x = torch.empty(4, 65600, dtype=torch.float16, device="meta")
    gm = W.fuse(WideSoftmax(), [x])
    assert not fused_nodes(gm)
    assert [target_name(n.target) for n in gm.graph.nodes if n.op == "call_function"] == ["_softmax", "mul"]


@pytest.mark.parametrize("transposed, swap", [(False, True), (True, True), (True, False)])
def test_bias_gradient_behind_a_head_merge_lowers_correctly(transposed, swap, monkeypatch):
    """A batched product over B * H heads, merged into [B * S, H * D] by a permuted
    store, with the bias gradient (sum over every row) on top: per column and
    over the batches that agree modulo H.  The transposed product ([D, S] per
    head) is computed with its operands exchanged and is then the same problem;
    with the exchange switched off the same sum runs along the rows with the
    same fold.  One kernel, values from the IR interpreter."""
    monkeypatch.setattr(EVTFuser, "allow_transpose", swap)
    mod, inputs = W.head_merge_bias_grad(B=2, H=3, S=40, D=16, K=24, transposed=transposed)
    gm = W.fuse(mod, inputs)
    (n,) = fused_nodes(gm)
    assert not [x for x in gm.graph.nodes if x.op == "call_function" and target_name(x.target) in ("sum", "clone", "bmm")]
    assert n.target.transposed == (transposed and swap)
    assert n.target.problem == ((16, 40, 24, 6) if transposed and not swap else (40, 16, 24, 6))
    (red,) = n.target.ir.reduces.values()
    assert (red.axis, red.fold, red.fold_step, red.fold_count) == ("row" if transposed and not swap else "col", "mod", 3, 2)
    got = run_emulated(gm, inputs)
    ref = evt_oracle.eval_fp32(mod, inputs)
    for o, r in zip(got, ref):
        assert tuple(o.shape) == tuple(r.shape)
        assert evt_oracle.max_rel_err(o.float(), r) <= 5e-3


@pytest.mark.parametrize("batched", [False, True], ids=["mm", "bmm"])
def test_column_major_outputs_are_computed_transposed(batched, monkeypatch):
    """A result stored as [N, M] (permute + copy behind the epilogue) makes the
    fused op exchange its operands and compute C^T = B^T A^T, as the reference's
    `transposed` problems do (evt_fuser.py:573-596): the full-tensor load and
    store then run along the kernel's n, the row vector becomes a per-row value,
    the sum over all rows a sum along each row (the batched product's row maximum
    a per-column maximum).  With the exchange switched off the same graph lowers
    to strided accesses; both agree with eager fp32."""
    mod, inputs = W.column_major_store(batched)
    M, N, K = inputs[0].shape[-2], inputs[1].shape[-1], inputs[0].shape[-1]
    for swap in (True, False):
        monkeypatch.setattr(EVTFuser, "allow_transpose", swap)
        gm = W.fuse(mod, inputs)
        (n,) = fused_nodes(gm)
        op = n.target
        assert op.transposed == swap
        assert op.problem[:3] == ((N, M, K) if swap else (M, N, K))
        assert (op.a_kc, op.b_kc) == ((False, True) if swap else (True, False))    # the same memory, read the other way
        full = [s.strides for s in op.ir.slots if s.domain == "tile" and s.kind == "aux"]
        assert len(full) == 2 and all((st.stride_n == 1) == swap for st in full)
        (red,) = op.ir.reduces.values()
        assert red.axis == (("col" if batched else "row") if swap else ("row" if batched else "col"))
        got = run_emulated(gm, inputs)
        ref = evt_oracle.eval_fp32(mod, inputs)
        assert len(got) == len(ref) == 2
        for o, r in zip(got, ref):
            assert tuple(o.shape) == tuple(r.shape)
            assert evt_oracle.max_rel_err(o.float(), r) <= 5e-3


@pytest.mark.parametrize("anchor", ["mm", "bmm"])
def test_random_trees_with_column_major_tensors_lower_transposed(anchor):
    """Seeded random epilogue trees whose full-size tensors are all stored [N, M]:
    one fused kernel computing the transposed product, values from the IR
    interpreter against eager fp32."""
    for seed in W.RANDOM_EPILOGUE_SEEDS[:6]:
        mod, inputs = W.random_epilogue(seed, anchor, column_major=True)
        gm = W.fuse(mod, inputs)
        (n,) = fused_nodes(gm)
        assert n.target.transposed
        got = run_emulated(gm, inputs)
        ref = evt_oracle.eval_fp32(mod, inputs)
        assert len(got) == len(ref)
        for o, r in zip(got, ref):
            assert tuple(o.shape) == tuple(r.shape)
            assert evt_oracle.max_rel_err(o.float(), r) <= 5e-3, (anchor, seed)


def test_column_major_output_beside_a_column_index_stays_untransposed():
    """A column index in the epilogue (here a gather along the row) has no
    counterpart in the transposed problem, where columns are rows: the
    column-major store is then kept as a strided store, and the values still
    agree with eager fp32."""
    aten = torch.ops.aten

    class StoreAndGather(torch.nn.Module):
        def forward(self, a, b, labels):
            out = aten.mm(a, b)
            t = aten.clone(aten.permute(aten.mul(out, 0.5), [1, 0]), memory_format=torch.contiguous_format)
            return t, aten.gather(out, 1, aten.unsqueeze(labels, 1))

    g = torch.Generator().manual_seed(3)
    inputs = [(torch.randn(72, 40, generator=g) * 0.5).half(), (torch.randn(40, 56, generator=g) * 0.5).half(),
              torch.randint(0, 56, (72,), generator=g)]
    gm = W.fuse(StoreAndGather(), inputs)
    (n,) = fused_nodes(gm)
    assert not n.target.transposed and n.target.problem[:2] == (72, 56)
    (st,) = [s.strides for s in n.target.ir.slots if s.role == "store" and s.domain == "tile"]
    assert (st.stride_m, st.stride_n) == (1, 72)
    for o, r in zip(run_emulated(gm, inputs), evt_oracle.eval_fp32(StoreAndGather(), inputs)):
        assert tuple(o.shape) == tuple(r.shape)
        assert evt_oracle.max_rel_err(o.float(), r) <= 5e-3


def test_walk_tiles_are_offered_and_refused_where_they_should(monkeypatch):
    """Tiles whose workgroups walk over several tiles of a row block: offered by
    the tuner only where the tiles outnumber the CUs, K is a multiple of bk and
    no per-column reduction sits in the epilogue; refused by the code generator
    otherwise."""
    from evt_ae_amd.autotuner import tune_workloads
    from evt_ae_amd.autotuner.tuner_base import force_tile
    from evt_ae_amd.codegen import TileConfig
    monkeypatch.setenv("EVT_TUNER_CACHE", "/nonexistent/tuner_cache.db")
    walks = {cfg: [t for t in tuner.candidates() if t.walk > 1] for cfg, tuner in tune_workloads._tuners()}
    assert walks[5] and all(t.pipe >= 2 and t.stages <= 3 for t in walks[5])      # 2048 tiles of 256 x 256
    assert any(t.walk == 8 and (t.bm, t.bn) == (256, 256) for t in walks[5])
    assert not walks[2] and not walks[3] and not walks[4]                          # one round of tiles / column sums
    tile = TileConfig(256, 256, 64, 4, 2, 2, True, 4, 2, 4)
    from dataclasses import replace
    from evt_ae_amd import jit, prebuild
    (node4,) = W.fused_nodes(W.fuse(W.CONFIGS[4].module(), prebuild._shapes_of(4, None)))
    assert node4.target.ir.col_state > 0
    with pytest.raises(NotImplementedError):           # per-column reduction in the epilogue
        jit.LazyModule(node4.target.ir, replace(node4.target.spec, tile=tile, k_exact=True))
    with force_tile(tile):
        gm = W.fuse(W.CONFIGS[5].module(), W.make_inputs(5, W.SMALL_SHAPES[5]))
    (node,) = W.fused_nodes(gm)
    assert node.target.tile == tile and node.target.spec.k_exact
    assert "_n4_kx" in node.target.module.name
    with pytest.raises(NotImplementedError):           # a module that must also take a K with a partial k-tile
        jit.LazyModule(node.target.ir, replace(node.target.spec, k_exact=False))


def test_a_vector_of_the_epilogue_leaves_the_kernel_as_a_row_store():
    """(1 - mask) * -10000 feeds the scores and is an output of its own: the kernel computes it per column, adds
    it, and the tiles that hold row 0 write it (one store per batch row of the mask, l // H)."""
    inputs = W.MaskedScores.inputs()
    gm = _check(W.MaskedScores, inputs)
    (node,) = fused_nodes(gm)
    ir = node.target.ir
    assert ir.epilogue_counts() == (0, 1, 0, 1, 0, 0, 1)
    (vec,) = [sl for sl in ir.slots if sl.role == "store" and sl.domain == "nvec"]
    assert (vec.strides.stride_m, vec.strides.stride_n, vec.strides.l_div) == (0, 1, W.MaskedScores.DIMS[1])
    assert not any(n.op == "call_function" and n.target in (aten.mul, aten.rsub) for n in gm.graph.nodes)
    assert "t.row(0, 0) == 0" in node.target.module.source


def test_one_kernel_writes_a_shared_vector_and_the_next_reads_it():
    inputs = W.TwoMaskedLayers.inputs()
    gm = _check(W.TwoMaskedLayers, inputs, n_fused=2)
    first, second = fused_nodes(gm)
    assert first.target.ir.epilogue_counts()[6] == 1 and second.target.ir.epilogue_counts()[6] == 0
    # the second kernel's row vector is the first one's output
    src = [a for a in second.args if isinstance(a, torch.fx.Node) and a.op == "call_function"]
    assert any(first in (a, *a.all_input_nodes, *(i for b in a.all_input_nodes for i in b.all_input_nodes)) for a in src)
    assert not any(n.op == "call_function" and n.target in (aten.mul, aten.rsub) for n in gm.graph.nodes)


def test_a_vector_that_feeds_the_partition_through_its_other_users_stays_outside():
    """If another user of the side expression is an ancestor of the partition, writing it from the kernel would
    close a cycle: it stays an eager node."""
    class Loop(torch.nn.Module):
        def forward(self, x, w, mask):
            ext = aten.mul(aten.rsub(mask, 1.0), -100.0)
            x2 = aten.add(x, ext)                    # reads ext and feeds the product
            return aten.add(aten.mm(x2, w), ext)
    g = torch.Generator().manual_seed(3)
    inputs = [torch.randn(40, 32, generator=g).half(), (torch.randn(32, 32, generator=g) * 0.2).half(),
              (torch.rand(32, generator=g) > 0.5).half()]
    gm = W.fuse(Loop(), inputs)
    (node,) = fused_nodes(gm)
    assert node.target.ir.epilogue_counts()[6] == 0
    assert any(n.op == "call_function" and n.target is aten.mul for n in gm.graph.nodes)
    # the eager nodes in front of the product round to fp16, which the product amplifies: a loose bound
    (got,), (ref,) = run_emulated(gm, inputs), evt_oracle.eval_fp32(Loop(), inputs)
    assert evt_oracle.max_rel_err(got.float(), ref) <= 5e-2
