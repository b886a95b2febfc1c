"""Front-end passes and the AOT-autograd glue without a GPU.

The decompositions are pinned by value: the joint graph after frontend +
decomposition + CSE (no fusion, so it runs on the CPU) must give the loss and
the gradients PyTorch's own autograd gives for the same fp32 model.  The
reference exercises these passes only inside whole-model GPU tests
(unittest/fx_passes/xmlcnn.py:48-62, 82-89).
"""
import operator

import pytest
import torch
from torch.fx import symbolic_trace

from tests import patterns as W
from evt_ae_amd.aot_helper import aot_capture, joint_optimization
from evt_ae_amd.evt_fuser import legalize_graph, target_name
from evt_ae_amd.passes import (GTLFrontend, pass_clean_up, pass_cse, pass_decomposition, pass_loss_elimination)
from evt_ae_amd.workloads import fused_nodes

aten = torch.ops.aten


def names_of(gm):
    return [target_name(n.target) for n in gm.graph.nodes if n.op == "call_function"]


def without_fusion(joint_module):
    joint_module, _ = GTLFrontend()(joint_module)
    pass_decomposition(joint_module, joint_module.graph)
    pass_cse(joint_module, joint_module.graph)
    return joint_module


@pytest.mark.parametrize("reduction", ["sum", "mean"])
def test_decomposed_joint_graph_matches_autograd(reduction):
    class Net(W.MLPClassifier):
        def forward(self, x, y):
            z = self.l2(torch.nn.functional.gelu(self.l1(x), approximate="tanh"))
            return torch.nn.functional.cross_entropy(z, y, reduction=reduction)

    g = torch.Generator().manual_seed(3)
    model = Net(24, 40, 12)
    x, y = torch.randn(16, 24, generator=g), torch.randint(0, 12, (16,), generator=g)
    box = aot_capture(model, (x, y), joint_compiler=without_fusion)
    ops = set(names_of(box["joint"]))
    assert not ops & {"addmm", "t", "detach", "_log_softmax", "_log_softmax_backward_data", "nll_loss_backward"}
    assert {"mm", "permute", "_softmax", "log", "one_hot", "ne", "gelu_backward"} <= ops
    # run the split graphs by hand: forward returns (loss, *saved), backward takes (*saved, tangent)
    primals = [p.detach() for p in model.parameters()] + [x, y]
    fw_out = box["fw"](*primals)
    loss, saved = fw_out[0], fw_out[1:]
    grads = box["bw"](*saved, torch.ones_like(loss))
    ref_loss = model(x, y)
    ref_grads = torch.autograd.grad(ref_loss, list(model.parameters()))
    assert torch.allclose(loss, ref_loss, rtol=1e-5, atol=1e-6)
    got = [t for t in grads if t is not None]
    assert len(got) == len(ref_grads)
    for a, b in zip(got, ref_grads):
        assert a.shape == b.shape
        assert torch.allclose(a, b, rtol=1e-4, atol=1e-6), float((a - b).abs().max())


def test_joint_graph_is_fused_and_split():
    """Five GEMMs and a softmax in the training step of the classifier: in the
    forward graph bias + GELU with the pre-activation saved, bias + cast, and
    softmax + log (both results leave: one for the loss, one for backward);
    in the backward graph the data gradient with GELU' and the bias gradient
    in one launch and two weight gradients.  No kernel mixes forward and
    backward nodes."""
    model, inputs = W.mlp_classifier()
    box = aot_capture(model, inputs)
    assert len(fused_nodes(box["joint"])) == 6
    fw, bw = box["fw"], box["bw"]
    assert len(fused_nodes(fw)) == 3 and len(fused_nodes(bw)) == 3
    softmax = fused_nodes(fw)[2].target
    assert type(softmax).__name__ == "FusedSoftmax" and softmax.partition_names == ["_softmax", "log"]
    assert "mm" not in names_of(fw) + names_of(bw) and "addmm" not in names_of(fw)
    first = fused_nodes(fw)[0].target
    assert first.ir.epilogue_counts()[1] == 1                       # the bias, broadcast along rows
    assert len([s for s in first.ir.slots if s.role == "store"]) == 2   # GELU output and pre-activation
    dgrad = [n.target for n in fused_nodes(bw) if any(s.role == "store" and s.domain != "tile" for s in n.target.ir.slots)]
    assert len(dgrad) == 1                                           # GELU' and the hidden bias gradient in one launch
    # no backward node leaked into the forward graph: it only needs the primals
    assert [n.name for n in fw.graph.nodes if n.op == "placeholder"] == [f"primals_{i}" for i in range(1, 7)]


def test_frontend_normalises_targets_views_and_expands():
    class M(torch.nn.Module):
        def forward(self, a, b, v):
            x = torch.ops.aten.add.Tensor(a, b)
            d = torch.ops.aten.detach.default(x)
            e = torch.ops.aten.expand.default(v, [4, 6])
            y = torch.ops.aten.mul.Tensor(d, e)                      # broadcasts by itself: expand goes
            e2 = torch.ops.aten.expand.default(v, [4, 6])
            z = torch.ops.aten.mm.default(e2, torch.ops.aten.t.default(y))   # a GEMM operand keeps its expand
            return torch.ops.aten.view.default(z, [-1, 2])

    gm = W.trace_module(M(), [torch.empty(4, 6), torch.empty(4, 6), torch.empty(1, 6)])
    gm, modified = GTLFrontend()(gm)
    assert modified
    calls = [n for n in gm.graph.nodes if n.op == "call_function"]
    assert all(not hasattr(n.target, "overloadpacket") for n in calls)          # suffixes gone
    assert names_of(gm).count("expand") == 1 and "detach" not in names_of(gm)
    view = [n for n in calls if target_name(n.target) == "view"][0]
    assert list(view.args[1]) == [8, 2]
    a, b, v = torch.randn(4, 6), torch.randn(4, 6), torch.randn(1, 6)
    assert torch.equal(gm(a, b, v), M()(a, b, v))


def test_cse_merges_pure_nodes_only():
    class M(torch.nn.Module):
        def forward(self, a):
            p = aten.permute(a, [1, 0])
            q = aten.permute(a, [1, 0])
            r1 = torch.rand_like(a)
            r2 = torch.rand_like(a)
            return aten.add(p, q), r1, r2

    gm = W.trace_module(M(), [torch.empty(3, 5)])
    pass_cse(gm)
    assert names_of(gm).count("permute") == 1 and names_of(gm).count("rand_like") == 2
    a = torch.randn(3, 5)
    assert torch.equal(gm(a)[0], 2 * a.t())


def test_permute_pairs_fold():
    class M(torch.nn.Module):
        def forward(self, w, x):
            t1 = aten.t(w)
            t2 = aten.t(t1)
            p = aten.permute(aten.permute(x, [2, 0, 1]), [0, 2, 1])
            return aten.mm(t2, t1), p

    gm = W.trace_module(M(), [torch.empty(4, 4), torch.empty(2, 3, 5)])
    pass_decomposition(gm)
    perms = [n for n in gm.graph.nodes if n.op == "call_function" and target_name(n.target) == "permute"]
    assert sorted(list(n.args[1]) for n in perms) == [[1, 0], [2, 1, 0]]
    w, x = torch.randn(4, 4), torch.randn(2, 3, 5)
    out = gm(w, x)
    assert torch.equal(out[0], w @ w.t()) and torch.equal(out[1], x.permute(2, 0, 1).permute(0, 2, 1))


def test_pow_of_one_is_the_value_itself():
    """The backward of x ** 2 as autograd writes it holds pow(x, 1), which ATen runs as a copy of x: the
    decomposition pass takes it out, and only it."""
    class P(torch.nn.Module):
        def forward(self, x, g):
            return aten.mul(aten.mul(aten.pow(x, 1.0), 2.0), g), aten.pow(x, 2), aten.pow(x, 1.5), aten.pow(x, 1)

    gp = W.trace_module(P(), [torch.empty(3, 5), torch.empty(3, 5)])
    pass_decomposition(gp)
    assert names_of(gp).count("pow") == 2
    x, g = torch.randn(3, 5).abs(), torch.randn(3, 5)
    out = gp(x, g)
    assert torch.equal(out[0], x * 2.0 * g) and torch.equal(out[1], x ** 2) and torch.equal(out[2], x ** 1.5)
    assert torch.equal(out[3], x)


def test_clean_up_and_loss_elimination():
    class M(torch.nn.Module):
        def forward(self, x, y):
            p = aten.permute(x, [1, 0])
            v = aten.view(aten.clone(p, memory_format=torch.contiguous_format), [-1])
            return aten.sum(aten.mul(v, y)), v

    gm = W.trace_module(M(), [torch.empty(3, 5), torch.empty(15)])

    class N(torch.nn.Module):
        def forward(self, x):
            p = aten.permute(x, [1, 0])
            return aten.view(p, [15])

    gn = symbolic_trace(N())                               # ShapeProp would already trip over the view
    pass_clean_up(gn)
    assert names_of(gn) == ["permute", "clone", "view"]
    x = torch.randn(3, 5)
    assert torch.equal(gn(x), x.t().reshape(15))            # a view of a permuted tensor would raise

    pass_loss_elimination(gm)
    assert "sum" not in names_of(gm) and "mul" not in names_of(gm)
    loss, v = gm(torch.randn(3, 5), torch.randn(15))
    assert float(loss) == 1.0 and v.shape == (15,)


def test_stable_legalize_moves_only_what_it_must():
    class M(torch.nn.Module):
        def forward(self, a, b):
            f1 = aten.add(a, 1.0)
            f2 = aten.mul(f1, 2.0)
            g1 = aten.add(b, 1.0)
            g2 = aten.mul(g1, f2)
            return f2, g2

    gm = symbolic_trace(M())
    nodes = {n.name: n for n in gm.graph.nodes}
    # make f1 read a node that is defined after it
    with gm.graph.inserting_after(nodes["mul_1"]):
        late = gm.graph.call_function(aten.neg, (nodes["a"],))
    nodes["add"].args = (late, 1.0)
    with pytest.raises(RuntimeError):
        gm.graph.lint()
    legalize_graph(gm)
    gm.graph.lint()
    order = [n.name for n in gm.graph.nodes]
    # the dependants of `late` moved behind it, in their old order; b's chain stayed in front
    assert order == ["a", "b", "add_1", "neg", "add", "mul", "mul_1", "output"]
    gm.recompile()
    a, b = torch.randn(3), torch.randn(3)
    f2, g2 = gm(a, b)
    assert torch.equal(f2, (-a + 1) * 2) and torch.equal(g2, (b + 1) * f2)


def test_aot_optimize_compiles_here_and_refuses_to_run_without_a_gpu():
    """Forward and backward graphs go through AOT autograd's own checks (saved
    activations need fake values on the nodes the passes created); the first
    fused launch then fails loudly: there is no CPU path."""
    if torch.cuda.is_available():
        pytest.skip("covered by the GPU training-step test")
    from evt_ae_amd.aot_helper import aot_optimize
    model, (x, y) = W.mlp_classifier()
    with pytest.raises(RuntimeError, match="HIP device only"):
        aot_optimize(model)(x, y)


def test_torch_compile_backend_traces_here():
    if torch.cuda.is_available():
        pytest.skip("covered by the GPU training-step test")
    from evt_ae_amd.aot_helper import evt_backend
    model, (x, y) = W.mlp_classifier()
    with pytest.raises(RuntimeError, match="HIP device only"):
        torch.compile(model, backend=evt_backend)(x, y)


def test_layer_norm_weight_and_bias_are_split_off():
    class M(torch.nn.Module):
        def forward(self, x, w, b):
            ln = aten.native_layer_norm(x, [64], w, b, 1e-5)
            return operator.getitem(ln, 0), operator.getitem(ln, 1), operator.getitem(ln, 2)

    x, w, b = torch.randn(6, 5, 64), torch.randn(64), torch.randn(64)
    gm = W.trace_module(M(), [x, w, b])
    pass_decomposition(gm)
    ln = [n for n in gm.graph.nodes if n.op == "call_function" and target_name(n.target) == "native_layer_norm"]
    assert len(ln) == 1 and ln[0].args[2] is None and ln[0].args[3] is None
    for got, ref in zip(gm(x, w, b), M()(x, w, b)):
        assert torch.allclose(got, ref, rtol=1e-5, atol=1e-6)
    # after the split the normalisation is a row-wise anchor with weight and bias in its epilogue
    from evt_ae_amd.passes import pass_fusion
    pass_fusion(gm, gm.graph)
    (node,) = fused_nodes(gm)
    assert type(node.target).__name__ == "FusedLayerNorm" and {"mul", "add"} <= set(node.target.partition_names)


def test_encoder_layer_joint_graph():
    """Every GEMM, batched product, softmax and forward layer norm of an encoder
    layer's training step is fused; forward and backward graphs each hold their
    own kernels (no forward kernel reads a backward value)."""
    model, inputs = W.encoder_layer(device="meta")     # meta follows the GPU's dtype rules (fp32 layer norm statistics)
    box = aot_capture(model, inputs)
    fw = [type(n.target).__name__ for n in fused_nodes(box["fw"])]
    bw = [type(n.target).__name__ for n in fused_nodes(box["bw"])]
    assert fw.count("FusedGEMM") == 4 and fw.count("FusedBMM") == 2 and fw.count("FusedSoftmax") == 1
    assert fw.count("FusedLayerNorm") == 2
    assert bw.count("FusedGEMM") == 7 and bw.count("FusedBMM") == 4 and bw.count("FusedSoftmaxBackward") == 1
    assert bw.count("FusedLayerNormBackward") == 2        # input, weight and bias gradients in one pass each
    left = {target_name(n.target) for g in (box["fw"], box["bw"]) for n in g.graph.nodes if n.op == "call_function"}
    assert not left & {"mm", "bmm", "addmm", "_softmax", "_softmax_backward_data", "native_layer_norm",
                       "native_layer_norm_backward", "gelu", "gelu_backward"}
    assert [n.name for n in box["fw"].graph.nodes if n.op == "placeholder"][-1].startswith("primals_")


def test_head_split_and_merge_are_read_and_written_in_place():
    """Separate Q / K / V projections (the reference's BERT): the chains
    view -> permute -> expand -> clone -> view in front of the batched products,
    shared between the forward product and the backward ones, are given to each
    product privately and folded into its operand strides (batch index in two
    levels), and the merge behind the products into the stores: no clone is
    left in either graph and the products' arguments are the projections' own
    outputs."""
    from evt_ae_amd.evt_fuser import FusedBMM
    model, inputs = W.encoder_layer(device="meta", fused_qkv=False)
    box = aot_capture(model, inputs)
    for g in (box["fw"], box["bw"]):
        names = [target_name(n.target) for n in g.graph.nodes if n.op == "call_function"]
        assert "clone" not in names and "bmm" not in names, names
    ops = [n.target for g in (box["fw"], box["bw"]) for n in fused_nodes(g) if isinstance(n.target, FusedBMM)]
    assert len(ops) == 6
    B, S, H, dh = 8, 128, 4, 64
    two_level = 0
    for op in ops:
        for div, s1, s2 in ((op.bdiva, op.bsa, op.bs2a), (op.bdivb, op.bsb, op.bs2b)):
            if div > 1:
                two_level += 1
                assert (div, s1, s2) == (H, S * H * dh, dh)
    assert two_level >= 8          # q, k, v and their gradients' partners: operands read straight from [B, S, H * dh]
    # the merged result is stored straight into [B, S, H * dh]
    pv = next(op for op in ops if op.problem == (S, dh, S, B * H) and any(s.strides.stride_l2 for s in op.ir.slots))
    (st,) = [s.strides for s in pv.ir.slots if s.role == "store"]
    assert (st.l_div, st.stride_l, st.stride_l2, st.stride_m, st.stride_n) == (H, S * H * dh, dh, H * dh, 1)


def test_fused_qkv_forward_reads_its_heads_in_place():
    """One [d, 3d] projection: q, k and v are `select`s (or an `unbind`) of a
    permuted view of its output; each batched product reads its operand inside
    that output through a base offset and two-level batch strides, so the
    forward graph holds no select, expand or clone."""
    from evt_ae_amd.evt_fuser import FusedBMM
    for model, inputs in (W.encoder_layer(device="meta"), W.decoder_block(device="meta")):
        box = aot_capture(model, inputs)
        names = [target_name(n.target) for n in box["fw"].graph.nodes if n.op == "call_function"]
        assert not {"clone", "select", "unbind", "expand", "bmm"} & set(names), names
        ops = [n.target for n in fused_nodes(box["fw"]) if isinstance(n.target, FusedBMM)]
        assert len(ops) == 2
        d = 256
        assert sorted((ops[0].offa, ops[0].offb)) == [0, d] and ops[1].offb == 2 * d       # q, k ; v
        assert ops[0].bdiva == ops[0].bdivb == ops[1].bdivb == 4 and ops[0].lda == ops[0].ldb == 3 * d


def test_select_backward_sum_becomes_a_stack():
    """The gradient of q, k, v = qkv[0], qkv[1], qkv[2]: three zero-filled tensors
    with one slice set, added up.  pass_decomposition turns the sum into one
    stack (same values), and an incomplete or mixed sum is left alone."""
    import operator
    from evt_ae_amd.passes import pass_decomposition
    aten = torch.ops.aten

    class Full(torch.nn.Module):
        def forward(self, a, b, c):
            s = [3, 2, 4]
            return aten.add(aten.add(aten.select_backward(a, s, 0, 0), aten.select_backward(b, s, 0, 1)),
                            aten.select_backward(c, s, 0, 2))

    class Partial(torch.nn.Module):
        def forward(self, a, b, c):
            s = [3, 2, 4]
            return aten.add(aten.add(aten.select_backward(a, s, 0, 0), aten.select_backward(b, s, 0, 1)),
                            aten.select_backward(c, s, 0, 1))

    ins = [torch.randn(2, 4) for _ in range(3)]
    for mod, want_stack in ((Full(), True), (Partial(), False)):
        gm = W.trace_module(mod, ins)
        pass_decomposition(gm, gm.graph)
        names = [target_name(n.target) for n in gm.graph.nodes if n.op == "call_function"]
        assert ("stack" in names) == want_stack and ("select_backward" in names) != want_stack, names
        assert torch.equal(gm(*ins), mod(*ins))


def test_stack_merge_becomes_a_cat_of_merged_parts():
    """stack -> permute -> clone -> view that merges the stacked axis into the last
    one (the gradient of a fused [d, 3d] projection) is rewritten into a cat of
    the parts, each permuted and merged by itself: same values, no stack; other
    permutes of a stack are left alone."""
    from evt_ae_amd.passes import pass_decomposition
    aten = torch.ops.aten
    B, H, S, D = 2, 3, 5, 4

    class Merge(torch.nn.Module):
        def forward(self, a, b, c):
            st = aten.stack([a, b, c], 0)
            return aten.view(aten.clone(aten.permute(st, [1, 3, 0, 2, 4]), memory_format=torch.contiguous_format),
                             [B * S, 3 * H * D])

    class Other(torch.nn.Module):
        def forward(self, a, b, c):
            st = aten.stack([a, b, c], 0)
            return aten.view(aten.clone(aten.permute(st, [1, 0, 3, 2, 4]), memory_format=torch.contiguous_format),
                             [B * 3, S * H * D])

    class MergeAndBias(torch.nn.Module):       # the bias gradient: sum over every row, through a regrouping view
        def forward(self, a, b, c):
            st = aten.stack([a, b, c], 0)
            m = aten.view(aten.clone(aten.permute(st, [1, 3, 0, 2, 4]), memory_format=torch.contiguous_format),
                          [B, S, 3 * H * D])
            rows = aten.view(m, [B * S, 3 * H * D])
            return rows, aten.sum(rows, [0], True)

    ins = [torch.randn(B, H, S, D) for _ in range(3)]
    for mod, rewritten in ((Merge(), True), (Other(), False)):
        gm = W.trace_module(mod, ins)
        pass_decomposition(gm, gm.graph)
        names = [target_name(n.target) for n in gm.graph.nodes if n.op == "call_function"]
        assert ("cat" in names) == rewritten and ("stack" in names) != rewritten, names
        assert torch.equal(gm(*ins), mod(*ins))
    gm = W.trace_module(MergeAndBias(), ins)
    pass_decomposition(gm, gm.graph)
    sums = [n for n in gm.graph.nodes if n.op == "call_function" and target_name(n.target) == "sum"]
    assert len(sums) == 3 and all(tuple(n.meta["tensor_meta"].shape) == (1, 1, H * D) for n in sums)
    for got, want in zip(gm(*ins), MergeAndBias()(*ins)):
        assert got.shape == want.shape and torch.allclose(got, want, atol=1e-5)


def test_dropout_in_a_training_step_is_fused_and_leaves_nothing_behind():
    """native_dropout becomes rand_like / ge / mul inside the GEMM epilogues; the
    masks are kernel outputs saved for backward.  fx keeps random ops alive as
    impure, so the fuser removes a fused partition's nodes itself: no stray
    rand_like (and with it no second, unfused copy of the GEMM chain) may remain."""
    model, inputs = W.dropout_block(device="meta")
    box = aot_capture(model, inputs)
    fw, bw = box["fw"], box["bw"]
    for gm in (fw, bw):
        left = [str(n.target) for n in gm.graph.nodes if n.op == "call_function" and not n.meta.get("evt")]
        assert not [t for t in left if "rand" in t or "aten.mm" in t or "gelu" in t or "dropout" in t], left
    parts = [n.target.partition_names for n in fused_nodes(fw)]
    assert sum("rand_like" in " ".join(p) for p in parts) == 2
    saved_masks = [n for n in fw.graph.nodes if n.op == "output"][0].args[0]
    bools = [a for a in saved_masks if hasattr(a, "meta") and getattr(a.meta.get("tensor_meta"), "dtype", None) == torch.bool]
    assert len(bools) == 2
