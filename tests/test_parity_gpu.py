"""Parity on the MI355X: the fused HIP kernels (called through the C ABI) against
the CPU oracle (PyTorch fp32 eager evaluation of the same fx subgraph).

Tolerances (the contract of the path): max relative error <= 2e-2 for fp16
outputs and <= 1e-3 for fp32 reduction outputs, measured as
max |out - ref| / max(|ref|, 1e-2 * rms(ref)).
"""
import ctypes

import numpy as np
import pytest
import torch

from tests import patterns as W
from evt_ae_amd.autotuner.tuner_base import force_tile
from evt_ae_amd.codegen import TileConfig
from evt_ae_amd.evt_fuser import EVTFuser
from oracle import evt_oracle
from evt_ae_amd.passes import target_name
from tests.util import fused_nodes, rand_slot

aten = torch.ops.aten

pytestmark = pytest.mark.gpu

FP16_TOL = 2e-2
REDUCTION_TOL = 1e-3


def _run(cfg, shapes, seed=None, tile=None):
    wl = W.CONFIGS[cfg]
    inputs = W.make_inputs(cfg, shapes, seed)
    if tile is None:
        gm = W.fuse(wl.module(), inputs)
    else:
        with force_tile(tile):
            gm = W.fuse(wl.module(), inputs)
        assert fused_nodes(gm)[0].target.tile == tile
    assert len(fused_nodes(gm)) == 1
    outs = gm(*[t.cuda() for t in inputs])
    outs = list(outs) if isinstance(outs, (tuple, list)) else [outs]
    torch.cuda.synchronize()
    return wl, inputs, gm, outs


def _compare(wl, outs, refs):
    assert len(outs) == len(refs)
    for i, (o, r) in enumerate(zip(outs, refs)):
        assert tuple(o.shape) == tuple(r.shape), (i, o.shape, r.shape)
        red = i in wl.reduction_outputs
        err = evt_oracle.max_rel_err(o, r)
        assert err <= (REDUCTION_TOL if red else FP16_TOL), f"{wl.name} output {i}: max rel err {err:.3e}"


@pytest.mark.parametrize("cfg", [1, 2, 3, 4, 5])
@pytest.mark.parametrize("shapes", ["small", "ragged", "unaligned"])
def test_configs_against_oracle(cfg, shapes):
    sh = {"small": W.SMALL_SHAPES, "ragged": W.RAGGED_SHAPES, "unaligned": W.UNALIGNED_SHAPES}[shapes][cfg]
    wl, inputs, gm, outs = _run(cfg, sh)
    _compare(wl, outs, evt_oracle.eval_fp32(wl.module(), inputs))


@pytest.mark.parametrize("cfg", [1, 2, 3, 4, 5])
@pytest.mark.parametrize("tile", W.pipeline_tiles(), ids=lambda t: t.tag())
def test_pipeline_variants_against_oracle(cfg, tile):
    """Every ping-pong main-loop variant and the one-wave-per-SIMD loop on shapes
    with several tiles in M, N and K, partial edge tiles and a K tail (one k-tile
    only for the batched config)."""
    wl, inputs, gm, outs = _run(cfg, W.PIPELINE_SHAPES[cfg], tile=tile)
    _compare(wl, outs, evt_oracle.eval_fp32(wl.module(), inputs))


@pytest.mark.parametrize("two_kernel", [False, True], ids=["in_kernel", "finalize_kernel"])
@pytest.mark.parametrize("case", W.walk_cases(), ids=lambda c: f"cfg{c[0]}_{c[2].tag()}_K{c[1].get('K', c[1].get('D'))}")
def test_walking_workgroups_against_oracle(case, two_kernel, monkeypatch):
    """Workgroups that compute several tiles of a row block in a row: the operand
    ring carried from tile to tile, the epilogue in the one free stage, per-row
    reductions folded over the walk into one partial per workgroup.  Runs of
    unequal length, partial edge tiles, and phase 2 in either place."""
    cfg, shapes, tile = case
    if two_kernel:
        if not W.CONFIGS[cfg].reduction_outputs:
            pytest.skip("no reduction in this epilogue")
        monkeypatch.setenv("EVT_TWO_KERNEL_REDUCE", "1")
    wl, inputs, gm, outs = _run(cfg, shapes, tile=tile)
    _compare(wl, outs, evt_oracle.eval_fp32(wl.module(), inputs))
    again = gm(*[t.cuda() for t in inputs])
    again = list(again) if isinstance(again, (tuple, list)) else [again]
    torch.cuda.synchronize()
    for a, b in zip(outs, again):
        assert torch.equal(a, b), "two launches of the same problem differ"


@pytest.mark.parametrize("cfg", [1, 2, 3, 4, 5])
def test_configs_full_size(cfg):
    """Headline sizes: against the oracle (its fp32 CPU evaluation finishes in
    seconds) and through size-independent properties of each subgraph."""
    wl, inputs, gm, outs = _run(cfg, None)
    refs = evt_oracle.eval_fp32(wl.module(), inputs)
    _compare(wl, outs, refs)
    if cfg == 2:
        s, m, l = outs
        sf = s.float()
        assert torch.all(l >= 1.0 - 1e-5)                       # the max term contributes exp(0) = 1
        assert torch.all(m + 1e-2 >= sf.amax(-1, keepdim=True))  # max of the unrounded >= rounded max - ulp
        lse = torch.logsumexp(sf, -1, keepdim=True)
        assert evt_oracle.max_rel_err(m + torch.log(l), lse) <= 2e-3
    if cfg == 3:
        o, mean, var = outs
        assert torch.all(var >= 0)
        v2, m2 = torch.var_mean(o.float(), dim=1, correction=0)  # recomputed from the stored fp16 tensor
        scale = o.float().pow(2).mean().sqrt()                   # fp16 rounding of o perturbs the mean by << scale
        assert torch.all((mean - m2).abs() <= 1e-3 * scale) and evt_oracle.max_rel_err(var, v2) <= 2e-3
    if cfg == 4:
        dp, db = outs
        chk = dp.double().sum(0).float()                        # checksum of the stored (fp16-rounded) tensor
        assert (db - chk).abs().max() <= 2e-3 * chk.abs().max()
    if cfg == 5:
        (loss,) = outs
        assert torch.all(loss > 0)


def test_reductions_are_deterministic_and_workspace_reusable():
    """The two-phase combine sums partials in tile order: repeated launches on
    the same workspace are bit-identical (the reference's atomics are not)."""
    for cfg in (3, 4, 5, 2):
        wl = W.CONFIGS[cfg]
        inputs = [t.cuda() for t in W.make_inputs(cfg, None if cfg != 5 else dict(M=256, N=8192, K=256))]
        gm = W.fuse(wl.module(), inputs)
        first = [o.clone() for o in gm(*inputs)] if cfg != 5 else [gm(*inputs).clone()]
        for _ in range(3):
            again = gm(*inputs)
            again = list(again) if isinstance(again, (tuple, list)) else [again]
            for a, b in zip(first, again):
                assert torch.equal(a, b)


@pytest.mark.parametrize("cfg,shapes", [(3, None), (4, None), (3, W.SPLIT_K_SHAPES[3])],
                         ids=["row_finalize", "column_finalize", "split_k"])
def test_exchange_between_workgroups_holds_over_many_launches(cfg, shapes):
    """Regression guard for the exchange of partial results between workgroups
    inside one kernel (device-scope stores, the wait for their acknowledgement,
    a relaxed arrival ticket, device-scope loads by the last arriver): 2000
    back-to-back launches on one shared workspace -- config 3 at full size (the
    last workgroup of a row block finishes the row statistics), config 4 at full
    size (per-column sums) and a split-K shape (accumulator tiles exchanged) --
    each compared bit for bit with the first launch; stops at the first mismatch."""
    wl = W.CONFIGS[cfg]
    inputs = W.make_inputs(cfg, shapes)
    gm = W.fuse(wl.module(), [t.to("meta") for t in inputs])
    (node,) = fused_nodes(gm)
    op = node.target
    placeholders = [n for n in gm.graph.nodes if n.op == "placeholder"]
    args = [inputs[placeholders.index(a)].cuda() for a in node.args]
    stream = torch.cuda.current_stream()
    module = op.module.ensure()
    batch, launches = 20, 2000
    sets = []
    for _ in range(batch + 1):
        stores = op.allocate_outputs("cuda")
        a, keep = op.build_arguments(stores, *args, block=op.new_argument_block())
        sets.append((stores, a, keep))
    ws_ptr, ws_bytes = op.workspace_for(sets[0][1], stream, "cuda")
    assert ws_bytes > 0
    module.launch(sets[batch][1], ws_ptr, ws_bytes, stream.cuda_stream)       # the reference launch
    torch.cuda.synchronize()
    first = sets[batch][0]
    done = 1
    while done < launches:
        for stores, a, _ in sets[:batch]:
            module.launch(a, ws_ptr, ws_bytes, stream.cuda_stream)
        torch.cuda.synchronize()
        for i, (stores, _, _) in enumerate(sets[:batch]):
            for name, t in stores.items():
                assert torch.equal(t.view(torch.uint8), first[name].view(torch.uint8)), \
                    f"config {cfg}: launch {done + i} differs from the first in '{name}'"
        done += batch


PATTERN_ATOL = 2e-1   # the reference's own criterion (unittest/evt_fuser/mm.py:28, bmm.py:27)


@pytest.mark.parametrize("name", ["mm1", "mm2", "mm3", "mm4", "mm5", "mm6", "mm7", "mm9", "mm10", "mm11", "bmm1", "bmm2", "bmm3"])
def test_reference_fuser_patterns(name):
    """The graph patterns of the reference's fuser tests, through pass_fusion,
    checked as the reference does (fused vs the same module run eagerly in
    fp16, atol 2e-1) and against the fp32 oracle."""
    cls, _ = W.REFERENCE_PATTERNS[name]
    inputs = W.pattern_inputs(name)
    dev = [t.cuda() for t in inputs]
    gm = W.fuse(cls(), inputs)
    assert len(fused_nodes(gm)) == 1
    outs = gm(*dev)
    outs = list(outs) if isinstance(outs, (tuple, list)) else [outs]
    eager = cls()(*dev)
    eager = list(eager) if isinstance(eager, (tuple, list)) else [eager]
    torch.cuda.synchronize()
    refs = evt_oracle.eval_fp32(cls(), inputs)
    for o, e, r in zip(outs, eager, refs):
        assert tuple(o.shape) == tuple(e.shape)
        assert torch.allclose(o.float(), e.float(), atol=PATTERN_ATOL, rtol=1e-2)
        err = evt_oracle.max_rel_err(o, r)
        assert err <= FP16_TOL, f"{name}: max rel err {err:.3e}"


def test_reference_dropout_test_verbatim():
    """unittest/evt_fuser/dropout.py:33-75 as written there: native_dropout in the
    module, pass_decomposition + pass_fusion, reference recomputed from the
    returned mask, the reference's tolerances and keep-rate window."""
    from evt_ae_amd.passes import pass_decomposition, pass_fusion
    inputs = [t.cuda() for t in W.pattern_inputs("dropout1")]
    view_9, primals_16, primals_17, permute_104 = inputs
    gm = W.fuse(W.Dropout1Undecomposed(), inputs, passes=[pass_decomposition, pass_fusion])
    (node,) = fused_nodes(gm)
    # fixed stream: the reference's +-1e-3 keep-rate window is 2.2 sigma wide for 2^20 elements
    node.target.rand_seed = 0xC0FFEE_0000_0001
    out, mask = gm(*inputs)
    mm_36 = torch.mm(view_9, primals_16.permute(1, 0))
    view_10 = (mm_36 + primals_17).view(512, 2, 1024)
    ref = view_10 * mask / 0.3 + permute_104
    assert torch.allclose(out, ref, atol=5e-1)        # the reference's check, against fp16 eager
    ref32 = ((view_9.float() @ primals_16.float().t() + primals_17.float()).view(512, 2, 1024)
             * mask / (1 - 0.7) + permute_104.float())
    assert evt_oracle.max_rel_err(out, ref32) <= FP16_TOL
    keep = torch.mean(mask.to(torch.float32)).item()
    assert 0.3 - 1e-3 < keep < 0.3 + 1e-3


@pytest.mark.parametrize("name", ["mm12", "dropout1", "softmax_dropout"])
def test_random_fuser_patterns(name):
    """rand_like fused into the epilogue (unittest/evt_fuser/mm.py:216-236,
    dropout.py:33-75; softmax_dropout: the same decomposed dropout behind a
    softmax anchor, 4-D probabilities, rows of 136).  The reference can only check the keep rate; here the
    generator's stream is replayed on the CPU (oracle/philox.py), so the masks
    must match bit for bit and the values to the fp16 tolerance, and two
    launches must draw different numbers."""
    cls, _ = W.RANDOM_PATTERNS[name]
    inputs = W.pattern_inputs(name)
    dev = [t.cuda() for t in inputs]
    gm = W.fuse(cls(), inputs)
    (node,) = fused_nodes(gm)
    op = node.target
    op.rand_seed = 0xC0FFEE_0000_0001
    masks = []
    for call in range(2):
        outs = list(gm(*dev))
        torch.cuda.synchronize()
        seed, offset = op.last_rand_state
        assert offset == call
        refs = evt_oracle.eval_fp32(cls(), inputs, rand=(seed, offset, rand_slot(op)))
        assert len(outs) == len(refs)
        for o, r in zip(outs, refs):
            assert tuple(o.shape) == tuple(r.shape)
            if r.dtype == torch.bool:
                assert o.dtype == torch.bool and torch.equal(o.cpu(), r)
            else:
                assert evt_oracle.max_rel_err(o, r) <= FP16_TOL
        masks.append(outs[1].cpu())
    if name != "mm12":
        assert not torch.equal(masks[0], masks[1])
    if name == "dropout1":
        keep = masks[0].float().mean().item()          # the reference's criterion (dropout.py:73-75)
        assert 0.3 - 1e-3 < keep < 0.3 + 1e-3


@pytest.mark.parametrize("two_kernel", [False, True])
def test_batch_folded_row_reductions(two_kernel, monkeypatch):
    """Per-row reductions that also fold batches: modulo (bmm.py partition 2 at a
    reduced size) and consecutive groups, with phase 2 inside the kernel and in
    the finalize kernel."""
    if two_kernel:
        monkeypatch.setenv("EVT_TWO_KERNEL_REDUCE", "1")
    cases = [(W.FoldConsecutiveBatches, W.fold_consecutive_inputs()), (W.BMMPartition2, W.pattern_inputs("bmm2")),
             # (max, sum-exp) and (count, mean, M2) states folding consecutive batches / batches modulo 3
             (W.FoldedLogSumExp, W.fold_consecutive_inputs()), (W.FoldedModuloVariance, W.fold_consecutive_inputs())]
    for cls, inputs in cases:
        gm = W.fuse(cls(), inputs)
        (node,) = fused_nodes(gm)
        assert any(r.fold for r in node.target.ir.reduces.values())
        outs = list(gm(*[t.cuda() for t in inputs]))
        again = list(gm(*[t.cuda() for t in inputs]))
        refs = evt_oracle.eval_fp32(cls(), inputs)
        for i, (o, o2, r) in enumerate(zip(outs, again, refs)):
            assert torch.equal(o, o2)
            assert evt_oracle.max_rel_err(o, r) <= (FP16_TOL if o.dtype != torch.float32 else evt_oracle.REDUCTION_TOL), (cls.__name__, i)


def test_launch_is_graph_capturable():
    """evt_launch allocates nothing and never synchronises, so a fused call with a
    cross-workgroup reduction can be captured in a HIP graph (the reference runs
    whole models from CUDA graphs, bert_modeling.py:170-182).  Every replay,
    with eager work and synchronisations in between, must reproduce the eager
    launch bit for bit (the workspace counters return to zero by themselves)."""
    wl = W.CONFIGS[3]
    inputs = [t.cuda() for t in W.make_inputs(3, W.SMALL_SHAPES[3])]
    gm = W.fuse(wl.module(), inputs)
    (node,) = fused_nodes(gm)
    op = node.target
    ph = [n for n in gm.graph.nodes if n.op == "placeholder"]
    args = [inputs[ph.index(a)] for a in node.args]
    eager = [o.clone() for o in op(*args)]
    torch.cuda.synchronize()
    outs = op.allocate_outputs("cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        a, keep = op.build_arguments(outs, *args)
        ws_ptr, ws_bytes = op.workspace_for(a, side, "cuda")     # allocated and initialised before capture
        for _ in range(2):
            op.module.launch(a, ws_ptr, ws_bytes, side.cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        op.module.launch(a, ws_ptr, ws_bytes, torch.cuda.current_stream().cuda_stream)
    for rep in range(4):
        for t in outs.values():
            t.zero_()
        _ = (inputs[0].float() @ inputs[1].float()).sum().item()   # unrelated eager work + a sync between replays
        graph.replay()
        torch.cuda.synchronize()
        for name, e in zip((op.output2store[op.get_output_name(o)] for o in op.outputs), eager):
            assert torch.equal(outs[name].view(-1), e.contiguous().view(-1)), (rep, name)


def test_graph_capture_of_a_fused_call_records_no_workspace_fill():
    """A fused call made through the op itself under torch.cuda.graph, on the capture's own stream, which the op
    has never seen: it takes the workspace that the first eager call cleared as a spare, so the graph holds the
    kernel alone (a recorded fill would run at every replay).  Every replay equals the eager call bit for bit; a
    second capture finds no spare and records the fill, with the same results."""
    wl = W.CONFIGS[3]
    inputs = [t.cuda() for t in W.make_inputs(3, W.SMALL_SHAPES[3])]
    gm = W.fuse(wl.module(), inputs)
    (node,) = fused_nodes(gm)
    op = node.target
    ph = [n for n in gm.graph.nodes if n.op == "placeholder"]
    args = [inputs[ph.index(a)] for a in node.args]
    assert op._spare_workspace is None
    eager = [o.clone() for o in op(*args)]
    torch.cuda.synchronize()
    assert op._spare_workspace is not None and len(op._workspace) == 1
    spare_ptr = op._spare_workspace.data_ptr()
    for capture in range(2):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=torch.cuda.Stream()):       # a stream of its own for each capture
            captured = op(*args)
        assert op._spare_workspace is None and len(op._workspace) == 2 + capture
        if capture == 0:
            assert spare_ptr in {w.data_ptr() for w in op._workspace.values()}
        for rep in range(3):
            for t in captured:
                t.zero_()
            _ = (inputs[0].float() @ inputs[1].float()).sum().item()   # unrelated eager work + a sync between replays
            graph.replay()
            torch.cuda.synchronize()
            for o, e in zip(captured, eager):
                assert torch.equal(o, e), (capture, rep)


def test_debug_mode_self_check():
    """MODE=DEBUG (evt_fuser.py:98-172): the first call compares the kernel with
    the eager anchor + extracted epilogue module and records the verdict."""
    for cfg in (1, 4):
        wl = W.CONFIGS[cfg]
        inputs = [t.cuda() for t in W.make_inputs(cfg, W.SMALL_SHAPES[cfg])]
        gm = W.fuse(wl.module(), inputs)
        (node,) = fused_nodes(gm)
        op = node.target
        op.mode = "DEBUG"
        gm(*inputs)
        assert op.launched
        report = op.last_reference_report
        assert len(report) == len(op.outputs)
        # eager runs in fp16 (two extra roundings), so elements near zero may miss the pure rtol 1e-2 test;
        # the report's pass rates are what a developer reads then
        assert all(r["match"] or r["atol_pass_rate"] > 0.999 or r["rtol_pass_rate"] > 0.98 for r in report), report


def test_golden_fixtures():
    """Committed input/output vectors (tests/golden): inputs are regenerated from
    the recorded seed, the kernels must reproduce the recorded outputs."""
    from pathlib import Path
    gold = np.load(Path(__file__).parent / "golden" / "configs_small.npz")
    for cfg in (1, 2, 3, 4, 5):
        wl, inputs, gm, outs = _run(cfg, W.GOLDEN_SHAPES[cfg])
        for i, t in enumerate(inputs):
            assert np.array_equal(gold[f"c{cfg}_in{i}"], t.numpy()), "input generator drifted from the fixture"
        refs = [torch.from_numpy(gold[f"c{cfg}_out{i}"]) for i in range(len(outs))]
        _compare(wl, outs, refs)


def test_bf16_operands():
    wl = W.CONFIGS[1]
    inputs = [t.bfloat16() for t in W.make_inputs(1, W.SMALL_SHAPES[1])]
    gm = W.fuse(wl.module(), inputs)
    out = gm(*[t.cuda() for t in inputs])
    ref = evt_oracle.eval_fp32(wl.module(), inputs)[0]
    assert evt_oracle.max_rel_err(out, ref) <= 4e-2   # bf16 store: 8 mantissa bits


@pytest.mark.parametrize("name", list(W.MULTI_ANCHOR_PATTERNS))
def test_multi_anchor_graphs(name):
    """Several GEMMs in one graph: the partitioner decides which epilogue takes
    the nodes they share (reference: pass_fusion.py:216-983), every GEMM becomes
    one fused launch, and the graph's results match the fp32 oracle.  Tensors
    that pass from one kernel to the next go through HBM in fp16."""
    cls, _ = W.MULTI_ANCHOR_PATTERNS[name]
    inputs = W.pattern_inputs(name)
    dev = [t.cuda() for t in inputs]
    gm = W.fuse(cls(), inputs)
    n_gemms = sum(1 for t in inputs if t.dim() == 2) // 2
    assert len(fused_nodes(gm)) == n_gemms
    outs = list(gm(*dev))
    torch.cuda.synchronize()
    refs = evt_oracle.eval_fp32(cls(), inputs)
    assert len(outs) == len(refs)
    for k, (o, r) in enumerate(zip(outs, refs)):
        assert tuple(o.shape) == tuple(r.shape)
        red = o.dim() == 1
        err = evt_oracle.max_rel_err(o, r)
        assert err <= (REDUCTION_TOL if red else FP16_TOL), f"{name} output {k}: max rel err {err:.3e}"


@pytest.mark.parametrize("dims", W.MaskedScores.GPU_DIMS, ids=lambda d: "x".join(map(str, d)))
def test_row_store_of_a_shared_mask(dims):
    """BERT's transformed attention mask, (1 - mask[B, 1, 1, S]) * -10000, is computed in the epilogue of the
    scores' product, added there, and written by the tiles that hold row 0 (the reference's row store,
    visitor_store.hpp:46-145): both outputs against the oracle, the stored vector exactly (one fp16 rounding of
    an exact value), and nothing but the fused kernel left in the graph."""
    inputs = W.MaskedScores.inputs(seed=5, dims=dims)
    mod = W.MaskedScores(dims)
    gm = W.fuse(mod, inputs)
    (node,) = fused_nodes(gm)
    assert node.target.ir.epilogue_counts() == (0, 1, 0, 1, 0, 0, 1)
    scores, ext = gm(*[t.cuda() for t in inputs])
    torch.cuda.synchronize()
    ref_scores, ref_ext = evt_oracle.eval_fp32(mod, inputs)
    assert tuple(ext.shape) == tuple(ref_ext.shape) and ext.dtype == torch.float16
    assert torch.equal(ext.cpu().float(), ref_ext.float())
    err = evt_oracle.max_rel_err(scores, ref_scores)
    assert err <= FP16_TOL, err
    again_scores, again_ext = gm(*[t.cuda() for t in inputs])
    torch.cuda.synchronize()
    assert torch.equal(again_scores, scores) and torch.equal(again_ext, ext)


@pytest.mark.parametrize("m,n", [(72, 48), (1000, 520)])
def test_one_kernel_writes_a_vector_the_next_one_reads(m, n):
    inputs = W.TwoMaskedLayers.inputs(seed=2, m=m, n=n)
    gm = W.fuse(W.TwoMaskedLayers(), inputs)
    first, second = fused_nodes(gm)
    assert first.target.ir.epilogue_counts()[6] == 1 and second.target.ir.epilogue_counts()[6] == 0
    out = gm(*[t.cuda() for t in inputs])
    out = out[0] if isinstance(out, (tuple, list)) else out
    torch.cuda.synchronize()
    (ref,) = evt_oracle.eval_fp32(W.TwoMaskedLayers(), inputs)
    err = evt_oracle.max_rel_err(out, ref)
    assert err <= FP16_TOL, err


@pytest.mark.parametrize("entry", ["aot_module", "torch.compile"])
def test_aot_training_step(entry):
    """A whole training step through AOT autograd, as the reference's model tests
    run it (unittest/fx_passes/xmlcnn.py:48-62, 82-89: frontend, decomposition,
    CSE and fusion on the joint graph, default_partition, fp16 parameters).
    Loss and gradients are checked against the same model in fp32, and with the
    reference's own criterion (more than 90 % of a gradient's elements within
    rtol 1e-1 of the eager fp16 run, xmlcnn.py:114-116)."""
    import copy
    from evt_ae_amd.aot_helper import aot_optimize, evt_backend
    model, (x, y) = W.mlp_classifier(device="cuda")
    master = copy.deepcopy(model).float()
    ref_loss = master(x.float(), y)
    ref_grads = torch.autograd.grad(ref_loss, list(master.parameters()))
    eager = copy.deepcopy(model)
    eager(x, y).backward()
    compiled = aot_optimize(model) if entry == "aot_module" else torch.compile(model, backend=evt_backend)
    for step in range(2):                       # the second call reuses the compiled graphs
        for p in model.parameters():
            p.grad = None
        loss = compiled(x, y)
        loss.backward()
        torch.cuda.synchronize()
        assert abs(float(loss) - float(ref_loss)) <= 2e-3 * abs(float(ref_loss)), (float(loss), float(ref_loss))
        for (name, p), g32, pe in zip(model.named_parameters(), ref_grads, eager.parameters()):
            assert p.grad is not None and p.grad.dtype == torch.float16 and p.grad.shape == g32.shape
            err = float((p.grad.float() - g32).norm() / g32.norm())
            assert err <= 1e-2, f"step {step} {name}: norm-wise error {err:.3e}"
            close = torch.isclose(p.grad, pe.grad, rtol=1e-1).float().mean().item()
            assert close > 0.9, f"step {step} {name}: {close:.3f} of the elements agree with eager fp16"


ROW_ATOL = {"softmax": 3e-3, "layernorm": 3e-2}   # the reference's criteria (softmax.py:28, layernorm.py:29)


@pytest.mark.parametrize("name", list(W.ROW_ANCHOR_PATTERNS))
def test_row_anchor_patterns(name):
    """Softmax / layer norm (forward and backward) as anchors with an epilogue
    behind them: the patterns of the reference's fuser tests
    (unittest/evt_fuser/softmax.py, softmax_backward.py, layernorm.py,
    layernorm_backward.py), one launch each, checked with the reference's
    absolute tolerance against the module run eagerly and with the parity
    contract's relative tolerance against the fp32 oracle."""
    cls, _ = W.ROW_ANCHOR_PATTERNS[name]
    inputs = W.pattern_inputs(name)
    dev = [t.cuda() for t in inputs]
    gm = W.fuse(cls(), inputs)
    assert len(fused_nodes(gm)) == 1
    assert not [n for n in gm.graph.nodes if n.op == "call_function"
                and n.target in (aten._softmax, aten._softmax_backward_data, aten.native_layer_norm,
                                 aten.native_layer_norm_backward)]
    outs = gm(*dev)
    outs = list(outs) if isinstance(outs, (tuple, list)) else [outs]
    eager = cls()(*dev)
    eager = list(eager) if isinstance(eager, (tuple, list)) else [eager]
    torch.cuda.synchronize()
    refs = evt_oracle.eval_fp32(cls(), inputs)
    atol = ROW_ATOL["softmax" if name.startswith("softmax") else "layernorm"]
    for k, (o, e, r) in enumerate(zip(outs, eager, refs)):
        assert tuple(o.shape) == tuple(e.shape) and o.dtype == e.dtype, f"{name} output {k}"
        assert torch.allclose(o.float(), e.float(), atol=atol, rtol=1e-2), f"{name} output {k} vs eager"
        stat = o.dtype == torch.float32 and o.numel() * 8 <= inputs[0].numel()      # per-row mean / rstd
        err = evt_oracle.max_rel_err(o, r)
        # the probabilities of a vocabulary-sized softmax lie below fp16's normal range (6.1e-5), where the output
        # format's spacing is 2^-24 whatever the value: there the bound is the relative one plus half that spacing
        d, rr = (o.float().cpu() - r).abs(), r.abs()
        denormal_ok = o.dtype == torch.float16 and bool((d <= FP16_TOL * rr + 2.0 ** -25).all())
        assert err <= (REDUCTION_TOL if stat else FP16_TOL) or denormal_ok, f"{name} output {k}: max rel err {err:.3e}"


@pytest.mark.parametrize("dtype", W.ROW_EDGE_DTYPES, ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("n", W.ROW_EDGE_LENGTHS)
@pytest.mark.parametrize("anchor", ["softmax", "softmax_backward", "layernorm", "layernorm_backward"])
def test_row_anchor_lengths_and_dtypes(anchor, n, dtype):
    """Bare row-wise anchors at the shortest (8) and longest (8192) supported row,
    at lengths that are no multiple of 8 or of the 16-byte access (24, 1000: the
    generic path), in fp16, bf16 and fp32, against the fp32 oracle."""
    mod, inputs = W.row_edge_case(anchor, n, dtype)
    gm = W.fuse(mod, inputs)
    (node,) = fused_nodes(gm)
    assert node.target.row_spec.max_n >= n
    outs = gm(*[t.cuda() for t in inputs])
    outs = list(outs) if isinstance(outs, (tuple, list)) else [outs]
    torch.cuda.synchronize()
    refs = evt_oracle.eval_fp32(mod, inputs)
    tol = {torch.float16: FP16_TOL, torch.bfloat16: FP16_TOL, torch.float32: REDUCTION_TOL}[dtype]
    for k, (o, r) in enumerate(zip(outs, refs)):
        assert tuple(o.shape) == tuple(r.shape)
        stat = k > 0                                  # layer norm's mean and rstd (fp32)
        err = evt_oracle.max_rel_err(o, r)
        assert err <= (REDUCTION_TOL if stat else tol), f"{anchor} n={n} {dtype} output {k}: max rel err {err:.3e}"


@pytest.mark.parametrize("anchor,n,dtype", W.ROW_LONG_CASES,
                         ids=[f"{a}-{n}-{str(d).split('.')[-1]}" for a, n, d in W.ROW_LONG_CASES])
def test_row_anchor_long_rows(anchor, n, dtype):
    """Rows longer than one wave can cache (8192): the row is spread over the
    2 .. 16 waves of a workgroup and each row reduction ends with an exchange
    through LDS.  Vocabulary-sized rows (30522, 50257), the longest rows each
    anchor takes, odd lengths, three element types, against the fp32 oracle."""
    mod, inputs = W.row_edge_case(anchor, n, dtype)
    gm = W.fuse(mod, inputs)
    (node,) = fused_nodes(gm)
    spec = node.target.row_spec
    assert spec.wpr > 1 and spec.max_n >= n
    outs = gm(*[t.cuda() for t in inputs])
    outs = list(outs) if isinstance(outs, (tuple, list)) else [outs]
    torch.cuda.synchronize()
    refs = evt_oracle.eval_fp32(mod, inputs)
    tol = {torch.float16: FP16_TOL, torch.bfloat16: FP16_TOL, torch.float32: REDUCTION_TOL}[dtype]
    for k, (o, r) in enumerate(zip(outs, refs)):
        assert tuple(o.shape) == tuple(r.shape)
        err = evt_oracle.max_rel_err(o, r)
        # probabilities of a 65536-wide softmax lie below fp16's normal range (6.1e-5), where the output format's
        # spacing is 2^-24 whatever the value: there the bound is the relative one plus half that spacing
        d, rr = (o.float().cpu() - r).abs(), r.abs()
        denormal_ok = dtype == torch.float16 and k == 0 and bool((d <= tol * rr + 2.0 ** -25).all())
        assert err <= (REDUCTION_TOL if k > 0 else tol) or denormal_ok, \
            f"{anchor} n={n} {dtype} output {k}: max rel err {err:.3e}"


_RANDOM_TREES = [(a, s) for a in W.RANDOM_EPILOGUE_ANCHORS for s in W.RANDOM_EPILOGUE_SEEDS[:12 if a == "mm" else 6]]


@pytest.mark.parametrize("anchor,seed", _RANDOM_TREES, ids=[f"{a}-{s}" for a, s in _RANDOM_TREES])
def test_random_epilogue_trees(anchor, seed):
    """Seeded random epilogue trees behind a 320 x 192 x 96 GEMM, a batch of three
    such products, a softmax and a layer norm over 320 x 192 (no multiples of the
    large tiles or of a lane group): 5 .. 9 element-wise steps from the fuser's
    vocabulary over the anchor's result, a same-shape tensor, a row vector, a
    column vector and immediates, one or two stored results, sometimes a sum over
    the rows or along them.  The whole tree must end up in one fused kernel and
    every output must match the fp32 oracle."""
    mod, inputs = W.random_epilogue(seed, anchor)
    gm = W.fuse(mod, inputs)
    (node,) = fused_nodes(gm)
    assert type(node.target).__name__ == {"mm": "FusedGEMM", "bmm": "FusedBMM", "softmax": "FusedSoftmax",
                                           "layernorm": "FusedLayerNorm"}[anchor]
    left = [n for n in gm.graph.nodes if n.op == "call_function" and target_name(n.target) not in ("getitem", "view")
            and n is not node]
    assert not left, left
    outs = gm(*[t.cuda() for t in inputs])
    outs = list(outs) if isinstance(outs, (tuple, list)) else [outs]
    torch.cuda.synchronize()
    refs = evt_oracle.eval_fp32(mod, inputs)
    assert len(outs) == len(refs)
    for k, (o, r) in enumerate(zip(outs, refs)):
        assert tuple(o.shape) == tuple(r.shape)
        reduced = r.numel() < inputs[2].numel()
        err = evt_oracle.max_rel_err(o, r)
        assert err <= (REDUCTION_TOL if reduced and o.dtype == torch.float32 else FP16_TOL), \
            f"{anchor} seed {seed} output {k}: max rel err {err:.3e}"


@pytest.mark.parametrize("seed", W.RANDOM_EPILOGUE_SEEDS[:6])
@pytest.mark.parametrize("anchor", ["mm", "bmm"])
def test_random_epilogue_trees_with_column_major_tensors(anchor, seed):
    """The same random trees with every full-size tensor of the epilogue stored
    [N, M]: the same-shape operand read through a permute, the results leaving
    through permute + copy.  The fused op computes the transposed product (row
    vector and column vector change roles, a sum along the rows becomes one over
    them); one kernel, every output against the fp32 oracle."""
    mod, inputs = W.random_epilogue(seed, anchor, column_major=True)
    gm = W.fuse(mod, inputs)
    (node,) = fused_nodes(gm)
    assert node.target.transposed
    left = [n for n in gm.graph.nodes if n.op == "call_function" and target_name(n.target) not in ("getitem", "view")
            and n is not node]
    assert not left, left
    outs = gm(*[t.cuda() for t in inputs])
    outs = list(outs) if isinstance(outs, (tuple, list)) else [outs]
    torch.cuda.synchronize()
    refs = evt_oracle.eval_fp32(mod, inputs)
    assert len(outs) == len(refs)
    for k, (o, r) in enumerate(zip(outs, refs)):
        assert tuple(o.shape) == tuple(r.shape)
        reduced = r.numel() < inputs[2].numel()
        err = evt_oracle.max_rel_err(o, r)
        assert err <= (REDUCTION_TOL if reduced and o.dtype == torch.float32 else FP16_TOL), \
            f"{anchor} seed {seed} output {k}: max rel err {err:.3e}"


@pytest.mark.parametrize("n", W.AFFINE_LN_LENGTHS)
def test_layer_norm_with_weight_and_bias_on_long_rows(n):
    """native_layer_norm with weight and bias (moved into the epilogue by
    pass_decomposition) on rows of 8192 (16 chunks in one wave), 12288 and 20480
    elements (rows over several waves; the [N] vectors are then read per row
    instead of being kept in registers)."""
    from evt_ae_amd.passes import pass_decomposition, pass_fusion
    mod, inputs = W.affine_layer_norm(n)
    gm = W.fuse(mod, inputs, passes=[pass_decomposition, pass_fusion])
    (node,) = fused_nodes(gm)
    assert type(node.target).__name__ == "FusedLayerNorm" and node.target.row_spec.max_n >= n
    outs = list(gm(*[t.cuda() for t in inputs]))
    torch.cuda.synchronize()
    refs = evt_oracle.eval_fp32(mod, inputs)
    for k, (o, r) in enumerate(zip(outs, refs)):
        assert tuple(o.shape) == tuple(r.shape)
        err = evt_oracle.max_rel_err(o, r)
        assert err <= (REDUCTION_TOL if k > 0 else FP16_TOL), f"n={n} output {k}: max rel err {err:.3e}"


@pytest.mark.parametrize("fused_qkv", [True, False], ids=["fused_qkv", "separate_qkv"])
def test_aot_encoder_layer_training_step(fused_qkv):
    """A transformer encoder layer, forward and backward, through AOT autograd
    with the joint pipeline (the reference's BERT flow, unittest/fx_passes/bert.py:
    frontend, decomposition, CSE, fusion, default_partition): projections with
    bias / residual / GELU epilogues, batched QK^T and PV products with their
    permutes and the 1/sqrt(d) scale, softmax and softmax backward, both layer
    norms with weight and bias, all as fused launches.  With separate Q / K / V
    projections (the reference's BERT) the head split and merge
    (view -> permute -> clone -> view around the batched products, forward and
    backward) are read and written in place through two-level batch strides: no
    copy kernel is left.  Loss and gradients against the same model in fp32."""
    import copy
    from evt_ae_amd.aot_helper import aot_capture, aot_optimize
    model, (x, target) = W.encoder_layer(device="cuda", fused_qkv=fused_qkv)
    box = aot_capture(copy.deepcopy(model), (x, target))
    kinds = [type(n.target).__name__ for n in fused_nodes(box["fw"])] + [type(n.target).__name__ for n in fused_nodes(box["bw"])]
    assert kinds.count("FusedGEMM") == (11 if fused_qkv else 15) and kinds.count("FusedBMM") == 6
    if not fused_qkv:
        left = [target_name(n.target) for g in (box["fw"], box["bw"]) for n in g.graph.nodes if n.op == "call_function"]
        assert "clone" not in left and "bmm" not in left, left
    assert kinds.count("FusedSoftmax") == 1 and kinds.count("FusedSoftmaxBackward") == 1
    assert kinds.count("FusedLayerNorm") == 2 and kinds.count("FusedLayerNormBackward") == 2
    master = copy.deepcopy(model).float()
    ref_loss = master(x.float(), target)
    ref_grads = torch.autograd.grad(ref_loss, list(master.parameters()))
    eager = copy.deepcopy(model)
    eager(x, target).backward()
    compiled = aot_optimize(model)
    loss = compiled(x, target)
    loss.backward()
    torch.cuda.synchronize()
    assert abs(float(loss) - float(ref_loss)) <= 5e-3 * abs(float(ref_loss)), (float(loss), float(ref_loss))
    for (name, p), g32, pe in zip(model.named_parameters(), ref_grads, eager.parameters()):
        assert p.grad is not None and p.grad.shape == g32.shape
        err = float((p.grad.float() - g32).norm() / g32.norm())
        err_eager = float((pe.grad.float() - g32).norm() / g32.norm())
        # no worse than the fp16 eager run of the same model (whose own rounding sets the scale), within 2e-2
        assert err <= max(2e-2, 2.0 * err_eager), f"{name}: norm-wise error {err:.3e} (eager fp16: {err_eager:.3e})"


@pytest.mark.parametrize("tile", [None, *W.SPLIT_K_TILES], ids=lambda t: "tuner" if t is None else TileConfig(*t).tag())
@pytest.mark.parametrize("cfg", list(W.SPLIT_K_SHAPES))
def test_split_k(cfg, tile, monkeypatch):
    """Few output tiles and a long K: several workgroups share a tile, leave their
    accumulators in the workspace and the last to arrive adds them in split order
    and runs the epilogue (with its own per-row / per-column reductions).  Checked
    against the oracle with the automatic split, with a forced odd split, with as
    many splits as there are k-tiles (which meet in two levels) and with splitting off; repeated launches are bit-identical (the order of the sum is
    fixed), and the automatic choice really splits.  With the tuner's tile, a
    ping-pong tile and a one-wave-per-SIMD tile."""
    shapes = W.SPLIT_K_SHAPES[cfg]
    wl = W.CONFIGS[cfg]
    inputs = W.make_inputs(cfg, shapes)
    refs = evt_oracle.eval_fp32(wl.module(), inputs)
    dev = [t.cuda() for t in inputs]
    if tile is None:
        gm = W.fuse(wl.module(), inputs)
    else:
        with force_tile(TileConfig(*tile)):
            gm = W.fuse(wl.module(), inputs)
        assert fused_nodes(gm)[0].target.tile == TileConfig(*tile)
    (node,) = fused_nodes(gm)
    op = node.target
    results = {}
    for mode in ("auto", "3", "40", "1"):     # "40": more than 16 splits meet in groups first (two levels)
        if mode == "auto":
            monkeypatch.delenv("EVT_SPLIT_K", raising=False)
        else:
            monkeypatch.setenv("EVT_SPLIT_K", mode)
        op._workspace.clear()                       # sized for the split in force
        outs = gm(*dev)
        outs = list(outs) if isinstance(outs, (tuple, list)) else [outs]
        torch.cuda.synchronize()
        _compare(wl, outs, refs)
        again = gm(*dev)
        again = list(again) if isinstance(again, (tuple, list)) else [again]
        torch.cuda.synchronize()
        for a, b in zip(outs, again):
            assert torch.equal(a, b), f"config {cfg} split {mode}: launches differ"
        results[mode] = [o.clone() for o in outs]
        if cfg == 1:        # no reduction in this epilogue: a workspace exists exactly when K is split
            assert bool(op._workspace) == (mode != "1"), mode
    monkeypatch.delenv("EVT_SPLIT_K", raising=False)
    tile = op.tile
    tiles = -(-op.problem[0] // tile.bm) * -(-op.problem[1] // tile.bn)
    assert tiles * 2 <= 256 and op.problem[2] >= 8 * tile.bk
    for o_auto, o_off in zip(results["auto"], results["1"]):
        assert evt_oracle.max_rel_err(o_auto, o_off.float()) <= 1e-2


@pytest.mark.parametrize("name", ["softmax_aux_load", "layernorm1", "layernorm_backward_full"])
def test_debug_mode_self_check_row_anchors(name):
    """MODE=DEBUG on the row-wise anchors: the first call runs the anchor eagerly
    (aten._softmax / native_layer_norm / native_layer_norm_backward), feeds its
    result to the extracted epilogue module and compares with the kernel
    (reference: FusedSoftmax.reference ... FusedLayerNormBackward.reference,
    evt_fuser.py:748-753, 884-890, 952-958)."""
    cls, _ = W.ROW_ANCHOR_PATTERNS[name]
    inputs = [t.cuda() for t in W.pattern_inputs(name)]
    gm = W.fuse(cls(), inputs)
    (node,) = fused_nodes(gm)
    op = node.target
    op.mode = "DEBUG"
    gm(*inputs)
    assert op.launched
    report = op.last_reference_report
    assert len(report) == len(op.outputs)
    assert all(r["match"] or r["atol_pass_rate"] > 0.999 or r["rtol_pass_rate"] > 0.98 for r in report), report


def test_aot_training_step_with_dropout():
    """Dropout in training mode through the joint pipeline: the masks are drawn in
    the GEMM epilogues (Philox, element-indexed) and saved for backward.  The
    split forward / backward graphs are run by hand so the masks can be read
    back; loss and gradients must equal the same block evaluated in fp32 with
    those masks, and the keep rate must be 1 - p."""
    import copy
    from evt_ae_amd.aot_helper import aot_capture
    model, (x, target) = W.dropout_block(device="cuda")
    box = aot_capture(copy.deepcopy(model), (x, target))
    fw, bw = box["fw"], box["bw"]
    primals = [p.detach() for p in model.parameters()] + [x, target]
    out = fw(*primals)
    loss, saved = out[0], list(out[1:])
    masks = [t for t in saved if t.dtype == torch.bool]
    assert [tuple(m.shape) for m in masks] == [(512, 512), (512, 256)]
    for m in masks:
        assert abs(m.float().mean().item() - (1 - W.DropoutBlock.P)) < 5e-3
    assert not torch.equal(masks[0][:, :256], masks[1])
    grads = [g for g in bw(*saved, torch.ones_like(loss)) if g is not None]
    torch.cuda.synchronize()
    master = copy.deepcopy(model).float()
    ref_loss = master.forward_with_masks(x.float(), target, masks[0].float(), masks[1].float())
    ref_grads = torch.autograd.grad(ref_loss, list(master.parameters()))
    assert abs(float(loss) - float(ref_loss)) <= 5e-3 * abs(float(ref_loss))
    assert len(grads) == len(ref_grads)
    for (name, _), g, r in zip(model.named_parameters(), grads, ref_grads):
        err = float((g.float() - r).norm() / r.norm())
        assert err <= 2e-2, f"{name}: norm-wise error {err:.3e}"


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_aot_decoder_block_with_attention_dropout(dtype):
    """A pre-layer-norm decoder block in training mode: the causal masked_fill
    runs as a `where` behind the Q K^T BMM, the attention-probability dropout is
    drawn behind the softmax anchor in the row kernel (same element-indexed
    Philox stream as the GEMM epilogues), and both layer norm backward ops are
    fused, the first layer's without an input gradient (x needs none).  Loss and gradients must equal the block evaluated in fp32 with the
    saved mask."""
    import copy
    from evt_ae_amd.aot_helper import aot_capture
    model, (x, target) = W.decoder_block(device="cuda", dtype=dtype)
    box = aot_capture(copy.deepcopy(model), (x, target))
    fw, bw = box["fw"], box["bw"]
    kinds = [type(n.target).__name__ for g in (fw, bw) for n in fused_nodes(g)]
    assert kinds.count("FusedSoftmax") == 1 and kinds.count("FusedSoftmaxBackward") == 1
    assert kinds.count("FusedLayerNorm") == 2 and kinds.count("FusedLayerNormBackward") == 2
    left = {str(n.target) for g in (fw, bw) for n in g.graph.nodes if n.op == "call_function"}
    assert not [t for t in left if "rand" in t or "masked_fill" in t or "dropout" in t or "aten.bmm" in t], left
    primals = [p.detach() for p in model.parameters()] + [x, target]
    out = fw(*primals)
    loss, saved = out[0], list(out[1:])
    (mask,) = [t for t in saved if t.dtype == torch.bool and t.dim() == 4]
    assert tuple(mask.shape) == (4, 4, 128, 128)
    assert abs(mask.float().mean().item() - (1 - W.DecoderBlock.P)) < 5e-3
    grads = [g for g in bw(*saved, torch.ones_like(loss)) if g is not None]
    torch.cuda.synchronize()
    master = copy.deepcopy(model).float()
    ref_loss = master.forward_with_masks(x.float(), target, mask.float())
    ref_grads = torch.autograd.grad(ref_loss, list(master.parameters()))
    tol = 2e-2 if dtype == torch.float16 else 6e-2      # bf16 carries 8 mantissa bits through every saved activation
    assert abs(float(loss) - float(ref_loss)) <= (5e-3 if dtype == torch.float16 else 2e-2) * abs(float(ref_loss))
    assert len(grads) == len(ref_grads)
    for (name, _), g, r in zip(model.named_parameters(), grads, ref_grads):
        err = float((g.float() - r).norm() / r.norm())
        assert err <= tol, f"{name}: norm-wise error {err:.3e}"


def test_bench_argument_sets_are_independent():
    """bench.py keeps several argument blocks per config side by side (rotating
    buffer sets): each must point at its own buffers, although an op called the
    ordinary way reuses one block."""
    import bench
    case = bench.Case(2, torch, W, fused_nodes)
    assert case.nsets >= 4
    blocks = [s[0] for s in case.sets]
    assert len({ctypes.addressof(b) for b in blocks}) == len(blocks)
    assert len({b.tensors[k].ptr for b in blocks for k in range(b.num_tensors)}) == len(blocks) * blocks[0].num_tensors
    for i in range(case.nsets):
        case.launch(i)
    torch.cuda.synchronize()
    first = case.outputs(0)
    assert all(float(o.float().abs().sum()) > 0 for o in first)
    for i in range(1, case.nsets):
        for a, b in zip(first, case.outputs(i)):
            assert torch.equal(a, b)


def test_tuning_at_trace_time(tmp_path, monkeypatch):
    """EVT_AUTOTUNE=1 with an empty cache: tracing times the candidate tiles on
    the device (here two of them, both built ahead of time), stores the faster
    with its time under the problem's key, and the next trace reads that row;
    the tuned op still agrees with the oracle."""
    import sqlite3
    from evt_ae_amd.autotuner.gemm_tuner import MMTuner
    cache = tmp_path / "tuner_cache.db"
    monkeypatch.setenv("EVT_TUNER_CACHE", str(cache))
    monkeypatch.setenv("EVT_AUTOTUNE", "1")
    tiles = [t for t in W.pipeline_tiles() if (t.bm, t.bn, t.stages, t.pipe) in ((256, 256, 2, 2), (128, 128, 3, 12))]
    assert len(tiles) == 2
    monkeypatch.setattr(MMTuner, "candidates", lambda self: list(tiles))
    monkeypatch.setattr(MMTuner, "warmup_iterations", 3)
    monkeypatch.setattr(MMTuner, "profile_iterations", 10)
    wl, inputs, gm, outs = _run(3, W.PIPELINE_SHAPES[3])
    op = fused_nodes(gm)[0].target
    assert op.tile in tiles
    con = sqlite3.connect(str(cache))
    rows = con.execute("SELECT key, us FROM best_config_mm").fetchall()
    con.close()
    assert len(rows) == 1 and rows[0][0].startswith("264_520_328_f16_f16_") and 0 < rows[0][1] < 1e4
    _compare(wl, outs, evt_oracle.eval_fp32(wl.module(), inputs))
    # the row is what an untuned trace now selects, without timing anything
    monkeypatch.setenv("EVT_AUTOTUNE", "0")
    monkeypatch.setattr(MMTuner, "profile", lambda self, tile: pytest.fail("timed a tile although a row exists"))
    again = fused_nodes(W.fuse(wl.module(), inputs))[0].target
    assert again.tile == op.tile


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
@pytest.mark.parametrize("swap", [True, False], ids=["operands_exchanged", "strided_store"])
@pytest.mark.parametrize("batched", [False, True], ids=["mm", "bmm"])
def test_column_major_outputs(batched, swap, dtype, monkeypatch):
    """gelu(a @ b + bias + r^T) stored as [N, M], with the sum over all rows (GEMM)
    or the maximum along every row (batched product) of the stored values: computed
    as C^T = B^T A^T with the operands exchanged (evt_fuser.py:573-596 in the
    reference), so that load and store are unit-stride along the kernel's n, and,
    with the exchange switched off, through strided accesses.  Both against eager
    fp32, and against each other."""
    mod, inputs = W.column_major_store(batched, dtype=dtype)
    tol = FP16_TOL      # 2e-2: wide enough for bf16's 8 mantissa bits as well
    monkeypatch.setattr(EVTFuser, "allow_transpose", swap)
    gm = W.fuse(mod, inputs)
    (node,) = fused_nodes(gm)
    assert node.target.transposed == swap and node.target.spec.bf16 == (dtype == torch.bfloat16)
    dev = [t.cuda() for t in inputs]
    outs = [o.clone() for o in gm(*dev)]
    torch.cuda.synchronize()
    refs = evt_oracle.eval_fp32(mod, inputs)
    assert len(outs) == len(refs) == 2
    for o, r in zip(outs, refs):
        assert tuple(o.shape) == tuple(r.shape)
        assert evt_oracle.max_rel_err(o, r) <= tol
    if swap:
        monkeypatch.setattr(EVTFuser, "allow_transpose", False)
        other = W.fuse(mod, inputs)(*dev)
        torch.cuda.synchronize()
        assert evt_oracle.max_rel_err(outs[0], other[0].float().cpu()) <= tol
        assert evt_oracle.max_rel_err(outs[1], other[1].float().cpu()) <= tol


@pytest.mark.parametrize("phase2", ["in_kernel", "finalize_kernel", "many_partials"])
@pytest.mark.parametrize("transposed, swap", [(False, True), (True, False), (True, True)],
                         ids=["per_column", "per_row", "operands_exchanged"])
def test_bias_gradient_behind_a_head_merge(transposed, swap, phase2, monkeypatch):
    """The backward pattern of an attention projection: batched product over
    B * H heads, result merged into [B * S, H * D] by the store, bias gradient
    = sum over all rows, i.e. per column (or, for the transposed product, per
    row; with the operands exchanged the transposed product is the per-column
    problem again) and over the batches that agree modulo H.  Several row tiles
    and several batches per result, combined by the last workgroup to arrive, by
    the finalize kernel on request, and by the finalize kernel because there are
    more partials per result (24 batches x the row tiles) than a workgroup
    combines; repeated launches are bit-identical."""
    monkeypatch.setattr(EVTFuser, "allow_transpose", swap)
    if phase2 == "finalize_kernel":
        monkeypatch.setenv("EVT_TWO_KERNEL_REDUCE", "1")
    many = phase2 == "many_partials"
    mod, inputs = W.head_merge_bias_grad(transposed=transposed, **(W.HEAD_MERGE_MANY_PARTIALS if many else {}))
    gm = W.fuse(mod, inputs)
    (node,) = fused_nodes(gm)
    (red,) = node.target.ir.reduces.values()
    per_row = transposed and not swap
    assert node.target.transposed == (transposed and swap)
    assert red.fold == "mod" and red.axis == ("row" if per_row else "col") and red.fold_count == (24 if many else 4)
    if many and not per_row:
        assert -(-node.target.problem[0] // node.target.tile.bm) * red.fold_count > 64
    dev = [t.cuda() for t in inputs]
    outs = [o.clone() for o in gm(*dev)]
    again = gm(*dev)
    torch.cuda.synchronize()
    refs = evt_oracle.eval_fp32(mod, inputs)
    for o, a, r in zip(outs, again, refs):
        assert torch.equal(o, a)
        assert tuple(o.shape) == tuple(r.shape)
        assert evt_oracle.max_rel_err(o, r) <= FP16_TOL
