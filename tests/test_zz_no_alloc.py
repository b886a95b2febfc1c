"""The entry point that allocates nothing (`evt_launch_static`): the partial
results and arrival counters of the cross-workgroup reductions live in a device
array that is part of the module instead of in a workspace of the caller's.
Called through the C ABI and compared bit for bit with `evt_launch` on the same
arguments -- two calls in a row, the second on a smaller problem, whose counters
lie where the first call left partial results."""
import ctypes

import pytest
import torch

from evt_ae_amd import jit
from tests import patterns as W
from evt_ae_amd.autotuner.tuner_base import force_tile
from evt_ae_amd.codegen import STATIC_SCRATCH_BYTES, TileConfig
from evt_ae_amd.workloads import fused_nodes

pytestmark = pytest.mark.gpu


def _launch_both(op, dev_inputs, arg_index):
    """Outputs of evt_launch and of evt_launch_static for one argument set."""
    stream = torch.cuda.current_stream()
    args = [dev_inputs[i] for i in arg_index]
    outs = []
    for static in (False, True):
        stores = op.allocate_outputs("cuda")
        for t in stores.values():
            t.view(torch.uint8).fill_(0xA5)     # stale contents must not survive
        a, keep = op.build_arguments(stores, *args, block=op.new_argument_block())
        module = op.module.ensure()
        if static:
            rc = module.lib.evt_launch_static(ctypes.byref(a), ctypes.c_void_p(stream.cuda_stream))
        else:
            ws_ptr, ws_bytes = op.workspace_for(a, stream, "cuda")
            rc = module.lib.evt_launch(ctypes.byref(a), ctypes.c_void_p(ws_ptr), ws_bytes, ctypes.c_void_p(stream.cuda_stream))
        assert rc == 0, rc
        torch.cuda.synchronize()
        outs.append({k: v.clone() for k, v in stores.items()})
        del keep
    return outs


def _op_for(cfg, shapes, tile):
    inputs = W.make_inputs(cfg, shapes)
    with force_tile(tile):
        gm = W.fuse(W.CONFIGS[cfg].module(), [t.to("meta") for t in inputs])
    (node,) = fused_nodes(gm)
    placeholders = [n for n in gm.graph.nodes if n.op == "placeholder"]
    return node.target, [t.cuda() for t in inputs], [placeholders.index(a) for a in node.args]


@pytest.mark.parametrize("cfg", list(W.NO_ALLOC_SHAPES))
def test_static_entry_point_matches_evt_launch(cfg):
    """Config 3 (per-row statistics over 4 column tiles, finished by the last workgroup of a row block) and
    config 4 (per-column sums over the row tiles): a first call, then a smaller problem through the same module."""
    tile = TileConfig(*W.NO_ALLOC_TILE)
    results = []
    for shapes in W.NO_ALLOC_SHAPES[cfg]:
        op, dev, idx = _op_for(cfg, shapes, tile)
        assert op.module.spec["static_scratch_bytes"] == STATIC_SCRATCH_BYTES
        a, keep = op.build_arguments(op.allocate_outputs("cuda"), *[dev[i] for i in idx], block=op.new_argument_block())
        need = op.module.workspace_bytes(a)
        assert 0 < need <= STATIC_SCRATCH_BYTES, need      # the kernels of this call do use the scratch array
        plain, static = _launch_both(op, dev, idx)
        for name in plain:
            assert torch.equal(plain[name].view(torch.uint8), static[name].view(torch.uint8)), (cfg, shapes, name)
        results.append(op.module.name)
    assert results[0] == results[1], "both problems must go through one module (one scratch array)"


def test_static_entry_point_refuses_what_does_not_fit():
    """The classifier at full size needs 6 MiB of partial results: refused before anything is enqueued."""
    cfg, shapes, tile = W.NO_ALLOC_TOO_BIG
    op, dev, idx = _op_for(cfg, shapes, TileConfig(*tile))
    a, keep = op.build_arguments(op.allocate_outputs("cuda"), *[dev[i] for i in idx], block=op.new_argument_block())
    assert op.module.workspace_bytes(a) > STATIC_SCRATCH_BYTES
    module = op.module.ensure()
    rc = module.lib.evt_launch_static(ctypes.byref(a), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == -5, rc                                      # EVT_ERR_SCRATCH
    torch.cuda.synchronize()


def test_static_entry_point_of_a_row_anchor():
    """Softmax with a per-column sum behind it: the row kernels' only scratch use (partials per workgroup)."""
    cls, _ = W.ROW_ANCHOR_PATTERNS["softmax_column_reduce"]
    inputs = W.pattern_inputs("softmax_column_reduce")
    gm = W.fuse(cls(), [t.to("meta") for t in inputs])
    (node,) = fused_nodes(gm)
    op = node.target
    placeholders = [n for n in gm.graph.nodes if n.op == "placeholder"]
    idx = [placeholders.index(a) for a in node.args]
    dev = [t.cuda() for t in inputs]
    plain, static = _launch_both(op, dev, idx)
    for name in plain:
        assert torch.equal(plain[name].view(torch.uint8), static[name].view(torch.uint8)), name


def test_static_entry_point_is_graph_capturable():
    """After one eager call on the device (which looks the array's address up), evt_launch_static can be recorded
    into a HIP graph: it enqueues fill kernels and the fused kernel, nothing else.  Every replay, with eager work
    and synchronisations in between, reproduces evt_launch bit for bit."""
    tile = TileConfig(*W.NO_ALLOC_TILE)
    op, dev, idx = _op_for(3, W.NO_ALLOC_SHAPES[3][0], tile)
    plain, static = _launch_both(op, dev, idx)                  # the eager warm-up call, outside capture
    args = [dev[i] for i in idx]
    outs = op.allocate_outputs("cuda")
    a, keep = op.build_arguments(outs, *args, block=op.new_argument_block())
    module = op.module.ensure()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        rc = module.lib.evt_launch_static(ctypes.byref(a), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0, rc
    for rep in range(3):
        for t in outs.values():
            t.view(torch.uint8).fill_(0x5A)
        _ = (dev[0].float().sum() + rep).item()                 # unrelated eager work and a synchronisation
        graph.replay()
        torch.cuda.synchronize()
        for name in plain:
            assert torch.equal(plain[name].view(torch.uint8), outs[name].view(torch.uint8)), (rep, name)
    del keep
