"""The joint-graph partitioner (evt_ae_amd/partitioner.py) without a GPU.

The integer program is pinned by exhaustive search on small multi-anchor
graphs: every assignment of candidate nodes to anchors is enumerated, the ones
whose partitions are closed and whose quotient graph is acyclic are kept, and
the largest on-chip volume among them must equal the program's optimum.  The
counterpart in the reference is the ILP of pass_fusion.py:216-983, which its
tests exercise only through whole models.
"""
import itertools
import operator

import networkx as nx
import pytest
import torch
from torch.fx.passes.tools_common import legalize_graph

from tests import patterns as W
from evt_ae_amd.evt_fuser import EVTFuser, packet, target_name
from evt_ae_amd.partitioner import AnchorPartitionILP, PartitionCache, _volume_bits
from evt_ae_amd.passes import Partitioning, _fusible, internal_volume_bits
from evt_ae_amd.workloads import fused_nodes

aten = torch.ops.aten
M, N, K = 128, 256, 64


def h(*shape):
    return torch.empty(*shape, dtype=torch.float16, device="meta")


TwoAnchorsMixedWidth, CrossedAnchors, ThreeAnchorsDiamond = (
    W.TwoAnchorsMixedWidth, W.CrossedAnchors, W.ThreeAnchorsDiamond)


def inputs_for(mod):
    if isinstance(mod, ThreeAnchorsDiamond):
        return [h(M, K), h(K, N)] * 3 + [h(N)]
    return [h(M, K), h(K, N)] * 2


def anchors_of(gm):
    return [n for n in gm.graph.nodes if n.op == "call_function" and packet(n.target) in EVTFuser.supported_targets]


def brute_force_optimum(gm):
    """Largest internal volume over every closed, acyclic assignment."""
    ilp = AnchorPartitionILP(gm, anchors_of(gm), _fusible)
    anchors = ilp.anchors
    cand = {s: ilp.candidates(s) for s in anchors}
    nodes = sorted({j for s in anchors for j in cand[s]}, key=ilp.index.__getitem__)
    owners = {j: [s for s in anchors if j in cand[s]] for j in nodes}
    best = -1
    for choice in itertools.product(*[[None] + owners[j] for j in nodes]):
        assign = dict(zip(nodes, choice))
        ok, total = True, 0
        for j, s in assign.items():
            if s is None:
                continue
            for i in j.all_input_nodes:
                if i is s:
                    total += _volume_bits(i)
                elif i in ilp._desc[s]:
                    if assign.get(i) is not s:        # closure: operands downstream of s stay inside
                        ok = False
                    else:
                        total += _volume_bits(i, j.args[1] if target_name(j.target) == "getitem" else None)
        if not ok:
            continue
        # quotient graph: one vertex per partition, one per unfused node
        part = {n: n for n in ilp.nodes}
        for j, s in assign.items():
            if s is not None:
                part[j] = s
        q = nx.DiGraph()
        for j in ilp.nodes:
            for i in j.all_input_nodes:
                if i in part and part[i] is not part[j]:
                    q.add_edge(part[i], part[j])
        if not nx.is_directed_acyclic_graph(q):
            continue
        best = max(best, total)
    return best


@pytest.mark.parametrize("mod", [TwoAnchorsMixedWidth, CrossedAnchors, ThreeAnchorsDiamond])
def test_ilp_matches_exhaustive_search(mod):
    gm = W.trace_module(mod(), inputs_for(mod()))
    best = brute_force_optimum(gm)
    ilp = AnchorPartitionILP(gm, anchors_of(gm), _fusible, cache=PartitionCache(path=""))
    assign = ilp.solve()
    assert ilp.last_objective == best
    # the reported objective is the volume of the assignment it returns
    parts = [[s.name] + [j.name for j in assign[s]] for s in ilp.anchors]
    assert internal_volume_bits(gm, parts) == best


def test_ilp_beats_graph_order_on_mixed_width():
    mod = TwoAnchorsMixedWidth()
    g = Partitioning("greedy")
    g(W.trace_module(mod, inputs_for(mod)))
    i = Partitioning("ilp")
    gm = i(W.trace_module(mod, inputs_for(mod)))
    assert g.objective_bits == 64 * M * N            # y1->z, y2->y2f, y2f->t
    assert i.objective_bits == 80 * M * N            # y2->y2f, y2f->t, t->z
    assert sorted(map(len, i.partitions)) == [1, 4]
    assert len(fused_nodes(gm)) == 2


def test_crossed_anchors_stay_orderable():
    mod = CrossedAnchors()
    p = Partitioning("ilp")
    gm = p(W.trace_module(mod, inputs_for(mod)))      # ensures() legalizes: a cycle would raise
    sizes = sorted(len(x) for x in p.partitions)
    assert sizes == [1, 2]                            # only one of e1 / e2 can be fused
    order = {n: k for k, n in enumerate(gm.graph.nodes)}
    for n in gm.graph.nodes:
        assert all(order[i] < order[n] for i in n.all_input_nodes)


def test_ilp_equals_greedy_on_single_anchor_graphs():
    """With one anchor there is nothing to arbitrate: both strategies must hand
    the fuser the same partition for every headline config and fuser pattern."""
    cases = [(W.CONFIGS[c].module(), W.make_inputs(c, W.SMALL_SHAPES[c])) for c in W.CONFIGS]
    cases += [(entry[0](), W.pattern_inputs(name)) for name, entry in W.REFERENCE_PATTERNS.items()]
    for mod, inputs in cases:
        metas = [t.to("meta") if isinstance(t, torch.Tensor) else t for t in inputs]
        a, b = Partitioning("greedy"), Partitioning("ilp")
        a(W.trace_module(mod, metas))
        b(W.trace_module(mod, metas))
        assert [sorted(p) for p in a.partitions] == [sorted(p) for p in b.partitions], type(mod).__name__
        assert a.objective_bits == b.objective_bits


def test_rejected_node_is_banned_and_solved_again():
    class ErfTail(torch.nn.Module):
        def forward(self, a, b, bias):
            y = aten.mm(a, b)
            x = aten.add(y, bias)
            e = aten.erf(x)                 # not an epilogue op: never a candidate
            return aten.mul(e, 2.0)

    class AlphaInTheMiddle(torch.nn.Module):
        def forward(self, a, b, bias):
            y = aten.mm(a, b)
            x = aten.add(y, bias)
            z = aten.add(x, bias, alpha=2.0)     # a candidate by target, turned down by the fuser
            return aten.relu(z)

    p = Partitioning("ilp")
    p(W.trace_module(ErfTail(), [h(M, K), h(K, N), h(N)]))
    assert [len(x) for x in p.partitions] == [2] and p.resolves == 0
    p = Partitioning("ilp")
    gm = p(W.trace_module(AlphaInTheMiddle(), [h(M, K), h(K, N), h(N)]))
    assert [len(x) for x in p.partitions] == [2] and p.resolves == 2     # relu, then the add with alpha
    assert len(fused_nodes(gm)) == 1
    assert p.objective_bits == 16 * M * N


def test_partition_cache_roundtrip(tmp_path):
    mod = ThreeAnchorsDiamond()
    path = str(tmp_path / "partitions.db")
    gm = W.trace_module(mod, inputs_for(mod))
    first = AnchorPartitionILP(gm, anchors_of(gm), _fusible, cache=PartitionCache(path))
    a = first.solve()
    assert not first.last_from_cache
    gm2 = W.trace_module(mod, inputs_for(mod))
    second = AnchorPartitionILP(gm2, anchors_of(gm2), _fusible, cache=PartitionCache(path))
    b = second.solve()
    assert second.last_from_cache
    assert {s.name: [j.name for j in v] for s, v in a.items()} == {s.name: [j.name for j in v] for s, v in b.items()}
    assert first.last_objective == second.last_objective
    # a different graph does not hit the entry
    other = TwoAnchorsMixedWidth()
    gm3 = W.trace_module(other, inputs_for(other))
    third = AnchorPartitionILP(gm3, anchors_of(gm3), _fusible, cache=PartitionCache(path))
    third.solve()
    assert not third.last_from_cache
