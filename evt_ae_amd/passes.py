"""Graph-level entry point that feeds the fuser: `pass_fusion(module, graph)`.

Mirror of the call surface of python/gtl/compiler/passes/pass_fusion.py:1383-1385
(`pass_fusion` -> `Partitioning` -> `EVTFuser.fusible / EVTFuser().trace`,
:1356-1374).  The reference decides partitions with an ILP over the whole joint
graph (:216-983); this backend covers the fused GEMM/BMM path only, so the
partitioner here grows one partition per mm/bmm anchor greedily: operand
permutes in front of the anchor (main-loop fusion, :1019-1030), then every
downstream node from FUSIBLE_TGT whose other operands do not depend on the
anchor, then small broadcast-side expressions that only feed the partition.
If the fuser rejects a partition (NotImplementedError) the partition is
shrunk from the end until it is accepted.
"""
from __future__ import annotations

import operator
from typing import List, Sequence, Set

import torch
from torch.fx import Graph, GraphModule, Node
from torch.fx.passes.tools_common import legalize_graph

from .evt_fuser import EVTFuser, packet, target_name

aten = torch.ops.aten

# ops the epilogue can absorb (reference list: pass_fusion.py:53-82, plus the
# reductions and index ops the MI355X epilogue adds)
FUSIBLE_TGT = {
    "add", "sub", "rsub", "mul", "div", "neg", "maximum", "minimum", "exp", "log", "sqrt", "rsqrt", "abs",
    "reciprocal", "gelu", "tanh", "relu", "sigmoid", "tanh_backward", "gelu_backward", "ge", "gt", "le", "lt",
    "ne", "eq", "where", "_to_copy", "to", "one_hot", "gather", "sum", "amax", "mean", "logsumexp", "var_mean",
    "getitem", "view", "_unsafe_view", "reshape", "unsqueeze", "squeeze", "permute", "clone", "expand",
    "detach", "alias", "contiguous", "rand_like",
}
_SMALL_SIDE = FUSIBLE_TGT - {"sum", "amax", "mean", "logsumexp", "var_mean", "gather", "one_hot", "getitem"}


def _fusible(node: Node) -> bool:
    return node.op == "call_function" and target_name(node.target) in FUSIBLE_TGT


def _descendants(anchor: Node) -> Set[Node]:
    seen, work = set(), [anchor]
    while work:
        n = work.pop()
        for u in n.users:
            if u not in seen:
                seen.add(u)
                work.append(u)
    return seen


def _grow(anchor: Node, taken: Set[Node]) -> List[Node]:
    part: List[Node] = []
    # main-loop fusion: a 2-D/3-D permute that only feeds the anchor
    for arg in anchor.args[:2]:
        if (isinstance(arg, Node) and arg.op == "call_function" and packet(arg.target) == aten.permute
                and len(arg.users) == 1 and arg not in taken):
            part.append(arg)
    part.append(anchor)
    inside = set(part)
    desc = _descendants(anchor)
    after = False
    for node in anchor.graph.nodes:
        if node is anchor:
            after = True
            continue
        if not after or node in taken or node not in desc or not _fusible(node):
            continue
        ins = node.all_input_nodes
        if not any(i in inside for i in ins):
            continue
        if any((i not in inside) and (i in desc) for i in ins):
            continue   # another operand depends on the anchor through unfused nodes
        if target_name(node.target) == "getitem" and node.args[0] not in inside:
            continue
        part.append(node)
        inside.add(node)
    # multi-output producers need all their getitems inside or none
    for node in list(part):
        if node.op == "call_function" and target_name(node.target) == "var_mean":
            if not all(u in inside for u in node.users):
                for u in [node] + list(node.users):
                    if u in inside:
                        inside.discard(u)
                        part.remove(u)
    # broadcast-side expressions (e.g. a mask built from a small tensor) whose
    # every user is inside the partition
    changed = True
    while changed:
        changed = False
        for node in list(inside):
            for i in node.all_input_nodes:
                if (i in inside or i in desc or i in taken or i.op != "call_function"
                        or target_name(i.target) not in _SMALL_SIDE or node is anchor
                        or (packet(node.target) == aten.permute and anchor in node.users)):
                    continue
                if all(u in inside for u in i.users):
                    inside.add(i)
                    changed = True
    return [n for n in anchor.graph.nodes if n in inside]


class Partitioning:
    """Callable pass object, as in the reference (pass_fusion.py:1185-1380)."""

    def __call__(self, graph_module: GraphModule) -> GraphModule:
        self.call(graph_module)
        self.ensures(graph_module)
        return graph_module

    def call(self, graph_module: GraphModule) -> None:
        graph = graph_module.graph
        anchors = [n for n in graph.nodes
                   if n.op == "call_function" and packet(n.target) in EVTFuser.supported_targets]
        taken: Set[Node] = set()
        self.partitions: List[List[str]] = []
        for anchor in anchors:
            if anchor in taken:
                continue
            part = _grow(anchor, taken)
            names = [n.name for n in part]
            while True:
                if not EVTFuser.fusible(names, graph_module):
                    break
                try:
                    EVTFuser().trace(graph_module, names)
                    self.partitions.append(names)
                    taken.update(n for n in part if n.name in names)
                    break
                except NotImplementedError:
                    # drop the last epilogue node (never the anchor or its operand permutes)
                    idx = names.index(anchor.name)
                    if len(names) - 1 <= idx:
                        break
                    names = names[:-1]

    def ensures(self, graph_module: GraphModule) -> None:
        legalize_graph(graph_module)
        graph_module.graph.eliminate_dead_code()
        graph_module.graph.lint()
        graph_module.recompile()


def pass_fusion(module: GraphModule, graph: Graph = None):
    return Partitioning()(module)
