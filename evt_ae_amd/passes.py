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


# ---------------------------------------------------------------------------
# pass_decomposition: the rewrites in front of the fuser that the fused
# GEMM/BMM path depends on
# ---------------------------------------------------------------------------

def _repropagate(module: GraphModule) -> None:
    """Refresh tensor_meta after a rewrite by running the graph on meta tensors
    shaped like the placeholders (no data, no device)."""
    from torch.fx.passes.shape_prop import ShapeProp
    metas = []
    for n in module.graph.nodes:
        if n.op == "placeholder":
            tm = n.meta.get("tensor_meta")
            if tm is None:
                return      # no shapes recorded: the caller runs ShapeProp itself
            metas.append(torch.empty(tuple(tm.shape), dtype=tm.dtype, device="meta"))
    ShapeProp(module).propagate(*metas)


def pass_decomposition(module: GraphModule, graph: Graph = None, disabled_ops: Sequence[str] = ()):
    """The subset of the reference's Decomposition pass
    (python/gtl/compiler/passes/pass_decomposition.py:192-502, entry :817) that
    the fused GEMM/BMM path needs, with the same replacements:

      addmm(b, x, w)                 -> add(mm(x, w), b)                         (:414-426)
      t(x) / transpose(x, i, j)      -> permute(x, dims)                         (:448-502)
      _unsafe_view(x, s)             -> view(x, s)                               (:463-475)
      rsub(x, y)                     -> sub(y, x)                                (:280-292)
      native_dropout(x, p, True)     -> mask = ge(rand_like(x), p);
                                        (mul(mul(x, mask), 1/(1-p)), mask)       (:350-379)
      native_dropout_backward(g,m,s) -> mul(mul(g, m), s)                        (:381-395)
      threshold_backward(g, y, t)    -> mul(g, gt(y, t))                         (:397-412; the reference
                                        writes ne(y, t), equal on ReLU outputs only)

    The reference's other decompositions (log_softmax, nll_loss, layer / batch
    norm, convolution, pooling) belong to anchors this backend does not provide
    and are left untouched."""
    graph = module.graph if graph is None else graph
    disabled = set(disabled_ops)
    changed = False
    for node in list(graph.nodes):
        if node.op != "call_function":
            continue
        name = target_name(node.target)
        if name in disabled:
            continue
        new = None
        with graph.inserting_before(node):
            if name == "addmm" and len(node.args) == 3 and not node.kwargs:
                b, x, w = node.args
                new = graph.call_function(aten.add, (graph.call_function(aten.mm, (x, w)), b))
            elif name == "t":
                new = graph.call_function(aten.permute, (node.args[0], [1, 0]))
            elif name == "transpose" and len(node.args) == 3:
                rank = len(node.meta["tensor_meta"].shape)
                dims = list(range(rank))
                i, j = node.args[1] % rank, node.args[2] % rank
                dims[i], dims[j] = j, i
                new = graph.call_function(aten.permute, (node.args[0], dims))
            elif name == "_unsafe_view":
                new = graph.call_function(aten.view, tuple(node.args))
            elif name == "rsub" and len(node.args) == 2 and node.kwargs.get("alpha", 1) == 1:
                new = graph.call_function(aten.sub, (node.args[1], node.args[0]))
            elif name == "native_dropout_backward":
                g, m, s = node.args
                new = graph.call_function(aten.mul, (graph.call_function(aten.mul, (g, m)), s))
            elif name == "threshold_backward":
                g, y, t = node.args
                new = graph.call_function(aten.mul, (g, graph.call_function(aten.gt, (y, t))))
            elif name == "native_dropout" and len(node.args) == 3 and node.args[2] is True:
                x, p = node.args[0], node.args[1]
                mask = graph.call_function(aten.ge, (graph.call_function(torch.rand_like, (x,)), p))
                out = graph.call_function(aten.mul, (graph.call_function(aten.mul, (x, mask)), 1. / (1 - p)))
                for user in list(node.users):     # getitem(dropout, 0 | 1)
                    if user.op == "call_function" and user.target is operator.getitem:
                        user.replace_all_uses_with(out if user.args[1] == 0 else mask)
                        graph.erase_node(user)
                if not node.users:
                    graph.erase_node(node)
                    changed = True
                continue
        if new is not None:
            node.replace_all_uses_with(new)
            graph.erase_node(node)
            changed = True
    if changed:
        graph.lint()
        module.recompile()
        _repropagate(module)
    return module
