"""Front-end passes that run on the joint forward/backward graph before the
fuser, as far as the fused GEMM/BMM path needs them.

Counterparts in the reference (python/gtl/compiler/passes/):
  GTLFrontend            pass_frontend.py:31-123, 131-192
  pass_cse               pass_cse.py
  pass_clean_up          pass_clean_up.py:24-55
  pass_loss_elimination  pass_eliminate_loss.py:24-37
Nodes these passes create inherit the forward/backward tag of the node they
replace, so that AOT autograd's partitioner still finds the boundary.
"""
from __future__ import annotations

import operator
from functools import reduce
from typing import Dict, Optional, Tuple

import torch
from torch.fx import Graph, GraphModule, Node

from .evt_fuser import packet, target_name

aten = torch.ops.aten

CARRIED_META = ("partitioner_tag", "seq_nr", "autograd_backward")

# consumers that broadcast their operands themselves, so an expand in front of
# them only restates the broadcast
_BROADCASTING = {"add", "sub", "rsub", "mul", "div", "maximum", "minimum", "where", "ge", "gt", "le", "lt", "ne",
                 "eq", "tanh_backward", "gelu_backward"}


def inherit_meta(new: Node, old: Node) -> Node:
    for k in CARRIED_META:
        if k in old.meta:
            new.meta[k] = old.meta[k]
    return new


class GTLFrontend:
    """Normalises the graph AOT autograd hands over:

      * `aten.add.Tensor` -> `aten.add`: overload suffixes are dropped, every
        later pass matches on the overload packet (pass_frontend.py:131-192);
      * `detach` / `alias` nodes are removed; `expand` nodes are removed where
        every consumer broadcasts by itself (the reference drops every expand,
        :44-47, 84-87; a GEMM operand or a view behind an expand still needs
        it, so those stay);
      * `view(x, [..., -1, ...])` gets its shape written out (:64-75).

    Called like the reference's pass object: `module, modified = GTLFrontend()(module)`.
    """

    transparent = ("detach", "alias", "lift_fresh_copy")

    def __init__(self) -> None:
        self.modified = False

    def __call__(self, graph_module: GraphModule) -> Tuple[GraphModule, bool]:
        self.modified = False
        graph = graph_module.graph
        for node in list(graph.nodes):
            if node.op != "call_function":
                continue
            name = target_name(node.target)
            if name in self.transparent and isinstance(node.args[0], Node):
                node.replace_all_uses_with(node.args[0])
                graph.erase_node(node)
                self.modified = True
                continue
            if name == "expand" and node.users and all(
                    u.op == "call_function" and target_name(u.target) in _BROADCASTING for u in node.users):
                node.replace_all_uses_with(node.args[0])
                graph.erase_node(node)
                self.modified = True
                continue
            pk = packet(node.target)
            if pk is not node.target and str(node.target).startswith("aten."):
                node.target = pk
                self.modified = True
            if name in ("view", "_unsafe_view", "reshape") and -1 in list(node.args[1]) and "tensor_meta" in node.meta:
                numel = reduce(lambda x, y: x * int(y), node.meta["tensor_meta"].shape, 1)
                known = reduce(lambda x, y: x * int(y), [d for d in node.args[1] if d != -1], 1)
                node.args = (node.args[0], [int(d) if d != -1 else numel // max(known, 1) for d in node.args[1]])
                self.modified = True
        graph.eliminate_dead_code()
        graph.lint()
        graph_module.recompile()
        return graph_module, self.modified


def _freeze(x):
    if isinstance(x, (list, tuple)):
        return tuple(_freeze(i) for i in x)
    if isinstance(x, dict):
        return tuple(sorted((k, _freeze(v)) for k, v in x.items()))
    if isinstance(x, Node):
        return ("node", x.name)
    if isinstance(x, slice):
        return ("slice", x.start, x.stop, x.step)
    if isinstance(x, (bool, int, float, complex)):
        return (type(x).__name__, x)      # 1, 1.0 and True compare equal but promote differently
    return x


_IMPURE = {"rand_like", "randn_like", "native_dropout", "bernoulli", "rand", "randn", "randint", "randperm",
           "normal", "uniform", "dropout"}
# fresh storage on every call: two of these must stay two tensors (something may write into one later)
_FACTORIES = {"empty", "empty_like", "empty_strided", "new_empty", "new_empty_strided", "new_zeros", "new_ones",
              "new_full", "zeros", "ones", "full", "zeros_like", "ones_like", "full_like", "clone", "arange"}


def _mergeable(node: Node) -> bool:
    """A pure function of its operands: not random, not a factory, and no mutable / out-variant schema."""
    name = target_name(node.target)
    if name in _IMPURE or name in _FACTORIES or name.endswith("_"):
        return False
    schema = getattr(node.target, "_schema", None)
    if schema is not None and getattr(schema, "is_mutable", False):
        return False
    return True



def pass_cse(module: GraphModule, graph: Graph = None) -> GraphModule:
    """Common-subexpression elimination over pure call_function nodes: a node
    with the same target and the same (already merged) operands as an earlier
    one is replaced by it.  Random ops, factory ops and ops with a mutable schema
    never merge, and Python scalars are keyed with their type."""
    graph = module.graph
    seen: Dict[tuple, Node] = {}
    for node in list(graph.nodes):
        if node.op != "call_function" or not _mergeable(node) or node.meta.get("evt"):
            continue
        try:
            key = (node.target, _freeze(node.args), _freeze(node.kwargs))
            hash(key)
        except TypeError:
            continue
        first = seen.get(key)
        if first is None:
            seen[key] = node
        else:
            node.replace_all_uses_with(first)
            graph.erase_node(node)
    graph.lint()
    module.recompile()
    return module


def pass_clean_up(module: GraphModule, graph: Graph = None) -> GraphModule:
    """pass_clean_up.py:24-55: `one_hot` results are cast to the dtype recorded
    for them unless a cast already follows, and a contiguous `clone` goes
    between a `permute` and a `view` that consumes it (a view of a permuted
    tensor is otherwise not expressible)."""
    graph = module.graph
    for node in list(graph.nodes):
        if node.op != "call_function":
            continue
        name = target_name(node.target)
        users = list(node.users)
        if name == "one_hot" and "tensor_meta" in node.meta:
            if len(users) == 1 and target_name(users[0].target) in ("to", "_to_copy"):
                continue
            with graph.inserting_after(node):
                cast = inherit_meta(graph.call_function(aten._to_copy, (node,),
                                                        {"dtype": node.meta["tensor_meta"].dtype}), node)
            cast.meta["tensor_meta"] = node.meta["tensor_meta"]
            for u in users:
                u.replace_input_with(node, cast)
        elif name == "permute":
            views = [u for u in users if u.op == "call_function" and target_name(u.target) == "view"]
            if not views:
                continue
            with graph.inserting_after(node):
                clone = inherit_meta(graph.call_function(aten.clone, (node,),
                                                         {"memory_format": torch.contiguous_format}), node)
            if "tensor_meta" in node.meta:
                clone.meta["tensor_meta"] = node.meta["tensor_meta"]
            for u in views:
                u.replace_input_with(node, clone)
    graph.lint()
    module.recompile()
    return module


def pass_loss_elimination(module: GraphModule, graph: Graph = None) -> GraphModule:
    """pass_eliminate_loss.py:24-37: the first result of the joint graph (the
    loss) is replaced by a constant tensor of ones, so that whatever only the
    loss value needs drops out as dead code.  Training loops that never read
    the loss use it; the default pipeline leaves the loss in."""
    graph = module.graph
    out = next(n for n in graph.nodes if n.op == "output")
    loss = out.all_input_nodes[0]
    tm = loss.meta.get("tensor_meta")
    if tm is None:
        raise ValueError("the loss node carries no tensor metadata")
    val = loss.meta.get("val")
    device = val.device if isinstance(val, torch.Tensor) else torch.device("cuda" if torch.cuda.is_available() else "cpu")
    from torch.utils._python_dispatch import _disable_current_modes
    with _disable_current_modes():
        ones = torch.ones(tuple(tm.shape), dtype=tm.dtype, device=device)
    module.register_buffer("_fake_loss_0", ones, persistent=False)
    with graph.inserting_before(loss):
        fake = inherit_meta(graph.get_attr("_fake_loss_0"), loss)
    fake.meta["tensor_meta"] = tm
    if "val" in loss.meta:
        fake.meta["val"] = loss.meta["val"]
    loss.replace_all_uses_with(fake)
    graph.eliminate_dead_code()
    graph.lint()
    module.recompile()
    return module
