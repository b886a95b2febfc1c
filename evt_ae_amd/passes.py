"""Graph-level entry point that feeds the fuser: `pass_fusion(module, graph)`.

Mirror of the call surface of python/gtl/compiler/passes/pass_fusion.py:1383-1385
(`pass_fusion` -> `Partitioning` -> `EVTFuser.fusible / EVTFuser().trace`,
:1356-1374).  The reference decides partitions with an ILP over the whole joint
graph (:216-983); this backend lowers the fused GEMM/BMM partitions only, so
every partition is one mm/bmm anchor, operand permutes in front of it
(main-loop fusion, :1019-1030), downstream nodes from FUSIBLE_TGT, and small
broadcast-side expressions that only feed the partition.  Which anchor gets
which downstream node is decided by the integer program in partitioner.py
(default) or greedily in graph order.  A partition the fuser rejects
(NotImplementedError) is shrunk from the end until it is accepted.
"""
from __future__ import annotations

import operator
import os
from typing import List, Sequence, Set

import torch
from torch.fx import Graph, GraphModule, Node

from .evt_fuser import EVTFuser, legalize_graph, operand_chain, operand_strides, packet, target_name
from .partitioner import same_phase
from .frontend_passes import (GTLFrontend, inherit_meta, pass_clean_up, pass_cse,  # noqa: F401  (one namespace,
                              pass_loss_elimination)                                # as gtl.compiler.passes)

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
# layout-only and generated values: nothing a kernel would compute once and hand to other kernels
LAYOUT_SIDE = {"view", "_unsafe_view", "reshape", "unsqueeze", "squeeze", "permute", "clone", "expand", "detach", "alias",
               "contiguous", "getitem", "rand_like"}


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


def _mainloop_permutes(anchor: Node, taken: Set[Node]) -> List[Node]:
    """Main-loop fusion: a permute that only feeds the anchor is read through
    the operand's strides (reference: pass_fusion.py:773-781, 1019-1030)."""
    out = []
    for arg in anchor.args[:2]:
        if packet(anchor.target) == aten.bmm and isinstance(arg, Node):
            # a whole chain of views / permutes / copies in front of a batched-product operand (the head split
            # of an attention layer), when it amounts to strided addressing the kernel can read in place
            chain, _ = operand_chain(arg, lambda n: n not in taken)
            if chain and any(target_name(n.target) in ("clone", "permute") for n in chain):
                shape = arg.meta["tensor_meta"].shape if "tensor_meta" in arg.meta else None
                st = operand_strides(chain, shape) if shape is not None and len(shape) == 3 else None
                if st is not None and (st.stride_n == 1 or st.stride_m == 1):
                    out.extend(chain)
                    continue
        if (isinstance(arg, Node) and arg.op == "call_function" and packet(arg.target) == aten.permute
                and len(arg.users) == 1 and arg not in taken):
            out.append(arg)
    return out


def _private_operand_chains(graph_module: GraphModule) -> None:
    """The layout chain in front of a batched-product operand can only be read in
    place when it feeds nothing else.  In a joint graph the split heads of an
    attention layer feed the forward product and, through a transpose, the
    backward products: every product whose operand chain amounts to strided
    addressing gets a private copy of the chain's (layout-only) nodes next to
    it, tagged with its own phase; what is left without users goes."""
    graph = graph_module.graph
    changed = False
    for anchor in [n for n in graph.nodes if n.op == "call_function" and packet(n.target) == aten.bmm]:
        for arg in list(anchor.args[:2]):
            if not isinstance(arg, Node) or "tensor_meta" not in arg.meta:
                continue
            if arg.meta["tensor_meta"].dtype not in (torch.float16, torch.bfloat16):
                continue        # not a product the fuser takes: a private chain would only add copies
            chain, src = [], arg
            while (isinstance(src, Node) and src.op == "call_function"
                   and target_name(src.target) in ("view", "_unsafe_view", "reshape", "permute", "expand", "clone", "select")):
                chain.append(src)
                src = src.args[0]
            chain.reverse()
            if not chain or all(len(n.users) == 1 for n in chain):
                continue
            if not any(target_name(n.target) == "clone" for n in chain):
                continue
            shape = tuple(arg.meta["tensor_meta"].shape)
            st = operand_strides(chain, shape) if len(shape) == 3 else None
            if st is None or not (st.stride_n == 1 or st.stride_m == 1):
                continue
            tags = {k: anchor.meta[k] for k in ("partitioner_tag", "seq_nr", "autograd_backward") if k in anchor.meta}
            x = src
            with graph.inserting_before(anchor):
                for n in chain:
                    y = graph.call_function(n.target, (x, *n.args[1:]), dict(n.kwargs))
                    y.meta = {k: v for k, v in n.meta.items() if k in ("tensor_meta", "val")}
                    y.meta.update(tags)
                    x = y
            anchor.replace_input_with(arg, x)
            changed = True
    if changed:
        graph.eliminate_dead_code()
        graph_module.recompile()


def _vector_along_n(node: Node) -> bool:
    """[N], [1, N], [B, 1, N], [B, 1, 1, N]: one value per column (and batch)."""
    tm = node.meta.get("tensor_meta")
    if tm is None or not hasattr(tm, "shape"):
        return False
    shape = [int(d) for d in tm.shape]
    if not shape or shape[-1] <= 1:
        return False
    middle = shape[1:-1] if len(shape) >= 3 else shape[:-1]
    return all(d == 1 for d in middle)


def _ancestors(nodes: Set[Node], stop: Node) -> Set[Node]:
    """Everything the `nodes` are computed from, not looking through `stop`."""
    seen: Set[Node] = set()
    work = [i for n in nodes for i in n.all_input_nodes if i is not stop]
    while work:
        n = work.pop()
        if n in seen or n is stop:
            continue
        seen.add(n)
        work.extend(n.all_input_nodes)
    return seen


def _absorb_side_expressions(anchor: Node, inside: Set[Node], desc: Set[Node], taken: Set[Node],
                             shared: Set[Node] = None) -> None:
    """Broadcast-side expressions (e.g. a mask built from a small tensor) whose
    every user is inside the partition join it.  They are not downstream of the
    anchor, so this cannot close a cycle between partitions.

    With `shared` (a set that receives them), a per-column vector that has users
    outside the partition as well joins it too and leaves the kernel as an
    output of its own -- the reference's row store (visitor_store.hpp:46-145):
    BERT's transformed attention mask is computed by the first attention
    product's kernel and read by the others.  None of its outside users may
    feed the partition; the caller checks the planned partitions as a whole
    for cycles."""
    # producers of the anchor's operands inside the partition (layout chains read through strides): what feeds
    # them is the operand's source tensor, never a side expression of the epilogue
    pre: Set[Node] = set()
    stack = [a for a in anchor.all_input_nodes if a in inside]
    while stack:
        n = stack.pop()
        if n not in pre:
            pre.add(n)
            stack.extend(a for a in n.all_input_nodes if a in inside)
    changed = True
    while changed:
        changed = False
        for node in list(inside):
            if node in pre:
                continue
            for i in node.all_input_nodes:
                if (i in inside or i in desc or i in taken or i.op != "call_function"
                        or target_name(i.target) not in _SMALL_SIDE or node is anchor
                        or (packet(node.target) == aten.permute and anchor in node.users)):
                    continue
                if all(u in inside for u in i.users):
                    inside.add(i)
                    changed = True
                elif (shared is not None and _vector_along_n(i) and same_phase(i, anchor)
                      and target_name(i.target) not in LAYOUT_SIDE
                      and not any(u in _ancestors(inside | {i}, i) for u in i.users if u not in inside)):
                    inside.add(i)
                    shared.add(i)
                    changed = True


def _quotient_is_acyclic(graph: Graph, groups: Sequence[Set[Node]]) -> bool:
    """Do the planned partitions, each taken as one node, leave the graph orderable?"""
    gid = {}
    for k, members in enumerate(groups):
        for n in members:
            gid[n] = ("p", k)
    succ, indeg = {}, {}
    for n in graph.nodes:
        a = gid.get(n, n)
        succ.setdefault(a, set())
        indeg.setdefault(a, 0)
    for n in graph.nodes:
        b = gid.get(n, n)
        for i in n.all_input_nodes:
            a = gid.get(i, i)
            if a != b and b not in succ[a]:
                succ[a].add(b)
                indeg[b] += 1
    ready = [a for a, d in indeg.items() if d == 0]
    done = 0
    while ready:
        a = ready.pop()
        done += 1
        for b in succ[a]:
            indeg[b] -= 1
            if indeg[b] == 0:
                ready.append(b)
    return done == len(indeg)


def _grow(anchor: Node, taken: Set[Node], shared: Set[Node] = None) -> List[Node]:
    part: List[Node] = _mainloop_permutes(anchor, taken)
    part.append(anchor)
    inside = set(part)
    desc = _descendants(anchor)
    after = False
    for node in anchor.graph.nodes:
        if node is anchor:
            after = True
            continue
        if not after or node in taken or node not in desc or not _fusible(node) or not same_phase(node, anchor):
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
    _absorb_side_expressions(anchor, inside, desc, taken, shared)
    return [n for n in anchor.graph.nodes if n in inside]


def internal_volume_bits(graph_module: GraphModule, partitions: Sequence[Sequence[str]]) -> int:
    """Bits of the anchor-downstream edges that the partitions keep on chip:
    the partitioner's objective (reference: pass_fusion.py:518-535)."""
    from .partitioner import _volume_bits
    by_name = {n.name: n for n in graph_module.graph.nodes}
    total = 0
    for names in partitions:
        nodes = [by_name[x] for x in names]
        anchor = next(n for n in nodes if n.op == "call_function" and packet(n.target) in EVTFuser.supported_targets)
        desc = _descendants(anchor) | {anchor}
        inside = set(nodes)
        for j in nodes:
            if j is anchor or j not in desc:
                continue
            for i in j.all_input_nodes:
                if i in inside and i in desc:
                    total += _volume_bits(i, j.args[1] if target_name(j.target) == "getitem" else None)
    return total


class Partitioning:
    """Callable pass object, as in the reference (pass_fusion.py:1185-1380).

    `strategy="ilp"` (default, or EVT_PARTITIONER) solves one integer program
    over all anchors of the graph; `"greedy"` grows the anchors one after the
    other in graph order.  Either way a partition the fuser turns down is
    shrunk from its end until it is accepted."""

    MAX_RESOLVES = 64

    def __init__(self, strategy: str = None) -> None:
        self.strategy = strategy or os.environ.get("EVT_PARTITIONER", "ilp")
        if self.strategy not in ("ilp", "greedy"):
            raise ValueError(f"unknown partitioning strategy {self.strategy!r}")
        self.partitions: List[List[str]] = []
        self.objective_bits = 0
        self.resolves = 0

    def __call__(self, graph_module: GraphModule) -> GraphModule:
        self.call(graph_module)
        self.ensures(graph_module)
        return graph_module

    def call(self, graph_module: GraphModule) -> None:
        graph = graph_module.graph
        _private_operand_chains(graph_module)
        anchors = [n for n in graph.nodes
                   if n.op == "call_function" and packet(n.target) in EVTFuser.supported_targets]
        planned = self.plan_ilp(graph_module, anchors) if self.strategy == "ilp" \
            else self.plan_greedy(graph_module, anchors)
        self.objective_bits = internal_volume_bits(graph_module, planned)
        self.partitions = []
        for names in planned:
            EVTFuser().trace(graph_module, names)
            self.partitions.append(names)

    # -- planning (no graph mutation) ---------------------------------------------
    @staticmethod
    def _accepted(graph_module: GraphModule, names: List[str]) -> bool:
        try:
            EVTFuser().trace(graph_module, names, dry_run=True)
            return True
        except NotImplementedError:
            return False

    def plan_greedy(self, graph_module: GraphModule, anchors: List[Node], share: bool = True) -> List[List[str]]:
        taken: Set[Node] = set()
        planned: List[List[str]] = []
        by_name = {n.name: n for n in graph_module.graph.nodes}
        any_shared = False
        for anchor in anchors:
            if anchor in taken:
                continue
            shared: Set[Node] = set()
            part = _grow(anchor, taken, shared if share else None)
            names = [n.name for n in part]
            if shared and not self._accepted(graph_module, names):
                # the fuser cannot write that vector from this kernel: it stays an input
                part = _grow(anchor, taken)
                names = [n.name for n in part]
                shared = set()
            while EVTFuser.fusible(names, graph_module):
                if self._accepted(graph_module, names):
                    planned.append(names)
                    taken.update(n for n in part if n.name in names)
                    any_shared |= bool(shared)
                    break
                # drop the last epilogue node (never the anchor or its operand permutes)
                if len(names) - 1 <= names.index(anchor.name):
                    break
                names = names[:-1]
        if any_shared and not _quotient_is_acyclic(graph_module.graph, [{by_name[x] for x in names} for names in planned]):
            return self.plan_greedy(graph_module, anchors, share=False)
        return planned

    def plan_ilp(self, graph_module: GraphModule, anchors: List[Node], share: bool = True) -> List[List[str]]:
        from .partitioner import AnchorPartitionILP
        reserved = {}
        for anchor in anchors:
            for p in _mainloop_permutes(anchor, set(reserved)):
                reserved[p] = anchor
        ilp = AnchorPartitionILP(graph_module, anchors, _fusible, reserved)
        dead: Set[Node] = set()            # anchors the fuser refuses even alone
        order = list(graph_module.graph.nodes)
        for self.resolves in range(self.MAX_RESOLVES):
            assign = ilp.solve()
            taken = set(reserved) | set(anchors)
            for s in anchors:
                taken.update(assign[s])
            planned, rejected, any_shared = [], False, False
            for s in anchors:
                if s in dead:
                    continue
                base = {s, *assign[s], *(p for p, a in reserved.items() if a is s)}
                inside, shared = set(base), set()
                _absorb_side_expressions(s, inside, ilp._desc[s], taken, shared if share else None)
                names = [n.name for n in order if n in inside]
                ok = self._accepted(graph_module, names)
                if not ok and shared:
                    # the fuser cannot write that vector from this kernel: it stays an input
                    inside, shared = set(base), set()
                    _absorb_side_expressions(s, inside, ilp._desc[s], taken)
                    names = [n.name for n in order if n in inside]
                    ok = self._accepted(graph_module, names)
                if ok:
                    planned.append(names)
                    taken.update(shared)         # one kernel writes it, the others read it
                    any_shared |= bool(shared)
                elif assign[s]:
                    ilp.ban(assign[s][-1], s)
                    rejected = True
                else:
                    dead.add(s)
            if not rejected:
                if any_shared:
                    by_name = {n.name: n for n in order}
                    if not _quotient_is_acyclic(graph_module.graph, [{by_name[x] for x in names} for names in planned]):
                        return self.plan_ilp(graph_module, anchors, share=False)
                self.ilp = ilp
                return planned
        raise RuntimeError("partitioning did not settle: the fuser kept turning partitions down")

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
    """Refresh tensor_meta after a rewrite without touching data: on the fake
    tensors AOT autograd recorded for the placeholders when there are any (they
    carry the real device, which `_to_copy(..., device=...)` nodes need), else
    on meta tensors shaped like the placeholders."""
    from torch._subclasses.fake_tensor import FakeTensor
    from torch.fx.passes.shape_prop import ShapeProp
    holders = [n for n in module.graph.nodes if n.op == "placeholder"]
    vals = [n.meta.get("val") for n in holders]
    if holders and all(isinstance(v, FakeTensor) for v in vals):
        class _WithVals(ShapeProp):
            # AOT autograd reads meta["val"] of whatever becomes a saved activation
            def run_node(self, n):
                result = super().run_node(n)
                n.meta["val"] = result
                return result
        _WithVals(module, fake_mode=vals[0].fake_mode).propagate(*vals)
        return
    metas = []
    for n in holders:
        tm = n.meta.get("tensor_meta")
        if tm is None:
            return      # no shapes recorded: the caller runs ShapeProp itself
        metas.append(torch.empty(tuple(tm.shape), dtype=tm.dtype, device="meta"))
    ShapeProp(module).propagate(*metas)


def _fold_permutes(graph: Graph) -> bool:
    """permute(permute(x, p), q) -> permute(x, p o q), or x when that is the
    identity (the transposes AOT autograd writes around weights come in such
    pairs; the reference folds them in pass_permute_propagation.py)."""
    changed = False
    for node in list(graph.nodes):
        if node.op != "call_function" or target_name(node.target) != "permute":
            continue
        src = node.args[0]
        if not (isinstance(src, Node) and src.op == "call_function" and target_name(src.target) == "permute"):
            continue
        p, q = [int(i) for i in src.args[1]], [int(i) for i in node.args[1]]
        rank = len(p)
        comp = [p[i % rank] % rank for i in q]
        if comp == list(range(rank)):
            node.replace_all_uses_with(src.args[0])
            graph.erase_node(node)
        else:
            node.args = (src.args[0], comp)
        if not src.users:
            graph.erase_node(src)
        changed = True
    return changed


def _stack_merge_to_cat(graph: Graph) -> bool:
    """stack([x_0 .. x_{n-1}], 0) -> permute -> clone -> view, where the permute
    leaves the stacked axis in front of the axes that the view merges into the
    last one (the gradient of a fused [d, 3d] projection: [3, B, H, S, D] ->
    [B, S, 3, H, D] -> [B * S, 3 * H * D]), is the concatenation along the last
    axis of the x_i, each permuted and merged by itself:
        cat([view(clone(permute(x_i, p')), [..., H * D]) for i], -1).
    One copy (the cat) instead of two (stack, clone), and the per-tensor
    permute / clone / view is a layout chain the producing kernel's store takes
    over."""
    changed = False
    for node in list(graph.nodes):
        if not (node.op == "call_function" and target_name(node.target) == "stack"):
            continue
        tensors = list(node.args[0])
        dim = int(node.args[1]) if len(node.args) > 1 else int(node.kwargs.get("dim", 0))
        if dim != 0 or len(node.users) != 1 or not all(isinstance(t, Node) and "tensor_meta" in t.meta for t in tensors):
            continue
        perm = next(iter(node.users))
        if not (perm.op == "call_function" and target_name(perm.target) == "permute" and len(perm.users) == 1):
            continue
        clone = next(iter(perm.users))
        if not (clone.op == "call_function" and target_name(clone.target) == "clone" and len(clone.users) == 1):
            continue
        view = next(iter(clone.users))
        if not (view.op == "call_function" and target_name(view.target) in ("view", "_unsafe_view", "reshape")):
            continue
        dims = [int(d) for d in perm.args[1]]
        rank = len(dims)
        k = dims.index(0)                        # where the stacked axis lands
        if k == 0 or k == rank - 1:
            continue
        src_shape = [int(x) for x in tensors[0].meta["tensor_meta"].shape]
        if any([int(x) for x in t.meta["tensor_meta"].shape] != src_shape for t in tensors):
            continue
        lead = [src_shape[d - 1] for d in dims[:k]]
        tail = 1
        for d in dims[k + 1:]:
            tail *= src_shape[d - 1]
        out_shape = [int(x) for x in view.args[1]]
        lead_numel = 1
        for x in lead:
            lead_numel *= x
        # the view must merge exactly the stacked axis and what follows it into its last axis
        rest = 1
        for x in out_shape[:-1]:
            rest *= x
        if out_shape[-1] != len(tensors) * tail or rest != lead_numel:
            continue
        sub = [d - 1 for d in dims[:k] + dims[k + 1:]]
        with graph.inserting_before(view):
            parts = []
            for t in tensors:
                p = inherit_meta(graph.call_function(aten.permute, (t, sub)), view)
                c = inherit_meta(graph.call_function(aten.clone, (p,), {"memory_format": torch.contiguous_format}), view)
                parts.append(inherit_meta(graph.call_function(aten.view, (c, out_shape[:-1] + [tail])), view))
            cat = inherit_meta(graph.call_function(aten.cat, (parts, -1)), view)
            for k_ in ("tensor_meta", "val"):
                if k_ in view.meta:
                    cat.meta[k_] = view.meta[k_]
        view.replace_all_uses_with(cat)
        # a sum over the rows of the concatenation (the fused projection's bias gradient) is the concatenation of
        # the parts' sums, and each of those joins the epilogue of the kernel that produces its part
        frontier = [cat]
        while frontier:
            x = frontier.pop()
            for user in list(x.users):
                name_u = target_name(user.target) if user.op == "call_function" else ""
                if name_u in ("view", "_unsafe_view", "reshape") and "tensor_meta" in user.meta \
                        and int(user.meta["tensor_meta"].shape[-1]) == out_shape[-1]:
                    frontier.append(user)            # regroups the rows only
                    continue
                if name_u != "sum" or len(user.args) < 2 or "tensor_meta" not in user.meta:
                    continue
                rank_x = len(x.meta["tensor_meta"].shape) if "tensor_meta" in x.meta else len(out_shape)
                if sorted(int(d) % rank_x for d in user.args[1]) != list(range(rank_x - 1)):
                    continue                         # not a sum over every row
                with graph.inserting_before(user):
                    sums = [inherit_meta(graph.call_function(aten.sum, (p_, list(range(len(out_shape) - 1)), True)), user)
                            for p_ in parts]
                    total = inherit_meta(graph.call_function(aten.cat, (sums, -1)), user)
                    total = inherit_meta(graph.call_function(aten.view, (total, [int(d) for d in user.meta["tensor_meta"].shape])), user)
                    for k_ in ("tensor_meta", "val"):
                        if k_ in user.meta:
                            total.meta[k_] = user.meta[k_]
                user.replace_all_uses_with(total)
        changed = True
    return changed


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

      _log_softmax(x, d, h)          -> log(_softmax(x, d, h))                   (:261-278)
      _log_softmax_backward_data     -> sub(g, mul(sum(g, d, keepdim), softmax)) (:428-446)
      nll_loss_backward (2-D, no weight, sum | mean)
                                     -> mul(mul(neg(one_hot(target)), tangent),
                                            unsqueeze(ne(target, ignore_index), 1)) [/ batch]   (:294-348;
                                        the reference compares with -1 instead of ignore_index)
      masked_fill(x, mask, v)        -> where(mask, v, x)                        (scalar v; not in the reference)
      pow(x, 1)                      -> x                                        (not in the reference)
      getitem(unbind(x, d), i)       -> select(x, d, i)                          (not in the reference)
      add of select_backward(g_i, s, d, i) over every i
                                     -> stack([g_0, g_1, ...], d)                (not in the reference)
      view(clone(permute(stack(xs, 0)))) that merges the stacked axis into the last one
                                     -> cat([view(clone(permute(x))) for x in xs], -1)   (not in the reference)
      native_layer_norm(x, s, w, b, eps)
                                     -> add(mul(native_layer_norm(x, s, None, None, eps)[0], w), b)   (:504-544)
    and permute(permute(x)) folded into one permute or none.  The reference's
    other decompositions (layer / batch norm, convolution, pooling, spmm)
    belong to anchors this backend does not provide and are left untouched."""
    graph = module.graph if graph is None else graph
    disabled = set(disabled_ops)
    changed = False
    for node in list(graph.nodes):
        if node.op != "call_function":
            continue
        name = target_name(node.target)
        if name in disabled:
            continue

        def mk(target, args, kwargs=None, _node=node):
            # nodes of a replacement stand where the replaced node stood, also
            # for the forward/backward split of the joint graph
            return inherit_meta(graph.call_function(target, tuple(args), kwargs or {}), _node)

        new = None
        with graph.inserting_before(node):
            if name == "addmm" and len(node.args) == 3 and not node.kwargs:
                b, x, w = node.args
                new = mk(aten.add, (mk(aten.mm, (x, w)), b))
            elif name == "t":
                new = mk(aten.permute, (node.args[0], [1, 0]))
            elif name == "transpose" and len(node.args) == 3:
                rank = len(node.meta["tensor_meta"].shape)
                dims = list(range(rank))
                i, j = node.args[1] % rank, node.args[2] % rank
                dims[i], dims[j] = j, i
                new = mk(aten.permute, (node.args[0], dims))
            elif name == "_unsafe_view":
                new = mk(aten.view, node.args)
            elif name == "rsub" and len(node.args) == 2 and node.kwargs.get("alpha", 1) == 1:
                new = mk(aten.sub, (node.args[1], node.args[0]))
            elif name == "native_dropout_backward":
                g, m, s = node.args
                new = mk(aten.mul, (mk(aten.mul, (g, m)), s))
            elif name == "threshold_backward":
                g, y, t = node.args
                new = mk(aten.mul, (g, mk(aten.gt, (y, t))))
            elif (name == "pow" and len(node.args) == 2 and isinstance(node.args[0], Node)
                  and type(node.args[1]) in (int, float) and node.args[1] == 1):
                # autograd writes pow(x, 1) into the backward of every x ** 2, and ATen runs it as a copy of x
                new = node.args[0]
            elif name == "masked_fill" and len(node.args) == 3 and isinstance(node.args[2], (int, float)):
                # a fill value under a mask is a select: where(mask, value, x) is in the epilogue vocabulary
                x, mask, value = node.args
                new = mk(aten.where, (mask, float(value), x))
            elif name == "_log_softmax" and len(node.args) == 3:
                x, dim, half_to_float = node.args
                new = mk(aten.log, (mk(aten._softmax, (x, dim, half_to_float)),))
            elif name == "_log_softmax_backward_data" and len(node.args) == 4:
                g, out, dim, _dtype = node.args
                # d log_softmax: g - softmax * sum(g); softmax is at hand when
                # `out` is the log(_softmax(x)) written above, else exp(out)
                if (isinstance(out, Node) and out.op == "call_function" and target_name(out.target) == "log"
                        and isinstance(out.args[0], Node) and target_name(out.args[0].target) == "_softmax"):
                    soft = out.args[0]
                else:
                    soft = mk(aten.exp, (out,))
                total = mk(aten.sum, (g, [dim], True))
                new = mk(aten.sub, (g, mk(aten.mul, (total, soft))))
            elif name == "nll_loss_backward" and len(node.args) == 7 and node.args[3] is None \
                    and node.args[4] in (1, 2) and "tensor_meta" in node.args[1].meta:
                tangent, logp, target, _w, reduction, ignore_index, _total = node.args
                shape = logp.meta["tensor_meta"].shape
                if len(shape) == 2:
                    grad = mk(aten.mul, (mk(aten.neg, (mk(aten.one_hot, (target, int(shape[-1]))),)), tangent))
                    keep = mk(aten.unsqueeze, (mk(aten.ne, (target, ignore_index)), 1))
                    new = mk(aten.mul, (grad, keep))
                    if reduction == 1:       # mean over the batch (labels equal to ignore_index are
                        new = mk(aten.div, (new, int(shape[0])))     # not discounted, as in the reference)
            elif name == "native_layer_norm" and len(node.args) == 5 and (node.args[2] is not None or node.args[3] is not None):
                # weight and bias become epilogue nodes of the normalisation (:504-544)
                x, shape, w, b, eps = node.args
                plain = mk(aten.native_layer_norm, (x, shape, None, None, eps))
                items = {i: mk(operator.getitem, (plain, i)) for i in range(3)}
                y = items[0]
                if w is not None:
                    y = mk(aten.mul, (y, w))
                if b is not None:
                    y = mk(aten.add, (y, b))
                for user in list(node.users):
                    if user.op == "call_function" and user.target is operator.getitem:
                        user.replace_all_uses_with(y if user.args[1] == 0 else items[int(user.args[1])])
                        graph.erase_node(user)
                if not node.users:
                    graph.erase_node(node)
                    changed = True
                continue
            elif name == "add" and len(node.args) == 2 and node.kwargs.get("alpha", 1) == 1:
                # add(add(select_backward(g0, s, d, 0), select_backward(g1, s, d, 1)), ...) over every index of d
                # is stack([g0, g1, ...], d): one copy instead of a zero-filled tensor per slice and the adds
                leaves, ok = [], True

                def collect(x):
                    nonlocal ok
                    if not (isinstance(x, Node) and x.op == "call_function" and len(x.users) == 1) and x is not node:
                        ok = False
                    elif target_name(x.target) == "select_backward":
                        leaves.append(x)
                    elif target_name(x.target) == "add" and len(x.args) == 2 and x.kwargs.get("alpha", 1) == 1:
                        collect(x.args[0])
                        collect(x.args[1])
                    else:
                        ok = False
                collect(node)
                if ok and leaves:
                    shape, dim = list(leaves[0].args[1]), int(leaves[0].args[2])
                    by_index = {int(x.args[3]): x.args[0] for x in leaves
                                if list(x.args[1]) == shape and int(x.args[2]) == dim}
                    if len(by_index) == len(leaves) == shape[dim] and sorted(by_index) == list(range(shape[dim])):
                        new = mk(aten.stack, ([by_index[i] for i in range(shape[dim])], dim))
            elif name == "unbind" and all(u.op == "call_function" and u.target is operator.getitem for u in node.users):
                # getitem(unbind(x, d), i) is select(x, d, i): a layout op the batched products read through
                x = node.args[0]
                dim = int(node.args[1]) if len(node.args) > 1 else int(node.kwargs.get("dim", 0))
                for user in list(node.users):
                    sel = inherit_meta(graph.call_function(aten.select, (x, dim, int(user.args[1]))), user)
                    for k in ("tensor_meta", "val"):
                        if k in user.meta:
                            sel.meta[k] = user.meta[k]
                    user.replace_all_uses_with(sel)
                    graph.erase_node(user)
                graph.erase_node(node)
                changed = True
                continue
            elif name == "native_dropout" and len(node.args) == 3 and node.args[2] is True:
                x, p = node.args[0], node.args[1]
                mask = mk(aten.ge, (mk(torch.rand_like, (x,)), p))
                out = mk(aten.mul, (mk(aten.mul, (x, mask)), 1. / (1 - p)))
                for user in list(node.users):     # getitem(dropout, 0 | 1)
                    if user.op == "call_function" and user.target is operator.getitem:
                        user.replace_all_uses_with(out if user.args[1] == 0 else mask)
                        graph.erase_node(user)
                if not node.users:
                    graph.erase_node(node)
                    changed = True
                continue
        if new is not None:
            for k in ("tensor_meta", "val"):     # same value: later rewrites of this sweep read its shape
                if k in node.meta and k not in new.meta:
                    new.meta[k] = node.meta[k]
            node.replace_all_uses_with(new)
            graph.erase_node(node)
            changed = True
    changed = _fold_permutes(graph) or changed
    if "stack" not in disabled:
        changed = _stack_merge_to_cat(graph) or changed
    if changed:
        graph.eliminate_dead_code()        # what a rewrite replaced piecewise (the adds under a stack, ...)
        graph.lint()
        module.recompile()
        _repropagate(module)
    return module
