"""Joint-graph partitioner for GEMM/BMM epilogues: an integer program that
assigns every fusible node to at most one anchor so that the tensor volume
kept on chip is largest and the fused kernels can still be ordered.

Counterpart of the reference's `ILPSolver` (python/gtl/compiler/passes/
pass_fusion.py:216-983: objective :518-535, one partition per node :541-549,
acyclic quotient graph through partition potentials :586-667, one unfusible
nucleus per partition :684-703, no main-loop fusion besides operand
transposes :760-815, reductions are leaves :817-842) restricted to the
partitions this backend lowers: one mm/bmm nucleus plus its epilogue.

Because every partition here is "an anchor and nodes downstream of it", the
program is indexed by anchor instead of by anonymous partition slots, which
removes the slot symmetry the reference breaks with (2.8)/(2.13):

    x[j,s] in {0,1}     node j is computed in the epilogue of anchor s;
                        only exists for j in R(s), the nodes reachable from s
                        through fusible nodes
    p[v]   in [0,n]     topological potential of graph node v

    max   sum_{s, j in R(s)}  x[j,s] * w(j,s)
          w(j,s) = bits of every operand of j that is s or lies in R(s)
                   (the edges that stop going through HBM, :288-313)
    s.t.  sum_s x[j,s] <= 1
          x[j,s] <= x[i,s]        for each operand i of j downstream of s
                                  (a partition is closed under paths from its
                                  anchor, so edge i->j is internal iff x[j,s])
          x[g,s]  = x[r,s]        g a getitem of a multi-output reduction r
          p[j] - p[i] + sum_s x[j,s][i in R(s)+s] >= 1     for each edge i->j
          |p[j] - p[s]| <= n (1 - x[j,s])                  (partitions share a potential)

The reference makes reductions leaves of their partition (:817-842); the
epilogue here also evaluates per-row and per-column expressions of finished
reductions (logsumexp minus a gathered logit, say), so R(s) keeps their users,
and what the epilogue cannot express is found by the fuser's dry run: the
caller bans that (node, anchor) pair and solves again.  Solved with scipy's HiGHS front
end (`scipy.optimize.milp`), as the reference does (:936-983).
"""
from __future__ import annotations

import hashlib
import json
import os
import sqlite3
from typing import Dict, List, Optional, Sequence, Set, Tuple

import numpy as np
import torch
from torch.fx import GraphModule, Node

from .evt_fuser import EVTFuser, packet, target_name

aten = torch.ops.aten

MULTI_OUTPUT = {"var_mean"}

_DTYPE_BITS = {torch.float16: 16, torch.bfloat16: 16, torch.float32: 32, torch.float64: 64, torch.bool: 8,
               torch.uint8: 8, torch.int8: 8, torch.int16: 16, torch.int32: 32, torch.int64: 64}


def _volume_bits(node: Node, index: Optional[int] = None) -> int:
    """Bits of the tensor a node produces (entry `index` of a tuple result);
    the edge weight of pass_fusion.py:288-313."""
    tm = node.meta.get("tensor_meta")
    if tm is None:
        val = node.meta.get("val")
        if isinstance(val, torch.Tensor):
            return int(val.numel()) * _DTYPE_BITS.get(val.dtype, 32)
        return 0
    if not hasattr(tm, "shape"):
        if index is None:
            return sum(_volume_bits_meta(t) for t in tm)
        tm = tm[index]
    return _volume_bits_meta(tm)


def _volume_bits_meta(tm) -> int:
    n = 1
    for d in tm.shape:
        n *= int(d)
    return n * _DTYPE_BITS.get(tm.dtype, 32)


def same_phase(node: Node, anchor: Node) -> bool:
    """In a joint forward/backward graph a kernel belongs to one side: a
    forward anchor that took a backward node into its epilogue would make the
    forward results wait for the incoming gradients.  AOT autograd tags every
    node of a joint graph; graphs without tags have one phase."""
    a, b = node.meta.get("partitioner_tag"), anchor.meta.get("partitioner_tag")
    return a is None or b is None or a == b


class PartitionCache:
    """Solved instances keyed by a digest of the program, in sqlite when
    `EVT_PARTITION_CACHE` names a file (the reference keeps its solutions in the
    `partitions` table of its cache file, pass_fusion.py:87-156), else in a
    dictionary that lives as long as the process."""

    _memory: Dict[str, List[List[int]]] = {}

    def __init__(self, path: Optional[str] = None) -> None:
        self.path = path if path is not None else os.environ.get("EVT_PARTITION_CACHE")
        if self.path:
            with self._connect() as con:
                con.execute("CREATE TABLE IF NOT EXISTS partitions (hash TEXT PRIMARY KEY, assignment TEXT NOT NULL)")

    def _connect(self) -> sqlite3.Connection:
        return sqlite3.connect(self.path, timeout=30)

    def fetch(self, key: str) -> Optional[List[List[int]]]:
        if not self.path:
            return self._memory.get(key)
        with self._connect() as con:
            row = con.execute("SELECT assignment FROM partitions WHERE hash = ?", (key,)).fetchone()
        return json.loads(row[0]) if row else None

    def insert(self, key: str, assignment: List[List[int]]) -> None:
        if not self.path:
            self._memory[key] = assignment
            return
        with self._connect() as con:
            con.execute("INSERT OR REPLACE INTO partitions (hash, assignment) VALUES (?, ?)",
                        (key, json.dumps(assignment)))


class AnchorPartitionILP:
    """Builds and solves the program above for one fx graph.

    `fusible(node)` says whether an epilogue may hold the node at all;
    `reserved` are nodes already claimed outside the program (operand
    transposes fused into an anchor's main loop): they are candidates for no
    epilogue and share their anchor's potential.
    """

    def __init__(self, graph_module: GraphModule, anchors: Sequence[Node], fusible,
                 reserved: Optional[Dict[Node, Node]] = None, cache: Optional[PartitionCache] = None) -> None:
        self.gm = graph_module
        self.nodes: List[Node] = [n for n in graph_module.graph.nodes if n.op == "call_function"]
        self.index = {n: i for i, n in enumerate(self.nodes)}
        self.anchors = list(anchors)
        self.anchor_set = set(self.anchors)
        self.fusible = fusible
        self.reserved = dict(reserved or {})
        self.cache = cache if cache is not None else PartitionCache()
        self.banned: Set[Tuple[Node, Node]] = set()      # (node, anchor) pairs the fuser rejected
        self.last_objective: Optional[float] = None
        self.last_from_cache = False
        self._desc = {s: self._descendants(s) for s in self.anchors}

    # -- candidate sets -------------------------------------------------------------
    @staticmethod
    def _descendants(anchor: Node) -> Set[Node]:
        seen, work = set(), [anchor]
        while work:
            n = work.pop()
            for u in n.users:
                if u not in seen:
                    seen.add(u)
                    work.append(u)
        return seen

    def ban(self, node: Node, anchor: Node) -> None:
        self.banned.add((node, anchor))

    def candidates(self, s: Node) -> List[Node]:
        """R(s): downstream nodes an epilogue of `s` could hold, in graph order."""
        desc = self._desc[s]
        inside: Set[Node] = {s}
        order: List[Node] = []
        for j in self.nodes:                      # graph order is topological
            if j not in desc or j in self.anchor_set or j in self.reserved or not self.fusible(j):
                continue
            if (j, s) in self.banned or not same_phase(j, s):
                continue
            ins = j.all_input_nodes
            if not any(i in inside for i in ins):
                continue
            # every operand downstream of the anchor must be inside as well
            if any((i in desc) and (i not in inside) for i in ins):
                continue
            name = target_name(j.target)
            ok = True
            for i in ins:
                if i in inside and i is not s and target_name(i.target) in MULTI_OUTPUT:
                    ok = ok and name == "getitem"          # only its getitems follow
            if name == "getitem" and j.args[0] not in inside:
                ok = False
            if ok:
                inside.add(j)
                order.append(j)
        # a multi-output reduction needs every getitem inside, or stays outside
        for r in [n for n in order if target_name(n.target) in MULTI_OUTPUT]:
            if not all(u in inside for u in r.users):
                for u in [r] + list(r.users):
                    if u in inside:
                        inside.discard(u)
                        order.remove(u)
        return order

    # -- the program ------------------------------------------------------------------
    def _build(self):
        R = {s: self.candidates(s) for s in self.anchors}
        xvar: Dict[Tuple[Node, Node], int] = {}
        for s in self.anchors:
            for j in R[s]:
                xvar[(j, s)] = len(xvar)
        nx_ = len(xvar)
        n = len(self.nodes)
        nvar = nx_ + n
        pv = lambda v: nx_ + self.index[v]

        c = np.zeros(nvar)
        rows: List[Dict[int, float]] = []
        lb: List[float] = []
        ub: List[float] = []

        def add(row, lo, hi):
            rows.append(row)
            lb.append(lo)
            ub.append(hi)

        by_node: Dict[Node, List[Node]] = {}
        for s in self.anchors:
            inside = set(R[s]) | {s}
            desc = self._desc[s]
            for j in R[s]:
                by_node.setdefault(j, []).append(s)
                w = 0
                for i in j.all_input_nodes:
                    if i not in inside:
                        continue
                    idx = j.args[1] if target_name(j.target) == "getitem" else None
                    w += _volume_bits(i, idx)
                    if i is not s:
                        add({xvar[(j, s)]: 1.0, xvar[(i, s)]: -1.0}, -np.inf, 0.0)       # closure
                c[xvar[(j, s)]] = -float(w)
                if target_name(j.target) == "getitem" and target_name(j.args[0].target) in MULTI_OUTPUT:
                    add({xvar[(j, s)]: 1.0, xvar[(j.args[0], s)]: -1.0}, 0.0, 0.0)
                # members share the anchor's potential
                add({pv(j): 1.0, pv(s): -1.0, xvar[(j, s)]: float(n)}, -np.inf, float(n))
                add({pv(s): 1.0, pv(j): -1.0, xvar[(j, s)]: float(n)}, -np.inf, float(n))
        for j, owners in by_node.items():
            if len(owners) > 1:
                add({xvar[(j, s)]: 1.0 for s in owners}, -np.inf, 1.0)

        # order: every edge climbs one potential level unless it is internal
        for j in self.nodes:
            for i in j.all_input_nodes:
                if i not in self.index:
                    continue
                if self.reserved.get(i) is j:
                    add({pv(j): 1.0, pv(i): -1.0}, 0.0, 0.0)
                    continue
                row = {pv(j): 1.0, pv(i): -1.0}
                for s in by_node.get(j, ()):
                    if i is s or (i, s) in xvar:
                        row[xvar[(j, s)]] = row.get(xvar[(j, s)], 0.0) + 1.0
                add(row, 1.0, np.inf)

        # objective in units of the greatest common divisor, as the reference labels edges (:428-436)
        g = 0
        for v in c[:nx_]:
            g = int(np.gcd(g, int(-v)))
        if g > 1:
            c[:nx_] /= g
        self._scale = max(g, 1)
        return R, xvar, c, rows, lb, ub, nx_, nvar

    def _digest(self, R, xvar, c, rows, lb, ub) -> str:
        h = hashlib.sha1()
        h.update(json.dumps([[self.index[j], self.index[s]] for (j, s) in xvar]).encode())
        h.update(np.asarray(c).tobytes())
        h.update(json.dumps([sorted(r.items()) for r in rows]).encode())
        h.update(np.asarray(lb).tobytes() + np.asarray(ub).tobytes())
        h.update(json.dumps([target_name(n.target) for n in self.nodes]).encode())
        return h.hexdigest()

    def solve(self) -> Dict[Node, List[Node]]:
        """anchor -> epilogue nodes (graph order)."""
        from scipy.optimize import Bounds, LinearConstraint, milp
        from scipy.sparse import csr_matrix

        R, xvar, c, rows, lb, ub, nx_, nvar = self._build()
        if nx_ == 0:
            self.last_objective = 0.0
            return {s: [] for s in self.anchors}
        key = self._digest(R, xvar, c, rows, lb, ub)
        pairs = list(xvar)
        cached = self.cache.fetch(key)
        self.last_from_cache = cached is not None
        if cached is not None:
            chosen = [tuple(p) for p in cached]
        else:
            data, ri, ci = [], [], []
            for r, row in enumerate(rows):
                for col, v in row.items():
                    ri.append(r)
                    ci.append(col)
                    data.append(v)
            A = csr_matrix((data, (ri, ci)), shape=(len(rows), nvar))
            integrality = np.concatenate([np.ones(nx_), np.zeros(nvar - nx_)])
            n = len(self.nodes)
            bounds = Bounds(np.zeros(nvar), np.concatenate([np.ones(nx_), np.full(nvar - nx_, float(n))]))
            res = milp(c, constraints=LinearConstraint(A, np.asarray(lb), np.asarray(ub)),
                       integrality=integrality, bounds=bounds)
            if not res.success:
                raise RuntimeError(f"partition program not solved: {res.message}")
            chosen = [(self.index[j], self.index[s]) for k, (j, s) in enumerate(pairs) if res.x[k] > 0.5]
            self.cache.insert(key, [list(p) for p in chosen])
        out: Dict[Node, List[Node]] = {s: [] for s in self.anchors}
        obj = 0.0
        for (ji, si) in chosen:
            j, s = self.nodes[ji], self.nodes[si]
            out[s].append(j)
            obj += -c[xvar[(j, s)]] * self._scale
        for s in out:
            out[s].sort(key=self.index.__getitem__)
        self.last_objective = obj
        return out
