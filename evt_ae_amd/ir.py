"""Epilogue-visitor-tree IR for the MI355X backend.

The reference builds its epilogue DAG through the un-vendored CUTLASS Python
package (`EVTFrontendBase.add_load_node / add_compute_node / add_store_node /
add_layout_node`, used at python/gtl/compiler/passes/evt_fuser.py:1323-1485) and
lets its pass manager classify every load as AuxLoad / RowBroadcast /
ColumnBroadcast / Scalar and every store as AuxStore / RowReduction /
ColumnReduction from broadcast shapes (class names at
python/gtl/compiler/autotuner/tuner_base.py:120-152).  That package is absent,
so this module is a re-derivation with the same vocabulary:

  * every value of the tree is evaluated once per element (l, m, n) of the
    accumulator's [L, M, N] iteration space, in fp32;
  * layout ops (view / permute / unsqueeze / squeeze / clone) never move data:
    they only change how a tensor's logical index is derived from (l, m, n).
    `Coord` carries that mapping as a vectorised integer function, and
    `fit_strides` turns it into the (stride_l, stride_m, stride_n, l_div)
    addressing the kernels use, verifying the fit on random probes;
  * reductions produce per-row ([L, M]) or per-column ([L, N]) values that may
    be post-processed by a small per-row / per-column expression graph.
"""
from __future__ import annotations

import hashlib
import json
from dataclasses import dataclass, field, replace
from typing import Callable, Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

# --------------------------------------------------------------------------
# coordinate functions
# --------------------------------------------------------------------------


class Coord:
    """Maps iteration-space coordinates to a logical flat index of a tensor.

    `fn(l, m, n)` takes int64 numpy arrays and returns the row-major flat index,
    in `shape`, of the element of this tensor that takes part in computing
    output element (l, m, n).
    """

    def __init__(self, shape: Sequence[int], fn: Callable):
        self.shape = tuple(int(s) for s in shape)
        self.fn = fn

    def numel(self) -> int:
        n = 1
        for s in self.shape:
            n *= s
        return n

    # -- layout transformations (consumer-side view of the same data) -------
    def reshape(self, new_shape: Sequence[int]) -> "Coord":
        new_shape = _resolve_shape(new_shape, self.numel())
        return Coord(new_shape, self.fn)

    def permute(self, dims: Sequence[int]) -> "Coord":
        old_shape = self.shape
        dims = [d % len(old_shape) for d in dims]
        new_shape = tuple(old_shape[d] for d in dims)
        old_fn = self.fn

        def fn(l, m, n):
            idx = np.unravel_index(old_fn(l, m, n), old_shape) if old_shape else ()
            new_idx = tuple(idx[d] for d in dims)
            return np.ravel_multi_index(new_idx, new_shape) if new_shape else np.zeros_like(l)

        return Coord(new_shape, fn)

    # -- producer-side: index of an operand that is broadcast to `self` -----
    def restrict(self, small_shape: Sequence[int]) -> "Coord":
        """Coordinate function of an operand of shape `small_shape` that is
        broadcast (numpy rules) against a tensor indexed by `self`."""
        big_shape = self.shape
        small_shape = tuple(int(s) for s in small_shape)
        if len(small_shape) > len(big_shape):
            # leading 1s may be dropped on the big side
            extra = len(small_shape) - len(big_shape)
            if any(s != 1 for s in small_shape[:extra]):
                raise NotImplementedError(
                    f"operand of shape {small_shape} is larger than the accumulator view {big_shape}")
            small_shape = small_shape[extra:]
        pad = len(big_shape) - len(small_shape)
        padded = (1,) * pad + small_shape
        for b, s in zip(big_shape, padded):
            if s != 1 and s != b:
                raise NotImplementedError(f"cannot broadcast {small_shape} to {big_shape}")
        big_fn = self.fn

        def fn(l, m, n):
            idx = np.unravel_index(big_fn(l, m, n), big_shape) if big_shape else ()
            sidx = tuple(np.zeros_like(i) if s == 1 else i for i, s in zip(idx, padded))
            return np.ravel_multi_index(sidx, padded) if padded else np.zeros_like(l)

        return Coord(small_shape, fn)

    def inverse_permute(self, dims: Sequence[int], src_shape: Sequence[int]) -> "Coord":
        """`self` indexes permute(src, dims); return the index into src."""
        src_shape = tuple(int(s) for s in src_shape)
        dims = [d % len(src_shape) for d in dims]
        my_shape = self.shape
        my_fn = self.fn

        def fn(l, m, n):
            idx = np.unravel_index(my_fn(l, m, n), my_shape)
            sidx = [None] * len(dims)
            for pos, d in enumerate(dims):
                sidx[d] = idx[pos]
            return np.ravel_multi_index(tuple(sidx), src_shape)

        return Coord(src_shape, fn)

    def inverse_select(self, dim: int, index: int, src_shape: Sequence[int]) -> "Coord":
        """`self` indexes select(src, dim, index); return the index into src."""
        src_shape = tuple(int(s) for s in src_shape)
        dim = dim % len(src_shape)
        index = index % src_shape[dim]
        my_shape = self.shape
        my_fn = self.fn

        def fn(l, m, n):
            flat = my_fn(l, m, n)
            idx = list(np.unravel_index(flat, my_shape)) if my_shape else []
            idx.insert(dim, np.full_like(flat, index))
            return np.ravel_multi_index(tuple(idx), src_shape)

        return Coord(src_shape, fn)

    def reduce(self, dims: Sequence[int], keepdim: bool) -> "Coord":
        """Index of the reduction result element that (l, m, n) contributes to."""
        shape = self.shape
        dims = sorted(d % len(shape) for d in dims)
        kept = tuple(1 if i in dims else s for i, s in enumerate(shape))
        out_shape = kept if keepdim else tuple(s for i, s in enumerate(shape) if i not in dims)
        my_fn = self.fn

        def fn(l, m, n):
            idx = np.unravel_index(my_fn(l, m, n), shape)
            ridx = tuple(np.zeros_like(i) if d in dims else i for d, i in enumerate(idx))
            return np.ravel_multi_index(ridx, kept)

        return Coord(out_shape, fn)


def _resolve_shape(shape, numel):
    shape = [int(s) for s in shape]
    if -1 in shape:
        known = 1
        for s in shape:
            if s != -1:
                known *= s
        shape[shape.index(-1)] = numel // max(known, 1)
    return tuple(shape)


def accum_coord(L: int, M: int, N: int, batched: bool) -> Coord:
    if batched:
        return Coord((L, M, N), lambda l, m, n: (l * M + m) * N + n)
    return Coord((M, N), lambda l, m, n: m * N + n)


@dataclass
class Strides:
    """offset(l, m, n) = (lb // l_div) * stride_l + (lb % l_div) * stride_l2 + m * stride_m + n * stride_n,
    lb = l % l_mod if l_mod else l."""
    stride_l: int
    stride_m: int
    stride_n: int
    l_div: int = 1
    l_mod: int = 0       # > 0: the batch index enters modulo l_mod (batches l and l + l_mod share elements)
    # batch index in two levels, l = outer * l_div + inner (a [B, S, H, D] tensor against L = B * H batches of
    # [S, D]): stride of the inner level; 0: the l_div consecutive batches share elements
    stride_l2: int = 0
    # operands only: elements in front of element (0, 0, 0) (a `select` of a larger tensor)
    base: int = 0

    def batch_index(self, l):
        lb = l % self.l_mod if self.l_mod else l
        return lb // self.l_div

    def batch_offset(self, l):
        lb = l % self.l_mod if self.l_mod else l
        return (lb // self.l_div) * self.stride_l + (lb % self.l_div) * self.stride_l2

    @property
    def kind(self) -> str:
        """Load classification, in the reference's terms
        (tuner_base.py:120-152): 'scalar', 'row' = RowBroadcast (an [N]
        vector), 'col' = ColumnBroadcast (an [M] vector), 'aux' = AuxLoad."""
        if self.stride_m == 0 and self.stride_n == 0 and self.stride_l == 0:
            return "scalar"
        if self.stride_m == 0 and self.stride_n != 0:
            return "row"
        if self.stride_n == 0:
            return "col"
        return "aux"


def fit_strides(coord: Coord, L: int, M: int, N: int, elem_strides: Optional[Sequence[int]] = None,
                seed: int = 0, allow_base: bool = False) -> Optional[Strides]:
    """Fit  offset(l, m, n) = (lb // l_div) * sl + (lb % l_div) * sl2 + m * sm + n * sn,
    lb = l % l_mod (or l), to `coord`.

    `elem_strides` are the memory strides of the tensor (default: contiguous).
    Returns None when the mapping is not of that form (checked on the corners,
    the unit steps, a few thousand random points and every point of the lines
    along l, m and n through six anchors)."""
    shape = coord.shape
    if elem_strides is None:
        elem_strides = []
        acc = 1
        for s in reversed(shape):
            elem_strides.append(acc)
            acc *= s
        elem_strides = tuple(reversed(elem_strides))

    def raw_offset(l, m, n):
        flat = coord.fn(np.asarray(l, dtype=np.int64), np.asarray(m, dtype=np.int64),
                        np.asarray(n, dtype=np.int64))
        if not shape:
            return np.zeros_like(flat)
        idx = np.unravel_index(flat, shape)
        off = np.zeros_like(flat)
        for i, s in zip(idx, elem_strides):
            off = off + i * s
        return off

    z = np.zeros(1, dtype=np.int64)
    base = int(raw_offset(z, z, z)[0])
    if base != 0 and not allow_base:
        return None

    def offset(l, m, n):
        return raw_offset(l, m, n) - base
    sm = int(offset(z, z + 1, z)[0]) if M > 1 else 0
    sn = int(offset(z, z, z + 1)[0]) if N > 1 else 0
    rng = np.random.default_rng(seed)
    npts = 4096
    pl = rng.integers(0, L, npts)
    pm = rng.integers(0, M, npts)
    pn = rng.integers(0, N, npts)
    # always include the far corner
    pl[0], pm[0], pn[0] = L - 1, M - 1, N - 1
    # ... and whole lines along each axis through a few anchors (the corners and two random points), so that a
    # mapping that leaves the affine form only in a late column / row / batch cannot slip through the sample:
    # O(L + M + N) points
    anchors = [(0, 0, 0), (L - 1, M - 1, N - 1), (L - 1, 0, N - 1), (0, M - 1, 0),
               (int(pl[1]), int(pm[1]), int(pn[1])), (int(pl[2]), int(pm[2]), int(pn[2]))]
    ll, mm, nn = [pl], [pm], [pn]
    for al, am, an in anchors:
        for axis, size in ((0, L), (1, M), (2, N)):
            line = np.arange(size, dtype=np.int64)
            ll.append(line if axis == 0 else np.full(size, al, dtype=np.int64))
            mm.append(line if axis == 1 else np.full(size, am, dtype=np.int64))
            nn.append(line if axis == 2 else np.full(size, an, dtype=np.int64))
    pl, pm, pn = np.concatenate(ll), np.concatenate(mm), np.concatenate(nn)
    want = offset(pl, pm, pn)

    def fits(st: Strides) -> bool:
        return np.array_equal(want, st.batch_offset(pl) + pm * sm + pn * sn)

    if L == 1:
        st = Strides(0, sm, sn, base=base)
        return st if fits(st) else None
    ls = np.arange(L, dtype=np.int64)
    offs = offset(ls, np.zeros_like(ls), np.zeros_like(ls))
    # one level: l_div consecutive batches share elements, then sl per group; possibly periodic in l
    sl, l_div, l_mod = 0, 1, 0
    nz = np.nonzero(offs)[0]
    if len(nz):
        l_div = int(nz[0])
        sl = int(offs[l_div])
        # periodic in l: the smallest period that divides L (a full period is no period)
        for period in range(l_div + 1, L):
            if L % period == 0 and np.array_equal(offs, offs[ls % period]):
                l_mod = period
                break
    st = Strides(sl, sm, sn, l_div, l_mod, base=base)
    if fits(st):
        return st
    # two levels: sl2 per batch until, at l = l_div, the offset jumps to sl
    step = int(offs[1])
    brk = np.nonzero(offs != ls * step)[0]
    if len(brk) and step:
        l_div = int(brk[0])
        st = Strides(int(offs[l_div]), sm, sn, l_div, 0, step, base)
        if L % l_div == 0 and fits(st):
            return st
    return None


# --------------------------------------------------------------------------
# DAG
# --------------------------------------------------------------------------

# elementwise ops: name -> arity
ELEMENTWISE = {
    "add": 2, "sub": 2, "mul": 2, "div": 2, "max": 2, "min": 2,
    "neg": 1, "exp": 1, "log": 1, "sqrt": 1, "rsqrt": 1, "abs": 1, "rcp": 1,
    "gelu_tanh": 1, "gelu_erf": 1, "tanh": 1, "relu": 1, "sigmoid": 1,
    "tanh_backward": 2, "gelu_backward_tanh": 2, "gelu_backward_erf": 2,
    "ge": 2, "gt": 2, "le": 2, "lt": 2, "ne": 2, "eq": 2,
    "cast_f16": 1, "cast_bf16": 1, "cast_f32": 1, "cast_bool": 1, "cast_int": 1,
    "where": 3,
}

# reduction kinds: name -> state components
REDUCE_STATE = {"sum": 1, "max": 1, "maxsumexp": 2, "welford": 3}

DTYPE_NAMES = {
    torch.float16: "f16", torch.bfloat16: "bf16", torch.float32: "f32",
    torch.bool: "bool", torch.int32: "i32", torch.int64: "i64", torch.uint8: "u8",
}
DTYPE_CTYPES = {
    "f16": "evt::f16", "bf16": "evt::bf16", "f32": "float", "bool": "bool",
    "i32": "int32_t", "i64": "int64_t", "u8": "uint8_t",
}


@dataclass
class Slot:
    """One tensor argument of the fused kernel (an EvtTensorArg at run time)."""
    name: str            # name of the fx node that is loaded / produced
    role: str            # 'load' | 'store'
    dtype: str           # key of DTYPE_CTYPES
    domain: str          # 'tile' | 'row' | 'col' : where it is accessed; stores also 'nvec' (see Store)
    kind: str            # loads: 'aux' | 'row' | 'col' | 'scalar' | 'rand' (no storage: generated); stores: 'aux' | 'row' | 'col'
    strides: Strides
    shape: Tuple[int, ...] = ()


@dataclass
class Node:
    name: str
    op: str                      # 'accum' | 'load' | 'imm' | 'colidx' | elementwise | 'rres'
    inputs: List[str] = field(default_factory=list)
    domain: str = "tile"         # 'tile' | 'row' | 'col' | 'const'
    slot: Optional[int] = None   # loads
    value: Optional[float] = None          # imm
    reduce: Optional[str] = None           # rres: name of the Reduce
    comp: int = 0                          # rres: state component


@dataclass
class Reduce:
    name: str
    kind: str            # key of REDUCE_STATE
    axis: str            # 'row' (over n, one value per row) | 'col' (over m, one per column)
    input: str
    state_offset: int = 0
    # a per-row reduction may also fold batches: 'mod' -> batches l, l + fold_step, ... (fold_count of them)
    # share one result (keyed by l % fold_step); 'div' -> fold_count consecutive batches do (keyed by l // fold_count)
    fold: str = ""
    fold_step: int = 1
    fold_count: int = 1


@dataclass
class Store:
    slot: int
    input: str
    # 'tile' | 'row' (one value per row: a reduction along the row) | 'col' (one per column: a reduction over the
    # rows) | 'nvec' (one per column, formed from [N] vectors and scalars alone: the reference's row store,
    # visitor_store.hpp:46-145 -- written once per batch by the tiles that hold row 0)
    domain: str


class EpilogueIR:
    """Topologically ordered epilogue DAG plus its tensor slots."""

    def __init__(self, L: int, M: int, N: int, batched: bool):
        self.L, self.M, self.N, self.batched = L, M, N, batched
        self.nodes: Dict[str, Node] = {}
        self.slots: List[Slot] = []
        self.reduces: Dict[str, Reduce] = {}
        self.stores: List[Store] = []
        self.scalars: List[float] = []
        self.rng_scalar: Optional[int] = None    # first of the four scalars that carry the rand_like seed / offset
        self.anchor_scalar: Optional[int] = None  # scalar that carries a row-wise anchor's own constant (layer norm eps)
        self.anchor_slots: List[int] = []         # load slots the anchor itself reads (layer norm backward: mean, rstd)
        self._imm_count = 0

    # -- construction -------------------------------------------------------
    def add_node(self, node: Node) -> Node:
        if node.name in self.nodes:
            raise ValueError(f"duplicate node {node.name}")
        self.nodes[node.name] = node
        return node

    def add_imm(self, value: float) -> str:
        name = f"imm_{self._imm_count}"
        self._imm_count += 1
        # immediates travel as run-time scalars so one module serves any value
        self.scalars.append(float(value))
        self.add_node(Node(name, "imm", domain="const", value=float(value), slot=len(self.scalars) - 1))
        return name

    def add_slot(self, slot: Slot) -> int:
        self.slots.append(slot)
        return len(self.slots) - 1

    def add_rand(self, name: str, strides: Strides, shape: Tuple[int, ...]) -> str:
        """Uniform [0, 1) numbers shaped like a tensor of `shape` (rand_like): a
        load slot without storage whose strides give the element index that
        seeds the generator.  The seed and the per-call offset travel as four
        run-time scalars (32-bit patterns), reserved once per module."""
        if self.rng_scalar is None:
            self.rng_scalar = len(self.scalars)
            self.scalars += [0.0, 0.0, 0.0, 0.0]
        k = self.add_slot(Slot(name, "load", "f32", "tile", "rand", strides, tuple(shape)))
        self.add_node(Node(name, "load", domain="tile", slot=k))
        return name

    def add_anchor_scalar(self, value: float) -> int:
        self.anchor_scalar = len(self.scalars)
        self.scalars.append(float(value))
        return self.anchor_scalar

    def domain_of(self, names: Sequence[str]) -> str:
        """Join of operand domains.

        const (immediates) < flex (anything computed from loads only) <
        tile | row | col.  A per-element value that consumes a reduction
        result is 'bad': legal to build (the softmax-statistics rewrite removes
        such nodes) but an error if still live at `finalize`."""
        doms = {self.nodes[n].domain for n in names}
        if "bad" in doms:
            return "bad"
        doms -= {"const"}
        if not doms:
            return "const"
        doms -= {"flex"}
        if not doms:
            return "flex"
        if len(doms) > 1:
            return "bad"
        return doms.pop()

    def add_compute(self, name: str, op: str, inputs: Sequence[str]) -> Node:
        if op not in ELEMENTWISE:
            raise NotImplementedError(f"unsupported elementwise op {op}")
        if len(inputs) != ELEMENTWISE[op]:
            raise ValueError(f"{op} expects {ELEMENTWISE[op]} operands, got {len(inputs)}")
        return self.add_node(Node(name, op, list(inputs), self.domain_of(inputs)))

    def add_reduce(self, name: str, kind: str, axis: str, input: str) -> Reduce:
        r = Reduce(name, kind, axis, input)
        self.reduces[name] = r
        return r

    # -- analysis -------------------------------------------------------------
    def live_nodes(self) -> List[str]:
        """Nodes reachable from stores (through reductions), in insertion order."""
        live = set()
        work = [s.input for s in self.stores]
        while work:
            n = work.pop()
            if n in live:
                continue
            live.add(n)
            node = self.nodes[n]
            work.extend(node.inputs)
            if node.op == "rres":
                work.append(self.reduces[node.reduce].input)
        return [n for n in self.nodes if n in live]

    def live_reduces(self) -> List[Reduce]:
        live = set(self.live_nodes())
        used = {self.nodes[n].reduce for n in live if self.nodes[n].op == "rres"}
        return [r for r in self.reduces.values() if r.name in used]

    # -- transposed problems ---------------------------------------------------
    def wants_transpose(self) -> bool:
        """True when every full-tensor access of the epilogue is strided along n and
        the stores are unit-stride along m: the output is column-major, and
        computing C^T = B^T A^T instead gives the kernel unit-stride (vector,
        check-free) accesses.  The counterpart of the reference's `transposed`
        problems (python/gtl/compiler/passes/evt_fuser.py:573-596)."""
        if self.M <= 1 or self.N <= 1:
            return False
        tile = [s for s in self.slots if s.domain == "tile" and s.kind == "aux"]
        stores = [s for s in tile if s.role == "store"]
        if not stores:
            return False
        if any(n.op == "colidx" for n in self.nodes.values()):
            return False            # there is no row-index value to take its place
        if any(st.domain == "nvec" for st in self.stores):
            return False            # a per-column vector store has no per-row counterpart
        for r in self.reduces.values():
            if r.axis == "row" and (r.kind not in ("sum", "max") or r.fold == "div"):
                return False        # per-column reductions are sums and maxima, folded modulo only
        return all(s.strides.stride_n != 1 for s in tile) and all(s.strides.stride_m == 1 for s in stores)

    def transpose(self) -> None:
        """Exchange the roles of m and n everywhere: the IR then describes the
        epilogue of the transposed product (call finalize() again afterwards)."""
        swap = {"row": "col", "col": "row"}
        self.M, self.N = self.N, self.M
        for s in self.slots:
            s.strides = replace(s.strides, stride_m=s.strides.stride_n, stride_n=s.strides.stride_m)
            s.domain = swap.get(s.domain, s.domain)
            s.kind = swap.get(s.kind, s.kind)
        for n in self.nodes.values():
            n.domain = swap.get(n.domain, n.domain)
        for r in self.reduces.values():
            r.axis = swap[r.axis]
        for st in self.stores:
            st.domain = swap.get(st.domain, st.domain)

    def finalize(self) -> None:
        """Dead-code elimination, state packing, validation."""
        live = self.live_nodes()
        self.nodes = {n: self.nodes[n] for n in live}
        reds = {}
        row_off = col_off = 0
        for r in self.reduces.values():
            used = any(n.op == "rres" and n.reduce == r.name for n in self.nodes.values())
            if not used:
                continue
            if r.axis == "row":
                r.state_offset = row_off
                row_off += REDUCE_STATE[r.kind]
            else:
                r.state_offset = col_off
                col_off += REDUCE_STATE[r.kind]
            reds[r.name] = r
        self.reduces = reds
        self.row_state, self.col_state = row_off, col_off
        # drop unused slots (e.g. loads that only fed dead nodes), keep order
        used_slots = sorted({n.slot for n in self.nodes.values() if n.op == "load"} |
                            {s.slot for s in self.stores} | set(self.anchor_slots))
        remap = {old: new for new, old in enumerate(used_slots)}
        self.slots = [self.slots[i] for i in used_slots]
        for n in self.nodes.values():
            if n.op == "load":
                n.slot = remap[n.slot]
        for s in self.stores:
            s.slot = remap[s.slot]
        self.anchor_slots = [remap[k] for k in self.anchor_slots]
        # validation
        for n in self.nodes.values():
            if n.domain == "bad":
                raise NotImplementedError(
                    f"node {n.name} mixes per-element values with reduction results; only the "
                    "softmax-statistics pattern (amax -> sub -> exp -> sum) is fused")
        for r in self.reduces.values():
            if self.nodes[r.input].domain not in ("tile", "flex", "const"):
                raise NotImplementedError("reduction of a reduction result")
            if r.axis == "col" and r.kind not in ("sum", "max"):
                raise NotImplementedError(f"per-column {r.kind} reduction")
        for s in self.stores:
            have = self.nodes[s.input].domain
            if have != ("flex" if s.domain == "nvec" else s.domain):
                raise NotImplementedError(
                    f"store of {s.input}: value domain {have} does not match tensor domain {s.domain}")
        for dom, bad_stride in (("row", "stride_n"), ("col", "stride_m"), ("nvec", "stride_m")):
            for name in self.closure([s.input for s in self.stores if s.domain == dom]):
                n = self.nodes[name]
                if n.op == "load" and getattr(self.slots[n.slot].strides, bad_stride) != 0:
                    raise NotImplementedError(
                        f"per-{dom} expression loads {n.name}, which varies along the reduced axis")

    def closure(self, roots: Sequence[str]) -> List[str]:
        """Nodes needed to evaluate `roots`, stopping at reduction results,
        in topological (insertion) order."""
        need = set()
        work = list(roots)
        while work:
            n = work.pop()
            if n in need:
                continue
            need.add(n)
            work.extend(self.nodes[n].inputs)
        return [n for n in self.nodes if n in need]

    # -- identity -------------------------------------------------------------
    def structure(self) -> dict:
        """Shape-independent description: what the generated code depends on."""
        return {
            "batched": self.batched,
            "nodes": [[n.name, n.op, n.inputs, n.domain, n.slot, n.reduce, n.comp]
                      for n in self.nodes.values()],
            "slots": [[s.name, s.role, s.dtype, s.domain, s.kind] for s in self.slots],
            "reduces": [[r.name, r.kind, r.axis, r.input, r.state_offset, r.fold] for r in self.reduces.values()],
            "stores": [[s.slot, s.input, s.domain] for s in self.stores],
            "rng_scalar": self.rng_scalar,
            **({"anchor_scalar": self.anchor_scalar, "anchor_slots": self.anchor_slots}
               if self.anchor_scalar is not None or self.anchor_slots else {}),
        }

    def key(self) -> str:
        return hashlib.sha256(json.dumps(self.structure(), sort_keys=True).encode()).hexdigest()[:16]

    def epilogue_counts(self) -> Tuple[int, ...]:
        """The 7 epilogue-node counts of the reference's tuner key
        (tuner_base.py:120-131): aux_load, row_broadcast, column_broadcast,
        aux_store, row_reduction ([N] result), column_reduction ([M] result),
        row_store."""
        c = {"aux_load": 0, "row": 0, "col": 0, "aux_store": 0, "rowred": 0, "colred": 0, "rowstore": 0}
        for s in self.slots:
            if s.role == "load":
                if s.kind == "aux":
                    c["aux_load"] += 1
                elif s.kind == "row":
                    c["row"] += 1
                elif s.kind == "col":
                    c["col"] += 1
            else:
                if s.domain == "tile":
                    c["aux_store"] += 1
                elif s.domain == "nvec":
                    c["rowstore"] += 1
                elif s.domain == "col":
                    c["rowred"] += 1      # reference naming: RowReduction -> [N] vector
                else:
                    c["colred"] += 1      # ColumnReduction -> [M] vector
        return (c["aux_load"], c["row"], c["col"], c["aux_store"], c["rowred"], c["colred"], c["rowstore"])
