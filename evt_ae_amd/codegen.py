"""HIP code generator: EpilogueIR + tile configuration -> one kernel module.

Replaces the un-vendored CUTLASS Python emitter that the reference drives
through `plan.compile(...)` / `operation.epilogue_type(visitor_args)`
(python/gtl/compiler/passes/evt_fuser.py:515-518, :539-546).  The generated
translation unit instantiates the hand-written main loop
(csrc/evt_gemm.hpp) with an `Epi` struct whose `tile()` is straight-line code
over the accumulator registers, and exports the C ABI of include/evt_amd.h.
"""
from __future__ import annotations

import json
from dataclasses import dataclass, asdict
from typing import Dict, List, Optional

from .ir import DTYPE_CTYPES, REDUCE_STATE, EpilogueIR, Node


@dataclass(frozen=True)
class TileConfig:
    """Workgroup tile of the main loop (the analogue of the reference tuner's
    (threadblock shape, stages, warp count, swizzle) tuple,
    python/gtl/compiler/autotuner/gemm_tuner.py:31-44)."""
    bm: int = 256
    bn: int = 256
    bk: int = 64
    wm: int = 4
    wn: int = 2
    stages: int = 2
    dma: bool = True
    group_m: int = 4
    # 0: plain ring; 1: look-ahead ring with pinned instruction order (stages >= 3);
    # 2: ping-pong, the two waves of a SIMD alternate MFMA and LDS-read phases (8 waves, stages >= 2);
    # 3: ping-pong with one barrier per k-tile; 4 + flags: as 3 with 1 = the barrier inside group 0's MFMA phase,
    # 2 = group 0 issues its transfers between its LDS reads, 4 = group 1 as well (stages >= 3);
    # 12: one wave per SIMD (4 waves, stages >= 2): each wave interleaves the MFMAs of a k sub-step with the LDS
    # reads of the next; 64 x 64 wave tiles on a 128 x 128 tile instead of the 64 x 32 of eight waves;
    # 16 + p (p = 2 ... 11): ping-pong loop p with each k-tile's depth split between the two wave groups, which
    # then share loop wave tiles of twice the rows (a quarter fewer LDS reads per MFMA) and add their accumulators
    # behind the loop
    pipe: int = 0
    # > 1: a workgroup computes this many consecutive tiles of a row block, the operand ring running on from one
    # into the next, and per-row reductions leave one partial per workgroup (ping-pong pipelines, no per-column
    # reduction in the epilogue); pays when the tiles outnumber the CUs several times
    walk: int = 1

    def tag(self) -> str:
        return (f"{self.bm}x{self.bn}x{self.bk}_w{self.wm}x{self.wn}_s{self.stages}"
                f"_{'dma' if self.dma else 'safe'}_g{self.group_m}" + (f"_p{self.pipe}" if self.pipe else "")
                + (f"_n{self.walk}" if self.walk > 1 else ""))

    def stage_bytes(self) -> int:
        return (self.bm + self.bn) * self.bk * 2

    def lds_bytes(self) -> int:
        return self.stages * self.stage_bytes()


@dataclass(frozen=True)
class KernelSpec:
    a_kc: bool          # A contiguous along K (row-major [M, K])
    b_kc: bool          # B contiguous along K (column-major, i.e. stored [N, K])
    bf16: bool
    tile: TileConfig
    # K is a multiple of the tile's bk for every launch of the module: the global -> LDS transfers then carry no
    # per-lane test against K (measured 2-3 % on 8192 x 1024 x 4096)
    k_exact: bool = False
    # The traced problem has tiles on the matrix's edge (M or N no multiple of the tile): the module then carries
    # a third instantiation of the epilogue, the interior tiles' buffer accesses with lanes outside the matrix
    # masked.  Modules for problems without edge tiles leave it out: its mere presence costs the short
    # HBM-bound kernels 10 % (attention scores, 64 x 512 x 512 x 64: 10.7 -> 12.1 us with it compiled in)
    edge: bool = False

    @staticmethod
    def for_problem(K: int, a_kc: bool, b_kc: bool, bf16: bool, tile: TileConfig,
                    M: Optional[int] = None, N: Optional[int] = None) -> "KernelSpec":
        edge = bool(M is not None and N is not None and (M % tile.bm or N % tile.bn))
        return KernelSpec(a_kc, b_kc, bf16, tile, bool(tile.dma and K % tile.bk == 0), edge)

    def tag(self) -> str:
        return self.tile.tag() + ("_kx" if self.k_exact else "") + ("_e" if self.edge else "")


def reduction_lds_bytes(t: "TileConfig", row_state: int, col_state: int) -> int:
    """LDS the epilogue's reductions need inside the operand stages: the per-wave row states [wn][bm] and the
    column states [max(wm, shares)][bn] side by side (each followed by a flag), and for phase 2 of a per-row
    reduction one state per thread."""
    need = 0
    if row_state:
        need += t.wn * t.bm * row_state * 4 + 16
    if col_state:
        need += max(t.wm, max(1, t.wm * t.wn * 64 // t.bn)) * t.bn * col_state * 4 + 16
    if row_state:   # + per wave and half one float per row: a row's first-pass result on its way back to its lanes
        need = (need + 15) // 16 * 16 + t.wm * t.wn * 2 * (t.bm // t.wm // 2) * 4
    return max(need, t.wm * t.wn * 64 * row_state * 4)


ABI_VERSION = 5            # EVT_ABI_VERSION of include/evt_amd.h
STATIC_SCRATCH_BYTES = 1 << 20


def emit_static_scratch(e: "_Emitter", needed: bool) -> None:
    """File-scope device array that takes the workspace's place in `evt_launch_static`, and the per-device
    look-up of its address (each GPU that loads the module holds its own copy).  A module whose kernels never use
    a workspace (`needed` false) carries no array."""
    e("// ---- evt_launch_static: the entry point that allocates nothing ------------------------------------------")
    e("namespace {")
    if not needed:
        e("constexpr int64_t kScratchBytes = 0;   // this module's kernels use no workspace: no array")
        e("[[maybe_unused]] int scratch_for_stream(void* stream, void** out) { (void)stream; *out = nullptr; return EVT_OK; }")
        e("}  // namespace")
        return
    e(f"constexpr int64_t kScratchBytes = {STATIC_SCRATCH_BYTES};")
    e("static __device__ __align__(256) unsigned char scratch[kScratchBytes];")
    e("constexpr int kMaxDevices = 64;")
    e("void* scratch_address[kMaxDevices];   // device address of `scratch` on each GPU, looked up on first use")
    e("std::mutex scratch_mutex;")
    e("// `scratch` names a host-side stand-in; kernels, fills and copies take the address this returns: the array's")
    e("// address on the GPU that `stream` belongs to (the current one for the null stream).  The first call per GPU")
    e("// looks the address up with that GPU current, which may load the code object: it has to happen outside a")
    e("// stream capture.")
    e("int scratch_for_stream(void* stream, void** out) {")
    e("  int cur = -1, dev = -1;")
    e("  const hipError_t e0 = hipGetDevice(&cur);")
    e("  if (e0 != hipSuccess) return (int)e0;")
    e("  dev = cur;")
    e("  if (stream) {")
    e("    const hipError_t es = hipStreamGetDevice((hipStream_t)stream, &dev);")
    e("    if (es != hipSuccess) return (int)es;")
    e("  }")
    e("  if (dev < 0 || dev >= kMaxDevices) return EVT_ERR_RANGE;")
    e("  std::lock_guard<std::mutex> lock(scratch_mutex);")
    e("  if (!scratch_address[dev]) {")
    e("    void* ptr = nullptr;")
    e("    if (dev != cur) { const hipError_t e2 = hipSetDevice(dev); if (e2 != hipSuccess) return (int)e2; }")
    e("    const hipError_t e1 = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));")
    e("    if (dev != cur) (void)hipSetDevice(cur);")
    e("    if (e1 != hipSuccess) return (int)e1;")
    e("    if (!ptr) return EVT_ERR_WORKSPACE;")
    e("    scratch_address[dev] = ptr;")
    e("  }")
    e("  *out = scratch_address[dev];")
    e("  return EVT_OK;")
    e("}")
    e("}  // namespace")


_BINARY = {
    "add": "({a} + {b})", "sub": "({a} - {b})", "mul": "({a} * {b})",
    "div": "__fdividef({a}, {b})", "max": "fmaxf({a}, {b})", "min": "fminf({a}, {b})",
    "tanh_backward": "evt::op_tanh_backward({a}, {b})",
    "gelu_backward_tanh": "evt::op_gelu_backward_tanh({a}, {b})",
    "gelu_backward_erf": "evt::op_gelu_backward_erf({a}, {b})",
    "ge": "(({a} >= {b}) ? 1.f : 0.f)", "gt": "(({a} > {b}) ? 1.f : 0.f)",
    "le": "(({a} <= {b}) ? 1.f : 0.f)", "lt": "(({a} < {b}) ? 1.f : 0.f)",
    "ne": "(({a} != {b}) ? 1.f : 0.f)", "eq": "(({a} == {b}) ? 1.f : 0.f)",
}
_UNARY = {
    "neg": "(-{a})", "exp": "evt::op_exp({a})", "log": "evt::op_log({a})",
    "sqrt": "sqrtf({a})", "rsqrt": "rsqrtf({a})", "abs": "fabsf({a})", "rcp": "evt::op_rcp({a})",
    "gelu_tanh": "evt::op_gelu_tanh({a})", "gelu_erf": "evt::op_gelu_erf({a})",
    "tanh": "evt::op_tanh({a})", "relu": "evt::op_relu({a})", "sigmoid": "evt::op_sigmoid({a})",
    "cast_f16": "evt::round_to<evt::f16>({a})", "cast_bf16": "evt::round_to<evt::bf16>({a})",
    "cast_f32": "({a})", "cast_bool": "(({a} != 0.f) ? 1.f : 0.f)", "cast_int": "truncf({a})",
}

_IDENTITY = {"sum": "0.f", "max": "-INFINITY"}


def _cname(name: str) -> str:
    return "v_" + "".join(ch if ch.isalnum() else "_" for ch in name)


class _Emitter:
    def __init__(self):
        self.lines: List[str] = []
        self.ind = 0

    def __call__(self, text: str = ""):
        for line in text.split("\n"):
            self.lines.append(("  " * self.ind + line) if line else "")

    def indent(self):
        self.ind += 1

    def dedent(self):
        self.ind -= 1

    def text(self) -> str:
        return "\n".join(self.lines) + "\n"


class Codegen:
    def __init__(self, ir: EpilogueIR, spec: KernelSpec, module_name: str, clock_probe: bool = False):
        self.ir = ir
        self.spec = spec
        self.name = module_name
        # diagnostic build: workgroup 0 times its main loop and its epilogue with the shader-clock and the
        # constant 100 MHz counters, and the module exports evt_clock_probe_read
        self.clock_probe = clock_probe
        # variance of every node: does it vary along m / along n?
        self.var_m: Dict[str, bool] = {}
        self.var_n: Dict[str, bool] = {}
        for n in ir.nodes.values():
            if n.op in ("accum",):
                vm, vn = True, True
            elif n.op == "colidx":
                vm, vn = False, True
            elif n.op == "load":
                st = ir.slots[n.slot].strides
                vm = st.stride_m != 0 or st.stride_l != 0
                vn = st.stride_n != 0
                # a batch-dependent value is re-read per row slot only if it also
                # depends on m; a pure batch scalar is workgroup-uniform
                vm = st.stride_m != 0
                if ir.slots[n.slot].kind == "rand":
                    vm, vn = True, True
            elif n.op in ("imm", "rres"):
                vm, vn = False, False
            elif n.op == "rowval":      # per-row value an anchor hands over (layer norm: mean, rstd)
                vm, vn = True, False
            elif n.op == "anchorval":   # further per-element value of a row-wise anchor (layer norm backward: g, xhat)
                vm, vn = True, True
            else:
                vm = any(self.var_m[i] for i in n.inputs)
                vn = any(self.var_n[i] for i in n.inputs)
            self.var_m[n.name], self.var_n[n.name] = vm, vn

    # -- expression helpers ---------------------------------------------------
    def ref(self, name: str, idx: str = "ni") -> str:
        return f"{_cname(name)}[{idx}]" if self.var_n[name] else _cname(name)

    def expr(self, n: Node, idx: str = "ni") -> str:
        a = [self.ref(i, idx) for i in n.inputs]
        if n.op in _BINARY:
            return _BINARY[n.op].format(a=a[0], b=a[1])
        if n.op in _UNARY:
            return _UNARY[n.op].format(a=a[0])
        if n.op == "where":
            return f"(({a[0]} != 0.f) ? {a[1]} : {a[2]})"
        raise NotImplementedError(n.op)

    def slot_off(self, k: int, batch: str = "t.batch") -> str:
        if batch == "t.batch" and getattr(self, "_tile_offsets", False):
            return f"bo_{k}"      # computed once at the top of tile()
        return f"evt::batch_offset({batch}, p.t{k}_lm, p.t{k}_ld, p.t{k}_sl, p.t{k}_sl2)"

    # -- sections ---------------------------------------------------------------
    def emit_params(self, e: _Emitter):
        e("struct Params {")
        e.indent()
        for k, s in enumerate(self.ir.slots):
            const = "const " if s.role == "load" else ""
            e(f"{const}{DTYPE_CTYPES[s.dtype]}* t{k};  // {s.role} {s.kind} '{s.name}'")
            e(f"int64_t t{k}_sl, t{k}_sl2, t{k}_sm, t{k}_sn; int t{k}_ld; int t{k}_lm; int t{k}_vec;")
        e(f"float s[{max(1, len(self.ir.scalars))}];")
        e("int fast;   // every per-element tensor is unit-stride / vector-aligned: interior tiles skip all checks")
        e.dedent()
        e("};")

    def emit_combine(self, e: _Emitter, axis: str):
        e(f"static EVT_DEV void {axis}_combine(float* a, const float* b) {{")
        e.indent()
        for r in self.ir.reduces.values():
            if r.axis != axis:
                continue
            o = r.state_offset
            if r.kind == "sum":
                e(f"a[{o}] += b[{o}];")
            elif r.kind == "max":
                e(f"a[{o}] = fmaxf(a[{o}], b[{o}]);")
            elif r.kind == "maxsumexp":
                e(f"evt::combine_maxsumexp(a[{o}], a[{o + 1}], b[{o}], b[{o + 1}]);")
            elif r.kind == "welford":
                e(f"evt::combine_welford(a[{o}], a[{o + 1}], a[{o + 2}], b[{o}], b[{o + 1}], b[{o + 2}]);")
        e("(void)a; (void)b;")
        e.dedent()
        e("}")

    def emit_identity(self, e: _Emitter, axis: str):
        e(f"static EVT_DEV void {axis}_identity(float* a) {{")
        e.indent()
        for r in self.ir.reduces.values():
            if r.axis != axis:
                continue
            o = r.state_offset
            if r.kind == "sum":
                e(f"a[{o}] = 0.f;")
            elif r.kind == "max":
                e(f"a[{o}] = -INFINITY;")
            elif r.kind == "maxsumexp":
                e(f"a[{o}] = -INFINITY; a[{o + 1}] = 0.f;")
            elif r.kind == "welford":
                e(f"a[{o}] = 0.f; a[{o + 1}] = 0.f; a[{o + 2}] = 0.f;")
        e("(void)a;")
        e.dedent()
        e("}")

    def emit_finalize(self, e: _Emitter, axis: str):
        idx = "row" if axis == "row" else "col"
        stride = "sm" if axis == "row" else "sn"
        e(f"static EVT_DEV void {axis}_finalize(const Params& p, int batch, int {idx}, const float* st) {{")
        e.indent()
        stores = [s for s in self.ir.stores if s.domain == axis]
        for name in self.ir.closure([s.input for s in stores]):
            n = self.ir.nodes[name]
            c = _cname(name)
            if n.op == "imm":
                e(f"const float {c} = p.s[{n.slot}];")
            elif n.op == "rres":
                r = self.ir.reduces[n.reduce]
                e(f"const float {c} = st[{r.state_offset + n.comp}];")
            elif n.op == "load":
                k = n.slot
                e(f"const float {c} = evt::ld_f32(p.t{k}, {self.slot_off(k, 'batch')} + (int64_t){idx} * p.t{k}_{stride});")
            else:
                a = [_cname(i) for i in n.inputs]
                if n.op in _BINARY:
                    ex = _BINARY[n.op].format(a=a[0], b=a[1])
                elif n.op in _UNARY:
                    ex = _UNARY[n.op].format(a=a[0])
                elif n.op == "where":
                    ex = f"(({a[0]} != 0.f) ? {a[1]} : {a[2]})"
                else:
                    raise NotImplementedError(f"{n.op} in a per-{axis} expression")
                e(f"const float {c} = {ex};")
        for s in stores:
            k = s.slot
            e(f"evt::st_f32(p.t{k}, {self.slot_off(k, 'batch')} + (int64_t){idx} * p.t{k}_{stride}, {_cname(s.input)});")
        e("(void)p; (void)batch; (void)st;")
        e.dedent()
        e("}")

    def onehot_label(self, r) -> str | None:
        """A per-row sum of where(label == column index, x, 0) -- a gather along the row -- has at most one
        non-zero term per row, and for most (wave, tile) pairs none: the name of the per-row `label` value if `r`
        is such a sum and the label's value can be formed from per-row loads alone, else None."""
        ir = self.ir
        if r.axis != "row" or r.kind != "sum" or r.fold:
            return None
        n = ir.nodes[r.input]
        if n.op != "where" or len(n.inputs) != 3:
            return None
        hit, _x, zero = (ir.nodes[i] for i in n.inputs)
        if zero.op != "imm" or ir.scalars[zero.slot] != 0.0 or hit.op != "eq":
            return None
        a, b = hit.inputs
        if ir.nodes[a].op == "colidx":
            a, b = b, a
        if ir.nodes[b].op != "colidx":
            return None
        for name in ir.closure([a]):
            m = ir.nodes[name]
            if self.var_n[name] or m.op in ("accum", "rres", "rowval", "anchorval", "colidx"):
                return None
            if m.op == "load" and ir.slots[m.slot].kind not in ("col", "scalar"):
                return None
            if m.op not in ("load", "imm", "where") and m.op not in _UNARY and m.op not in _BINARY:
                return None
        return a

    def emit_onehot_vote(self, e: _Emitter, labels: List[str]):
        """`oh_hit`: does the label of this lane's row(s) of the wave tile name one of this wave's columns?  (The
        loads go out at the top of the tile; the vote over the wave is taken where the answer is needed.)"""
        ir = self.ir
        e("bool oh_hit = false;")
        e("#pragma unroll")
        e("for (int j = 0; j < (Cfg::TM + 63) / 64; ++j) {")
        e.indent()
        e("const int lr = t.lane + 64 * j, vr = t.row_u + lr;")
        e("const bool vok = lr < Cfg::TM && vr < t.M;")
        for name in ir.closure(labels):
            n = ir.nodes[name]
            c = "q" + _cname(name)
            if n.op == "imm":
                e(f"const float {c} = p.s[{n.slot}];")
            elif n.op == "load":
                k = n.slot
                if ir.slots[k].kind == "col":
                    e(f"const float {c} = vok ? evt::ld_f32(p.t{k}, bo_{k} + (int64_t)vr * p.t{k}_sm) : -1.f;")
                else:
                    e(f"const float {c} = evt::ld_f32(p.t{k}, 0);")
            else:
                a = ["q" + _cname(i) for i in n.inputs]
                if n.op in _BINARY:
                    ex = _BINARY[n.op].format(a=a[0], b=a[1])
                elif n.op in _UNARY:
                    ex = _UNARY[n.op].format(a=a[0])
                else:
                    ex = f"(({a[0]} != 0.f) ? {a[1]} : {a[2]})"
                e(f"const float {c} = {ex};")
        for lab in labels:
            c = "q" + _cname(lab)
            e(f"oh_hit |= vok && {c} >= (float)t.col_u && {c} < (float)(t.col_u + Cfg::TN);")
        e.dedent()
        e("}")

    def emit_tile(self, e: _Emitter):
        ir = self.ir
        tile_stores = [s for s in ir.stores if s.domain == "tile"]
        row_reds = [r for r in ir.reduces.values() if r.axis == "row"]
        col_reds = [r for r in ir.reduces.values() if r.axis == "col"]
        vec_stores = [s for s in ir.stores if s.domain == "nvec"]
        roots = [s.input for s in tile_stores] + [r.input for r in ir.reduces.values()] + [s.input for s in vec_stores]
        need = ir.closure(roots)
        hoisted = [n for n in need if not self.var_m[n]]
        # One-hot row sums (a gather along the row) are collected in a pass of their own, which a wave skips when
        # none of its rows' labels names one of its columns (wave tiles of two or more 32-row blocks)
        onehot: Dict[str, str] = {}
        if self.spec is not None and self.spec.tile.bm // self.spec.tile.wm // 32 >= 2 and not col_reds:
            for r in row_reds:
                lab = self.onehot_label(r)
                if lab is not None:
                    onehot[r.name] = lab
        main_roots = [s.input for s in tile_stores] + [r.input for r in ir.reduces.values() if r.name not in onehot]
        inner = [n for n in ir.closure(main_roots) if self.var_m[n]]
        oh_inner = [n for n in ir.closure([ir.reduces[name].input for name in onehot]) if self.var_m[n]]

        aux_nodes = [n for n in inner if ir.nodes[n].op == "load" and ir.slots[ir.nodes[n].slot].kind == "aux"]
        e("template <class Cfg, class Tile, bool FAST>")
        e("static EVT_DEV void tile(const Params& p, const Tile& t, const evt::GemmArgs& g, "
          "const evt::f32x16 (&acc)[Cfg::MI][Cfg::NI]) {")
        e.indent()
        e("constexpr int MI = Cfg::MI, NI = Cfg::NI;")
        if row_reds or col_reds:
            e("__syncthreads();  // all waves are done reading the last operand tile from LDS")
        # each tensor's batch offset once per tile (it holds a division; left inside the row loops it is redone
        # for every row)
        for k in range(len(ir.slots)):
            e(f"[[maybe_unused]] const int64_t bo_{k} = evt::batch_offset(t.batch, p.t{k}_lm, p.t{k}_ld, p.t{k}_sl, p.t{k}_sl2);")
        self._tile_offsets = True
        # one value per row (column vectors): check-free path through buffer loads, the row's offset in a scalar
        col_loads = sorted({ir.nodes[n].slot for n in inner + oh_inner if ir.nodes[n].op == "load" and ir.slots[ir.nodes[n].slot].kind == "col"})
        for k in col_loads:
            e(f"[[maybe_unused]] __amdgpu_buffer_rsrc_t rc_{k};")
            e(f"[[maybe_unused]] uint32_t vc_{k} = 0;")
            e(f"[[maybe_unused]] const uint32_t cp_{k} = (uint32_t)p.t{k}_sm * (uint32_t)sizeof(*p.t{k});")
            e("if constexpr (FAST) {")
            e(f"  rc_{k} = evt::make_rsrc((const char*)(p.t{k} + bo_{k} + (int64_t)t.row_u * p.t{k}_sm));")
            e(f"  vc_{k} = (uint32_t)(t.row_l * (int)p.t{k}_sm) * (uint32_t)sizeof(*p.t{k});")
            e("}")
        # hoisted values
        for name in hoisted:
            self.emit_node(e, ir.nodes[name], hoisted=True)
        if vec_stores:
            # one value per column, formed from [N] vectors and scalars alone: written once per batch, by the
            # lanes that hold row 0
            e("if (t.row(0, 0) == 0) {")
            e.indent()
            for s_ in vec_stores:
                k = s_.slot
                e("#pragma unroll")
                e(f"for (int ni = 0; ni < NI; ++ni) if (t.col_ok(ni)) "
                  f"evt::st_f32(p.t{k}, bo_{k} + (int64_t)t.col(ni) * p.t{k}_sn, {self.ref(s_.input)});")
            e.dedent()
            e("}")
        if onehot:
            self.emit_onehot_vote(e, sorted(set(onehot.values())))
        if col_reds:
            e(f"float cst[NI][{ir.col_state}];")
            e("#pragma unroll")
            e("for (int ni = 0; ni < NI; ++ni) {")
            e.indent()
            for r in col_reds:
                e(f"cst[ni][{r.state_offset}] = {_IDENTITY[r.kind]};")
            e.dedent()
            e("}")
        # check-free path: wave-uniform row base (scalar registers) + one per-lane offset per tensor
        for k in [ir.nodes[n].slot for n in aux_nodes] + [s_.slot for s_ in tile_stores]:
            e(f"[[maybe_unused]] __amdgpu_buffer_rsrc_t rs_{k};   // this wave's corner of the tile (scalar registers)")
            e(f"[[maybe_unused]] uint32_t vo_{k} = 0;              // this lane's byte offset inside a row")
            e(f"[[maybe_unused]] const uint32_t rp_{k} = (uint32_t)p.t{k}_sm * (uint32_t)sizeof(*p.t{k});   // row pitch in bytes")
            e("if constexpr (FAST) {")
            e(f"  rs_{k} = evt::make_rsrc((const char*)(p.t{k} + {self.slot_off(k)} + (int64_t)t.row_u * p.t{k}_sm + t.col_u));")
            e(f"  vo_{k} = (uint32_t)(t.row_l * (int)p.t{k}_sm + t.col_l) * (uint32_t)sizeof(*p.t{k});")
            e("}")
        # With a cross-workgroup reduction in the same epilogue, the arrival ticket has to wait until this wave's
        # earlier stores are acknowledged; the output-tile values of a small wave tile are therefore kept in
        # registers and stored after the ticket instead of in front of it.
        defer = bool(tile_stores) and bool(row_reds or col_reds)
        e(f"constexpr bool DEFER = {'true' if defer else 'false'} && MI * NI <= 4;")
        for s_ in tile_stores:
            # kept in the storage type (rounded once, as a direct store would): half the registers for 16-bit outputs
            e(f"[[maybe_unused]] typename evt::StorageRow<{DTYPE_CTYPES[ir.slots[s_.slot].dtype]}, NI>::type sv_{s_.slot}[DEFER ? MI : 1][16];")
        # per-row reductions work on all rows of the wave tile at once (evt::rows_*): the loops below only collect
        # the values
        # With one 32-row block per wave (MI = 1) each row is reduced as it is produced (ROW_BY_ROW), which runs under
        # the row's stores; larger wave tiles collect the values and reduce all rows together afterwards
        e("constexpr bool ROW_BY_ROW = MI == 1;")
        if onehot:
            e('static_assert(!ROW_BY_ROW, "the separate pass of one-hot row sums is generated for wave tiles of two or more row blocks");')
        for r in row_reds:
            if r.kind in ("sum", "max"):
                e(f"[[maybe_unused]] float rp_{_cname(r.name)}[16 * MI];")
            else:
                e(f"[[maybe_unused]] float rx_{_cname(r.name)}[ROW_BY_ROW ? 1 : 16 * MI][NI];")
        if any(r.kind == "welford" for r in row_reds):
            e("[[maybe_unused]] const float wcnt = (float)t.wave_cols();")
            e("[[maybe_unused]] const float wrcnt = wcnt > 0.f ? 1.f / wcnt : 0.f;")
        # rows are processed in batches of MB x 16: the full-tensor loads of a batch are all issued before its
        # arithmetic and stores (loads do not move above stores by themselves), so a batch costs one round trip
        # to HBM; two 32-row blocks per batch keep the staging registers bounded on the largest wave tiles
        # The staging registers of a batch sit next to the accumulators (16 MI NI per lane) and the epilogue's own
        # values: with several full tensors to read, a batch shrinks to one 32-row block, then to 8 or 4 of its 16
        # rows per lane, so that nothing spills (three residuals on a 256 x 256 tile spilled 576 bytes per lane with
        # fixed batches of two blocks and ran 118 us where the unfused sequence takes 81)
        stage_words = " + ".join(f"(int)sizeof({DTYPE_CTYPES[ir.slots[ir.nodes[n].slot].dtype]})" for n in aux_nodes) or "0"
        e(f"constexpr int STAGE_BYTES_PER_ROW = NI * ({stage_words});     // per lane and row of the wave tile")
        e("constexpr int STAGE_BUDGET = (256 - 16 * MI * NI - 104 > 16 ? 256 - 16 * MI * NI - 104 : 16) * 4;   // bytes per lane")
        e("constexpr int STAGE_ROWS = STAGE_BYTES_PER_ROW == 0 ? 32 : STAGE_BUDGET / STAGE_BYTES_PER_ROW;")
        e("constexpr int MB = (MI >= 2 && STAGE_ROWS >= 32) ? 2 : 1;")
        e("constexpr int VB = STAGE_ROWS >= 16 ? 16 : STAGE_ROWS >= 8 ? 8 : 4;    // rows of a block per batch")
        e('static_assert(MI % MB == 0, "row blocks per wave must be 1 or even");')
        e("#pragma unroll")
        e("for (int mb = 0; mb < MI; mb += MB) {")
        e.indent()
        e("#pragma unroll")
        e("for (int vb = 0; vb < 16; vb += VB) {")
        e.indent()
        if aux_nodes:
            for name in aux_nodes:
                k = ir.nodes[name].slot
                e(f"{DTYPE_CTYPES[ir.slots[k].dtype]} rb_{_cname(name)}[MB][VB][NI];")
            e("#pragma unroll")
            e("for (int mo = 0; mo < MB; ++mo) {")
            e.indent()
            e("#pragma unroll")
            e("for (int vi = 0; vi < VB; ++vi) {")
            e.indent()
            e("const int v = vb + vi;")
            e("const int row = t.row(mb + mo, v);")
            e("const bool rok = t.row_ok(row);")
            for name in aux_nodes:
                k = ir.nodes[name].slot
                e(f"if constexpr (FAST) evt::row_load<Tile>(t, rok, rs_{k}, vo_{k}, (uint32_t)Tile::row_step(mb + mo, v) * rp_{k}, "
                  f"rb_{_cname(name)}[mo][vi]);")
                e(f"else evt::aux_load<false>(t, p.t{k}, {self.slot_off(k)} + (int64_t)row * p.t{k}_sm + (int64_t)t.col0 * p.t{k}_sn, "
                  f"p.t{k}_sn, p.t{k}_vec, rok, rb_{_cname(name)}[mo][vi]);")
            e.dedent()
            e("}")
            e.dedent()
            e("}")
        e("#pragma unroll")
        e("for (int mo = 0; mo < MB; ++mo) {")
        e.indent()
        e("const int mi = mb + mo;")
        for name in aux_nodes:
            k = ir.nodes[name].slot
            e(f"const {DTYPE_CTYPES[ir.slots[k].dtype]} (&r_{_cname(name)})[VB][NI] = rb_{_cname(name)}[mo];")
        e("#pragma unroll")
        e("for (int vi = 0; vi < VB; ++vi) {")
        e.indent()
        e("const int v = vb + vi;")
        e("const int row = t.row(mi, v);")
        e("const bool rok = t.row_ok(row);")
        for name in inner:
            self.emit_node(e, ir.nodes[name], hoisted=False)
        for s in tile_stores:
            k = s.slot
            src = s.input
            if not self.var_n[src]:
                e(f"float b_{k}[NI];")
                e(f"#pragma unroll\nfor (int ni = 0; ni < NI; ++ni) b_{k}[ni] = {_cname(src)};")
                arr = f"b_{k}"
            else:
                arr = _cname(src)
            e("if constexpr (DEFER) {")
            e(f"  #pragma unroll\n  for (int ni = 0; ni < NI; ++ni) sv_{k}[mi][v][ni] = evt::to_storage<{DTYPE_CTYPES[ir.slots[k].dtype]}>({arr}[ni]);")
            e("} else {")
            e.indent()
            self.emit_tile_store(e, k, arr)
            e.dedent()
            e("}")
        if row_reds and not onehot:
            e("if constexpr (ROW_BY_ROW) {")
            e.indent()
            e(f"float rst[{ir.row_state}];")
            for r in row_reds:
                self.emit_row_reduce(e, r)
            e(f"evt::row_state_to_lds<Cfg, {ir.row_state}>(t, mi, v, rst);")
            e.dedent()
            e("} else {")
            e.indent()
        for r in row_reds:
            if r.name in onehot:
                continue
            c, x = _cname(r.name), self.ref(r.input)
            if r.kind == "sum":
                e(f"{{ float a = 0.f;\n#pragma unroll\nfor (int ni = 0; ni < NI; ++ni) a += t.col_ok(ni) ? {x} : 0.f;\nrp_{c}[mi * 16 + v] = a; }}")
            elif r.kind == "max":
                e(f"{{ float a = -INFINITY;\n#pragma unroll\nfor (int ni = 0; ni < NI; ++ni) a = t.col_ok(ni) ? fmaxf(a, {x}) : a;\nrp_{c}[mi * 16 + v] = a; }}")
            else:
                e(f"#pragma unroll\nfor (int ni = 0; ni < NI; ++ni) rx_{c}[mi * 16 + v][ni] = {x};")
        if row_reds and not onehot:
            e.dedent()
            e("}")
        for r in col_reds:
            x = lambda: self.ref(r.input)  # noqa: E731
            o = r.state_offset
            e("#pragma unroll")
            e("for (int ni = 0; ni < NI; ++ni) {")
            e.indent()
            if r.kind == "sum":
                e(f"cst[ni][{o}] += (rok && t.col_ok(ni)) ? {x()} : 0.f;")
            else:
                e(f"cst[ni][{o}] = (rok && t.col_ok(ni)) ? fmaxf(cst[ni][{o}], {x()}) : cst[ni][{o}];")
            e.dedent()
            e("}")
        e.dedent()
        e("}")
        e.dedent()
        e("}")
        e.dedent()
        e("}")
        e.dedent()
        e("}")
        if row_reds and onehot:      # the other reductions first: the vote's loads travel meanwhile
            for r in row_reds:
                if r.name in onehot:
                    continue
                c, o = _cname(r.name), r.state_offset
                if r.kind in ("sum", "max"):
                    e(f"evt::rows_simple<Cfg, {ir.row_state}, {'true' if r.kind == 'max' else 'false'}>(t, rp_{c}, {o});")
                elif r.kind == "maxsumexp":
                    e(f"evt::rows_maxsumexp<Cfg, {ir.row_state}, {ir.col_state}>(t, rx_{c}, {o});")
                elif r.kind == "welford":
                    e(f"evt::rows_welford<Cfg, {ir.row_state}, {ir.col_state}>(t, rx_{c}, {o});")
                else:
                    raise NotImplementedError(r.kind)
        if onehot:
            e("const bool oh_any = __builtin_amdgcn_ballot_w64(oh_hit) != 0;   // wave-uniform")
            e("if (oh_any) {")
            e.indent()
            e("#pragma unroll")
            e("for (int mi = 0; mi < MI; ++mi) {")
            e.indent()
            e("#pragma unroll")
            e("for (int v = 0; v < 16; ++v) {")
            e.indent()
            e("const int row = t.row(mi, v);")
            e("const bool rok = t.row_ok(row);")
            for name in oh_inner:
                self.emit_node(e, ir.nodes[name], hoisted=False)
            for name in onehot:
                r = ir.reduces[name]
                c, x = _cname(r.name), self.ref(r.input)
                e(f"{{ float a = 0.f;\n#pragma unroll\nfor (int ni = 0; ni < NI; ++ni) a += t.col_ok(ni) ? {x} : 0.f;\nrp_{c}[mi * 16 + v] = a; }}")
            e("(void)row; (void)rok;")
            e.dedent()
            e("}")
            e.dedent()
            e("}")
            e.dedent()
            e("}")
        if row_reds:
            e("if constexpr (!ROW_BY_ROW) {")
            e.indent()
        for r in row_reds:
            c, o = _cname(r.name), r.state_offset
            if r.name in onehot:
                # no label of this wave's rows names one of its columns: every term is zero
                e(f"if (oh_any) evt::rows_simple<Cfg, {ir.row_state}, false>(t, rp_{c}, {o});")
                e(f"else evt::rows_fill<Cfg, {ir.row_state}>(t, {o}, 0.f);")
            elif onehot:
                pass        # emitted above
            elif r.kind in ("sum", "max"):
                e(f"evt::rows_simple<Cfg, {ir.row_state}, {'true' if r.kind == 'max' else 'false'}>(t, rp_{c}, {o});")
            elif r.kind == "maxsumexp":
                e(f"evt::rows_maxsumexp<Cfg, {ir.row_state}, {ir.col_state}>(t, rx_{c}, {o});")
            elif r.kind == "welford":
                e(f"evt::rows_welford<Cfg, {ir.row_state}, {ir.col_state}>(t, rx_{c}, {o});")
            else:
                raise NotImplementedError(r.kind)
        if row_reds:
            e.dedent()
            e("}")
            e("const int row_ticket = evt::row_reduce_publish<Cfg, Epi>(p, t, g);")
        if col_reds:
            e("const int col_ticket = evt::col_reduce_publish<Cfg, Epi>(p, t, g, cst);")
        if defer:
            e("if constexpr (DEFER) {")
            e.indent()
            e("#pragma unroll")
            e("for (int mi = 0; mi < MI; ++mi) {")
            e.indent()
            e("#pragma unroll")
            e("for (int v = 0; v < 16; ++v) {")
            e.indent()
            e("const int row = t.row(mi, v);")
            e("const bool rok = t.row_ok(row);")
            for s_ in tile_stores:
                e(f"float dv_{s_.slot}[NI];")
                e(f"#pragma unroll\nfor (int ni = 0; ni < NI; ++ni) dv_{s_.slot}[ni] = evt::from_storage(sv_{s_.slot}[mi][v][ni]);")
                self.emit_tile_store(e, s_.slot, f"dv_{s_.slot}")
            e("(void)row; (void)rok;")
            e.dedent()
            e("}")
            e.dedent()
            e("}")
            e.dedent()
            e("}")
        # the deferred stores above travel while the arrival tickets do
        if row_reds:
            e("const bool row_last = evt::row_reduce_arrived<Cfg, Epi>(t, g, row_ticket);")
        if col_reds:
            e("const bool col_last = evt::col_reduce_arrived<Cfg, Epi>(t, g, col_ticket);")
        if row_reds:
            e("if (row_last) evt::row_reduce_complete<Cfg, Epi>(p, t, g);")
        if col_reds:
            e("if (col_last) evt::col_reduce_complete<Cfg, Epi>(p, t, g);")
        e("(void)p; (void)t; (void)g; (void)acc;")
        e.dedent()
        e("}")
        self._tile_offsets = False

    def emit_tile_store(self, e: _Emitter, k: int, arr: str):
        """Store the NI values `arr` of row (mi, v) to tile slot k (inside the row loops)."""
        e(f"if constexpr (FAST) evt::row_store<Tile, {DTYPE_CTYPES[self.ir.slots[k].dtype]}>(t, rok, rs_{k}, vo_{k}, (uint32_t)Tile::row_step(mi, v) * rp_{k}, {arr});")
        e(f"else evt::aux_store<false>(t, p.t{k}, {self.slot_off(k)} + (int64_t)row * p.t{k}_sm + (int64_t)t.col0 * p.t{k}_sn, "
          f"p.t{k}_sn, p.t{k}_vec, rok, {arr});")

    def emit_node(self, e: _Emitter, n: Node, hoisted: bool):
        c = _cname(n.name)
        vn = self.var_n[n.name]
        if n.op == "imm":
            e(f"const float {c} = p.s[{n.slot}];")
        elif n.op == "accum":
            e(f"float {c}[NI];")
            e(f"#pragma unroll\nfor (int ni = 0; ni < NI; ++ni) {c}[ni] = acc[mi][ni][v];")
        elif n.op == "colidx":
            e(f"float {c}[NI];")
            e(f"#pragma unroll\nfor (int ni = 0; ni < NI; ++ni) {c}[ni] = (float)t.col(ni);")
        elif n.op == "load":
            k = n.slot
            s = self.ir.slots[k]
            base = self.slot_off(k)
            if s.kind == "rand":
                r = self.ir.rng_scalar
                e(f"float {c}[NI];")
                e(f"evt::rand_row<Tile>((uint64_t)__builtin_bit_cast(uint32_t, p.s[{r}]) | ((uint64_t)__builtin_bit_cast(uint32_t, p.s[{r + 1}]) << 32), "
                  f"__builtin_bit_cast(uint32_t, p.s[{r + 2}]), {k}u + 16u * __builtin_bit_cast(uint32_t, p.s[{r + 3}]), "
                  f"{base} + (int64_t)row * p.t{k}_sm + (int64_t)t.col0 * p.t{k}_sn, p.t{k}_sn, {c});")
            elif s.kind == "aux":
                e(f"float {c}[NI];")
                e(f"#pragma unroll\nfor (int ni = 0; ni < NI; ++ni) {c}[ni] = (float)r_{c}[vi][ni];")
            elif s.kind == "row":
                e(f"float {c}[NI];")
                e(f"#pragma unroll\nfor (int ni = 0; ni < NI; ++ni) {c}[ni] = t.col_ok(ni) ? "
                  f"evt::ld_f32(p.t{k}, {base} + (int64_t)t.col(ni) * p.t{k}_sn) : 0.f;")
            elif s.kind == "col":
                if hoisted:   # depends on the batch only
                    e(f"const float {c} = evt::ld_f32(p.t{k}, {base});")
                else:
                    ct = DTYPE_CTYPES[s.dtype]
                    e(f"float {c};")
                    e(f"if constexpr (FAST) {c} = evt::buffer_ld_f32<{ct}>(rc_{k}, (Tile::FULL || rok) ? vc_{k} : evt::kOobOffset, (uint32_t)Tile::row_step(mi, v) * cp_{k});")
                    e(f"else {c} = rok ? evt::ld_f32(p.t{k}, {base} + (int64_t)row * p.t{k}_sm) : 0.f;")
            else:
                e(f"const float {c} = evt::ld_f32(p.t{k}, 0);")
        elif n.op == "rres":
            raise NotImplementedError("reduction result used per element")
        else:
            if vn:
                e(f"float {c}[NI];")
                e(f"#pragma unroll\nfor (int ni = 0; ni < NI; ++ni) {c}[ni] = {self.expr(n)};")
            else:
                e(f"const float {c} = {self.expr(n)};")

    def emit_row_reduce(self, e: _Emitter, r):
        o = r.state_offset
        vn = self.var_n[r.input]
        x = self.ref(r.input)
        e("{")
        e.indent()
        if not vn:
            # value constant along n: materialise so the generic code applies
            e(f"float xv[NI];\n#pragma unroll\nfor (int ni = 0; ni < NI; ++ni) xv[ni] = {x};")
            x = "xv[ni]"
        if r.kind == "sum":
            e("float part = 0.f;")
            e(f"#pragma unroll\nfor (int ni = 0; ni < NI; ++ni) part += t.col_ok(ni) ? {x} : 0.f;")
            e(f"rst[{o}] = evt::half_wave_sum(part);")
        elif r.kind == "max":
            e("float part = -INFINITY;")
            e(f"#pragma unroll\nfor (int ni = 0; ni < NI; ++ni) part = t.col_ok(ni) ? fmaxf(part, {x}) : part;")
            e(f"rst[{o}] = evt::half_wave_max(part);")
        elif r.kind == "maxsumexp":
            e("float mx = -INFINITY;")
            e(f"#pragma unroll\nfor (int ni = 0; ni < NI; ++ni) mx = t.col_ok(ni) ? fmaxf(mx, {x}) : mx;")
            e("mx = evt::half_wave_max(mx);")
            e("float se = 0.f;")
            e("const float mxs = mx * evt::kLog2e;")
            e(f"#pragma unroll\nfor (int ni = 0; ni < NI; ++ni) se += t.col_ok(ni) ? evt::op_exp_minus({x}, mxs) : 0.f;")
            e(f"rst[{o}] = mx; rst[{o + 1}] = evt::half_wave_sum(se);")
        elif r.kind == "welford":
            e("const float cnt = wcnt;")
            e("float sx = 0.f;")
            e(f"#pragma unroll\nfor (int ni = 0; ni < NI; ++ni) sx += t.col_ok(ni) ? {x} : 0.f;")
            e("sx = evt::half_wave_sum(sx);")
            e("const float mean = sx * wrcnt;")
            e("float sq = 0.f;")
            e(f"#pragma unroll\nfor (int ni = 0; ni < NI; ++ni) {{ const float d = {x} - mean; sq += t.col_ok(ni) ? d * d : 0.f; }}")
            e(f"rst[{o}] = cnt; rst[{o + 1}] = mean; rst[{o + 2}] = evt::half_wave_sum(sq);")
        e.dedent()
        e("}")

    # -- module -------------------------------------------------------------------
    def module_spec(self) -> dict:
        t = self.spec.tile
        return {
            "abi": ABI_VERSION,
            "name": self.name,
            # what evt_launch_static can hold in place of a workspace (0: these kernels never use one)
            "static_scratch_bytes": STATIC_SCRATCH_BYTES if self.uses_workspace() else 0,
            "tile": asdict(t),
            "a_k_contiguous": self.spec.a_kc,
            "k_multiple_of": self.spec.tile.bk if self.spec.k_exact else 1,   # launches with another K are refused
            "b_k_contiguous": self.spec.b_kc,
            "element": "bf16" if self.spec.bf16 else "f16",
            "batched": self.ir.batched,
            "row_state": self.ir.row_state,
            "col_state": self.ir.col_state,
            "tensors": [{"name": s.name, "role": s.role, "dtype": s.dtype, "kind": s.kind,
                         "domain": s.domain} for s in self.ir.slots],
            "num_scalars": len(self.ir.scalars),
            # scalars[rng_scalars .. +3] = 32-bit patterns of (seed low, seed high, offset, stream id) for rand_like
            "rng_scalars": self.ir.rng_scalar,
        }

    def uses_workspace(self) -> bool:
        """Can a launch of this module need a workspace: cross-tile reductions, or split-K (rings of two or more
        stages outside a walk)?"""
        t = self.spec.tile
        return bool(self.ir.row_state or self.ir.col_state or (t.stages > 1 and t.walk == 1))

    def source(self) -> str:
        ir, sp, t = self.ir, self.spec, self.spec.tile
        e = _Emitter()
        e("// Generated by evt_ae_amd.codegen -- do not edit.")
        e(f"// module {self.name}")
        if self.clock_probe:
            e("#define EVT_CLOCK_PROBE 1")
        e('#include "evt_epilogue.hpp"')
        e('#include "evt_amd.h"')
        e("#include <stdlib.h>")
        e("#include <mutex>")
        e("")
        e("namespace {")
        e("struct Epi {")
        e.indent()
        e(f"static constexpr int ROW_STATE = {ir.row_state};")
        e(f"static constexpr int COL_STATE = {ir.col_state};")
        e(f"static constexpr bool EDGE_TILES = {'true' if sp.edge else 'false'};   // KernelSpec.edge")
        self.emit_params(e)
        self.emit_combine(e, "row")
        self.emit_combine(e, "col")
        self.emit_identity(e, "row")
        self.emit_identity(e, "col")
        self.emit_finalize(e, "row")
        self.emit_finalize(e, "col")
        self.emit_tile(e)
        e.dedent()
        e("};")
        b = lambda x: "true" if x else "false"  # noqa: E731
        tile_io = any((sl.role == "store" and sl.domain == "tile") or (sl.role == "load" and sl.kind == "aux") for sl in ir.slots)
        if t.pipe == 12 and (t.wm * t.wn != 4 or not t.dma or t.stages < 2 or t.walk > 1):
            raise NotImplementedError("the one-wave-per-SIMD loop needs four waves, the 16-byte transfers, two or more "
                                      "stages and one tile per workgroup")
        if t.pipe >= 16:
            mi, ni = t.bm // t.wm // 32, t.bn // t.wn // 32
            if (not 18 <= t.pipe <= 27 or t.wm * t.wn != 8 or t.wm % 2 or not t.dma or t.stages < 2 or t.walk > 1 or t.bk % 32
                    or 2 * mi * ni > 8 or 8 * mi * ni * 4096 > t.lds_bytes()):
                raise NotImplementedError("split k-tiles need a ping-pong loop of eight waves in an even number of rows, "
                                          "loop wave tiles of at most eight 32 x 32 blocks, one tile per workgroup and "
                                          "LDS stages that hold one exchange of the accumulators")
        if t.walk > 1 and (t.pipe < 2 or not t.dma or ir.col_state or not sp.k_exact):
            raise NotImplementedError("a walk over tiles needs a ping-pong pipeline, K a multiple of bk and an epilogue "
                                      "without per-column reduction")
        e(f"using Cfg = evt::GemmCfg<{t.bm}, {t.bn}, {t.bk}, {t.wm}, {t.wn}, {b(sp.a_kc)}, {b(sp.b_kc)}, "
          f"{b(t.dma)}, {t.stages}, {b(sp.bf16)}, {t.group_m}, {t.pipe}, {b(tile_io)}, {b(t.walk > 1)}, {b(sp.k_exact)}>;")
        e(f"constexpr int kNumTensors = {len(ir.slots)};")
        e(f"constexpr int kNumScalars = {len(ir.scalars)};")
        red_lds = reduction_lds_bytes(t, ir.row_state, ir.col_state)
        e(f"static_assert((Cfg::WALK ? Cfg::STAGE_BYTES : Cfg::LDS_BYTES) >= {red_lds}, "
          "\"reduction exchange area exceeds the operand LDS\");")
        e("")
        e("int fill(const EvtArgs* a, evt::GemmArgs& g, Epi::Params& p) {")
        e.indent()
        e("if (!a || !a->A || !a->B) return EVT_ERR_BAD_ARGS;")
        e("if (a->num_tensors != kNumTensors || a->num_scalars != kNumScalars) return EVT_ERR_BAD_ARGS;")
        e("if (a->M <= 0 || a->N <= 0 || a->K <= 0 || a->L <= 0) return EVT_ERR_BAD_ARGS;")
        e("if (a->split_k < 0 || (a->flags & ~(EVT_FLAG_TWO_KERNEL_REDUCE | EVT_FLAG_ROW_WG_PER_CU_MASK))) return EVT_ERR_BAD_ARGS;")
        e("const bool two_kernel_reduce = (a->flags & EVT_FLAG_TWO_KERNEL_REDUCE) != 0;")
        e("g.M = a->M; g.N = a->N; g.K = a->K; g.L = a->L;")
        e("g.A = (const char*)a->A; g.lda = a->lda; g.bsA = a->batch_stride_A;")
        e("g.B = (const char*)a->B; g.ldb = a->ldb; g.bsB = a->batch_stride_B;")
        e("if (a->batch_div_A < 0 || a->batch_div_B < 0 || a->batch_div_A > 0x7fffffff || a->batch_div_B > 0x7fffffff) return EVT_ERR_BAD_ARGS;")
        e("g.bdivA = a->batch_div_A > 1 ? (int)a->batch_div_A : 1; g.bs2A = a->batch_div_A > 1 ? a->batch_stride2_A : 0;")
        e("g.bdivB = a->batch_div_B > 1 ? (int)a->batch_div_B : 1; g.bs2B = a->batch_div_B > 1 ? a->batch_stride2_B : 0;")
        e("g.tiles_m = (a->M + Cfg::BM - 1) / Cfg::BM;")
        e("g.tiles_n = (a->N + Cfg::BN - 1) / Cfg::BN;")
        e("// tiles per workgroup along a row block (Cfg::WALK); the ring needs a full set of k-tiles to carry over")
        e("if (Cfg::K_EXACT && a->K % Cfg::BK) return EVT_ERR_ALIGNMENT;   // this module has no code for a partial k-tile")
        e(f"g.walk = (Cfg::WALK && a->K / Cfg::BK >= Cfg::STAGES) ? {t.walk} : 1;")
        e("g.parts_n = (g.tiles_n + g.walk - 1) / g.walk;")
        e("g.workspace = nullptr;")
        e("g.row_fold_mod = 0; g.row_fold_step = 1; g.row_fold_count = 1;")
        folds = {(r.fold) for r in ir.reduces.values() if r.axis == "row"}
        if folds - {""}:
            # batches fold into one per-row result the way the reduction's output tensor shares elements between them
            (fold,) = folds
            k = next(s_.slot for s_ in ir.stores if s_.domain == "row")
            e(f"{{ const EvtTensorArg& x = a->tensors[{k}];")
            if fold == "mod":
                e("  if (x.l_mod <= 0 || x.l_div != 1 || a->L % x.l_mod) return EVT_ERR_BAD_ARGS;")
                e("  g.row_fold_mod = 1; g.row_fold_step = (int)x.l_mod; g.row_fold_count = a->L / (int)x.l_mod; }")
            else:
                e("  if (x.l_mod != 0 || x.l_div <= 1 || a->L % x.l_div) return EVT_ERR_BAD_ARGS;")
                e("  g.row_fold_count = (int)x.l_div; }")
        e("// few partials: the last workgroup to arrive combines them; many: a finalize kernel does")
        e("g.row_inkernel = (g.parts_n * g.row_fold_count <= evt::kMaxInKernelRowPartials && !two_kernel_reduce && "
          "(int64_t)g.parts_n * a->M * Epi::ROW_STATE * 4 < 0x7fffffffLL) ? 1 : 0;   // the last arriver reads with 32-bit offsets")
        e("g.col_fold_step = 1; g.col_fold_count = 1;")
        col_folds = {r.fold for r in ir.reduces.values() if r.axis == "col"} - {""}
        if col_folds:
            # batches that agree modulo l_mod of the reduction's output tensor fold into one per-column result;
            # few partials are combined by the last workgroup to arrive, many by the finalize kernel
            k = next(s_.slot for s_ in ir.stores if s_.domain == "col")
            e(f"{{ const EvtTensorArg& x = a->tensors[{k}];")
            e("  if (x.l_mod <= 0 || x.l_div != 1 || a->L % x.l_mod) return EVT_ERR_BAD_ARGS;")
            e("  g.col_fold_step = (int)x.l_mod; g.col_fold_count = a->L / (int)x.l_mod;")
            e("}")
        e("g.col_inkernel = (g.tiles_m * g.col_fold_count <= evt::kMaxInKernelPartials && !two_kernel_reduce) ? 1 : 0;")
        e("// Split-K: when the output tiles cannot fill the chip and K is long, several workgroups share a tile")
        e("// (EvtArgs.split_k: 0 = decide here, 1 = off, n = n splits)")
        e("g.splits = 1; g.split_group = 0; g.k_chunk = (a->K + Cfg::BK - 1) / Cfg::BK * Cfg::BK;")
        if t.stages > 1 and t.walk == 1:
            e("{")
            e("  const int want = a->split_k;")
            e("  static const int cus = [] { int dev = 0, n = 0; if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, "
              "hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256; return n; }();")
            e("  const int kt = (a->K + Cfg::BK - 1) / Cfg::BK;")
            e("  const int64_t tiles = (int64_t)g.tiles_m * g.tiles_n * a->L;")
            e("  int s = 1;")
            e("  if (want > 1) s = want < kt ? want : kt;")
            e("  // automatic: small outputs only, a split per CU the tiles leave idle, four k-tiles or more each, while the")
            e("  // exchange stays small -- every split writes a whole fp32 tile and the last arrivers read them back, which")
            e("  // costs more than idle CUs once it runs to megabytes: at most 4 Mi elements over all splits (1024 x 1024 x")
            e("  // 4096 on 128 x 128 tiles measured 22 us with 4 splits, 40 us with 8, 30 us unsplit; 64 x 64 x 736389 takes")
            e("  // a split per CU)")
            e("  else if (want == 0 && tiles * 2 <= cus && kt >= 8 && (int64_t)a->M * a->N * a->L <= (1 << 20)) {")
            e("    s = (int)(cus / tiles); if (s > kt / 4) s = kt / 4;")
            e("    const int64_t cap = (4 << 20) / (tiles * Cfg::BM * Cfg::BN); if (s > cap) s = cap < 1 ? 1 : (int)cap;")
            e("  }")
            e("  if (s >= 2) {")
            e("    const int chunk = (kt + s - 1) / s;")
            e("    g.splits = (kt + chunk - 1) / chunk;      // every split has work")
            e("    g.k_chunk = chunk * Cfg::BK;")
            e("    // more than 16 splits meet in groups first: nobody reads more than 16 + 16 tiles alone")
            e("    if (g.splits > 16) g.split_group = g.splits > 128 ? 16 : (g.splits + 7) / 8 < 4 ? 4 : (g.splits + 7) / 8;")
            e("  }")
            e("}")
        e("if ((int64_t)g.tiles_m * g.tiles_n * a->L * g.splits > 0x7fffffffLL) return EVT_ERR_RANGE;")
        e("if (a->N > (1 << 24)) return EVT_ERR_RANGE;   // column indices are carried as fp32")
        e("// a row's partial state is addressed with a 32-bit buffer offset inside its (batch, part) block")
        e("if (Epi::ROW_STATE > 0 && (int64_t)a->M * Epi::ROW_STATE * 4 >= 0x7fffffffLL) return EVT_ERR_RANGE;")
        if t.stages == 1:
            e("if (a->K > Cfg::BK) return EVT_ERR_RANGE;   // single-stage variant: K must fit one tile")
        if t.dma:
            e("// fast path: 16-byte global->LDS transfers, buffer range check for the tails")
            e("if (((uintptr_t)a->A | (uintptr_t)a->B) & 15) return EVT_ERR_ALIGNMENT;")
            e("if ((a->lda | a->ldb | a->batch_stride_A | a->batch_stride_B | g.bs2A | g.bs2B) & 7) return EVT_ERR_ALIGNMENT;")
            if sp.a_kc:
                e("if (a->K & 7) return EVT_ERR_ALIGNMENT;")
                e("if ((int64_t)Cfg::BM * a->lda * 2 >= 0x7fffffffLL) return EVT_ERR_RANGE;")
            else:
                e("// whole 8-element chunks are read along M: rows padded to a multiple of 8 make room for the last one")
                e("if ((a->M & 7) && a->lda < ((a->M + 7) & ~(int64_t)7)) return EVT_ERR_ALIGNMENT;")
                e("if ((int64_t)Cfg::BK * a->lda * 2 >= 0x7fffffffLL) return EVT_ERR_RANGE;")
            if sp.b_kc:
                e("if (a->K & 7) return EVT_ERR_ALIGNMENT;")
                e("if ((int64_t)Cfg::BN * a->ldb * 2 >= 0x7fffffffLL) return EVT_ERR_RANGE;")
            else:
                e("if ((a->N & 7) && a->ldb < ((a->N + 7) & ~(int64_t)7)) return EVT_ERR_ALIGNMENT;")
                e("if ((int64_t)Cfg::BK * a->ldb * 2 >= 0x7fffffffLL) return EVT_ERR_RANGE;")
        for k, s in enumerate(ir.slots):
            ct = DTYPE_CTYPES[s.dtype]
            e(f"{{ const EvtTensorArg& x = a->tensors[{k}];")
            if s.kind == "rand":   # generated values: no storage behind this slot
                e("  if (x.l_div <= 0 || x.l_mod < 0) return EVT_ERR_BAD_ARGS;")
            else:
                e("  if (!x.ptr || x.l_div <= 0 || x.l_mod < 0) return EVT_ERR_BAD_ARGS;")
            e(f"  p.t{k} = ({'const ' if s.role == 'load' else ''}{ct}*)x.ptr;")
            e(f"  p.t{k}_sl = x.stride_l; p.t{k}_sl2 = x.stride_l2; p.t{k}_sm = x.stride_m; p.t{k}_sn = x.stride_n; "
              f"p.t{k}_ld = (int)x.l_div; p.t{k}_lm = (int)x.l_mod;")
            e(f"  p.t{k}_vec = (x.stride_n == 1 ? 1 : 0) | ((x.stride_n == 1 && ((uintptr_t)x.ptr % (sizeof({ct}) * Cfg::NI)) == 0 && "
              f"x.stride_m % Cfg::NI == 0 && x.stride_l % Cfg::NI == 0 && x.stride_l2 % Cfg::NI == 0) ? 2 : 0); }}")
        e("for (int i = 0; i < kNumScalars; ++i) p.s[i] = a->scalars[i];")
        tile_slots = [k for k, sl in enumerate(ir.slots)
                      if (sl.role == "store" and sl.domain == "tile") or (sl.role == "load" and sl.kind == "aux")]
        col_slots = [k for k, sl in enumerate(ir.slots) if sl.role == "load" and sl.kind == "col"]
        cond = " && ".join(
            [f"(p.t{k}_vec & 1) && (!(Cfg::ADJACENT && sizeof(*p.t{k}) == 2 && (Cfg::NI == 2 || Cfg::NI == 4 || Cfg::NI == 8)) || (p.t{k}_vec & 2))"
             f" && p.t{k}_sm >= 0 && p.t{k}_sm < (1 << 20)"
             for k in tile_slots] +
            [f"p.t{k}_sm >= 0 && p.t{k}_sm < (1 << 20)" for k in col_slots]) or "true"
        e(f"p.fast = ({cond}) ? 1 : 0;")
        e("return EVT_OK;")
        e.dedent()
        e("}")
        e("}  // namespace")
        e("")
        e('extern "C" int evt_abi_version(void) { return EVT_ABI_VERSION; }')
        spec_json = json.dumps(self.module_spec(), sort_keys=True)
        e(f'extern "C" const char* evt_module_spec(void) {{ return R"evtjson({spec_json})evtjson"; }}')
        e('extern "C" int64_t evt_workspace_bytes(const EvtArgs* a) {')
        e("  evt::GemmArgs g; Epi::Params p;")
        e("  const int rc = fill(a, g, p);")
        e("  if (rc != EVT_OK) return rc;")
        e("  return evt::ws_layout_split<Cfg, Epi::ROW_STATE, Epi::COL_STATE>(g).total();")
        e("}")
        e('extern "C" int evt_workspace_init(void* ws, int64_t bytes, void* stream) {')
        e("  if (bytes <= 0) return EVT_OK;")
        e("  if (!ws || (bytes & 3)) return EVT_ERR_WORKSPACE;")
        e("  // arrival counters start at zero (a fill kernel, so the call can be captured in a graph)")
        e("  hipLaunchKernelGGL(evt::evt_fill_zero_kernel, dim3(64), dim3(256), 0, (hipStream_t)stream, (uint32_t*)ws, bytes / 4);")
        e("  return (int)hipGetLastError();")
        e("}")
        e("static int enqueue(evt::GemmArgs& g, const Epi::Params& p, void* ws, void* stream) {")
        e("  g.workspace = (char*)ws;")
        e("  const unsigned grid = (unsigned)((int64_t)g.tiles_m * g.parts_n * g.L * g.splits);")
        e("  hipLaunchKernelGGL((evt::evt_gemm_kernel<Cfg, Epi>), dim3(grid), dim3(Cfg::THREADS), 0, (hipStream_t)stream, g, p);")
        e("  const int err = (int)hipGetLastError();")
        e("  if (err != 0) return err;")
        e("  return evt::launch_finalize<Epi>(p, g, (hipStream_t)stream);")
        e("}")
        e('extern "C" int evt_launch(const EvtArgs* a, void* ws, int64_t ws_bytes, void* stream) {')
        e("  evt::GemmArgs g; Epi::Params p;")
        e("  const int rc = fill(a, g, p);")
        e("  if (rc != EVT_OK) return rc;")
        e("  const int64_t need = evt::ws_layout_split<Cfg, Epi::ROW_STATE, Epi::COL_STATE>(g).total();")
        e("  if (need > 0 && (!ws || ws_bytes < need || ((uintptr_t)ws & 15))) return EVT_ERR_WORKSPACE;   // 16-byte aligned")
        e("  return enqueue(g, p, ws, stream);")
        e("}")
        emit_static_scratch(e, self.uses_workspace())
        e('extern "C" int evt_launch_static(const EvtArgs* a, void* stream) {')
        e("  evt::GemmArgs g; Epi::Params p;")
        e("  const int rc = fill(a, g, p);")
        e("  if (rc != EVT_OK) return rc;")
        e("  const evt::WsLayout wl = evt::ws_layout_split<Cfg, Epi::ROW_STATE, Epi::COL_STATE>(g);")
        e("  const int64_t need = wl.total();")
        e("  if (need > kScratchBytes) return EVT_ERR_SCRATCH;   // this problem's partial results do not fit the static array")
        e("  void* ws = nullptr;")
        e("  if (need > 0) {")
        e("    const int rs = scratch_for_stream(stream, &ws);")
        e("    if (rs != EVT_OK) return rs;")
        e("    // The array keeps the last call's contents, and another problem size lays its counters out elsewhere:")
        e("    // the arrival counters of this launch start at zero (fill kernels, not memset nodes).  Partial results")
        e("    // and split-K tiles are written by every launch before it reads them and need no clearing.")
        e("    const int64_t regions[2][2] = {{0, wl.counter_bytes}, {wl.counter_bytes + wl.row_bytes + wl.col_bytes, wl.split_counter_bytes}};")
        e("    for (const auto& r : regions) {")
        e("      if (r[1] <= 0) continue;")
        e("      const unsigned blocks = (unsigned)((r[1] / 4 + 255) / 256 < 64 ? (r[1] / 4 + 255) / 256 : 64);")
        e("      hipLaunchKernelGGL(evt::evt_fill_zero_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (uint32_t*)((char*)ws + r[0]), r[1] / 4);")
        e("      const int ef = (int)hipGetLastError();")
        e("      if (ef != 0) return ef;")
        e("    }")
        e("  }")
        e("  return enqueue(g, p, ws, stream);")
        e("}")
        if self.clock_probe:
            e("// out[0..3] = main-loop shader cycles, main-loop 100 MHz ticks, epilogue shader cycles, epilogue ticks")
            e("// of workgroup 0 in the most recent launch (synchronises the device)")
            e('extern "C" int evt_clock_probe_read(uint64_t* out) {')
            e("  return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(evt::evt_clock_probe), 4 * sizeof(uint64_t));")
            e("}")
        return e.text()


@dataclass(frozen=True)
class RowSpec:
    """Row-wise reduce-apply anchor (csrc/evt_rowwise.hpp): which anchor, how a
    row is spread over a wave, and the element type of the anchor operands.
    The analogue of the reference's (rows_per_cta, warp_count, cache_input)
    tuple (python/gtl/compiler/autotuner/softmax_tuner.py)."""
    op: str             # "softmax" | "softmax_backward" | "layernorm" | "layernorm_backward"
    ch: int             # chunks of lpr * wpr * 8 columns cached per lane
    lpr: int            # lanes per row inside a wave (power of two, <= 64)
    elt: str            # "f16" | "bf16" | "f32"
    wpr: int = 1        # waves per row (power of two, <= 16; above 1 a workgroup holds one row)

    OPS = ("softmax", "softmax_backward", "layernorm", "layernorm_backward")

    def tag(self) -> str:
        return f"{self.op}_{self.elt}_ch{self.ch}_lpr{self.lpr}" + (f"_w{self.wpr}" if self.wpr > 1 else "")

    @property
    def max_n(self) -> int:
        return self.ch * self.lpr * self.wpr * 8

    @staticmethod
    def registers(op: str, elt: str, ch: int, lookahead: bool, col_state: int = 0) -> float:
        """Registers per lane that hold row data: the fp32 working copies (two
        for the backward anchors), the operands as loaded, twice when the next
        row is fetched ahead, layer norm backward's weight, and the partials
        of the epilogue's per-column reductions (`col_state` words per column)."""
        two = 2 if op in ("softmax_backward", "layernorm_backward") else 1
        weight = ch * 8 if op == "layernorm_backward" else 0      # this lane's columns of the weight, kept across rows
        return ch * 8 * two * (1 + (1.0 if elt == "f32" else 0.5) * (2 if lookahead else 1)) + weight + col_state * ch * 8

    @staticmethod
    def for_row_length(op: str, n: int, elt: str, col_state: int = 0) -> "RowSpec":
        """Smallest lane group that holds the row in two chunks per lane (four
        for softmax), a full wave with up to 16 chunks for longer rows.  Rows longer
        than 8192 go over 2 .. 16 waves, as few as keep the row data within
        three quarters of the registers a lane can have at that workgroup size
        (16 waves: 128 registers and no fetch ahead)."""
        # softmax holds one operand and little else: four chunks per lane, so more rows per wave, measured 12 %
        # faster on 512-wide rows; the anchors with two operands or two reductions lose with more than two
        per_lane = 4 if op == "softmax" else 2
        lpr = 8
        while lpr < 64 and (n + lpr * 8 - 1) // (lpr * 8) > per_lane:
            lpr *= 2
        ch = (n + lpr * 8 - 1) // (lpr * 8)
        if ch <= 16:
            return RowSpec(op, ch, lpr, elt)
        for wpr, budget in ((2, 192), (4, 192), (8, 192), (16, 96)):
            ch = (n + wpr * 512 - 1) // (wpr * 512)
            if ch <= 16 and RowSpec.registers(op, elt, ch, wpr < 16, col_state) <= budget:
                return RowSpec(op, ch, 64, elt, wpr)
        raise NotImplementedError(f"rows of {n} {elt} elements do not fit the register-cached {op} kernel")


class RowCodegen(Codegen):
    """EpilogueIR behind a row-wise anchor -> one kernel module with the same
    five C entry points as the GEMM modules.  The generated `Epi::row()` walks
    this lane's chunks of 8 columns; values that do not vary along the row are
    computed once in front of the chunk loop."""

    def __init__(self, ir: EpilogueIR, spec: RowSpec, module_name: str):
        super().__init__(ir, None, module_name)
        self.row_spec = spec
        for r in ir.reduces.values():
            # a sum / max over all rows is carried in registers and combined in two phases; a reduction along
            # the row would be a second pass over the anchor's own axis
            if r.axis != "col" or r.kind not in ("sum", "max"):
                raise NotImplementedError(f"per-row reduction {r.name} behind a row-wise anchor")
        if ir.col_state and ir.L != 1:
            raise NotImplementedError("per-column reduction behind a row-wise anchor: the rows must form one batch")
        if ir.col_state and spec.wpr == 1 and ir.col_state * spec.ch * spec.lpr * 8 * 4 > 65536:
            raise NotImplementedError("per-column reduction behind a row-wise anchor: the waves' partials of a row of "
                                      f"{spec.max_n} elements do not fit the LDS")
        if ir.col_state and spec.wpr > 1:
            # a row over several waves: every lane carries the partials of its own columns in registers, next to
            # the row data (three quarters of the lane's registers at most, as for the row data alone)
            budget = 96 if spec.wpr == 16 else 192
            if RowSpec.registers(spec.op, spec.elt, spec.ch, spec.wpr < 16, ir.col_state) > budget:
                raise NotImplementedError("per-column reduction behind a row-wise anchor: the partials of a row of "
                                          f"{spec.max_n} elements over {spec.wpr} waves do not fit the registers")
        # a kernel that reduces over the rows runs 8 waves per workgroup: as many rows in flight per CU from half
        # the workgroups, so half the partials for the second phase (16 waves would cap a wave at 128 registers,
        # which spills the layer norm backward kernel)
        self.waves = spec.wpr if spec.wpr > 1 else (8 if ir.col_state else 4)
        for n in ir.nodes.values():
            if n.op == "colidx":
                raise NotImplementedError(f"{n.op} behind a row-wise anchor")
        self.anchor_values = 1 + max([n.comp for n in ir.nodes.values() if n.op == "anchorval"], default=-1)
        # [N] vectors shared by every row (weight, bias, ...): read once per wave, not once per row
        self.hoisted = [n.name for n in ir.nodes.values() if n.op == "load" and ir.slots[n.slot].kind == "row"
                        and ir.slots[n.slot].strides.stride_l == 0 and n.slot not in ir.anchor_slots]
        if spec.wpr > 1 or spec.ch * len(self.hoisted) > 8:
            # long rows: the registers (8 per chunk and vector) go to the row itself; next to 4 KB and more of row
            # data per lane group the vectors' trip from L2 once per row is small
            self.hoisted = []

    def slot_row_off(self, k: int) -> str:
        return f"o_{k}"

    def emit_row(self, e: _Emitter):
        ir = self.ir
        tile_stores = [s for s in ir.stores if s.domain == "tile"]
        row_stores = [s for s in ir.stores if s.domain == "row"]
        col_reds = list(ir.reduces.values())
        need = ir.closure([s.input for s in tile_stores + row_stores] + [r.input for r in col_reds])
        outer = [n for n in need if not self.var_n[n]]
        inner = [n for n in need if self.var_n[n]]
        nh = len(self.hoisted)
        e(f"static constexpr int NH = {nh};   // row vectors kept in registers across the rows of a wave")
        e("template <class Cfg, int FAST, class Ctx>")
        e(f"static EVT_DEV void hoist(const Params& p, const Ctx& t, float (&hz)[{max(nh, 1)}][Cfg::CH][8]) {{")
        e.indent()
        if nh:
            e("#pragma unroll")
            e("for (int c = 0; c < Cfg::CH; ++c) {")
            e.indent()
            e("const int nv = t.valid(c);")
            e("const int n0 = t.col0(c);")
            for i, name in enumerate(self.hoisted):
                k = ir.nodes[name].slot
                e("if (nv > 0) {")
                e(f"  if (FAST == 2 || (FAST == 1 && nv == 8)) evt::load8v(p.t{k} + n0, hz[{i}][c]);")
                e(f"  else evt::load8s(p.t{k} + (int64_t)n0 * p.t{k}_sn, p.t{k}_sn, p.t{k}_vec != 0, nv, hz[{i}][c]);")
                e("} else {")
                e(f"  #pragma unroll\n  for (int j = 0; j < 8; ++j) hz[{i}][c][j] = 0.f;")
                e("}")
            e.dedent()
            e("}")
        e("(void)p; (void)t; (void)hz;")
        e.dedent()
        e("}")
        e("template <class Cfg, int FAST, class Ctx>")
        e(f"static EVT_DEV void row(const Params& p, const Ctx& t, const float (&acc)[Cfg::CH][8], const float (&rv)[2], "
          f"const float (&av)[{max(self.anchor_values, 1)}][Cfg::CH][8], "
          f"const float (&hz)[{max(nh, 1)}][Cfg::CH][8], float (&cst)[{max(ir.col_state, 1)}][Cfg::CH][8], "
          f"float (&rsv)[{max(len(row_stores), 1)}]) {{")
        e.indent()
        for k, s in enumerate(ir.slots):
            # a single batch (the common 2-D case) needs none of batch_offset's divisions
            e(f"const int64_t o_{k} = (t.L == 1 ? (int64_t)0 : evt::batch_offset(t.l, p.t{k}_lm, p.t{k}_ld, p.t{k}_sl, p.t{k}_sl2)) + (int64_t)t.m * p.t{k}_sm;")
        # one row per wave: its tensors' rows as buffer resources (chunk_body(buffer=True))
        buffered = sorted({ir.nodes[n].slot for n in inner if ir.nodes[n].op == "load" and n not in self.hoisted
                           and ir.slots[ir.nodes[n].slot].kind != "rand"} | {s_.slot for s_ in tile_stores})
        for k in buffered:
            e(f"[[maybe_unused]] __amdgpu_buffer_rsrc_t rs_{k};")
            e(f"if constexpr (FAST == 2 && Cfg::RPW == 1) rs_{k} = evt::make_rsrc(evt::wave_uniform(p.t{k} + o_{k}));")
        for name in outer:
            n = ir.nodes[name]
            c = _cname(name)
            if n.op == "imm":
                e(f"const float {c} = p.s[{n.slot}];")
            elif n.op == "rowval":
                e(f"const float {c} = rv[{n.comp}];")
            elif n.op == "load":
                e(f"const float {c} = evt::ld_f32(p.t{n.slot}, o_{n.slot});")
            elif n.op == "accum":
                raise NotImplementedError("accumulator used as a per-row value")
            else:
                e(f"const float {c} = {self.expr(n, 'j')};")
        e("#pragma unroll")
        e("for (int c = 0; c < Cfg::CH; ++c) {")
        e.indent()
        e("const int nv = t.valid(c);")
        e("const int n0 = t.col0(c);")

        def chunk_body(vector: bool, buffer: bool = False):
            """The epilogue on this lane's 8 columns of chunk c: whole groups through 16-byte accesses (check-free
            instantiation only), the group that straddles the row end element by element."""
            for name in inner:
                n = ir.nodes[name]
                c = _cname(name)
                e(f"float {c}[8];")
                if n.op == "accum":
                    e(f"#pragma unroll\nfor (int j = 0; j < 8; ++j) {c}[j] = acc[c][j];")
                elif n.op == "anchorval":
                    e(f"#pragma unroll\nfor (int j = 0; j < 8; ++j) {c}[j] = av[{n.comp}][c][j];")
                elif n.op == "load" and ir.slots[n.slot].kind == "rand":
                    k, r = n.slot, ir.rng_scalar
                    e(f"evt::rand8((uint64_t)__builtin_bit_cast(uint32_t, p.s[{r}]) | ((uint64_t)__builtin_bit_cast(uint32_t, p.s[{r + 1}]) << 32), "
                      f"__builtin_bit_cast(uint32_t, p.s[{r + 2}]), {k}u + 16u * __builtin_bit_cast(uint32_t, p.s[{r + 3}]), o_{k} + (int64_t)n0 * p.t{k}_sn, p.t{k}_sn, {c});")
                elif n.op == "load" and name in self.hoisted:
                    e(f"#pragma unroll\nfor (int j = 0; j < 8; ++j) {c}[j] = hz[{self.hoisted.index(name)}][c][j];")
                elif n.op == "load":
                    k = n.slot
                    if buffer:
                        e(f"evt::load8v_b<std::remove_cv_t<std::remove_pointer_t<decltype(p.t{k})>>>(rs_{k}, "
                          f"nv > 0 ? (uint32_t)n0 * (uint32_t)sizeof(*p.t{k}) : evt::kOobOffset, {c});")
                    elif vector:
                        e(f"evt::load8v(p.t{k} + o_{k} + n0, {c});")
                    else:
                        e(f"evt::load8s(p.t{k} + o_{k} + (int64_t)n0 * p.t{k}_sn, p.t{k}_sn, p.t{k}_vec != 0, nv, {c});")
                else:
                    e(f"#pragma unroll\nfor (int j = 0; j < 8; ++j) {c}[j] = {self.expr(n, 'j')};")
            for s in tile_stores:
                k = s.slot
                src = _cname(s.input)
                if not self.var_n[s.input]:
                    e(f"float b_{k}[8];\n#pragma unroll\nfor (int j = 0; j < 8; ++j) b_{k}[j] = {src};")
                    src = f"b_{k}"
                if buffer:
                    e(f"evt::store8v_b<std::remove_pointer_t<decltype(p.t{k})>>(rs_{k}, "
                      f"nv > 0 ? (uint32_t)n0 * (uint32_t)sizeof(*p.t{k}) : evt::kOobOffset, {src});")
                elif vector:
                    e(f"evt::store8v(p.t{k} + o_{k} + n0, {src});")
                else:
                    e(f"evt::store8s(p.t{k} + o_{k} + (int64_t)n0 * p.t{k}_sn, p.t{k}_sn, p.t{k}_vec != 0, nv, {src});")
            for r in col_reds:
                x = f"{_cname(r.input)}[j]" if self.var_n[r.input] else _cname(r.input)
                o = r.state_offset
                e("#pragma unroll")
                if r.kind == "sum":
                    e(f"for (int j = 0; j < 8; ++j) cst[{o}][c][j] += j < nv ? {x} : 0.f;")
                else:
                    e(f"for (int j = 0; j < 8; ++j) cst[{o}][c][j] = j < nv ? fmaxf(cst[{o}][c][j], {x}) : cst[{o}][c][j];")

        # FAST 2: every group is whole; FAST 1: whole groups and the one that straddles the row end; 0: generic
        e("if constexpr (FAST == 2 && Cfg::RPW == 1) {")
        e.indent()
        chunk_body(True, buffer=True)      # every lane, no branch: lanes without columns are dropped by the range check
        e.dedent()
        e("} else if constexpr (FAST == 2) {")
        e.indent()
        e("if (nv > 0) {")
        e.indent()
        chunk_body(True)
        e.dedent()
        e("}")
        e.dedent()
        e("} else {")
        e.indent()
        e("if (FAST == 1 && nv == 8) {")
        e.indent()
        chunk_body(True)
        e.dedent()
        e("} else if (nv > 0) {")
        e.indent()
        chunk_body(False)
        e.dedent()
        e("}")
        e.dedent()
        e("}")
        e.dedent()
        e("}")
        # one value per row (mean, rstd, ...): handed back to the kernel, which collects the values of the rows a
        # wave visits and stores them together (row_store_one below)
        for i, s in enumerate(row_stores):
            if self.var_n[s.input]:
                raise NotImplementedError("per-row output of a per-element value")
            e(f"rsv[{i}] = {_cname(s.input)};")
        e("(void)p; (void)t; (void)acc; (void)rv; (void)av; (void)hz; (void)cst; (void)rsv;")
        e.dedent()
        e("}")
        e(f"static constexpr int NRS = {len(row_stores)};   // per-row outputs")
        esize = {"f16": 2, "bf16": 2, "f32": 4, "i32": 4, "i64": 8, "bool": 1, "u8": 1, "i8": 1}
        nst = sum(max(1, esize[ir.slots[s_.slot].dtype] // 2) for s_ in tile_stores)
        e("// store instructions row() issues per chunk of a row when every lane stores without a branch (16 bytes each)")
        e(f"static constexpr int CHUNK_STORES = {nst};")
        e("// per-row output number i of row (l, m); L: number of batches")
        e("static EVT_DEV void row_store_one(const Params& p, int L, int l, int m, int i, float v) {")
        e.indent()
        for i, s in enumerate(row_stores):
            k = s.slot
            e(f"if (i == {i}) evt::st_f32(p.t{k}, (L == 1 ? (int64_t)0 : evt::batch_offset(l, p.t{k}_lm, p.t{k}_ld, p.t{k}_sl, p.t{k}_sl2)) + (int64_t)m * p.t{k}_sm, v);")
        e("(void)p; (void)L; (void)l; (void)m; (void)i; (void)v;")
        e.dedent()
        e("}")

    def module_spec(self) -> dict:
        sp = self.row_spec
        return {
            "abi": ABI_VERSION,
            "name": self.name,
            # what evt_launch_static can hold in place of a workspace (0: this kernel never uses one)
            "static_scratch_bytes": STATIC_SCRATCH_BYTES if self.ir.col_state else 0,
            "anchor": sp.op,
            "row": {"chunks": sp.ch, "lanes_per_row": sp.lpr * sp.wpr, "waves_per_row": sp.wpr, "max_n": sp.max_n},
            "element": sp.elt,
            "batched": self.ir.batched,
            "row_state": 0,
            "col_state": self.ir.col_state,
            "tensors": [{"name": s.name, "role": s.role, "dtype": s.dtype, "kind": s.kind,
                         "domain": s.domain} for s in self.ir.slots],
            "num_scalars": len(self.ir.scalars),
            "rng_scalars": self.ir.rng_scalar,
            # scalars[anchor_scalars] = eps of a layer norm anchor
            "anchor_scalars": self.ir.anchor_scalar,
            # layer norm backward: tensor slots of the forward pass's mean and rstd
            "anchor_tensors": list(self.ir.anchor_slots),
        }

    def source(self) -> str:
        ir, sp = self.ir, self.row_spec
        op_id = RowSpec.OPS.index(sp.op)
        elt_id = {"f16": 0, "bf16": 1, "f32": 2}[sp.elt]
        two = sp.op in ("softmax_backward", "layernorm_backward")
        stats = sp.op == "layernorm_backward"
        e = _Emitter()
        e("// Generated by evt_ae_amd.codegen -- do not edit.")
        e(f"// module {self.name}")
        e('#include "evt_rowwise.hpp"')
        e('#include "evt_amd.h"')
        e("#include <stdlib.h>")
        e("#include <mutex>")
        e("")
        e("namespace {")
        e("struct Epi {")
        e.indent()
        e(f"static constexpr int COL_STATE = {ir.col_state};")
        self.emit_params(e)
        self.emit_combine(e, "col")
        self.emit_identity(e, "col")
        self.emit_finalize(e, "col")
        self.emit_row(e)
        e.dedent()
        e("};")
        e(f"using Cfg = evt::RowCfg<{op_id}, {sp.ch}, {sp.lpr}, {elt_id}, {self.anchor_values}, {self.waves}, {sp.wpr}>;")
        e(f"constexpr int kNumTensors = {len(ir.slots)};")
        e(f"constexpr int kNumScalars = {len(ir.scalars)};")
        e(f"constexpr int kEltBytes = {4 if sp.elt == 'f32' else 2};")
        e("int fill(const EvtArgs* a, evt::RowArgs& g, Epi::Params& p) {")
        e.indent()
        e("if (!a || !a->A) return EVT_ERR_BAD_ARGS;")
        if two:
            e("if (!a->B) return EVT_ERR_BAD_ARGS;")
        e("if (a->num_tensors != kNumTensors || a->num_scalars != kNumScalars) return EVT_ERR_BAD_ARGS;")
        e("if (a->M <= 0 || a->N <= 0 || a->L <= 0) return EVT_ERR_BAD_ARGS;")
        e("if (a->N > Cfg::CH * Cfg::SPAN) return EVT_ERR_RANGE;       // the row must fit this module's register cache")
        e("if (((int64_t)a->L * a->M + Cfg::ROWS - 1) / Cfg::ROWS > 0x7fffffffLL) return EVT_ERR_RANGE;")
        e("g.M = a->M; g.N = a->N; g.L = a->L;")
        e("g.A = (const char*)a->A; g.lda = a->lda; g.bsA = a->batch_stride_A;")
        e("g.B = (const char*)a->B; g.ldb = a->ldb; g.bsB = a->batch_stride_B;")
        e("if (a->lda < a->N) return EVT_ERR_BAD_ARGS;")
        e("// 16-byte accesses need dword alignment only")
        e("g.vecA = (((uintptr_t)a->A | (uintptr_t)(a->lda * kEltBytes) | (uintptr_t)(a->batch_stride_A * kEltBytes)) & 3) == 0;")
        e("g.vecB = (((uintptr_t)a->B | (uintptr_t)(a->ldb * kEltBytes) | (uintptr_t)(a->batch_stride_B * kEltBytes)) & 3) == 0;")
        e("g.mean = nullptr; g.rstd = nullptr; g.gamma = nullptr; g.vecG = 0; g.colws = nullptr;")
        if ir.col_state:
            e("if (a->L != 1) return EVT_ERR_BAD_ARGS;      // the per-column reductions run over every row")
        e(f"g.fast = (g.vecA && {'g.vecB && ' if two else ''}a->N >= 8) ? ((a->N & 7) == 0 ? 2 : 1) : 0;")
        e(f"g.eps = {'a->scalars[%d]' % ir.anchor_scalar if ir.anchor_scalar is not None else '0.f'};")
        if stats:
            # the forward statistics are two fp32 load slots with one value per row, contiguous over all rows
            km, kr = ir.anchor_slots[:2]
            e(f"if (!a->tensors[{km}].ptr || !a->tensors[{kr}].ptr) return EVT_ERR_BAD_ARGS;")
            e(f"if (a->tensors[{km}].stride_m != 1 || a->tensors[{kr}].stride_m != 1) return EVT_ERR_BAD_ARGS;")
            e(f"g.mean = (const float*)a->tensors[{km}].ptr; g.rstd = (const float*)a->tensors[{kr}].ptr;")
            if len(ir.anchor_slots) > 2:     # the weight, applied to the incoming gradient
                kg = ir.anchor_slots[2]
                e(f"if (!a->tensors[{kg}].ptr || a->tensors[{kg}].stride_n != 1) return EVT_ERR_BAD_ARGS;")
                e(f"g.gamma = (const char*)a->tensors[{kg}].ptr; g.vecG = ((uintptr_t)g.gamma & 3) == 0;")
        for k, s in enumerate(ir.slots):
            ct = DTYPE_CTYPES[s.dtype]
            e(f"{{ const EvtTensorArg& x = a->tensors[{k}];")
            if s.kind == "rand":   # generated values: no storage behind this slot
                e("  if (x.l_div <= 0 || x.l_mod < 0) return EVT_ERR_BAD_ARGS;")
            else:
                e("  if (!x.ptr || x.l_div <= 0 || x.l_mod < 0) return EVT_ERR_BAD_ARGS;")
            e(f"  p.t{k} = ({'const ' if s.role == 'load' else ''}{ct}*)x.ptr;")
            e(f"  p.t{k}_sl = x.stride_l; p.t{k}_sl2 = x.stride_l2; p.t{k}_sm = x.stride_m; p.t{k}_sn = x.stride_n; "
              f"p.t{k}_ld = (int)x.l_div; p.t{k}_lm = (int)x.l_mod;")
            e(f"  p.t{k}_vec = (x.stride_n == 1 && (((uintptr_t)x.ptr | (uintptr_t)(x.stride_m * (int64_t)sizeof({ct})) | "
              f"(uintptr_t)(x.stride_l * (int64_t)sizeof({ct})) | (uintptr_t)(x.stride_l2 * (int64_t)sizeof({ct}))) & 3) == 0) ? 1 : 0; }}")
        for name in self.hoisted:
            k = ir.nodes[name].slot
            e(f"if (a->tensors[{k}].stride_l != 0 || a->tensors[{k}].stride_m != 0) return EVT_ERR_BAD_ARGS;   // read once per wave")
        e("for (int i = 0; i < kNumScalars; ++i) p.s[i] = a->scalars[i];")
        # slots read or written per element (their kind says they vary along the row; strides are run-time values)
        vec_slots = [k for k, sl in enumerate(ir.slots) if k not in ir.anchor_slots and
                     ((sl.role == "load" and sl.kind in ("aux", "row")) or (sl.role == "store" and sl.domain == "tile"))]
        cond = " && ".join(f"p.t{k}_vec" for k in vec_slots) or "1"
        e(f"p.fast = ({cond}) ? g.fast : 0;   // every per-element tensor of the epilogue is unit-stride and dword aligned too")
        e("return EVT_OK;")
        e.dedent()
        e("}")
        e("}  // namespace")
        e("")
        e('extern "C" int evt_abi_version(void) { return EVT_ABI_VERSION; }')
        spec_json = json.dumps(self.module_spec(), sort_keys=True)
        e(f'extern "C" const char* evt_module_spec(void) {{ return R"evtjson({spec_json})evtjson"; }}')
        e("// workgroups per CU before waves start walking over several rows (0: one pass, a workgroup per Cfg::ROWS rows);")
        e("// walking pays when row vectors are kept in registers across the rows of a wave, and bounds the number of")
        e("// partials of a per-column reduction")
        has_row_outputs = any(s_.domain == "row" for s_ in ir.stores)
        # per-row outputs leave in batches only when a wave visits several consecutive rows (measured on a layer norm
        # over 131072 x 1024: 128 us with a workgroup per four rows, 107 / 102.5 / 107 us with 16 / 32 / 48
        # workgroups per CU)
        default_cap = 4 if ir.col_state else (32 if has_row_outputs else (16 if self.hoisted else 0))
        if 1 < sp.wpr < 16:
            # a row per workgroup: 8 waves per CU walk over the rows, each fetching its next row ahead (measured
            # on 4096 x 30528: 100 us against 108 us with a workgroup per row)
            default_cap = 8 // sp.wpr
        e("static unsigned grid_for(const evt::RowArgs& g, int flags) {")
        e("  // EvtArgs.flags carries the caller's choice (EVT_FLAG_ROW_WG_PER_CU); the module reads no environment")
        e(f"  int per_cu = (flags & EVT_FLAG_ROW_WG_PER_CU_MASK) ? ((flags & EVT_FLAG_ROW_WG_PER_CU_MASK) >> 8) - 1 : {default_cap};")
        e("  static const int cus = [] { int dev = 0, n = 0; if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, "
          "hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256; return n; }();")
        if ir.col_state:
            e("  if (per_cu <= 0) per_cu = 4;   // a per-column reduction needs a bounded number of partials")
        e("  const int64_t want = ((int64_t)g.L * g.M + Cfg::ROWS - 1) / Cfg::ROWS;")
        e("  return (unsigned)((per_cu <= 0 || want < (int64_t)cus * per_cu) ? want : (int64_t)cus * per_cu);")
        e("}")
        e('extern "C" int64_t evt_workspace_bytes(const EvtArgs* a) {')
        e("  evt::RowArgs g; Epi::Params p;")
        e("  const int rc = fill(a, g, p);")
        e("  if (rc != EVT_OK) return rc;")
        e("  // partials of the per-column reductions, one per (workgroup, state word, column); nothing else is staged")
        e("  return (int64_t)grid_for(g, a->flags) * Epi::COL_STATE * g.N * 4;")
        e("}")
        e('extern "C" int evt_workspace_init(void* ws, int64_t bytes, void* stream) {')
        e("  (void)ws; (void)bytes; (void)stream;      // no counters: every partial is written before it is read")
        e("  return EVT_OK;")
        e("}")
        e("static int enqueue(evt::RowArgs& g, const Epi::Params& p, unsigned grid, void* ws, void* stream);")
        e('extern "C" int evt_launch(const EvtArgs* a, void* ws, int64_t ws_bytes, void* stream) {')
        e("  evt::RowArgs g; Epi::Params p;")
        e("  const int rc = fill(a, g, p);")
        e("  if (rc != EVT_OK) return rc;")
        e("  const unsigned grid = grid_for(g, a->flags);")
        e("  const int64_t need = (int64_t)grid * Epi::COL_STATE * g.N * 4;")
        e("  if (need > 0 && (!ws || ws_bytes < need)) return EVT_ERR_WORKSPACE;")
        e("  return enqueue(g, p, grid, ws, stream);")
        e("}")
        emit_static_scratch(e, bool(ir.col_state))
        e('extern "C" int evt_launch_static(const EvtArgs* a, void* stream) {')
        e("  evt::RowArgs g; Epi::Params p;")
        e("  const int rc = fill(a, g, p);")
        e("  if (rc != EVT_OK) return rc;")
        e("  const unsigned grid = grid_for(g, a->flags);")
        e("  const int64_t need = (int64_t)grid * Epi::COL_STATE * g.N * 4;")
        e("  if (need > kScratchBytes) return EVT_ERR_SCRATCH;")
        e("  void* ws = nullptr;")
        e("  if (need > 0) {   // partials only, each written before it is read: nothing to clear")
        e("    const int rs = scratch_for_stream(stream, &ws);")
        e("    if (rs != EVT_OK) return rs;")
        e("  }")
        e("  return enqueue(g, p, grid, ws, stream);")
        e("}")
        e("static int enqueue(evt::RowArgs& g, const Epi::Params& p, unsigned grid, void* ws, void* stream) {")
        e("  g.colws = (float*)ws;")
        e("  if (p.fast == 2) hipLaunchKernelGGL((evt::evt_row_kernel<Cfg, Epi, 2>), dim3(grid), dim3(Cfg::THREADS), 0, (hipStream_t)stream, g, p);")
        e("  else if (p.fast == 1) hipLaunchKernelGGL((evt::evt_row_kernel<Cfg, Epi, 1>), dim3(grid), dim3(Cfg::THREADS), 0, (hipStream_t)stream, g, p);")
        e("  else hipLaunchKernelGGL((evt::evt_row_kernel<Cfg, Epi, 0>), dim3(grid), dim3(Cfg::THREADS), 0, (hipStream_t)stream, g, p);")
        e("  int err = (int)hipGetLastError();")
        e("  if (err != 0 || Epi::COL_STATE == 0) return err;")
        e("  hipLaunchKernelGGL((evt::evt_row_col_finalize_kernel<Epi>), dim3((g.N + evt::kColFinalizeCols - 1) / evt::kColFinalizeCols), dim3(1024), 0, (hipStream_t)stream, g, p, (int)grid);")
        e("  return (int)hipGetLastError();")
        e("}")
        return e.text()


def generate(ir: EpilogueIR, spec, module_name: str, clock_probe: bool = False) -> str:
    if isinstance(spec, RowSpec):
        return RowCodegen(ir, spec, module_name).source()
    return Codegen(ir, spec, module_name, clock_probe).source()
