"""EVT fuser: turns a partition of a torch.fx graph into one fused GEMM/BMM +
epilogue kernel node.

Host-side mirror of python/gtl/compiler/passes/evt_fuser.py of the reference:
the same public surface (`EVTFuser.supported_targets`, `EVTFuser.fusible`,
`EVTFuser(...).trace(gm, partition_names)`, the `visit_*` op vocabulary
:1308-1485, `FusedOpBase.__call__(*epilogue_inputs, A, B) -> list[Tensor]`
:190-267, `FusedGEMM` :453-558, `FusedBMM` :561-697), re-homed on this
package's own IR, code generator and C-ABI kernel modules instead of the
un-vendored CUTLASS Python package.
"""
from __future__ import annotations

import ctypes
import operator
import zlib
import os
from contextlib import nullcontext
from dataclasses import replace
from typing import Any, Dict, List, Optional, Sequence, Tuple

import torch
from torch.fx import Node
from torch.fx.graph_module import GraphModule
from torch.utils._python_dispatch import _len_torch_dispatch_stack, _pop_mode_temporarily

from . import jit
from .autotuner.bmm_tuner import BMMTuner
from .autotuner.gemm_tuner import MMTuner
from .codegen import KernelSpec, RowSpec, TileConfig
from .ir import (DTYPE_NAMES, Coord, EpilogueIR, Node as IRNode, Slot, Store, Strides, accum_coord,
                 fit_strides)

aten = torch.ops.aten

LAYOUT_TARGETS = {"view", "_unsafe_view", "reshape", "unsqueeze", "squeeze", "permute", "clone", "expand",
                  "detach", "alias", "contiguous"}


def packet(target):
    """aten.add.Tensor -> aten.add (the reference strips overload suffixes in
    its front end, python/gtl/compiler/passes/pass_frontend.py:131-192)."""
    return getattr(target, "overloadpacket", target)


def target_name(target) -> str:
    name = getattr(packet(target), "__name__", str(target))
    return name.split(".")[0]


def node_shape_dtype(node: Node) -> Tuple[Tuple[int, ...], torch.dtype]:
    if "tensor_meta" in node.meta:
        tm = node.meta["tensor_meta"]
        if not hasattr(tm, "shape"):
            raise ValueError(f"{node.name} produces several tensors")
        return tuple(int(s) for s in tm.shape), tm.dtype
    if "val" in node.meta and isinstance(node.meta["val"], torch.Tensor):
        v = node.meta["val"]
        return tuple(int(s) for s in v.shape), v.dtype
    raise ValueError(f"node {node.name} carries no shape metadata (run ShapeProp first)")


def legalize_graph(graph_module: GraphModule) -> GraphModule:
    """Stable topological sort of the graph, in place: every node is moved
    behind its latest operand and otherwise keeps its place.  (torch.fx's own
    legalize_graph sorts breadth first, which interleaves the forward and
    backward halves of a joint graph; the forward/backward partitioner of
    AOT autograd goes by node position, as the reference's flow does through
    `default_partition`, python/gtl/helper/aot_helper.py:24-28.)"""
    graph = graph_module.graph
    pos = {n: k for k, n in enumerate(graph.nodes)}
    pending = list(graph.nodes)
    placed: set = set()
    order: List[Node] = []
    waiting: Dict[Node, List[Node]] = {}

    def place(n: Node):
        stack = [n]
        while stack:
            m = stack.pop()
            missing = [i for i in m.all_input_nodes if i not in placed]
            if missing:
                # wait for the operand that comes last in the present order
                waiting.setdefault(max(missing, key=pos.__getitem__), []).append(m)
                continue
            order.append(m)
            placed.add(m)
            stack.extend(reversed(waiting.pop(m, [])))

    for n in pending:
        place(n)
    if len(order) != len(pending):
        rest = [n.name for n in pending if n not in placed]
        raise RuntimeError("the graph has a cycle through " + ", ".join(rest[:8]))
    out = [n for n in order if n.op == "output"]
    order = [n for n in order if n.op != "output"] + out
    prev = None
    for n in order:
        if prev is None:
            if n.prev is not graph._root:
                graph._root.append(n)
        elif n.prev is not prev:
            prev.append(n)
        prev = n
    return graph_module


def _tensor_meta(shape: Sequence[int], dtype: torch.dtype):
    from torch.fx.passes.shape_prop import _extract_tensor_metadata
    return _extract_tensor_metadata(torch.empty(tuple(shape), dtype=dtype, device="meta"))


def _contig_strides(shape: Sequence[int]) -> Tuple[int, ...]:
    st, acc = [], 1
    for s in reversed(shape):
        st.append(acc)
        acc *= int(s)
    return tuple(reversed(st))


# ---------------------------------------------------------------------------
# run-time objects placed in the graph
# ---------------------------------------------------------------------------


def rand_stream_id(anchor_name: str) -> int:
    """Stream id of a fused op's rand_like tensors: a 28-bit hash of its anchor
    node's name.  Names are unique inside a graph, so two fused ops of one model
    draw unrelated numbers, and they do not change from trace to trace, so the
    same model traced again with the same seed draws the same masks (a count of
    the ops created in the process would depend on every earlier trace, dry runs
    included)."""
    return (zlib.crc32(anchor_name.encode()) & 0x0FFFFFFF) or 1


def launch_switches() -> Tuple[int, int]:
    """(EvtArgs.split_k, EvtArgs.flags) from the host's environment, read at
    every call: EVT_SPLIT_K=1|n turns split-K off / asks for n splits,
    EVT_TWO_KERNEL_REDUCE=1 finishes cross-tile reductions in the finalize
    kernel, EVT_ROW_WG_PER_CU=n sets the workgroups per CU of the row-wise
    kernels.  The kernel modules themselves read no environment."""
    if _ENV_BYTES:      # the usual case, nothing set: three dictionary look-ups
        d = _ENV_DATA
        if d.get(b"EVT_SPLIT_K") is None and d.get(b"EVT_TWO_KERNEL_REDUCE") is None and d.get(b"EVT_ROW_WG_PER_CU") is None:
            return 0, 0
    split, two, per_cu = _env("EVT_SPLIT_K"), _env("EVT_TWO_KERNEL_REDUCE"), _env("EVT_ROW_WG_PER_CU")
    flags = jit.EVT_FLAG_TWO_KERNEL_REDUCE if two == "1" else 0
    if per_cu:
        flags |= jit.evt_flag_row_wg_per_cu(max(0, min(254, int(per_cu))))
    return (max(0, int(split)) if split else 0), flags


_ENV_DATA = getattr(os.environ, "_data", None)        # the mapping behind os.environ (bytes keys on POSIX)
_ENV_BYTES = isinstance(_ENV_DATA, dict) and os.name == "posix"


def _env(name: str) -> Optional[str]:
    """os.environ.get(name) without its per-call encoding and wrapping: these switches are read at every launch."""
    if isinstance(_ENV_DATA, dict):
        v = _ENV_DATA.get(name.encode() if os.name == "posix" else name.upper())
        return None if v is None else (v.decode() if isinstance(v, bytes) else v)
    return os.environ.get(name)


class FusedOpBase:
    """Callable placed in the fx graph.  `fused(*epilogue_inputs, A, B)` returns
    the list of partition outputs (reference: evt_fuser.py:62-279)."""

    def __init__(self, node: Node, epilogue_visitor: "EVTFuser") -> None:
        self.node = node
        self.outputs = epilogue_visitor.outputs
        self.output2store = epilogue_visitor.output2store
        self.inputs = [i for i in epilogue_visitor.inputs if i is not node]
        self.input_names = epilogue_visitor.input_names
        self.post_reshape_permute = epilogue_visitor.post_reshape_permute
        self.stream = None
        self.mode = os.environ.get("MODE", "RUN")
        self.launched = False
        self.partition_names = epilogue_visitor.partition_names
        self.reference_module: GraphModule = epilogue_visitor.reference_gm
        self.rtol = 1e-2
        self.atol = 1e-3
        self.ir: EpilogueIR = epilogue_visitor.ir
        # kernel-tensor bookkeeping filled by the visitor
        self.slot_sources = epilogue_visitor.slot_sources      # slot -> ('input', idx) | ('output', store name)
        self.store_meta = epilogue_visitor.store_meta          # store name -> (shape, dtype)
        self._workspace = {}
        self._spare_workspace = None     # cleared at the first eager call, for the first graph capture (workspace_for)
        # rand_like stream: 64-bit seed (torch's global seed at the time of the call unless `rand_seed` is set), a
        # 32-bit offset that advances by one per launch, so successive calls draw different numbers, and a stream
        # id of the op's own (rand_stream_id: from the anchor node's name) that goes into the generator's counter
        # next to the slot index: two fused ops with rand_like tensors of equal shape draw unrelated numbers, as
        # eager PyTorch does.  The offset is a launch argument: a captured HIP graph replays the mask it was captured with.
        self._rand_seed: Optional[int] = None
        self.rand_stream = rand_stream_id(node.name)
        self.rand_offset = 0
        self.last_rand_state: Optional[Tuple[int, int]] = None   # (seed, offset) the most recent launch used

    @property
    def rand_seed(self) -> int:
        seed = torch.initial_seed() if self._rand_seed is None else self._rand_seed
        return int(seed) & 0xFFFFFFFFFFFFFFFF

    @rand_seed.setter
    def rand_seed(self, value: Optional[int]) -> None:
        self._rand_seed = value

    def rand_salt(self, slot: int) -> int:
        """Fourth counter word of the generator for rand_like slot `slot` of this op."""
        return (slot + 16 * self.rand_stream) & 0xFFFFFFFF

    # -- to be provided by subclasses -----------------------------------------
    module: jit.KernelModule
    problem: Tuple[int, int, int, int]   # M, N, K, L
    num_anchor_inputs = 2                 # trailing call arguments that belong to the anchor itself

    def operands(self, A: torch.Tensor, B: torch.Tensor):
        """-> (A, lda, batch_stride_A, B, ldb, batch_stride_B) ready for the kernel."""
        raise NotImplementedError("Should be Overwritten by child class")

    def build_arguments(self, visitor_args: Dict[str, torch.Tensor], *args, block=None) -> Tuple[jit.EvtArgs, list]:
        """Marshal operands and epilogue tensors into the C-ABI argument block
        (the counterpart of GemmArguments / BmmArguments2x +
        operation.epilogue_type(visitor_args), evt_fuser.py:539-544, :674-678).
        Returns the block and the tensors it points into (keep them alive).
        Without `block` the op's one reused block is filled, valid until the
        next call; a caller that keeps several argument sets side by side
        passes a block of its own (`new_argument_block()`) for each."""
        M, N, K, L = self.problem
        K = getattr(self, "kernel_k", K)         # operands padded along K (FusedGEMM.pad)
        A, lda, bsa, B, ldb, bsb = self.operands(args[-2], args[-1])
        a = block if block is not None else self.argument_block()
        a.M, a.N, a.K, a.L = M, N, K, L
        a.A, a.lda, a.batch_stride_A = A.data_ptr(), lda, bsa
        a.B, a.ldb, a.batch_stride_B = B.data_ptr(), ldb, bsb
        a.split_k, a.flags = launch_switches()
        keep = [A, B]
        self.fill_epilogue_arguments(a, keep, visitor_args, args)
        return a, keep

    def argument_block(self) -> jit.EvtArgs:
        """The op's argument block.  The launch call reads it before it returns, so
        one block per op is reused from call to call; what never changes (slot
        counts, strides, immediates) is written once."""
        a = getattr(self, "_evt_args", None)
        if a is None:
            a = self._evt_args = self.new_argument_block()
        return a

    def new_argument_block(self) -> jit.EvtArgs:
        """A block with everything but the per-call pointers filled in."""
        a = jit.EvtArgs()
        a.batch_div_A = a.batch_div_B = 1
        a.num_tensors = len(self.ir.slots)
        a.num_scalars = len(self.ir.scalars)
        for k, slot in enumerate(self.ir.slots):
            ta = a.tensors[k]
            ta.ptr = None
            ta.stride_l, ta.stride_m, ta.stride_n = slot.strides.stride_l, slot.strides.stride_m, slot.strides.stride_n
            ta.l_div = slot.strides.l_div
            ta.l_mod = slot.strides.l_mod
            ta.stride_l2 = slot.strides.stride_l2
        for i, sc in enumerate(self.ir.scalars):
            a.scalars[i] = sc
        # per call: (slot, where its tensor comes from)
        self._slot_plan = [(k, *self.slot_sources[k]) for k, slot in enumerate(self.ir.slots) if slot.kind != "rand"]
        return a

    def fill_epilogue_arguments(self, a: jit.EvtArgs, keep: list, visitor_args: Dict[str, torch.Tensor], args) -> None:
        """Tensor pointers of the epilogue's slots (shared by every anchor); a
        rand slot has no storage, its strides alone seed the generator."""
        tensors = a.tensors
        first_anchor = len(args) - self.num_anchor_inputs
        for k, kind, ref in self._slot_plan:
            if kind == "input":
                t = args[ref]
            elif kind == "anchor":
                t = args[first_anchor + ref]
            else:
                t = visitor_args[ref]
            keep.append(t)
            tensors[k].ptr = t.data_ptr()
        if self.ir.rng_scalar is not None:
            # 32-bit patterns, not float values: written through an integer view of the scalar array
            bits = (ctypes.c_uint32 * jit.EVT_MAX_SCALARS).from_buffer(a, jit.EvtArgs.scalars.offset)
            r = self.ir.rng_scalar
            seed = self.rand_seed
            bits[r], bits[r + 1] = seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF
            bits[r + 2], bits[r + 3] = self.rand_offset & 0xFFFFFFFF, self.rand_stream
            self.last_rand_state = (seed, self.rand_offset & 0xFFFFFFFF)
            self.rand_offset += 1

    def workspace_for(self, a: jit.EvtArgs, stream, device) -> Tuple[int, int]:
        """Device workspace for cross-workgroup reductions, one per stream,
        zero-filled once (launches leave it clean)."""
        # the size depends on the problem (fixed per op) and on the block's split-K / reduction switches
        mode = (a.split_k, a.flags)
        cached = getattr(self, "_ws_bytes", None)
        if cached is None or cached[0] != mode:
            cached = self._ws_bytes = (mode, self.module.workspace_bytes(a))
        ws_bytes = cached[1]
        if not ws_bytes:
            return 0, 0
        key = stream if isinstance(stream, int) else stream.cuda_stream      # a raw stream handle or a torch stream
        ws = self._workspace.get(key)
        if ws is None or ws.numel() < ws_bytes:
            # what torch says about "the current stream" holds for this launch only if it goes to that stream
            index = torch.device(device).index
            index = torch.cuda.current_device() if index is None else index
            current = key == _raw_current_stream(index)
            capturing = current and torch.cuda.is_current_stream_capturing()
            spare = self._spare_workspace
            if capturing and spare is not None and spare.numel() >= ws_bytes and spare.device.index == index:
                # A fill recorded into the graph would run at every replay, although launches leave the workspace
                # clean (measured on an encoder layer's training step: eight fills, 63 of 840 us per replay), and
                # nothing outside the graph may be waited for while a capture is open.  The capture takes the spare
                # that the op's first eager call cleared; without one (no eager call before the capture, or a
                # second capture) the fill is recorded, which is correct and only slower.
                ws, self._spare_workspace = spare, None
            else:
                ws = torch.empty(ws_bytes, dtype=torch.uint8, device=device)
                self.module.workspace_init(ws.data_ptr(), ws_bytes, key)
                if current and not capturing and (spare is None or spare.numel() < ws_bytes):
                    # cleared now and waited for once, so that it is clean whenever a capture takes it
                    spare = self._spare_workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=device)
                    self.module.workspace_init(spare.data_ptr(), ws_bytes, key)
                    torch.cuda.synchronize(spare.device)
            self._workspace[key] = ws
        return ws.data_ptr(), ws_bytes

    def allocate_outputs(self, device) -> Dict[str, torch.Tensor]:
        # one buffer per distinct store; reduction outputs need no zero fill
        # (the reference zero-fills them for its atomics, evt_fuser.py:217-225)
        return {name: torch.empty(shape, dtype=dtype, device=device)
                for name, (shape, dtype) in self.store_meta.items()}

    def call(self, visitor_args: Dict[str, torch.Tensor], stream, *args) -> Any:
        """`stream`: a torch stream or a raw HIP stream handle."""
        a, keep = self.build_arguments(visitor_args, *args)
        ws_ptr, ws_bytes = self.workspace_for(a, stream, keep[0].device)
        self.module.launch(a, ws_ptr, ws_bytes, stream if isinstance(stream, int) else stream.cuda_stream)

    def get_output_name(self, output: Node) -> str:
        return "accum" if output is self.node else output.name

    def result_shape(self, name: str) -> Tuple[int, ...]:
        """Shape of the tensor `__call__` returns for output `name`: the stored tensor's, seen through the views
        and permutes that follow the store."""
        shape = tuple(self.store_meta[self.output2store[name]][0])
        for op, arg in self.post_reshape_permute.get(name, ()):
            shape = tuple(int(d) for d in arg) if op == "view" else tuple(shape[int(i)] for i in arg)
        return shape

    def __call__(self, *args_):
        if not _hip_device_present():
            raise RuntimeError("the fused EVT kernels run on a HIP device only; none is available")
        # every microsecond here is paid per launch: no copies of what is contiguous already, no stream context
        # unless the op has a stream of its own, the result plan (store, views / permutes) worked out once
        args = [a if (not isinstance(a, torch.Tensor) or a.is_contiguous()) else a.contiguous() for a in args_]
        if self.stream is not None:
            self.stream.wait_stream(torch.cuda.current_stream())
            stream = self.stream
        else:
            # the current stream's raw handle: torch.cuda.current_stream() builds a Stream object and resolves
            # the device three times over, 8 us per call where this takes a fraction of one
            index = args[-1].device.index
            stream = _raw_current_stream(torch.cuda.current_device() if index is None else index)

        with (torch.cuda.stream(stream) if self.stream is not None else nullcontext()):
            visitor_args = self.allocate_outputs(args[-1].device)
            self.call(visitor_args, stream, *args)

            if self.stream is not None:
                for arg in args:
                    if isinstance(arg, torch.Tensor):
                        arg.record_stream(self.stream)

            plan = getattr(self, "_result_plan", None)
            if plan is None:
                plan = self._result_plan = [
                    (self.output2store[self.get_output_name(o)], tuple(self.post_reshape_permute.get(self.get_output_name(o), ())))
                    for o in self.outputs]
            results = []
            for store, ops in plan:
                out = visitor_args[store]
                for op, arg in ops:
                    out = out.view(arg) if op == "view" else out.permute(arg)
                results.append(out)

            if self.mode == "DEBUG" and not self.launched:
                self.launched = True
                self.reference(args, results)
            return results

    def anchor_eager(self, A: torch.Tensor, B: torch.Tensor) -> torch.Tensor:
        """The anchor (mm / bmm with its fused operand permutes) run eagerly."""
        raise NotImplementedError("Should be Overwritten by child class")

    def reference(self, args, results):
        """MODE=DEBUG self check on the first call (reference: evt_fuser.py:551-553,
        :688-689 -> reference_base)."""
        return self.reference_base(args, results)

    @staticmethod
    def pass_rate(out: torch.Tensor, ref: torch.Tensor, criteria: dict) -> float:
        return float(torch.sum(torch.isclose(out, ref, **criteria)) / max(out.numel(), 1))

    def reference_base(self, args, results, verbose: bool = True) -> List[dict]:
        """In-situ checker (reference: FusedOpBase.reference_base,
        evt_fuser.py:98-172): run the anchor eagerly in the operands' dtype, feed
        it as `accum` to the extracted epilogue module together with the
        partition inputs, and compare every output of the fused kernel with
        allclose(rtol=self.rtol); on a mismatch report maximum absolute /
        relative error and the atol / rtol pass rates.  Returns one record per
        output; nothing is raised (the reference prints and drops into a
        debugger)."""
        accum = self.anchor_eager(*args[len(args) - self.num_anchor_inputs:])
        named = dict(zip(self.input_names, args[:len(self.input_names)]))
        inputs = {n.name: named[n.name] for n in self.reference_module.graph.nodes
                  if n.op == "placeholder" and n.name != "accum"}
        with torch.no_grad():
            refs = self.reference_module(accum=accum, **inputs)
        report = []
        for output, out, ref in zip(self.outputs, results, refs):
            o = out.contiguous().view(-1)
            r = ref.contiguous().view(-1).to(o.dtype) if ref.dtype != o.dtype else ref.contiguous().view(-1)
            rec = {"name": self.get_output_name(output), "match": bool(torch.allclose(o, r, rtol=self.rtol))}
            if not rec["match"] and o.dtype != torch.bool:
                of, rf = o.float(), r.float()
                rec.update(max_abs=float(torch.max(torch.abs(of - rf))),
                           max_rel=float(torch.max(torch.abs(of - rf) / torch.abs(rf).clamp_min(1e-30))),
                           atol_pass_rate=self.pass_rate(of, rf, {"atol": self.atol, "rtol": 0.0}),
                           rtol_pass_rate=self.pass_rate(of, rf, {"rtol": self.rtol, "atol": 0.0}))
                if verbose:
                    print(f"!!!!!!!!!!!!!!result mismatch: {rec['name']}!!!!!!!!!!!!!!")
                    print("maximum abs error: ", rec["max_abs"])
                    print("maximum relative error: ", rec["max_rel"])
                    print("atol passed rate: ", rec["atol_pass_rate"])
                    print("rtol passed rate: ", rec["rtol_pass_rate"])
            report.append(rec)
        self.last_reference_report = report
        return report

    def get_src(self, node: Node) -> Node:
        if packet(node.target) in self.mainloop_fusion_targets and node.name in self.partition_names:
            return node.args[0]
        return node

    def get_alignment(self, dim: int) -> int:
        for a in (8, 4, 2):
            if dim % a == 0:
                return a
        return 1


# layout-only ops between a tensor in memory and a batched-product operand (the head split of an attention layer:
# view [B, S, H, D] -> permute [0, 2, 1, 3] -> expand -> clone -> view [B * H, S, D])
_OPERAND_CHAIN_OPS = ("view", "_unsafe_view", "reshape", "permute", "expand", "clone", "unsqueeze", "squeeze", "select")


def operand_chain(node, allowed=None) -> Tuple[List[Node], Any]:
    """The layout-only nodes, each with one user, that end in the operand
    `node`, in graph order, and the tensor they start from."""
    chain: List[Node] = []
    while (isinstance(node, Node) and node.op == "call_function" and target_name(node.target) in _OPERAND_CHAIN_OPS
           and len(node.users) == 1 and (allowed is None or allowed(node))):
        chain.append(node)
        node = node.args[0]
    chain.reverse()
    return chain, node


def operand_strides(chain: Sequence[Node], shape3: Sequence[int]) -> Optional[Strides]:
    """Addressing of the operand [L, R, C] that `chain` produces inside the
    (contiguous) tensor the chain starts from: offset(l, r, c) = (l // l_div)
    * stride_l + (l % l_div) * stride_l2 + r * stride_m + c * stride_n, or None
    when the chain does not reduce to that form (a copy is needed then)."""
    L, R, C = (int(x) for x in shape3)
    coord = Coord((L, R, C), lambda l, m, n: (l * R + m) * C + n)
    for node in reversed(chain):
        in_shape, _ = node_shape_dtype(node.args[0])
        if target_name(node.target) == "permute":
            coord = coord.inverse_permute([int(d) for d in node.args[1]], in_shape)
        elif target_name(node.target) == "select":
            coord = coord.inverse_select(int(node.args[1]), int(node.args[2]), in_shape)
        else:
            numel = 1
            for d in in_shape:
                numel *= int(d)
            if numel != coord.numel():        # an expand that broadcasts
                return None
            coord = coord.reshape(in_shape)
    st = fit_strides(coord, L, R, C, allow_base=True)
    if st is None or st.l_mod:
        return None
    return st


_HIP_PRESENT: Optional[bool] = None


_raw_current_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None) or (
    lambda index: torch.cuda.current_stream(index).cuda_stream)


def _hip_device_present() -> bool:
    """torch.cuda.is_available(), asked once (a fused op runs thousands of times per second)."""
    global _HIP_PRESENT
    if _HIP_PRESENT is None:
        _HIP_PRESENT = bool(torch.cuda.is_available())
    return _HIP_PRESENT


def _dma_ok(a_kc: bool, b_kc: bool, M: int, N: int, K: int, lda: int, ldb: int, bsa: int, bsb: int) -> bool:
    """The fast global->LDS path moves 16-byte chunks: every operand row must
    start on a 16-byte boundary and the contiguous extent must be a multiple
    of 8 elements (the same role as the reference's alignment_A/B = 8 case,
    evt_fuser.py:502-512)."""
    if (lda | ldb | bsa | bsb) & 7:
        return False
    if (a_kc or b_kc) and K % 8:
        return False
    if not a_kc and M % 8:
        return False
    if not b_kc and N % 8:
        return False
    return True


class FusedGEMM(FusedOpBase):
    """epilogue_visitor(A @ B, args) as one kernel (reference: evt_fuser.py:453-558)."""
    __name__ = "cutlass_gemm_with_visitor"
    target = aten.mm
    mainloop_fusion_targets = [aten.permute]
    pad_min_flops = 1e9          # products below this keep the element-wise path: the copies would cost more

    def __init__(self, node: Node, epilogue_visitor: "EVTFuser") -> None:
        super().__init__(node, epilogue_visitor)
        lhs_node, rhs_node = node.args[0], node.args[1]
        lhs_shape, dtype = node_shape_dtype(lhs_node)
        rhs_shape, _ = node_shape_dtype(rhs_node)
        M, K = lhs_shape[-2:]
        N = rhs_shape[-1]
        # A column-major output is computed as C^T = B^T A^T (reference: the `transposed` problems of
        # evt_fuser.py:573-596): the operands change places, and what was row-major is read as column-major.
        self.transposed = bool(getattr(epilogue_visitor, "transposed", False))
        if self.transposed:
            lhs_node, rhs_node = rhs_node, lhs_node
            M, N = N, M
        self.lhs_layout = self.get_src_layout(lhs_node)
        self.rhs_layout = self.get_src_layout(rhs_node)
        self.A = self.get_src(lhs_node)
        self.B = self.get_src(rhs_node)
        self.args = [self.A, self.B]
        self.problem = (M, N, K, 1)
        if dtype not in (torch.float16, torch.bfloat16):
            raise NotImplementedError(f"GEMM operands of dtype {dtype}")
        if self.transposed:     # the new A is the old B seen as [N, K], the new B the old A seen as [K, M]
            self.a_kc = self.lhs_layout == "ColumnMajor"
            self.b_kc = self.rhs_layout == "RowMajor"
        else:
            self.a_kc = self.lhs_layout == "RowMajor"
            self.b_kc = self.rhs_layout == "ColumnMajor"
        self.lda = K if self.a_kc else M
        self.ldb = K if self.b_kc else N
        dma = _dma_ok(self.a_kc, self.b_kc, M, N, K, self.lda, self.ldb, 0, 0)
        # Extents that break the transfer path's 16-byte rule (ViT's patch embedding: K = 588) would fall back to the
        # element-wise path, several times slower.  A product large enough to pay for two copy kernels runs on
        # zero-padded copies of its operands instead: rows padded to a multiple of 8 elements, K to a multiple of 8
        # (zero columns / rows add nothing to the product; the output keeps its M and N).
        self.pad = None
        if not dma and 2.0 * M * N * K >= self.pad_min_flops:
            r8 = lambda v: (v + 7) & ~7      # noqa: E731
            Kp = r8(K) if (self.a_kc or self.b_kc) else K
            self.pad = (Kp, Kp if self.a_kc else r8(M), Kp if self.b_kc else r8(N))
            self.kernel_k, self.lda, self.ldb = self.pad
            dma = True
            K = Kp

        self.align_A = self.get_alignment(K if self.a_kc else M)
        self.align_B = self.get_alignment(K if self.b_kc else N)
        self.align_C = self.get_alignment(N)

        with (_pop_mode_temporarily() if _len_torch_dispatch_stack() > 0 else nullcontext()):
            tuner = MMTuner((M, N, K, 1), self.a_kc, self.b_kc, dtype == torch.bfloat16, dma, self.ir)
            tile = tuner.get_best_config()
            self.tile = tile
            self.spec = KernelSpec.for_problem(K, self.a_kc, self.b_kc, dtype == torch.bfloat16, tile,
                                               self.problem[0], self.problem[1])
            self.module = jit.load_module(self.ir, self.spec)

    def operands(self, A, B):
        A = A.contiguous()
        B = B.contiguous()
        if self.pad is not None:
            M, N, K, _ = self.problem
            Kp, lda, ldb = self.pad
            pad = torch.nn.functional.pad
            # (last-axis padding, then rows): one copy kernel per operand that needs it
            if self.a_kc:
                A = pad(A, (0, lda - K)) if lda != K else A
            elif lda != M or Kp != K:
                A = pad(A, (0, lda - M, 0, Kp - K))
            if self.b_kc:
                B = pad(B, (0, ldb - K)) if ldb != K else B
            elif ldb != N or Kp != K:
                B = pad(B, (0, ldb - N, 0, Kp - K))
        if self.tile.dma:
            # the global->LDS path moves 16-byte chunks: a contiguous view that starts at an odd storage offset is
            # copied into a fresh (aligned) allocation instead of failing the launch, as eager would simply work
            if A.data_ptr() & 15:
                A = A.clone()
            if B.data_ptr() & 15:
                B = B.clone()
        return A, self.lda, 0, B, self.ldb, 0

    def anchor_eager(self, A, B):
        C = torch.mm(A if self.a_kc else A.t(), B.t() if self.b_kc else B)
        return C.t() if self.transposed else C

    def get_src_layout(self, node: Node) -> str:
        if packet(node.target) == aten.permute and node.name in self.partition_names:
            indices = [int(i) for i in node.args[1]]
            if indices == [0, 1]:
                return "RowMajor"
            if indices == [1, 0]:
                return "ColumnMajor"
            raise ValueError(f"Invalid permutation: {indices}")
        return "RowMajor"


class FusedBMM(FusedOpBase):
    """Batched variant; A/B may be 3-D permutations of their source tensors
    (reference: evt_fuser.py:561-697, python/gtl/ops/bmm.py:23-64), or come out
    of any chain of views, permutes and copies that amounts to strided
    addressing with a batch index in two levels (the head split / merge of an
    attention layer), which the kernel then reads in place."""
    __name__ = "cutlass_bmm_with_visitor"
    target = aten.bmm
    mainloop_fusion_targets = [aten.permute]

    def __init__(self, node: Node, epilogue_visitor: "EVTFuser") -> None:
        super().__init__(node, epilogue_visitor)
        lhs_node, rhs_node = node.args[0], node.args[1]
        lhs_shape, dtype = node_shape_dtype(lhs_node)
        rhs_shape, _ = node_shape_dtype(rhs_node)
        L, M, K = lhs_shape
        N = rhs_shape[-1]
        if dtype not in (torch.float16, torch.bfloat16):
            raise NotImplementedError(f"BMM operands of dtype {dtype}")

        # the layout-only producers of each operand that belong to the partition, and the operand's strides
        # inside the (contiguous) tensor they start from
        inside = lambda n: n.name in self.partition_names      # noqa: E731
        self.chain_A, self.A = operand_chain(lhs_node, inside)
        self.chain_B, self.B = operand_chain(rhs_node, inside)
        sa = operand_strides(self.chain_A, lhs_shape)
        sb = operand_strides(self.chain_B, rhs_shape)
        # A column-major output is computed as C^T = B^T A^T (reference: evt_fuser.py:573-596): the operands change
        # places, each seen transposed (its m and n strides exchanged).
        self.transposed = bool(getattr(epilogue_visitor, "transposed", False))
        if self.transposed:
            flip = lambda st: None if st is None else replace(st, stride_m=st.stride_n, stride_n=st.stride_m)   # noqa: E731
            self.chain_A, self.chain_B, self.A, self.B = self.chain_B, self.chain_A, self.B, self.A
            sa, sb = flip(sb), flip(sa)
            M, N = N, M
        self.problem = (M, N, K, L)
        self.args = [self.A, self.B]
        self.copy_A = self.copy_B = False
        self.bdiva, self.bs2a, self.bdivb, self.bs2b = 1, 0, 1, 0
        if sa is not None and sa.stride_n == 1 and (M == 1 or sa.stride_m >= K):
            self.a_kc, self.lda = True, (sa.stride_m if M > 1 else K)
        elif sa is not None and sa.stride_m == 1 and (K == 1 or sa.stride_n >= M):
            self.a_kc, self.lda = False, (sa.stride_n if K > 1 else M)
        else:   # batch-last source and the like: make the operand contiguous first (evt_fuser.py:663-672)
            self.copy_A, self.a_kc, self.lda, sa = True, True, K, Strides(M * K, K, 1)
        if sb is not None and sb.stride_m == 1 and (N == 1 or sb.stride_n >= K):
            self.b_kc, self.ldb = True, (sb.stride_n if N > 1 else K)
        elif sb is not None and sb.stride_n == 1 and (K == 1 or sb.stride_m >= N):
            self.b_kc, self.ldb = False, (sb.stride_m if K > 1 else N)
        else:
            self.copy_B, self.b_kc, self.ldb, sb = True, False, N, Strides(K * N, N, 1)
        self.bsa, self.bdiva, self.bs2a, self.offa = sa.stride_l, sa.l_div, sa.stride_l2, sa.base
        self.bsb, self.bdivb, self.bs2b, self.offb = sb.stride_l, sb.l_div, sb.stride_l2, sb.base
        self.lhs_layout = "RowMajor" if self.a_kc else "ColumnMajor"
        self.rhs_layout = "ColumnMajor" if self.b_kc else "RowMajor"
        dma = _dma_ok(self.a_kc, self.b_kc, M, N, K, self.lda, self.ldb,
                      self.bsa | self.bs2a | self.offa, self.bsb | self.bs2b | self.offb)

        with (_pop_mode_temporarily() if _len_torch_dispatch_stack() > 0 else nullcontext()):
            tuner = BMMTuner(self.problem, self.a_kc, self.b_kc, dtype == torch.bfloat16, dma, self.ir)
            tile = tuner.get_best_config()
            self.tile = tile
            self.spec = KernelSpec.for_problem(K, self.a_kc, self.b_kc, dtype == torch.bfloat16, tile,
                                               self.problem[0], self.problem[1])
            self.module = jit.load_module(self.ir, self.spec)

    # kept for callers that ask which 3-D permutation an operand went through
    @property
    def permute_A(self) -> List[int]:
        return self._single_permute(self.chain_A)

    @property
    def permute_B(self) -> List[int]:
        return self._single_permute(self.chain_B)

    @staticmethod
    def _single_permute(chain) -> List[int]:
        if len(chain) == 1 and target_name(chain[0].target) == "permute":
            return [int(i) for i in chain[0].args[1]]
        return [0, 1, 2]

    @staticmethod
    def _replay(chain, x):
        """The operand as eager PyTorch computes it from its source tensor."""
        for node in chain:
            x = node.target(x, *node.args[1:], **node.kwargs)
        return x

    def operands(self, A, B):
        # a copied operand is laid out as the kernel's [L, M, K] / [L, K, N]; in a transposed problem the eager
        # chain yields it the other way round
        if self.copy_A:
            A = self._replay(self.chain_A, A)
            A = (A.transpose(1, 2) if self.transposed else A).contiguous()
        if self.copy_B:
            B = self._replay(self.chain_B, B)
            B = (B.transpose(1, 2) if self.transposed else B).contiguous()
        if self.tile.dma:
            # as in FusedGEMM.operands: a source tensor that starts at an odd storage offset is copied into a fresh
            # (aligned) allocation; the strides inside it and the base offset of a `select` (both multiples of 8
            # elements, or the element-wise module was chosen) carry over
            if A.data_ptr() & 15:
                A = A.clone()
            if B.data_ptr() & 15:
                B = B.clone()
        return A, self.lda, self.bsa, B, self.ldb, self.bsb

    def build_arguments(self, visitor_args, *args, block=None):
        a, keep = super().build_arguments(visitor_args, *args, block=block)
        a.batch_div_A, a.batch_stride2_A = self.bdiva, self.bs2a
        a.batch_div_B, a.batch_stride2_B = self.bdivb, self.bs2b
        if self.offa:       # the operand starts inside its source tensor (a `select`): elements of 2 bytes
            a.A = a.A + 2 * self.offa
        if self.offb:
            a.B = a.B + 2 * self.offb
        return a, keep

    def anchor_eager(self, A, B):
        if self.transposed:     # A, B are the original right and left operands
            return torch.bmm(self._replay(self.chain_B, B), self._replay(self.chain_A, A))
        return torch.bmm(self._replay(self.chain_A, A), self._replay(self.chain_B, B))


def _unsupported_anchor(name: str, where: str):
    class _Stub(FusedOpBase):
        __doc__ = (f"{name}: anchor outside this backend's scope (the fused GEMM/BMM path); "
                   f"reference: evt_fuser.py:{where}.")

        def __init__(self, *a, **k) -> None:
            raise NotImplementedError(f"{name} is not provided by the MI355X GEMM/BMM backend")
    _Stub.__name__ = name
    _Stub.__qualname__ = name
    return _Stub


FusedConvFprop = _unsupported_anchor("FusedConvFprop", "282-365")
FusedConvDgrad = _unsupported_anchor("FusedConvDgrad", "368-450")
FusedSpmm = _unsupported_anchor("FusedSpmm", "973-1035")

class FusedRowOp(FusedOpBase):
    """Common part of the row-wise reduce-apply anchors (softmax, layer norm
    and their backward passes over the last axis): `fused(*epilogue_inputs,
    *anchor_operands)`.  The anchor's result takes the place of the GEMM
    accumulator in front of the same epilogue tree; rows are r = l * M + m of
    the operand viewed as [L, M, N]."""

    row_op = ""

    def __init__(self, node: Node, epilogue_visitor: "EVTFuser") -> None:
        super().__init__(node, epilogue_visitor)
        v = epilogue_visitor
        self.args = list(v.anchor_operands)
        self.num_anchor_inputs = len(self.args)
        _, dtype = node_shape_dtype(self.args[0])
        if dtype not in (torch.float16, torch.bfloat16, torch.float32):
            raise NotImplementedError(f"{self.row_op} operands of dtype {dtype}")
        self.problem = (v.M, v.N, 1, v.L)
        # (a per-column reduction of the epilogue keeps its partials in registers next to the row: rows over several
        # waves then take more waves)
        self.row_spec = RowSpec.for_row_length(self.row_op, v.N, DTYPE_NAMES[dtype], self.ir.col_state)
        self.spec = self.row_spec
        self.module = jit.load_module(self.ir, self.row_spec)

    def build_arguments(self, visitor_args: Dict[str, torch.Tensor], *args, block=None) -> Tuple[jit.EvtArgs, list]:
        M, N, _, L = self.problem
        ops = [t.contiguous() for t in args[len(args) - self.num_anchor_inputs:]]
        a = block if block is not None else self.argument_block()
        a.M, a.N, a.K, a.L = M, N, 1, L
        a.A, a.lda, a.batch_stride_A = ops[0].data_ptr(), N, M * N
        a.split_k, a.flags = launch_switches()
        if len(ops) > 1:
            a.B, a.ldb, a.batch_stride_B = ops[1].data_ptr(), N, M * N
        keep = list(ops)
        self.fill_epilogue_arguments(a, keep, visitor_args, args)
        return a, keep


class FusedSoftmax(FusedRowOp):
    """aten._softmax over the last axis + epilogue (reference: evt_fuser.py:700-762)."""
    __name__ = "cutlass_softmax_with_visitor"
    target = aten._softmax
    row_op = "softmax"

    def anchor_eager(self, x):
        return aten._softmax(x, -1, self.node.args[2])


class FusedSoftmaxBackward(FusedRowOp):
    """aten._softmax_backward_data over the last axis + epilogue (reference: evt_fuser.py:765-826)."""
    __name__ = "cutlass_softmax_backward_with_visitor"
    target = aten._softmax_backward_data
    row_op = "softmax_backward"

    def anchor_eager(self, grad, out):
        return aten._softmax_backward_data(grad, out, -1, self.node.args[3])


class FusedLayerNorm(FusedRowOp):
    """aten.native_layer_norm over the last axis, without weight and bias (they
    are epilogue nodes), + epilogue; mean and rstd are per-row outputs
    (reference: evt_fuser.py:829-902)."""
    __name__ = "cutlass_layernorm_with_visitor"
    target = aten.native_layer_norm
    row_op = "layernorm"

    def anchor_eager(self, x):
        return aten.native_layer_norm(x, list(self.node.args[1]), None, None, self.node.args[4])


class FusedLayerNormBackward(FusedRowOp):
    """aten.native_layer_norm_backward + epilogue: the input gradient and, when
    the output mask asks for them, the weight and bias gradients as per-column
    sums of the same pass; operands: gradient, forward input, mean, rstd and
    optionally the weight (reference: evt_fuser.py:905-970, input gradient only)."""
    __name__ = "cutlass_layernorm_backward_with_visitor"
    target = aten.native_layer_norm_backward
    row_op = "layernorm_backward"

    def anchor_eager(self, grad, x, mean, rstd, gamma=None):
        mask = [bool(b) for b in self.node.args[7]]
        bias = torch.zeros_like(gamma) if (gamma is not None and mask[2]) else None
        return aten.native_layer_norm_backward(grad, x, list(self.node.args[2]), mean, rstd, gamma, bias, mask)





# ---------------------------------------------------------------------------
# the fuser
# ---------------------------------------------------------------------------


class EVTFuser:
    """Entry point: `EVTFuser.fusible(partition, gm)` and
    `EVTFuser().trace(gm, partition)` (reference: evt_fuser.py:1038-1235)."""

    supported_targets = [aten.mm, aten.bmm, aten._softmax, aten._softmax_backward_data, aten.native_layer_norm,
                         aten.native_layer_norm_backward]
    row_targets = {aten._softmax: FusedSoftmax, aten._softmax_backward_data: FusedSoftmaxBackward,
                   aten.native_layer_norm: FusedLayerNorm, aten.native_layer_norm_backward: FusedLayerNormBackward}
    # compute C^T = B^T A^T when the outputs are column-major (tests switch it off to reach the strided stores)
    allow_transpose = True

    def __init__(self, element_compute=torch.float32, **kwargs):
        self.element_compute = element_compute
        self.mode = os.environ.get("MODE", "RUN")

    @staticmethod
    def get_node_with_name(name: str, graph_module: GraphModule) -> Node:
        for node in graph_module.graph.nodes:
            if node.name == name:
                return node
        raise ValueError(f"{name} is not in the graph.")

    @staticmethod
    def fusible(partition: Sequence[str], graph_module: GraphModule) -> bool:
        for node_name in partition:
            node = EVTFuser.get_node_with_name(node_name, graph_module)
            if node.op == "call_function" and packet(node.target) in EVTFuser.supported_targets:
                return True
        return False

    # -- tracing ------------------------------------------------------------------
    def trace(self, graph_module: GraphModule, partition_: Sequence[str], dry_run: bool = False):
        """Lower one partition to a fused kernel and splice it into the graph.
        With `dry_run` the analysis runs (and raises NotImplementedError for
        a partition the epilogue cannot express) but the graph is left alone."""
        self.partition_names = list(partition_)
        try:
            graph_module.graph.lint()
        except Exception:
            legalize_graph(graph_module)
        in_partition = set(self.partition_names)
        partition = [n for n in graph_module.graph.nodes if n.name in in_partition]

        # Step 1: anchor = the heavy op; producers of the anchor inside the
        # partition are main-loop fusions (operand permutes), not epilogue
        anchor = None
        for node in partition:
            if node.op == "call_function" and packet(node.target) in self.supported_targets:
                anchor = node
        if anchor is None:
            raise ValueError("partition holds no supported anchor")
        self.anchor = anchor
        if packet(anchor.target) in (aten.native_layer_norm, aten.native_layer_norm_backward):
            # a tuple cannot leave the kernel: the getitems of the anchor always belong to its partition
            extra = [u for u in anchor.users if u not in partition]
            if any(u.op != "call_function" or u.target is not operator.getitem for u in extra):
                raise NotImplementedError(f"{anchor.name}: result used other than through getitem")
            members = set(partition) | set(extra)
            partition = [n for n in graph_module.graph.nodes if n in members]
            self.partition_names = [n.name for n in partition]
        # producers of the anchor's operands inside the partition (layout-only chains) are read through the
        # operands' strides: main-loop fusion, not epilogue
        pre: set = set()
        stack = [a for a in anchor.all_input_nodes if a in partition]
        while stack:
            n = stack.pop()
            if n not in pre:
                pre.add(n)
                stack.extend(a for a in n.all_input_nodes if a in partition)
        epilogue_partition = [n for n in partition if n is not anchor and n not in pre]
        epi_set = set(epilogue_partition)

        # Step 2: inputs and outputs of the epilogue, in graph order
        inputs: List[Node] = []
        for node in epilogue_partition:
            for inp in node.all_input_nodes:
                if inp not in epi_set and inp not in inputs:
                    inputs.append(inp)
        outputs: List[Node] = []
        for node in epilogue_partition:
            if any(user not in epi_set for user in node.users):
                outputs.append(node)
        store_anchor = any(user not in epi_set for user in anchor.users) or not epilogue_partition
        if store_anchor:
            outputs.insert(0, anchor)
        self.inputs = inputs
        self.outputs = outputs
        self.outputs_subgraph = set(outputs)
        self.reference_gm = self._extract_reference(graph_module, anchor, epilogue_partition, inputs, outputs)

        # Steps 3 and 4: the epilogue IR and its stores.  A row-wise anchor on a tensor of rank 3 or more is
        # first viewed as [L, M, N] (what broadcasts along a middle axis need); if the epilogue cannot be
        # expressed that way (a reduction over every row, say), as one batch of L * M rows
        try:
            fused_kernel = self._lower(anchor, epilogue_partition, epi_set, inputs, outputs, flatten=False)
        except NotImplementedError:
            if packet(anchor.target) not in self.row_targets or getattr(self, "L", 1) == 1:
                raise
            fused_kernel = self._lower(anchor, epilogue_partition, epi_set, inputs, outputs, flatten=True)

        # Step 5: compose the fused kernel and rewire the graph
        if dry_run:
            return fused_kernel
        args = [i for i in inputs if i is not anchor] + fused_kernel.args
        graph_module.graph.inserting_after(anchor)
        fused_node = graph_module.graph.call_function(fused_kernel, args=tuple(args))
        # the forward/backward split of AOT autograd reads these tags and wants
        # tensor metadata on every tensor-valued node
        carried = {k: anchor.meta[k] for k in ("partitioner_tag", "seq_nr", "autograd_backward") if k in anchor.meta}
        fused_node.meta = {"evt": True, **carried}
        graph_module.graph.inserting_after(fused_node)
        for idx, output_node in enumerate(outputs):
            get_item_node = graph_module.graph.call_function(operator.getitem, args=(fused_node, idx))
            graph_module.graph.inserting_after(get_item_node)
            shape, dtype = node_shape_dtype(output_node)
            get_item_node.meta = {"tensor_meta": _tensor_meta(shape, dtype), **carried}
            out_meta = {k: v for k, v in output_node.meta.items()
                        if k in ("tensor_meta", "val", "partitioner_tag", "seq_nr", "autograd_backward")}
            name = "accum" if output_node is anchor else output_node.name
            if tuple(fused_kernel.result_shape(name)) == tuple(shape):
                # the kernel's result has the node's shape already: no view node (an aten call per output and launch)
                get_item_node.meta.update(out_meta)
                view_node = get_item_node
            else:
                view_node = graph_module.graph.call_function(aten.view, args=(get_item_node, list(shape)))
                view_node.meta = out_meta
            if output_node is anchor:
                for user in list(anchor.users):
                    if user not in epi_set and user is not fused_node:
                        user.replace_input_with(anchor, view_node)
            else:
                output_node.replace_all_uses_with(view_node)
            graph_module.graph.inserting_after(view_node)
        # The partition's own nodes are dead now.  Remove them here rather than leave it to dead-code elimination:
        # fx keeps random ops (rand_like) alive as impure, and a stranded rand_like would keep its operand -- the
        # whole unfused chain up to the GEMM -- running next to the fused kernel.
        for node in reversed(partition):
            if not node.users:
                graph_module.graph.erase_node(node)
        self.fused_kernel = fused_kernel
        return fused_kernel

    def _lower(self, anchor: Node, epilogue_partition, epi_set, inputs, outputs, flatten: bool):
        """Steps 3 and 4 of `trace`: the epilogue IR and its stores for one
        choice of the (L, M) split of a row-wise anchor's rows."""
        # Step 3: build the IR
        tgt = packet(anchor.target)
        self.anchor_operands: List[Node] = []
        self.pending_multi: Dict[Node, Dict[int, str]] = {}
        self.pending_coords: Dict[Node, Dict[int, Coord]] = {}
        self.anchor_slot_nodes: List[Node] = []
        self.coords: Dict[Node, Coord] = {}
        self.ir_name: Dict[Node, str] = {}
        if tgt in self.row_targets:
            self._begin_row_anchor(anchor, tgt, flatten)
        else:
            (ashape, adtype) = node_shape_dtype(anchor)
            batched = tgt == aten.bmm
            if batched:
                L, M, N = ashape
            else:
                L, (M, N) = 1, ashape
            self.L, self.M, self.N = L, M, N
            self.ir = EpilogueIR(L, M, N, batched)
            self.ir.add_node(IRNode("accum", "accum", domain="tile"))
            self.coords[anchor] = accum_coord(L, M, N, batched)
            self.ir_name[anchor] = "accum"
        self.full = self._accum_dependents(anchor, epi_set)
        self.load_cache: Dict[Tuple[str, Tuple[int, ...]], str] = {}
        self.input_index = {n: i for i, n in enumerate(x for x in inputs if x is not anchor)}
        self.input_names = [n.name for n in inputs if n is not anchor]
        self.input_nodes = [n for n in inputs if n is not anchor]
        self.slot_sources: Dict[int, Tuple[str, Any]] = {}

        for node in epilogue_partition:
            if node in self.full:
                self.visit(node)

        # Step 4: stores
        self.output2store: Dict[str, str] = {}
        self.post_reshape_permute: Dict[str, List[Tuple[str, Any]]] = {}
        self.store_meta: Dict[str, Tuple[Tuple[int, ...], torch.dtype]] = {}
        store_key: Dict[Tuple, str] = {}
        for out in outputs:
            self._insert_store(out, store_key)
        self.ir.finalize()
        # a column-major output: compute the transposed product instead (operands exchanged by the fused op), so
        # that the stores run along the kernel's n
        self.transposed = False
        if self.allow_transpose and tgt not in self.row_targets and self.ir.wants_transpose():
            self.ir.transpose()
            self.ir.finalize()
            self.transposed = True
        # slot indices may have been compacted by finalize(): rebuild the map
        self._rebuild_slot_sources()
        self.return_names = [o.name for o in outputs]
        self.reduction_names = [s.name for s in self.ir.slots if s.role == "store" and s.domain != "tile"]

        return self.get_fused_node(anchor)

    def _begin_row_anchor(self, anchor: Node, tgt, flatten: bool = False) -> None:
        """Geometry, accumulator and anchor operands of a row-wise anchor: the
        operand is viewed as [L, M, N] with N its last axis (the reference
        canonicalises these anchors to rank 3, pass_fusion.py:1187-1342)."""
        x = anchor.args[0] if tgt is not aten.native_layer_norm_backward else anchor.args[1]
        shape, dtype = node_shape_dtype(x)
        rank = len(shape)
        if rank < 2:
            raise NotImplementedError(f"{anchor.name}: row-wise anchor on a rank-{rank} tensor")
        if tgt in (aten._softmax, aten._softmax_backward_data):
            dim = int(anchor.args[1] if tgt is aten._softmax else anchor.args[2])
            if dim % rank != rank - 1:
                raise NotImplementedError(f"{anchor.name}: softmax over an axis other than the last")
        else:
            nshape = list(anchor.args[1] if tgt is aten.native_layer_norm else anchor.args[2])
            if [int(d) for d in nshape] != [int(shape[-1])]:
                raise NotImplementedError(f"{anchor.name}: layer norm over more than the last axis")
        N = int(shape[-1])
        M = int(shape[-2])
        L = 1
        for d in shape[:-2]:
            L *= int(d)
        if flatten:          # all rows as one batch: what a reduction over every row needs
            L, M = 1, L * M
        batched = L > 1
        self.L, self.M, self.N = L, M, N
        self.ir = EpilogueIR(L, M, N, batched)
        self.ir.add_node(IRNode("accum", "accum", domain="tile"))
        full = Coord(tuple(shape), lambda l, m, n: (l * M + m) * N + n)
        self.coords[anchor] = full
        if tgt is aten._softmax:
            self.anchor_operands = [anchor.args[0]]
            self.ir_name[anchor] = "accum"
        elif tgt is aten._softmax_backward_data:
            self.anchor_operands = [anchor.args[0], anchor.args[1]]
            self.ir_name[anchor] = "accum"
        elif tgt is aten.native_layer_norm:
            if anchor.args[2] is not None or anchor.args[3] is not None:
                raise NotImplementedError(f"{anchor.name}: weight and bias belong in the epilogue "
                                          "(pass_decomposition splits them off)")
            self.anchor_operands = [anchor.args[0]]
            self.ir.add_anchor_scalar(float(anchor.args[4]))
            self.ir.add_node(IRNode("ln_mean", "rowval", domain="row", comp=0))
            self.ir.add_node(IRNode("ln_rstd", "rowval", domain="row", comp=1))
            self.pending_multi[anchor] = {0: "accum", 1: "ln_mean", 2: "ln_rstd"}
            stat = full.reduce([rank - 1], True)
            self.pending_coords[anchor] = {1: stat, 2: stat}
        else:
            grad, xin, _, mean, rstd, gamma, _beta, mask = anchor.args[:8]
            mask = [bool(b) for b in mask]
            # (with mask[0] unset -- the input needs no gradient -- the kernel still forms it in registers, the
            # weight / bias sums share its row statistics; it is simply not stored)
            if (mask[1] or mask[2]) and L != 1:
                # weight / bias gradients are sums over every row: one batch of rows
                raise NotImplementedError(f"{anchor.name}: weight / bias gradients need the rows as one batch")
            self.anchor_operands = [grad, xin, mean, rstd] + ([gamma] if gamma is not None else [])
            for node_, st_, dt_, kind_ in ((mean, Strides(M, 1, 0), "f32", "col"), (rstd, Strides(M, 1, 0), "f32", "col")):
                if node_shape_dtype(node_)[1] != torch.float32:
                    raise NotImplementedError(f"{anchor.name}: statistics must be fp32")
                k = self.ir.add_slot(Slot(node_.name, "load", dt_, "tile", kind_, st_, node_shape_dtype(node_)[0]))
                self.ir.anchor_slots.append(k)
            if gamma is not None:
                gshape, gdtype = node_shape_dtype(gamma)
                if gdtype != dtype or tuple(gshape) != (N,):
                    raise NotImplementedError(f"{anchor.name}: weight must be an [N] vector of the operands' dtype")
                k = self.ir.add_slot(Slot(gamma.name, "load", DTYPE_NAMES[gdtype], "tile", "row", Strides(0, 0, 1), (N,)))
                self.ir.anchor_slots.append(k)
            self.anchor_slot_nodes = [mean, rstd] + ([gamma] if gamma is not None else [])
            self.pending_multi[anchor] = {0: "accum"}
            if mask[1] or mask[2]:
                # dweight = sum_rows g * xhat, dbias = sum_rows g: per-column reductions of two more per-element
                # values the anchor hands to the epilogue (the incoming gradient and the normalised input)
                self.ir.add_node(IRNode("ln_g", "anchorval", domain="tile", comp=0))
                self.ir.add_node(IRNode("ln_xhat", "anchorval", domain="tile", comp=1))
                per_column = full.reduce(list(range(rank - 1)), False)
                self.pending_coords[anchor] = {}
                if mask[1]:
                    self.ir.add_compute("ln_gx", "mul", ["ln_g", "ln_xhat"])
                    self.ir.add_reduce("ln_dw_red", "sum", "col", "ln_gx")
                    self.ir.add_node(IRNode("ln_dw", "rres", domain="col", reduce="ln_dw_red", comp=0))
                    self.pending_multi[anchor][1] = "ln_dw"
                    self.pending_coords[anchor][1] = per_column
                if mask[2]:
                    self.ir.add_reduce("ln_db_red", "sum", "col", "ln_g")
                    self.ir.add_node(IRNode("ln_db", "rres", domain="col", reduce="ln_db_red", comp=0))
                    self.pending_multi[anchor][2] = "ln_db"
                    self.pending_coords[anchor][2] = per_column

    @staticmethod
    def _extract_reference(graph_module: GraphModule, anchor: Node, epilogue_partition, inputs, outputs) -> GraphModule:
        """The epilogue as a module of its own: placeholder `accum` for the anchor's
        result plus one placeholder per partition input, returning the
        partition's outputs in order (the reference's `reference_gm`, consumed by
        FusedOpBase.reference_base, evt_fuser.py:98-126)."""
        import torch.fx as fx
        g = fx.Graph()
        env: Dict[Node, Node] = {anchor: g.placeholder("accum")}
        for inp in inputs:
            if inp is not anchor:
                env[inp] = g.placeholder(inp.name)
        for node in epilogue_partition:
            env[node] = g.node_copy(node, lambda n: env[n])
        g.output(tuple(env[o] for o in outputs))
        return GraphModule(graph_module, g)

    def _accum_dependents(self, anchor: Node, epi_set) -> set:
        full = {anchor}
        changed = True
        order = [n for n in anchor.graph.nodes if n in epi_set]
        while changed:
            changed = False
            for n in order:
                if n not in full and any(i in full for i in n.all_input_nodes):
                    full.add(n)
                    changed = True
        return full

    def _rebuild_slot_sources(self):
        self.slot_sources = {}
        for k, slot in enumerate(self.ir.slots):
            if slot.kind == "rand":
                self.slot_sources[k] = ("rand", None)
            elif k in self.ir.anchor_slots:
                j = self.ir.anchor_slots.index(k)
                self.slot_sources[k] = ("anchor", self.anchor_operands.index(self.anchor_slot_nodes[j]))
            elif slot.role == "load":
                node = next(n for n in self.input_nodes if n.name == slot.name)
                self.slot_sources[k] = ("input", self.input_index[node])
            else:
                self.slot_sources[k] = ("output", slot.name)

    # -- stores ---------------------------------------------------------------------
    def _insert_store(self, out: Node, store_key: Dict[Tuple, str]):
        name = "accum" if out is self.anchor else out.name
        shape, dtype = node_shape_dtype(out)
        if dtype not in DTYPE_NAMES:
            raise NotImplementedError(f"output dtype {dtype}")
        if out not in self.ir_name or out not in self.coords:
            # an output no other node of the epilogue reads and that does not depend on the accumulator: its
            # elements as the accumulator's coordinates see them
            coord = accum_coord(self.L, self.M, self.N, self.ir.batched).restrict(shape)
            self.ir_name[out] = self._materialize(out, coord)
            self.coords.setdefault(out, coord)
        value = self.ir_name[out]
        domain = self.ir.nodes[value].domain
        if domain == "flex":
            # formed from the epilogue's inputs alone.  One value per column (the reference's row store,
            # visitor_store.hpp:46-145: BERT's transformed attention mask leaves its first use that way) is
            # written by the tiles that hold row 0; anything else stays outside
            st0 = fit_strides(self.coords[out], self.L, self.M, self.N)
            if (st0 is None or st0.stride_m != 0 or st0.stride_n == 0 or self.M <= 0
                    or packet(self.anchor.target) in self.row_targets):
                raise NotImplementedError(
                    f"output {out.name} does not depend on the accumulator; keep it outside the partition")
            domain = "nvec"
        if domain not in ("tile", "row", "col", "nvec"):
            raise NotImplementedError(
                f"output {out.name} does not depend on the accumulator; keep it outside the partition")
        # find the tensor to materialise: the output itself, or (if its layout
        # is not strided in (l, m, n)) the node before trailing view/permute
        # ops, which are then applied as free views on the stored tensor
        # (the reference's post_reshape_permute, evt_fuser.py:247-255)
        node, post = out, []
        while True:
            st = fit_strides(self.coords[node], self.L, self.M, self.N)
            if st is not None:
                break
            tname = target_name(node.target) if node.op == "call_function" else ""
            src = node.args[0] if node.args and isinstance(node.args[0], Node) else None
            if tname not in LAYOUT_TARGETS or src is None or src not in self.coords:
                raise NotImplementedError(f"output {out.name}: layout is not expressible with (l, m, n) strides")
            nshape, _ = node_shape_dtype(node)
            if tname == "permute":
                post.insert(0, ("permute", [int(i) for i in node.args[1]]))
            elif tname in ("clone", "contiguous"):
                raise NotImplementedError(f"output {out.name}: materialised permutation is not strided in (l, m, n)")
            else:
                post.insert(0, ("view", list(nshape)))
            node = src
        sshape, _ = node_shape_dtype(node)
        key = (value, st.stride_l, st.stride_m, st.stride_n, st.l_div, st.l_mod, st.stride_l2, dtype, domain)
        if key in store_key:
            self.output2store[name] = store_key[key]
            stored_shape = self.store_meta[store_key[key]][0]
            if tuple(stored_shape) != tuple(sshape):
                post.insert(0, ("view", list(sshape)))
        else:
            store_key[key] = name
            self.output2store[name] = name
            self.store_meta[name] = (tuple(sshape), dtype)
            kind = {"tile": "aux", "row": "col", "col": "row", "nvec": "row"}[domain]
            k = self.ir.add_slot(Slot(name, "store", DTYPE_NAMES[dtype], domain, kind, st, tuple(sshape)))
            self.ir.stores.append(Store(k, value, domain))
        if post:
            self.post_reshape_permute[name] = post

    # -- operand materialisation (top-down) -----------------------------------------
    def _operand(self, arg, consumer_coord: Coord) -> str:
        """IR value name for operand `arg` of a node indexed by `consumer_coord`."""
        if isinstance(arg, (int, float, bool)):
            return self.ir.add_imm(float(arg))
        if not isinstance(arg, Node):
            raise NotImplementedError(f"operand {arg!r}")
        if arg in self.ir_name and arg in self.coords:
            return self.ir_name[arg]
        shape, dtype = node_shape_dtype(arg)
        return self._materialize(arg, consumer_coord.restrict(shape))

    def _materialize(self, node: Node, coord: Coord) -> str:
        """Value of a tensor that does not depend on the accumulator, indexed
        through `coord` (derived from its consumer)."""
        shape, dtype = node_shape_dtype(node)
        in_epilogue = node.name in self.partition_names and node.op == "call_function" and node is not self.anchor
        if not in_epilogue or node in self.inputs:
            # a kernel input: classify by how its offset varies with (l, m, n)
            st = fit_strides(coord, self.L, self.M, self.N)
            if st is None:
                raise NotImplementedError(f"input {node.name}: broadcast pattern is not strided in (l, m, n)")
            key = (node.name, (st.stride_l, st.stride_m, st.stride_n, st.l_div, st.l_mod, st.stride_l2))
            if key in self.load_cache:
                return self.load_cache[key]
            if dtype not in DTYPE_NAMES:
                raise NotImplementedError(f"input dtype {dtype}")
            if node not in self.input_index:
                raise NotImplementedError(f"{node.name} is used by the epilogue but is not a partition input")
            k = self.ir.add_slot(Slot(node.name, "load", DTYPE_NAMES[dtype], "tile", st.kind, st, shape))
            name = node.name if node.name not in self.ir.nodes else f"{node.name}_ld{k}"
            self.ir.add_node(IRNode(name, "load", domain="flex", slot=k))
            self.load_cache[key] = name
            return name
        tname = target_name(node.target)
        src = node.args[0] if node.args and isinstance(node.args[0], Node) else None
        if tname in ("view", "_unsafe_view", "reshape", "unsqueeze", "squeeze", "clone", "detach", "alias",
                     "contiguous", "expand"):
            sshape, _ = node_shape_dtype(src)
            if tname == "expand":
                return self._materialize(src, coord.restrict(sshape))
            return self._materialize(src, coord.reshape(sshape))
        if tname == "permute":
            sshape, _ = node_shape_dtype(src)
            return self._materialize(src, coord.inverse_permute([int(i) for i in node.args[1]], sshape))
        # elementwise on small tensors: evaluate per element from its operands
        self.coords[node] = coord
        self.visit(node)
        return self.ir_name[node]

    # -- node visitors (reference vocabulary: evt_fuser.py:1308-1485) ----------------
    def visit(self, node: Node):
        if node.op in ("placeholder", "get_attr"):
            return
        if node.op == "call_function":
            name = target_name(node.target)
            fn = getattr(self, f"visit_{name}", None)
            if fn is None:
                raise NotImplementedError(f"Doesn't support target {node.target}")
            return fn(node)

    def _coord_for(self, node: Node) -> Coord:
        """Coordinate function of an elementwise node: inherited from its
        accumulator-dependent operand (shapes equal up to broadcasting)."""
        if node in self.coords:
            return self.coords[node]
        shape, _ = node_shape_dtype(node)
        numel = 1
        for s in shape:
            numel *= s
        for arg in node.all_input_nodes:
            if arg in self.coords and arg in self.full:
                c = self.coords[arg]
                if c.numel() == numel:
                    return Coord(shape, c.fn)
        raise NotImplementedError(f"{node.name}: result is larger than its accumulator-dependent operand")

    def _visit_compute(self, node: Node, op: str, args: Optional[Sequence] = None):
        coord = self._coord_for(node)
        self.coords[node] = coord
        operands = [self._operand(a, coord) for a in (node.args if args is None else args)]
        name = node.name
        self.ir.add_compute(name, op, operands)
        self.ir_name[node] = name
        return name

    def _visit_layout(self, node: Node, fn):
        src = node.args[0]
        self.coords[node] = fn(self.coords[src])
        self.ir_name[node] = self.ir_name[src]
        return self.ir_name[node]

    def visit_add(self, node: Node):
        args = list(node.args)
        alpha = node.kwargs.get("alpha", 1)
        if alpha != 1:
            raise NotImplementedError("add with alpha")
        return self._visit_compute(node, "add", args)

    def visit_sub(self, node: Node):
        if node.kwargs.get("alpha", 1) != 1:
            raise NotImplementedError("sub with alpha")
        return self._visit_compute(node, "sub")

    def visit_rsub(self, node: Node):
        return self._visit_compute(node, "sub", [node.args[1], node.args[0]])

    def visit_mul(self, node: Node):
        return self._visit_compute(node, "mul")

    def visit_div(self, node: Node):
        return self._visit_compute(node, "div")

    def visit_neg(self, node: Node):
        return self._visit_compute(node, "neg")

    def visit_maximum(self, node: Node):
        return self._visit_compute(node, "max")

    def visit_minimum(self, node: Node):
        return self._visit_compute(node, "min")

    def visit_exp(self, node: Node):
        return self._visit_compute(node, "exp")

    def visit_log(self, node: Node):
        return self._visit_compute(node, "log")

    def visit_sqrt(self, node: Node):
        return self._visit_compute(node, "sqrt")

    def visit_rsqrt(self, node: Node):
        return self._visit_compute(node, "rsqrt")

    def visit_abs(self, node: Node):
        return self._visit_compute(node, "abs")

    def visit_reciprocal(self, node: Node):
        return self._visit_compute(node, "rcp")

    def visit_gelu(self, node: Node):
        # the reference drops the `approximate` keyword (evt_fuser.py:1377-1378);
        # here it selects the functor, as PyTorch defines it
        approx = node.kwargs.get("approximate", "none")
        return self._visit_compute(node, "gelu_tanh" if approx == "tanh" else "gelu_erf", node.args[:1])

    def visit_tanh(self, node: Node):
        return self._visit_compute(node, "tanh")

    def visit_relu(self, node: Node):
        return self._visit_compute(node, "relu")

    def visit_sigmoid(self, node: Node):
        return self._visit_compute(node, "sigmoid")

    def visit_tanh_backward(self, node: Node):
        return self._visit_compute(node, "tanh_backward")

    def visit_gelu_backward(self, node: Node):
        approx = node.kwargs.get("approximate", "none")
        return self._visit_compute(node, "gelu_backward_tanh" if approx == "tanh" else "gelu_backward_erf",
                                   node.args[:2])

    def visit_ge(self, node: Node):
        return self._visit_compute(node, "ge")

    def visit_gt(self, node: Node):
        return self._visit_compute(node, "gt")

    def visit_le(self, node: Node):
        return self._visit_compute(node, "le")

    def visit_lt(self, node: Node):
        return self._visit_compute(node, "lt")

    def visit_ne(self, node: Node):
        return self._visit_compute(node, "ne")

    def visit_eq(self, node: Node):
        return self._visit_compute(node, "eq")

    def visit_where(self, node: Node):
        return self._visit_compute(node, "where")

    def visit_rand_like(self, node: Node):
        """Uniform [0, 1) numbers shaped like an accumulator-dependent tensor
        (the reference's FunctionalOp.Rand, evt_fuser.py:1383-1384).  The values
        come from a counter-based generator indexed by the element's row-major
        position in the rand_like tensor, so they do not depend on the tile
        configuration; seed and per-call offset are run-time scalars."""
        coord = self._coord_for(node)
        self.coords[node] = coord
        st = fit_strides(coord, self.L, self.M, self.N)
        if st is None or st.kind != "aux":
            raise NotImplementedError("rand_like of a tensor that is not laid out over (l, m, n)")
        shape, _ = node_shape_dtype(node)
        self.ir.add_rand(node.name, st, shape)
        self.ir_name[node] = node.name
        self.full.add(node)
        return node.name

    def visit__to_copy(self, node: Node):
        dtype = node.kwargs.get("dtype", None)
        return self._visit_cast(node, dtype)

    def visit_to(self, node: Node):
        dtype = node.args[1] if len(node.args) > 1 and isinstance(node.args[1], torch.dtype) else node.kwargs.get("dtype")
        return self._visit_cast(node, dtype)

    def _visit_cast(self, node: Node, dtype):
        op = {torch.float16: "cast_f16", torch.bfloat16: "cast_bf16", torch.float32: "cast_f32",
              torch.bool: "cast_bool", torch.int32: "cast_int", torch.int64: "cast_int", None: "cast_f32"}.get(dtype)
        if op is None:
            raise NotImplementedError(f"cast to {dtype}")
        src = node.args[0]
        _, sdtype = node_shape_dtype(src)
        if op == "cast_f32" or (sdtype == dtype):
            # widening (or no-op) casts do not change the fp32 value
            if src in self.coords and src in self.ir_name:
                self.coords[node] = Coord(node_shape_dtype(node)[0], self.coords[src].fn)
                self.ir_name[node] = self.ir_name[src]
                return self.ir_name[node]
        return self._visit_compute(node, op, node.args[:1])

    def visit_one_hot(self, node: Node):
        """one_hot(label, num_classes)[..., n] == (label == n); the class axis is
        the GEMM N axis (reference: VisitorComputeOneHot,
        src/cuda/epilogue/threadblock/visitor_compute.hpp:98-145)."""
        num_classes = node.kwargs.get("num_classes", node.args[1] if len(node.args) > 1 else -1)
        shape, _ = node_shape_dtype(node)
        if int(num_classes) != self.N or shape[-1] != self.N:
            raise NotImplementedError("one_hot whose class axis is not the GEMM N axis")
        coord = self._coord_for(node) if node in self.coords else None
        if coord is None:
            raise NotImplementedError("one_hot must be consumed by an accumulator-dependent node")
        labels = node.args[0]
        lshape, _ = node_shape_dtype(labels)
        label_val = self._materialize(labels, coord.restrict(tuple(lshape) + (1,)))
        if "colidx" not in self.ir.nodes:
            self.ir.add_node(IRNode("colidx", "colidx", domain="tile"))
        self.ir.add_compute(node.name, "eq", [label_val, "colidx"])
        self.ir_name[node] = node.name
        return node.name

    def visit_gather(self, node: Node):
        """gather(x, -1, index[..., 1]) of an accumulator-dependent x along the N
        axis: sum_n x[n] * (index == n), a per-row reduction."""
        x, dim, index = node.args[0], node.args[1], node.args[2]
        xshape, _ = node_shape_dtype(x)
        ishape, _ = node_shape_dtype(index)
        if dim % len(xshape) != len(xshape) - 1 or ishape[-1] != 1 or xshape[-1] != self.N:
            raise NotImplementedError("gather other than one index per row along N")
        cx = self.coords[x]
        label_val = self._materialize(index, cx.restrict(ishape))
        if "colidx" not in self.ir.nodes:
            self.ir.add_node(IRNode("colidx", "colidx", domain="tile"))
        hit = f"{node.name}_hit"
        self.ir.add_compute(hit, "eq", [label_val, "colidx"])
        sel = f"{node.name}_sel"
        zero = self.ir.add_imm(0.0)
        self.ir.add_compute(sel, "where", [hit, self.ir_name[x], zero])
        (n,) = self._reduce(node, sel, cx, [len(xshape) - 1], True, "sum")
        self.ir_name[node] = n
        return n

    # -- reductions ------------------------------------------------------------------
    def _reduce(self, node: Node, value: str, coord: Coord, dims, keepdim: bool, kind: str,
                comps: Sequence[int] = (0,)):
        rc = coord.reduce(dims, keepdim)
        st = fit_strides(rc, self.L, self.M, self.N)
        if st is None:
            raise NotImplementedError(f"{node.name}: reduction result is not strided in (l, m, n)")
        numel = rc.numel()
        fold, fold_step, fold_count = "", 1, 1
        if st.stride_n == 0 and numel == self.L * self.M:
            axis = "row"
        elif st.stride_n == 0 and st.l_mod and st.l_div == 1 and numel == st.l_mod * self.M:
            # also summed over the batches that agree modulo l_mod (e.g. a [S, B, H*D] view of a BMM over
            # L = B*H batches, reduced over S and B: unittest/evt_fuser/bmm.py:48-67)
            axis, fold, fold_step, fold_count = "row", "mod", st.l_mod, self.L // st.l_mod
        elif st.stride_n == 0 and not st.l_mod and st.l_div > 1 and not st.stride_l2 and numel == (self.L // st.l_div) * self.M:
            axis, fold, fold_step, fold_count = "row", "div", 1, st.l_div     # l_div consecutive batches summed
        elif st.stride_m == 0 and numel == self.L * self.N and (self.L == 1 or st.stride_l != 0):
            axis = "col"
        elif (st.stride_m == 0 and st.stride_n != 0 and st.l_mod and st.l_div == 1 and not st.stride_l2
              and numel == st.l_mod * self.N and kind in ("sum", "max")):
            # per column, and over the batches that agree modulo l_mod: the bias gradient behind a batched product
            # whose result is merged back into [B, S, H * D] (sum over B and S for every head and column)
            axis, fold, fold_step, fold_count = "col", "mod", st.l_mod, self.L // st.l_mod
        else:
            raise NotImplementedError(
                f"{node.name}: reduces over something other than the N axis (optionally with batches folded) "
                f"or exactly the M axis")
        if fold and axis == "col" and kind not in ("sum", "max"):
            raise NotImplementedError(f"{node.name}: per-column {kind} reduction that also folds batches")
        # (a per-row reduction of any kind may fold batches: the partial states of the batches that share a result
        # go through the workspace and are merged with the kind's own combine operator, in batch order)
        for other in self.ir.reduces.values():
            if other.axis == axis and (other.fold, other.fold_step, other.fold_count) != (fold, fold_step, fold_count):
                raise NotImplementedError(f"{node.name}: per-{axis} reductions of one epilogue fold batches differently")
        rname = f"{node.name}_red"
        red = self.ir.add_reduce(rname, kind, axis, value)
        red.fold, red.fold_step, red.fold_count = fold, fold_step, fold_count
        names = []
        for c in comps:
            n = f"{node.name}_r{c}"
            self.ir.add_node(IRNode(n, "rres", domain=axis, reduce=rname, comp=c))
            names.append(n)
        self.coords[node] = rc
        return names

    @staticmethod
    def _dims(arg, rank):
        if arg is None or arg == []:
            return list(range(rank))
        if isinstance(arg, int):
            return [arg]
        return [int(a) for a in arg]

    def visit_sum(self, node: Node):
        x = node.args[0]
        shape, _ = node_shape_dtype(x)
        dims = self._dims(node.args[1] if len(node.args) > 1 else None, len(shape))
        keepdim = bool(node.args[2]) if len(node.args) > 2 else bool(node.kwargs.get("keepdim", False))
        value = self.ir_name[x]
        fused = self._match_softmax_stats(x, dims)
        if fused is not None:
            base, amax_node = fused
            rname = self.ir.nodes[self.ir_name[amax_node]].reduce
            # upgrade the row max to the (max, sum-exp) pair; this sum is its
            # second component
            self.ir.reduces[rname].kind = "maxsumexp"
            n = f"{node.name}_r1"
            self.ir.add_node(IRNode(n, "rres", domain="row", reduce=rname, comp=1))
            self.coords[node] = self.coords[x].reduce(dims, keepdim)
            self.ir_name[node] = n
            return n
        (n,) = self._reduce(node, value, self.coords[x], dims, keepdim, "sum")
        self.ir_name[node] = n
        return n

    def _match_softmax_stats(self, x: Node, dims) -> Optional[Tuple[Node, Node]]:
        """x == exp(sub(s, amax(s, dims, keepdim=True))) with the amax already a
        per-row max reduction of the same s -> (s, amax node)."""
        if x.op != "call_function" or target_name(x.target) != "exp":
            return None
        sub = x.args[0]
        if not isinstance(sub, Node) or sub.op != "call_function" or target_name(sub.target) != "sub":
            return None
        s, m = sub.args[0], sub.args[1]
        if not isinstance(m, Node) or not isinstance(s, Node) or m not in self.ir_name:
            return None
        mval = self.ir.nodes.get(self.ir_name[m])
        if mval is None or mval.op != "rres" or mval.comp != 0:
            return None
        red = self.ir.reduces[mval.reduce]
        if red.kind not in ("max", "maxsumexp") or red.axis != "row" or red.input != self.ir_name.get(s):
            return None
        shape, _ = node_shape_dtype(x)
        if sorted(d % len(shape) for d in dims) != [len(shape) - 1]:
            return None
        return s, m

    def visit_amax(self, node: Node):
        x = node.args[0]
        shape, _ = node_shape_dtype(x)
        dims = self._dims(node.args[1] if len(node.args) > 1 else None, len(shape))
        keepdim = bool(node.args[2]) if len(node.args) > 2 else bool(node.kwargs.get("keepdim", False))
        (n,) = self._reduce(node, self.ir_name[x], self.coords[x], dims, keepdim, "max")
        self.ir_name[node] = n
        return n

    def visit_mean(self, node: Node):
        x = node.args[0]
        shape, _ = node_shape_dtype(x)
        dims = self._dims(node.args[1] if len(node.args) > 1 else None, len(shape))
        keepdim = bool(node.args[2]) if len(node.args) > 2 else bool(node.kwargs.get("keepdim", False))
        (s,) = self._reduce(node, self.ir_name[x], self.coords[x], dims, keepdim, "sum")
        count = 1
        for d in dims:
            count *= shape[d]
        inv = self.ir.add_imm(1.0 / count)
        self.ir.add_compute(node.name, "mul", [s, inv])
        self.ir_name[node] = node.name
        return node.name

    def visit_logsumexp(self, node: Node):
        x = node.args[0]
        shape, _ = node_shape_dtype(x)
        dims = self._dims(node.args[1], len(shape))
        keepdim = bool(node.args[2]) if len(node.args) > 2 else bool(node.kwargs.get("keepdim", False))
        m, l = self._reduce(node, self.ir_name[x], self.coords[x], dims, keepdim, "maxsumexp", (0, 1))
        if self.ir.reduces[f"{node.name}_red"].axis != "row":
            raise NotImplementedError("logsumexp over the M axis")
        self.ir.add_compute(f"{node.name}_log", "log", [l])
        self.ir.add_compute(node.name, "add", [m, f"{node.name}_log"])
        self.ir_name[node] = node.name
        return node.name

    def visit_var_mean(self, node: Node):
        """var_mean(x, dims, correction=c, keepdim=k) -> (var, mean); consumed
        through getitem."""
        x = node.args[0]
        shape, _ = node_shape_dtype(x)
        dims = self._dims(node.args[1] if len(node.args) > 1 else node.kwargs.get("dim"), len(shape))
        keepdim = bool(node.kwargs.get("keepdim", False))
        correction = node.kwargs.get("correction", 1)
        if "unbiased" in node.kwargs:
            correction = 1 if node.kwargs["unbiased"] else 0
        n, mean, m2 = self._reduce(node, self.ir_name[x], self.coords[x], dims, keepdim, "welford", (0, 1, 2))
        if self.ir.reduces[f"{node.name}_red"].axis != "row":
            raise NotImplementedError("var_mean over the M axis")
        denom = n
        if correction:
            c = self.ir.add_imm(float(correction))
            denom = f"{node.name}_dof"
            self.ir.add_compute(denom, "sub", [n, c])
        var = f"{node.name}_var"
        self.ir.add_compute(var, "div", [m2, denom])
        self.pending_multi[node] = {0: var, 1: mean}
        return var

    def visit_getitem(self, node: Node):
        src, idx = node.args
        if src not in self.pending_multi:
            raise NotImplementedError(f"getitem of {src.name}")
        if int(idx) not in self.pending_multi[src]:
            raise NotImplementedError(f"getitem {int(idx)} of {src.name}")
        self.ir_name[node] = self.pending_multi[src][int(idx)]
        own = self.pending_coords.get(src, {}).get(int(idx))
        self.coords[node] = own if own is not None else Coord(node_shape_dtype(node)[0], self.coords[src].fn)
        return self.ir_name[node]

    # -- layout ops: no data movement, only index bookkeeping -----------------------
    def visit_view(self, node: Node):
        shape, _ = node_shape_dtype(node)
        return self._visit_layout(node, lambda c: c.reshape(shape))

    visit__unsafe_view = visit_view
    visit_reshape = visit_view
    visit_unsqueeze = visit_view
    visit_squeeze = visit_view

    def visit_permute(self, node: Node):
        dims = [int(i) for i in node.args[1]]
        return self._visit_layout(node, lambda c: c.permute(dims))

    def visit_clone(self, node: Node):
        return self._visit_layout(node, lambda c: c)

    visit_detach = visit_clone
    visit_alias = visit_clone
    visit_contiguous = visit_clone

    def visit_expand(self, node: Node):
        shape, _ = node_shape_dtype(node)
        src_shape, _ = node_shape_dtype(node.args[0])
        n1 = n2 = 1
        for s in shape:
            n1 *= s
        for s in src_shape:
            n2 *= s
        if n1 != n2:
            raise NotImplementedError("expand that enlarges an accumulator-dependent tensor")
        return self._visit_layout(node, lambda c: c.reshape(shape))

    # -- main-loop op ------------------------------------------------------------------
    def get_fused_node(self, node: Node):
        tgt = packet(node.target)
        if tgt == aten.mm:
            return FusedGEMM(node, self)
        if tgt == aten.bmm:
            return FusedBMM(node, self)
        if tgt in self.row_targets:
            return self.row_targets[tgt](node, self)
        raise NotImplementedError()
