"""CPU interpreter of the epilogue IR.  TEST INFRASTRUCTURE ONLY.

Evaluates an `EpilogueIR` (duck-typed: .nodes, .slots, .reduces, .stores,
.scalars, .L/.M/.N) on fp32 torch tensors exactly as the generated kernels are
specified to: every node once per (l, m, n), loads through the fitted
(batch index, m, n) strides, reductions over the N axis ('row') or the M axis
('col'), per-row / per-column post expressions, one rounding per store.  Used
by the CPU tests to check that `EVTFuser.trace` (the host-side mirror of
python/gtl/compiler/passes/evt_fuser.py:1065-1235) lowers a graph to an IR
whose meaning is the graph's.
"""
from __future__ import annotations

from typing import Dict, List

import torch

_TORCH_DTYPE = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32, "bool": torch.bool,
                "i32": torch.int32, "i64": torch.int64, "u8": torch.uint8}


def _gelu_tanh(x):
    return torch.nn.functional.gelu(x, approximate="tanh")


def _apply(op: str, a: List[torch.Tensor]) -> torch.Tensor:
    f = torch.float32
    if op == "add": return a[0] + a[1]
    if op == "sub": return a[0] - a[1]
    if op == "mul": return a[0] * a[1]
    if op == "div": return a[0] / a[1]
    if op == "max": return torch.maximum(a[0], a[1])
    if op == "min": return torch.minimum(a[0], a[1])
    if op == "neg": return -a[0]
    if op == "exp": return torch.exp(a[0])
    if op == "log": return torch.log(a[0])
    if op == "sqrt": return torch.sqrt(a[0])
    if op == "rsqrt": return torch.rsqrt(a[0])
    if op == "abs": return torch.abs(a[0])
    if op == "rcp": return 1.0 / a[0]
    if op == "gelu_tanh": return _gelu_tanh(a[0])
    if op == "gelu_erf": return torch.nn.functional.gelu(a[0])
    if op == "tanh": return torch.tanh(a[0])
    if op == "relu": return torch.relu(a[0])
    if op == "sigmoid": return torch.sigmoid(a[0])
    if op == "tanh_backward": return a[0] * (1 - a[1] * a[1])
    if op == "gelu_backward_tanh": return torch.ops.aten.gelu_backward(a[0], a[1], approximate="tanh")
    if op == "gelu_backward_erf": return torch.ops.aten.gelu_backward(a[0], a[1], approximate="none")
    if op == "ge": return (a[0] >= a[1]).to(f)
    if op == "gt": return (a[0] > a[1]).to(f)
    if op == "le": return (a[0] <= a[1]).to(f)
    if op == "lt": return (a[0] < a[1]).to(f)
    if op == "ne": return (a[0] != a[1]).to(f)
    if op == "eq": return (a[0] == a[1]).to(f)
    if op == "cast_f16": return a[0].half().float()
    if op == "cast_bf16": return a[0].bfloat16().float()
    if op == "cast_f32": return a[0]
    if op == "cast_bool": return (a[0] != 0).to(f)
    if op == "cast_int": return torch.trunc(a[0])
    if op == "where": return torch.where(a[0] != 0, a[1], a[2])
    raise NotImplementedError(op)


def _gather_strided(t: torch.Tensor, st, L, M, N) -> torch.Tensor:
    """Full [L, M, N] fp32 tensor of the slot's values at each iteration point."""
    flat = t.reshape(-1)
    l = torch.arange(L).view(L, 1, 1)
    m = torch.arange(M).view(1, M, 1)
    n = torch.arange(N).view(1, 1, N)
    off = st.batch_offset(l) + m * st.stride_m + n * st.stride_n
    return flat[off.reshape(-1)].reshape(L, M, N).to(torch.float32)


def interpret(ir, accum: torch.Tensor, slot_tensors: Dict[int, torch.Tensor]) -> Dict[int, torch.Tensor]:
    """accum: fp32 [L, M, N] (or [M, N]); slot_tensors: load slot -> CPU tensor.
    Returns store slot -> flat tensor holding the stored values (dtype of the slot)."""
    L, M, N = ir.L, ir.M, ir.N
    acc = accum.reshape(L, M, N).to(torch.float32)
    val: Dict[str, torch.Tensor] = {}
    for name, node in ir.nodes.items():
        if node.op == "accum":
            val[name] = acc
        elif node.op == "imm":
            val[name] = torch.full((1, 1, 1), float(torch.tensor(ir.scalars[node.slot], dtype=torch.float32)))
        elif node.op == "colidx":
            val[name] = torch.arange(N, dtype=torch.float32).view(1, 1, N).expand(L, M, N)
        elif node.op == "load":
            val[name] = _gather_strided(slot_tensors[node.slot], ir.slots[node.slot].strides, L, M, N)
        elif node.op == "rres":
            r = ir.reduces[node.reduce]
            x = val[r.input].expand(L, M, N)
            fold = getattr(r, "fold", "")
            if fold:
                # Batches that share a result are reduced together: bring them side by side in front of the reduced
                # axis ([groups, members, M, N]), reduce over members and the axis, and let every member carry the
                # total.  'mod': batch l = j * step + key belongs to group key; 'div': l = key * count + j.
                cnt = r.fold_count
                g4 = x.reshape(cnt, L // cnt, M, N).transpose(0, 1) if fold == "mod" else x.reshape(L // cnt, cnt, M, N)
                dims = (1, 3) if r.axis == "row" else (1, 2)
            else:
                g4 = x.reshape(L, 1, M, N)
                dims = (1, 3) if r.axis == "row" else (1, 2)
            if r.kind == "sum":
                out = g4.sum(dims, keepdim=True)
            elif r.kind == "max":
                out = g4.amax(dims, keepdim=True)
            elif r.kind == "maxsumexp":
                mx = g4.amax(dims, keepdim=True)
                out = mx if node.comp == 0 else torch.exp(g4 - mx).sum(dims, keepdim=True)
            elif r.kind == "welford":
                cnt_el = g4.shape[dims[0]] * g4.shape[dims[1]]
                mean = g4.mean(dims, keepdim=True)
                out = (torch.full_like(mean, float(cnt_el)) if node.comp == 0 else mean if node.comp == 1
                       else ((g4 - mean) ** 2).sum(dims, keepdim=True))
            else:
                raise NotImplementedError(r.kind)
            tail = (M, 1) if r.axis == "row" else (1, N)
            if fold:
                members = g4.shape[1]
                out = out.expand(g4.shape[0], members, *tail)
                out = out.transpose(0, 1).reshape(L, *tail) if fold == "mod" else out.reshape(L, *tail)
            else:
                out = out.reshape(L, *tail)
            val[name] = out
        else:
            val[name] = _apply(node.op, [val[i] for i in node.inputs])
    outs: Dict[int, torch.Tensor] = {}
    l = torch.arange(L).view(L, 1, 1)
    m = torch.arange(M).view(1, M, 1)
    n = torch.arange(N).view(1, 1, N)
    for s in ir.stores:
        slot = ir.slots[s.slot]
        st = slot.strides
        v = val[s.input].expand(L, M, N)
        off = (st.batch_offset(l) + m * st.stride_m + n * st.stride_n).expand(L, M, N)
        size = int(off.max()) + 1
        buf = torch.zeros(size, dtype=torch.float32)
        buf[off.reshape(-1)] = v.reshape(-1)
        dt = _TORCH_DTYPE[slot.dtype]
        outs[s.slot] = (buf != 0) if dt == torch.bool else buf.to(dt)
    return outs
