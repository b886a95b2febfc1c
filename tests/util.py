"""Shared helpers for the tests."""
from __future__ import annotations

import torch

from evt_ae_amd.evt_fuser import FusedBMM, FusedGEMM, FusedOpBase
from oracle import ir_interp, philox

aten = torch.ops.aten


from evt_ae_amd.workloads import fused_nodes  # noqa: E402,F401


def emulate_fused(op: FusedOpBase, *args):
    """What `FusedOpBase.__call__` returns, computed on CPU from the op's IR
    with the IR interpreter instead of the HIP kernel."""
    args = [a.contiguous() if isinstance(a, torch.Tensor) else a for a in args]
    A, B = args[-2].float(), args[-1].float()
    if isinstance(op, FusedGEMM):
        Al = A if op.a_kc else A.t()
        Bl = B.t() if op.b_kc else B
        acc = Al @ Bl
    else:
        acc = op.anchor_eager(A, B)        # replays the operands' layout chains
        if op.transposed:                  # the IR describes the epilogue of the transposed product
            acc = acc.transpose(1, 2)
    loads = {}
    for k, slot in enumerate(op.ir.slots):
        kind, ref = op.slot_sources[k]
        if kind == "input":
            loads[k] = args[ref]
        elif kind == "rand":   # the numbers the kernel generates for this launch
            numel = 1
            for d in slot.shape:
                numel *= d
            loads[k] = torch.from_numpy(philox.uniform(op.rand_seed, op.rand_offset, op.rand_salt(k), numel))
    if op.ir.rng_scalar is not None:
        op.last_rand_state = (op.rand_seed, op.rand_offset & 0xFFFFFFFF)
        op.rand_offset += 1
    stored = ir_interp.interpret(op.ir, acc, loads)
    visitor = {}
    for k, slot in enumerate(op.ir.slots):
        if slot.role == "store":
            shape, dtype = op.store_meta[slot.name]
            numel = 1
            for s in shape:
                numel *= s
            flat = stored[k]
            assert flat.numel() == numel, (slot.name, flat.numel(), shape)
            visitor[slot.name] = flat.view(shape)
    results = []
    for out in op.outputs:
        name = op.get_output_name(out)
        t = visitor[op.output2store[name]]
        for kind, arg in op.post_reshape_permute.get(name, ()):
            t = t.view(arg) if kind == "view" else t.permute(arg)
        results.append(t)
    return results


def run_emulated(gm, inputs):
    """Run a fused GraphModule on CPU with every fused node emulated."""
    import types
    patched = []
    for n in fused_nodes(gm):
        op = n.target
        patched.append((op, op.__class__.__call__))
    # FusedOpBase.__call__ is looked up on the class: patch per instance via a subclass
    for op, _ in patched:
        op.__class__ = type("Emulated" + op.__class__.__name__, (op.__class__,),
                            {"__call__": lambda self, *a: emulate_fused(self, *a)})
    try:
        out = gm(*inputs)
    finally:
        for op, _ in patched:
            op.__class__ = op.__class__.__mro__[1]
    return list(out) if isinstance(out, (tuple, list)) else [out]


def rand_slot(op: FusedOpBase) -> int:
    """Generator salt (slot index + 16 x the op's stream id) of the op's single rand_like slot."""
    (k,) = [k for k, s in enumerate(op.ir.slots) if s.kind == "rand"]
    return op.rand_salt(k)


def fake_argument_block(op: FusedOpBase):
    """The op's argument block with made-up (aligned, non-null) pointers: what the host side of a module needs
    to run its checks and size its workspace without any device memory."""
    from evt_ae_amd.evt_fuser import FusedRowOp
    a = op.new_argument_block()
    M, N, K, L = op.problem
    a.M, a.N, a.K, a.L = M, N, getattr(op, "kernel_k", K), L
    a.A, a.B = 0x7000_0000_0000, 0x7100_0000_0000
    if isinstance(op, FusedRowOp):
        a.lda = a.ldb = N
        a.batch_stride_A = a.batch_stride_B = M * N
    else:
        a.lda, a.ldb = op.lda, op.ldb
        a.batch_stride_A, a.batch_stride_B = getattr(op, "bsa", 0), getattr(op, "bsb", 0)
        if isinstance(op, FusedBMM):
            a.batch_div_A, a.batch_stride2_A = op.bdiva, op.bs2a
            a.batch_div_B, a.batch_stride2_B = op.bdivb, op.bs2b
    for k in range(a.num_tensors):
        a.tensors[k].ptr = 0x7200_0000_0000 + (k << 36)
    return a
