"""CPU oracle for the fused GEMM/BMM + epilogue path.  TEST INFRASTRUCTURE ONLY:
imported by tests/, by __graft_entry__.smoke() and by bench.py's cpu_baseline
leg as the checker / the timed CPU baseline, never by the product path.

What it restates.  The reference's arithmetic for this path lives in an
un-vendored dependency (thirdparty/cutlass, fork apuaaChen/cutlass branch
3.2_fix, commit unpinned; call sites python/gtl/compiler/passes/
evt_fuser.py:481-486, :515-518, :539-546) and the reference's own tests hold no
numeric vectors (unittest/evt_fuser/mm.py:28 compares against the same module
run eagerly, atol 2e-1, on unseeded random inputs).  The specified oracle is
therefore PyTorch's own eager evaluation, in fp32, of the same fx subgraph on
the fp16-rounded inputs:

  * `eval_fp32`      runs the ATen-level module on CPU with every floating
                     input widened to fp32 (semantics the fused kernel follows:
                     fp32 intermediates, one rounding per store;
                     src/cuda/epilogue/threadblock/visitor.hpp:221-226,
                     visitor_store.hpp:99-112);
  * `closed_form`    an independent numpy float64 restatement of each headline
                     subgraph from its mathematical definition (no torch), used
                     to pin `eval_fp32`;
  * `gemm_bruteforce` a pure-Python triple loop for tiny shapes that pins the
                     operand-index conventions of both.

Pinned by tests/test_oracle.py: closed forms vs eval_fp32 on seeded inputs,
brute force on tiny ragged shapes, identity/ones-matrix cases, GELU special
values and odd symmetry, finite-difference GELU', softmax shift invariance and
sum-to-one, LayerNorm affine invariance and constant rows, exact integer column
sums, CE of uniform logits = log N, and the committed golden fixtures.
Parity unpinned (no reference vector exists, see above): which GELU flavour the
fork's ActivationOp.Gelu / DGelu denote -- this oracle follows the graph's
`approximate` keyword as PyTorch defines it.
"""
from __future__ import annotations

import contextlib
import math
from typing import Dict, List, Sequence, Tuple

import numpy as np
import torch

FP16_TOL = 2e-2        # max relative error, fp16 outputs
REDUCTION_TOL = 1e-3   # max relative error, fp32 reduction outputs
TAU_FACTOR = 1e-2      # floor of the relative-error denominator, x rms(ref)


# ---------------------------------------------------------------------------
# PyTorch fp32 eager evaluation of the subgraph
# ---------------------------------------------------------------------------

def widen(t):
    if isinstance(t, torch.Tensor) and t.dtype in (torch.float16, torch.bfloat16):
        return t.float()
    return t


@contextlib.contextmanager
def philox_rand_like(seed: int, offset: int, salt: int):
    """Inside the block `torch.rand_like(x)` returns the numbers the fused kernels
    generate for a rand_like tensor shaped like x (oracle/philox.py) under the
    given (seed, offset) and slot salt, instead of drawing from torch's generator."""
    from . import philox
    orig = torch.rand_like

    def replay(x, *a, **k):
        u = philox.uniform(seed, offset, salt, x.numel())
        return torch.from_numpy(u).view(x.shape).to(dtype=torch.float32)
    torch.rand_like = replay
    try:
        yield
    finally:
        torch.rand_like = orig


class _Fp32DtypeFlags(torch.overrides.TorchFunctionMode):
    """`aten._softmax(x, dim, half_to_float)` and `aten._softmax_backward_data(g, y,
    dim, input_dtype)` name the fp16 storage type of the graph; on the widened
    fp32 inputs of the oracle the flags have to say fp32."""

    def __torch_function__(self, func, types, args=(), kwargs=None):
        kwargs = kwargs or {}
        pk = getattr(func, "overloadpacket", func)
        if pk is torch.ops.aten._softmax and args[0].dtype == torch.float32:
            args = (args[0], args[1], False)
        elif pk is torch.ops.aten._softmax_backward_data and args[0].dtype == torch.float32:
            args = (args[0], args[1], args[2], torch.float32)
        return func(*args, **kwargs)


def eval_fp32(module: torch.nn.Module, inputs: Sequence[torch.Tensor], rand=None) -> List[torch.Tensor]:
    """Eager fp32 evaluation on CPU of `module` on the (already fp16-rounded) inputs.
    rand = (seed, offset, salt): replay the kernels' random stream for rand_like."""
    with torch.no_grad(), _Fp32DtypeFlags(), (philox_rand_like(*rand) if rand is not None else contextlib.nullcontext()):
        out = module(*[widen(t.cpu() if isinstance(t, torch.Tensor) else t) for t in inputs])
    if isinstance(out, torch.Tensor):
        out = [out]
    return [o.float() if o.is_floating_point() else o for o in out]


# ---------------------------------------------------------------------------
# error metric of the parity contract
# ---------------------------------------------------------------------------

def max_rel_err(out, ref) -> float:
    """max |out - ref| / max(|ref|, tau), tau = 1e-2 * rms(ref)."""
    out = np.asarray(out.detach().cpu().float().numpy() if isinstance(out, torch.Tensor) else out, dtype=np.float64)
    ref = np.asarray(ref.detach().cpu().float().numpy() if isinstance(ref, torch.Tensor) else ref, dtype=np.float64)
    if out.shape != ref.shape:
        raise AssertionError(f"shape mismatch {out.shape} vs {ref.shape}")
    if not np.all(np.isfinite(out)):
        return float("inf")
    rms = math.sqrt(float(np.mean(ref * ref))) if ref.size else 0.0
    tau = max(TAU_FACTOR * rms, 1e-30)
    return float(np.max(np.abs(out - ref) / np.maximum(np.abs(ref), tau))) if ref.size else 0.0


def check(out, ref, reduction: bool) -> Tuple[bool, float]:
    if isinstance(ref, torch.Tensor) and ref.dtype == torch.bool:
        ok = bool(torch.equal(out.cpu().bool(), ref))
        return ok, 0.0 if ok else float("inf")
    err = max_rel_err(out, ref)
    return err <= (REDUCTION_TOL if reduction else FP16_TOL), err


# ---------------------------------------------------------------------------
# numpy float64 closed forms
# ---------------------------------------------------------------------------

def _f64(t) -> np.ndarray:
    return t.detach().cpu().to(torch.float64).numpy() if isinstance(t, torch.Tensor) else np.asarray(t, np.float64)


def gelu_tanh(x: np.ndarray) -> np.ndarray:
    """0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3)))"""
    return 0.5 * x * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x ** 3)))


def gelu_tanh_grad(x: np.ndarray) -> np.ndarray:
    """d/dx gelu_tanh(x) = 0.5 (1 + t) + 0.5 x (1 - t^2) sqrt(2/pi) (1 + 0.134145 x^2)"""
    c = math.sqrt(2.0 / math.pi)
    t = np.tanh(c * (x + 0.044715 * x ** 3))
    return 0.5 * (1.0 + t) + 0.5 * x * (1.0 - t * t) * c * (1.0 + 3 * 0.044715 * x * x)


def closed_form(cfg: int, inputs: Sequence[torch.Tensor]) -> List[np.ndarray]:
    """Outputs of headline subgraph `cfg` from its definition, in float64."""
    if cfg == 1:
        x, w, b = map(_f64, inputs)
        return [gelu_tanh(x @ w + b)]
    if cfg == 2:
        q, k = map(_f64, inputs)
        s = np.einsum("lmd,lnd->lmn", q, k) * 0.125
        m = s.max(-1, keepdims=True)
        return [s, m, np.exp(s - m).sum(-1, keepdims=True)]
    if cfg == 3:
        x, w, b, r = map(_f64, inputs)
        o = x @ w + b + r
        mean = o.mean(1)
        return [o, mean, ((o - mean[:, None]) ** 2).mean(1)]
    if cfg == 4:
        dy, w, p = map(_f64, inputs)
        dp = (dy @ w.T) * gelu_tanh_grad(p)
        return [dp, dp.sum(0)]
    if cfg == 5:
        h, w = _f64(inputs[0]), _f64(inputs[1])
        labels = inputs[2].cpu().numpy().astype(np.int64)
        z = h @ w
        m = z.max(1)
        lse = m + np.log(np.exp(z - m[:, None]).sum(1))
        return [lse - z[np.arange(z.shape[0]), labels]]
    raise KeyError(cfg)


def gemm_bruteforce(a, b) -> np.ndarray:
    """C[i][j] = sum_k A[i][k] B[k][j] with Python loops (tiny shapes only)."""
    a, b = _f64(a), _f64(b)
    M, K = a.shape
    K2, N = b.shape
    assert K == K2
    c = np.zeros((M, N))
    for i in range(M):
        for j in range(N):
            acc = 0.0
            for k in range(K):
                acc += a[i, k] * b[k, j]
            c[i, j] = acc
    return c


# ---------------------------------------------------------------------------
# two-phase reduction algebra (what the kernels' combine steps must satisfy)
# ---------------------------------------------------------------------------

def combine_maxsumexp(a: Tuple[float, float], b: Tuple[float, float]) -> Tuple[float, float]:
    m = max(a[0], b[0])
    la = 0.0 if a[0] == -math.inf else a[1] * math.exp(a[0] - m)
    lb = 0.0 if b[0] == -math.inf else b[1] * math.exp(b[0] - m)
    return m, la + lb


def combine_welford(a: Tuple[float, float, float], b: Tuple[float, float, float]) -> Tuple[float, float, float]:
    """Chan, Golub, LeVeque parallel (count, mean, M2) update."""
    n = a[0] + b[0]
    if n == 0:
        return 0.0, 0.0, 0.0
    d = b[1] - a[1]
    return n, a[1] + d * b[0] / n, a[2] + b[2] + d * d * a[0] * b[0] / n
