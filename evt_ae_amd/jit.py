"""Compile, cache and load generated kernel modules.

Replaces the un-vendored `cutlass.backend.compiler` (nvcc/nvrtc JIT with a
sqlite `compiled_cache.db`; call sites python/gtl/compiler/passes/
evt_fuser.py:515-518, :738-746).  A module is identified by the SHA-256 of its
generated source and compile flags; the shared object is kept in-tree under
`evt_ae_amd/_kernels/` so that modules built ahead of time travel with the
source tree, and an sqlite index (`compiled_cache.db`) records what each file
is.  Loading goes through ctypes against the C ABI of include/evt_amd.h.
"""
from __future__ import annotations

import ctypes
import hashlib
import json
import re
import logging
import os
import sqlite3
import subprocess
import threading
from pathlib import Path
from typing import Dict, Optional

from .codegen import ABI_VERSION, KernelSpec, generate
from .ir import EpilogueIR

PKG_DIR = Path(__file__).resolve().parent
CSRC_DIR = Path(os.environ.get("EVT_CSRC_DIR", PKG_DIR / "csrc"))
INCLUDE_DIR = PKG_DIR.parent / "include"
KERNEL_DIR = Path(os.environ.get("EVT_KERNEL_DIR", PKG_DIR / "_kernels"))
CACHE_FILE = KERNEL_DIR / "compiled_cache.db"

EVT_ABI_VERSION = ABI_VERSION
EVT_MAX_TENSORS = 16
EVT_MAX_SCALARS = 16

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-shared", "-fPIC",
    # packed-fp32 VALU forms are kept off on this hardware pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-value", "-Wno-unknown-attributes",
    # The epilogue's row loops are written to be unrolled in full: the accumulators are indexed by their loop
    # counters and must stay in registers.  Past the compiler's default size limit for `#pragma unroll` a loop
    # stays rolled and the accumulators go to scratch memory (three residual loads on a 128 x 64 wave tile: 576
    # bytes of scratch per lane, 114 us instead of 53)
    "-mllvm", "-pragma-unroll-threshold=1000000",
] + os.environ.get("EVT_HIPCC_EXTRA", "").split()


class EvtTensorArg(ctypes.Structure):
    _fields_ = [("ptr", ctypes.c_void_p), ("stride_l", ctypes.c_int64), ("stride_m", ctypes.c_int64),
                ("stride_n", ctypes.c_int64), ("l_div", ctypes.c_int64), ("l_mod", ctypes.c_int64),
                ("stride_l2", ctypes.c_int64)]


class EvtArgs(ctypes.Structure):
    _fields_ = [("M", ctypes.c_int32), ("N", ctypes.c_int32), ("K", ctypes.c_int32), ("L", ctypes.c_int32),
                ("A", ctypes.c_void_p), ("lda", ctypes.c_int64), ("batch_stride_A", ctypes.c_int64),
                ("B", ctypes.c_void_p), ("ldb", ctypes.c_int64), ("batch_stride_B", ctypes.c_int64),
                ("batch_div_A", ctypes.c_int64), ("batch_stride2_A", ctypes.c_int64),
                ("batch_div_B", ctypes.c_int64), ("batch_stride2_B", ctypes.c_int64),
                ("num_tensors", ctypes.c_int32), ("num_scalars", ctypes.c_int32),
                ("split_k", ctypes.c_int32), ("flags", ctypes.c_int32),
                ("tensors", EvtTensorArg * EVT_MAX_TENSORS), ("scalars", ctypes.c_float * EVT_MAX_SCALARS)]


EVT_FLAG_TWO_KERNEL_REDUCE = 1
EVT_FLAG_ROW_WG_PER_CU_MASK = 0xFF00


def evt_flag_row_wg_per_cu(n: int) -> int:
    """EVT_FLAG_ROW_WG_PER_CU(n) of include/evt_amd.h."""
    return ((n + 1) & 0xFF) << 8

ERROR_NAMES = {-1: "EVT_ERR_BAD_ARGS", -2: "EVT_ERR_ALIGNMENT", -3: "EVT_ERR_WORKSPACE", -4: "EVT_ERR_RANGE",
               -5: "EVT_ERR_SCRATCH"}


class KernelModule:
    """A loaded fused-kernel shared object."""

    def __init__(self, path: Path):
        self.path = Path(path)
        self.lib = ctypes.CDLL(str(path), mode=ctypes.RTLD_LOCAL)
        self.lib.evt_abi_version.restype = ctypes.c_int
        self.lib.evt_module_spec.restype = ctypes.c_char_p
        self.lib.evt_workspace_bytes.restype = ctypes.c_int64
        self.lib.evt_workspace_bytes.argtypes = [ctypes.POINTER(EvtArgs)]
        self.lib.evt_workspace_init.restype = ctypes.c_int
        self.lib.evt_workspace_init.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]
        self.lib.evt_launch.restype = ctypes.c_int
        self.lib.evt_launch.argtypes = [ctypes.POINTER(EvtArgs), ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]
        self.lib.evt_launch_static.restype = ctypes.c_int
        self.lib.evt_launch_static.argtypes = [ctypes.POINTER(EvtArgs), ctypes.c_void_p]
        if self.lib.evt_abi_version() != EVT_ABI_VERSION:
            raise RuntimeError(f"{path}: ABI version mismatch")
        if hasattr(self.lib, "evt_clock_probe_read"):      # diagnostic builds only
            self.lib.evt_clock_probe_read.restype = ctypes.c_int
            self.lib.evt_clock_probe_read.argtypes = [ctypes.POINTER(ctypes.c_uint64)]
        self.spec = json.loads(self.lib.evt_module_spec().decode())

    def workspace_bytes(self, args: EvtArgs) -> int:
        n = self.lib.evt_workspace_bytes(ctypes.byref(args))
        if n < 0:
            raise RuntimeError(f"evt_workspace_bytes: {ERROR_NAMES.get(n, n)}")
        return n

    def workspace_init(self, ptr: int, nbytes: int, stream: int) -> None:
        rc = self.lib.evt_workspace_init(ctypes.c_void_p(ptr), nbytes, ctypes.c_void_p(stream))
        if rc != 0:
            raise RuntimeError(f"HIP Error {rc} in evt_workspace_init")

    def clock_probe_read(self):
        """(main-loop cycles, main-loop 100 MHz ticks, epilogue cycles, epilogue ticks) of workgroup 0 in the
        last launch; only modules generated with clock_probe=True export it."""
        if not hasattr(self.lib, "evt_clock_probe_read"):
            raise RuntimeError(f"{self.path.name} was not built with the clock probe")
        out = (ctypes.c_uint64 * 4)()
        rc = self.lib.evt_clock_probe_read(out)
        if rc != 0:
            raise RuntimeError(f"HIP Error {rc} in evt_clock_probe_read")
        return tuple(int(x) for x in out)

    def launch(self, args: EvtArgs, ws_ptr: int, ws_bytes: int, stream: int) -> None:
        rc = self.lib.evt_launch(ctypes.byref(args), ctypes.c_void_p(ws_ptr), ws_bytes, ctypes.c_void_p(stream))
        if rc < 0:
            raise RuntimeError(f"evt_launch rejected the arguments: {ERROR_NAMES.get(rc, rc)} ({self.path.name})")
        if rc > 0:
            # same error class as the reference raises on a failed launch
            # (python/gtl/ops/reduce_apply_operation.py:157-158)
            raise RuntimeError(f"HIP Error {rc} launching {self.path.name}")


    def launch_static(self, args: EvtArgs, stream: int) -> None:
        """evt_launch_static: partial results go to the module's own device array, nothing is allocated."""
        rc = self.lib.evt_launch_static(ctypes.byref(args), ctypes.c_void_p(stream))
        if rc < 0:
            raise RuntimeError(f"evt_launch_static rejected the arguments: {ERROR_NAMES.get(rc, rc)} ({self.path.name})")
        if rc > 0:
            raise RuntimeError(f"HIP Error {rc} launching {self.path.name}")


_loaded: Dict[str, KernelModule] = {}
_lock = threading.Lock()


def _db() -> sqlite3.Connection:
    KERNEL_DIR.mkdir(parents=True, exist_ok=True)
    con = sqlite3.connect(str(CACHE_FILE), timeout=60)
    con.execute("CREATE TABLE IF NOT EXISTS compiled_modules("
                "hash TEXT PRIMARY KEY, name TEXT, file TEXT, spec TEXT)")
    return con


def _included_headers(text: str, seen: Dict[str, bytes]) -> None:
    for name in re.findall(r'#include\s+"([^"]+)"', text):
        if name in seen:
            continue
        path = next((d / name for d in (CSRC_DIR, INCLUDE_DIR) if (d / name).exists()), None)
        if path is None:
            continue
        seen[name] = path.read_bytes()
        _included_headers(seen[name].decode(), seen)


def module_hash(source: str) -> str:
    """Digest of everything the binary depends on: the generated source, the
    compiler flags and the headers it includes (transitively)."""
    h = hashlib.sha256()
    h.update(source.encode())
    h.update(" ".join(HIPCC_FLAGS).encode())
    seen: Dict[str, bytes] = {}
    _included_headers(source, seen)
    for name in sorted(seen):
        h.update(seen[name])
    return h.hexdigest()[:20]


def compile_source(source: str, out: Path, extra_flags=()) -> None:
    out.parent.mkdir(parents=True, exist_ok=True)
    src = out.with_suffix(".hip")
    src.write_text(source)
    tmp = out.with_suffix(f".tmp{os.getpid()}.so")
    cmd = [HIPCC, *HIPCC_FLAGS, *extra_flags, f"-I{CSRC_DIR}", f"-I{INCLUDE_DIR}", str(src), "-o", str(tmp)]
    logging.getLogger("evt_ae_amd.jit").info("compiling %s", src.name)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{proc.stderr[-4000:]}")
    os.replace(tmp, out)


def _record(h: str, name: str, path: Path, spec_json: str) -> None:
    try:
        con = _db()
        with con:
            con.execute("INSERT OR REPLACE INTO compiled_modules VALUES (?,?,?,?)", (h, name, path.name, spec_json))
        con.close()
    except sqlite3.Error:
        pass   # the index is informational; the file name carries the hash


class LazyModule:
    """A kernel module identified at trace time and compiled / loaded on first
    use, so that tracing a graph never needs hipcc or a GPU.  Modules built
    ahead of time (evt_ae_amd.prebuild) are found by their hash."""

    def __init__(self, ir: EpilogueIR, spec, clock_probe: bool = False):
        from .codegen import Codegen, RowCodegen, RowSpec
        self.ir, self.kernel_spec = ir, spec
        if isinstance(spec, RowSpec):
            self.name = f"evt_row_{ir.key()}_{spec.tag()}"
            cg = RowCodegen(ir, spec, self.name)
        else:
            self.name = (f"evt_{'bmm' if ir.batched else 'gemm'}_{ir.key()}_{spec.tag()}"
                         + ("_probe" if clock_probe else ""))
            cg = Codegen(ir, spec, self.name, clock_probe)
        self.source = cg.source()
        self.spec_json = json.dumps(cg.module_spec(), sort_keys=True)
        self.hash = module_hash(self.source)
        self.path = KERNEL_DIR / f"evt_{self.hash}.so"
        self._mod: Optional[KernelModule] = None

    def build(self, force: bool = False) -> Path:
        if force or not self.path.exists():
            compile_source(self.source, self.path)
            _record(self.hash, self.name, self.path, self.spec_json)
        return self.path

    def ensure(self) -> KernelModule:
        if self._mod is None:
            self.build()
            with _lock:
                mod = _loaded.get(str(self.path))
                if mod is None:
                    mod = KernelModule(self.path)
                    _loaded[str(self.path)] = mod
                self._mod = mod
        return self._mod

    @property
    def spec(self) -> dict:
        return json.loads(self.spec_json)

    def workspace_bytes(self, args: EvtArgs) -> int:
        return self.ensure().workspace_bytes(args)

    def workspace_init(self, ptr: int, nbytes: int, stream: int) -> None:
        self.ensure().workspace_init(ptr, nbytes, stream)

    def launch(self, args: EvtArgs, ws_ptr: int, ws_bytes: int, stream: int) -> None:
        self.ensure().launch(args, ws_ptr, ws_bytes, stream)

    def launch_static(self, args: EvtArgs, stream: int) -> None:
        self.ensure().launch_static(args, stream)

    def clock_probe_read(self):
        return self.ensure().clock_probe_read()


_registry: Dict[str, LazyModule] = {}


def load_module(ir: EpilogueIR, spec: KernelSpec, clock_probe: bool = False) -> LazyModule:
    mod = LazyModule(ir, spec, clock_probe)
    with _lock:
        return _registry.setdefault(str(mod.path), mod)


def registered_modules():
    with _lock:
        return list(_registry.values())


def build_module(ir: EpilogueIR, spec: KernelSpec, force: bool = False) -> Path:
    return load_module(ir, spec).build(force)
