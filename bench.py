#!/usr/bin/env python3
"""Benchmark of the fused GEMM + epilogue path on one MI355X.

One "step" launches the fused kernel of each headline subgraph the metric's
target is quoted on (configs 1-4: FFN up-projection + GELU, attention scores +
softmax statistics, output projection + residual + LayerNorm statistics, FFN
backward + bias gradient), once each, on synthetic inputs of the documented
shapes and distributions that already sit in HBM.  Throughput is the sum of
their algorithmic FLOPs over the step time.  Config 5 (classifier +
cross-entropy) is measured and reported in the same line, outside `value`.

Per config the line also carries: TFLOP/s and fraction of the MI355X dense fp16
MFMA peak, algorithmic GB/s and fraction of HBM peak, the unfused GPU sequence
(rocBLAS/hipBLASLt GEMM + one eager kernel per epilogue op) timed in the same
run, and parity against the CPU oracle.  `cpu_baseline` is PyTorch's fp32 eager
evaluation of the same subgraphs on the host cores.

Launches go through the C ABI (evt_launch) on torch's current stream; inputs
and outputs rotate over several buffer sets (> 256 MB in total per config) so
the Infinity Cache does not stand in for HBM.
"""
import argparse
import json
import operator
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

PEAK_FP16_TFLOPS = 2516.6     # MI355X dense fp16 MFMA (256 CU x 4096 flop/clk x 2.4 GHz)
PEAK_HBM_GBS = 8000.0         # MI355X HBM3E
ROTATE_BYTES = 320 << 20
VALUE_CONFIGS = (1, 2, 3, 4)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


class Case:
    """One headline subgraph prepared for timing: fused op, rotating argument
    blocks, the unfused eager callable."""

    def __init__(self, cfg, torch, W, fused_nodes):
        self.cfg = cfg
        self.wl = W.CONFIGS[cfg]
        self.torch = torch
        self.cpu_inputs = W.make_inputs(cfg)
        gm = W.fuse(self.wl.module(), [t.to("meta") for t in self.cpu_inputs])
        (node,) = fused_nodes(gm)
        self.gm, self.op = gm, node.target
        # order of the fused node's arguments in terms of module inputs
        placeholders = [n for n in gm.graph.nodes if n.op == "placeholder"]
        self.arg_index = [placeholders.index(a) for a in node.args]
        per_set = sum(t.numel() * t.element_size() for t in self.cpu_inputs)
        per_set += sum(int(torch.tensor(s).prod()) * torch.empty(0, dtype=d).element_size()
                       for s, d in self.op.store_meta.values())
        self.nsets = max(4, -(-ROTATE_BYTES // per_set))
        self.sets = []
        stream = torch.cuda.current_stream()
        for _ in range(self.nsets):
            dev_in = [t.cuda() for t in self.cpu_inputs]
            args = [dev_in[i] for i in self.arg_index]
            outs = self.op.allocate_outputs("cuda")
            a, keep = self.op.build_arguments(outs, *args, block=self.op.new_argument_block())
            ws_ptr, ws_bytes = self.op.workspace_for(a, stream, "cuda")
            self.sets.append((a, keep, outs, dev_in, ws_ptr, ws_bytes))
        self.unfused = W.unfused_eager(cfg)
        self.module = self.op.module.ensure()

    def launch(self, i):
        a, _, _, _, ws_ptr, ws_bytes = self.sets[i % self.nsets]
        self.module.launch(a, ws_ptr, ws_bytes, self.torch.cuda.current_stream().cuda_stream)

    def clock_probe(self, jit, spin_seconds=0.3):
        """Run the diagnostic build of the same kernel under sustained load and read what workgroup 0 timed:
        shader clock (cycles per 100 MHz tick) and the split between main loop and epilogue."""
        probe = jit.load_module(self.op.ir, self.op.spec, clock_probe=True).ensure()
        stream = self.torch.cuda.current_stream().cuda_stream

        def fn(i):
            a, _, _, _, ws_ptr, ws_bytes = self.sets[i % self.nsets]
            probe.launch(a, ws_ptr, ws_bytes, stream)
        spin_up(self.torch, fn, spin_seconds)
        samples = []
        for i in range(8):
            fn(i)
            self.torch.cuda.synchronize()
            samples.append(probe.clock_probe_read())
        samples.sort(key=lambda s: s[1] + s[3])
        c_main, r_main, c_epi, r_epi = samples[len(samples) // 2]
        return {"shader_mhz": round(100.0 * (c_main + c_epi) / max(r_main + r_epi, 1), 0),
                "wg0_mainloop_us": round(r_main / 100.0, 2), "wg0_epilogue_us": round(r_epi / 100.0, 2),
                "wg0_mainloop_cycles": c_main, "wg0_epilogue_cycles": c_epi}

    def launch_unfused(self, i):
        return self.unfused(*self.sets[i % self.nsets][3])

    def outputs(self, i):
        _, _, outs, _, _, _ = self.sets[i % self.nsets]
        res = []
        for o in self.op.outputs:
            name = self.op.get_output_name(o)
            t = outs[self.op.output2store[name]]
            for kind, arg in self.op.post_reshape_permute.get(name, ()):
                t = t.view(arg) if kind == "view" else t.permute(arg)
            res.append(t)
        # module output order
        out_node = [n for n in self.gm.graph.nodes if n.op == "output"][0]
        ret = out_node.args[0]
        ret = list(ret) if isinstance(ret, (tuple, list)) else [ret]
        order = []
        for r in ret:   # each is getitem(fused, idx), or a view of one
            if r.target is operator.getitem:
                order.append(res[r.args[1]])
            else:
                gi = r.args[0]
                order.append(res[gi.args[1]].view(r.args[1]))
        return order


def spin_up(torch, fn, seconds=0.15):
    """Untimed: keep the GPU busy long enough for its clocks to settle."""
    t0 = time.perf_counter()
    i = 0
    while time.perf_counter() - t0 < seconds:
        for _ in range(20):
            fn(i)
            i += 1
        torch.cuda.synchronize()


class PowerMeter:
    """Socket power of GPU 0 as the amdgpu driver reports it (hwmon `power1_input`, or `power1_average`, in
    microwatts; `power1_cap` is the limit the part regulates to), read while a launch loop keeps the GPU busy.
    Telemetry the box does not expose reads as None; nothing here changes a setting."""

    def __init__(self, torch):
        import glob
        self.torch = torch
        self.path = self.cap_w = None
        cards = sorted(glob.glob("/sys/class/drm/card*/device"))
        try:
            p = torch.cuda.get_device_properties(0)
            want = "%04x:%02x:%02x." % (getattr(p, "pci_domain_id", 0), p.pci_bus_id, p.pci_device_id)
            mine = [c for c in cards if os.path.basename(os.path.realpath(c)).startswith(want)]
        except Exception:
            mine = []
        for card in mine or (cards if len(cards) == 1 else []):
            for hw in sorted(glob.glob(card + "/hwmon/hwmon*")):
                for name in ("power1_input", "power1_average"):
                    if self._read(os.path.join(hw, name)) is not None:
                        self.path = os.path.join(hw, name)
                        cap = self._read(os.path.join(hw, "power1_cap"))
                        self.cap_w = None if cap is None else round(cap / 1e6, 1)
                        return

    @staticmethod
    def _read(path):
        try:
            with open(path) as f:
                return int(f.read().strip())
        except (OSError, ValueError):
            return None

    def under_load(self, fn, seconds=2.0, batch=40):
        """Keep `fn(i)` launches queued for `seconds` (at most two batches ahead of the GPU) and read the power
        after every batch; the report covers the readings of the second half, when the sensor's average has
        caught up with the load."""
        if self.path is None:
            return None
        torch = self.torch
        events, readings, i = [], [], 0
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < seconds:
            for _ in range(batch):
                fn(i)
                i += 1
            ev = torch.cuda.Event()
            ev.record()
            events.append(ev)
            if len(events) > 2:
                events.pop(0).synchronize()
            w = self._read(self.path)
            if w is not None:
                readings.append((time.perf_counter() - t0, w / 1e6))
        torch.cuda.synchronize()
        late = sorted(w for t, w in readings if t >= seconds / 2)
        if not late:
            return None
        return {"socket_w": round(late[len(late) // 2], 1), "socket_w_max": round(late[-1], 1), "cap_w": self.cap_w,
                "readings": len(late), "seconds": seconds, "source": os.path.basename(self.path)}


def time_loop(torch, fn, steps, warmup, repeats=1):
    """ms per call: `steps` back-to-back calls between two HIP events on the launch stream, after a clock
    spin-up and `warmup` untimed calls; the median of `repeats` such regions."""
    spin_up(torch, fn)
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    samples = []
    for _ in range(repeats):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(steps):
            fn(i)
        e1.record()
        torch.cuda.synchronize()
        samples.append(e0.elapsed_time(e1) / steps)
    samples.sort()
    return samples[len(samples) // 2]


def time_graph(torch, fn, steps, warmup, span):
    """Same work replayed from a HIP graph of `span` consecutive calls (launch
    overhead removed).  Returns ms per call or None if capture is unavailable."""
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for i in range(3):
                fn(i)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for i in range(span):
                fn(i)
        reps = max(1, steps // span)
        for _ in range(max(1, warmup // span)):
            graph.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            graph.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / (reps * span)
    except Exception as exc:   # capture not possible: report the plain loop only
        log(f"[bench] graph capture unavailable: {exc!r}")
        torch.cuda.synchronize()
        return None


def bench_row_anchors(torch, W, steps, warmup):
    """The row-wise anchors (softmax / layer norm, forward and backward) on
    HBM-sized inputs: microseconds per launch from a HIP graph of rotating
    buffer sets, algorithmic bytes per second against the 8 TB/s HBM peak, and
    the same module run eagerly."""
    out = {}
    g = torch.Generator(device="cuda").manual_seed(0x50F7)
    for name, (cls, shapes, nbytes) in W.ROW_BENCH.items():
        nsets = max(3, -(-(1 << 30) // nbytes))        # more than 1 GiB in rotation: past the 256 MB cache
        sets = []
        for _ in range(nsets):
            ins = []
            for sh, dt in shapes:
                t = torch.randn(sh, generator=g, device="cuda", dtype=torch.float32)
                ins.append(t.to(dt))
            if name == "softmax_backward":
                ins[1] = torch.softmax(ins[1].float(), -1).half()
            if name == "layernorm_backward":
                x = ins[1].float()
                ins[2] = x.mean(-1, keepdim=True)
                ins[3] = torch.rsqrt(x.var(-1, unbiased=False, keepdim=True) + 1e-5)
                del x
            sets.append(ins)
        gm = W.fuse(cls(), sets[0])
        (node,) = W.fused_nodes(gm)
        eager = cls()
        fused_out = gm(*sets[0])
        eager_out = eager(*sets[0])
        fo = list(fused_out) if isinstance(fused_out, (tuple, list)) else [fused_out]
        eo = list(eager_out) if isinstance(eager_out, (tuple, list)) else [eager_out]
        err = max(float((a.float() - b.float()).abs().max() / b.float().abs().max().clamp_min(1e-30)) for a, b in zip(fo, eo))
        if not err <= 2e-2:
            sys.exit(f"bench.py: row anchor {name} disagrees with the eager module (norm-wise error {err:.3e})")
        del fused_out, eager_out, fo, eo
        ms = time_graph(torch, lambda i: gm(*sets[i % nsets]), steps, warmup, span=nsets * 2) or \
            time_loop(torch, lambda i: gm(*sets[i % nsets]), steps, warmup)
        ms_eager = time_loop(torch, lambda i: eager(*sets[i % nsets]), max(10, steps // 4), 3)
        out[name] = {"kernel": node.target.module.name, "rows_x_cols": [shapes[0][0][0] * (shapes[0][0][1] if len(shapes[0][0]) == 3 else 1),
                                                                     shapes[0][0][-1]],
                     "us": round(ms * 1e3, 2), "alg_bytes": nbytes, "alg_GBps": round(nbytes / (ms * 1e-3) / 1e9, 1),
                     "frac_hbm_peak": round(nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                     "eager_us": round(ms_eager * 1e3, 2), "speedup_vs_eager": round(ms_eager / ms, 3),
                     "normwise_err_vs_eager": err, "buffer_sets": nsets}
        log(f"[bench] row anchor {name}: {out[name]}")
        del sets, gm
        torch.cuda.empty_cache()
    return out


def bench_encoder_step(torch, W, iters=20, only=None):
    """One training step (forward + backward) of a BERT-large encoder layer in
    fp16, through AOT autograd with every GEMM / BMM / softmax / layer norm
    fused, against the same model run eagerly; both also replayed from a HIP
    graph, which removes the host-side launch cost of either.  `only` =
    "fused" | "eager" runs just that side in a plain loop (for kernel traces)."""
    import copy
    from evt_ae_amd.aot_helper import aot_optimize
    model, (x, target) = W.encoder_layer(device="cuda", **W.ENCODER_BENCH)
    eager = copy.deepcopy(model)
    fused = aot_optimize(model)

    def run(fn, params):
        def step():
            for p in params:
                p.grad = None
            fn(x, target).backward()
        for _ in range(3):
            step()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            step()
        e1.record()
        torch.cuda.synchronize()
        loop_ms = e0.elapsed_time(e1) / iters
        graph_ms = None
        try:
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                step()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            for p in params:
                p.grad = None
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                fn(x, target).backward()
            graph.replay()
            torch.cuda.synchronize()
            e0.record()
            for _ in range(iters):
                graph.replay()
            e1.record()
            torch.cuda.synchronize()
            graph_ms = e0.elapsed_time(e1) / iters
        except Exception as exc:
            log(f"[bench] encoder step: graph capture unavailable: {exc!r}")
            torch.cuda.synchronize()
        return loop_ms, graph_ms

    if only is not None:
        fn, params = (fused, list(model.parameters())) if only == "fused" else (eager, list(eager.parameters()))
        for _ in range(3 + iters):
            for p in params:
                p.grad = None
            fn(x, target).backward()
        torch.cuda.synchronize()
        return {"model": "post-LN encoder layer", **W.ENCODER_BENCH, "dtype": "f16", "only": only, "steps": 3 + iters}
    e_loop, e_graph = run(eager, list(eager.parameters()))
    f_loop, f_graph = run(fused, list(model.parameters()))
    ref = [p.grad.float() for p in eager.parameters()]
    got = [p.grad.float() for p in model.parameters()]
    # norm-wise per parameter.  The key projection's bias has no influence on a softmax over keys: its exact
    # gradient is zero and both runs return rounding noise, so a gradient far below the others' scale is measured
    # against that scale (1e-3 of the largest per-element RMS) instead of against its own norm
    rms = max(float(b.norm()) / b.numel() ** 0.5 for b in ref)
    err = max(float((a - b).norm()) / max(float(b.norm()), 1e-3 * rms * b.numel() ** 0.5, 1e-30) for a, b in zip(got, ref))
    best_e = min(t for t in (e_loop, e_graph) if t)
    best_f = min(t for t in (f_loop, f_graph) if t)
    out = {"model": "post-LN encoder layer", **W.ENCODER_BENCH, "dtype": "f16",
           "fused_ms": round(f_loop, 4), "fused_graph_ms": None if f_graph is None else round(f_graph, 4),
           "eager_ms": round(e_loop, 4), "eager_graph_ms": None if e_graph is None else round(e_graph, 4),
           "speedup_vs_eager": round(best_e / best_f, 3), "max_grad_normwise_diff_vs_eager": err}
    log(f"[bench] encoder layer training step: {out}")
    return out


def bench_reference_keys(torch, steps=30, only=None):
    """Every GEMM / BMM problem of the reference's tuner caches (tests/golden/reference_tuner_keys.json: shape,
    operand layouts and the seven node counts of its epilogue) at its real size: a synthetic epilogue with the
    key's counts, fused (the tile the tuner cache or the model picks), against the same module run unfused by
    PyTorch and against the library's GEMM alone.  µs per call, median of 3 regions of `steps` calls each."""
    from tests import patterns as P
    from evt_ae_amd.workloads import fused_nodes
    rows = []
    for table, key, case in P.reference_key_cases():
        if only and not any(o in key for o in only):
            continue
        g = torch.Generator(device="cuda").manual_seed(1234)
        ins = []
        for i, (shape, dt) in enumerate(P.counted_epilogue_shapes(case)):
            t = torch.empty(shape, dtype=dt, device="cuda")
            flat = t.view(-1)
            for lo in range(0, flat.numel(), 1 << 28):      # in pieces: the largest operands run to gigabytes
                n = min(1 << 28, flat.numel() - lo)
                flat[lo:lo + n] = (torch.randn(n, generator=g, device="cuda") * (0.02 if i == 1 else 1.0)).to(dt)
            ins.append(t)
        mod, _ = P.counted_epilogue(case)
        gm = P.fuse(mod, [t.to("meta") for t in ins])
        (node,) = fused_nodes(gm)
        outs = gm(*ins)
        with torch.no_grad():
            refs = mod(*ins)
        torch.cuda.synchronize()
        worst = 0.0
        for o, r in zip(outs, refs):      # a spot check against the unfused fp16 result; parity proper is the tests' job
            o, r = o.float().reshape(-1), r.float().reshape(-1)
            idx = torch.randint(0, o.numel(), (1 << 18,), device="cuda")
            worst = max(worst, float((o[idx] - r[idx]).abs().max() / r[idx].abs().max().clamp_min(1e-6)))
        if worst > 5e-2:
            sys.exit(f"bench.py: reference key {key}: fused and unfused results differ ({worst:.3e})")
        a, b = ins[0], ins[1]
        swap = (1, 2) if case["batched"] else (0, 1)
        A = a if case["a_row"] else a.transpose(*swap)
        B = b if case["b_row"] else b.transpose(*swap)
        mm = torch.bmm if case["batched"] else torch.mm
        us = time_loop(torch, lambda i: gm(*ins), steps, 10, 3) * 1e3
        with torch.no_grad():
            us_eager = time_loop(torch, lambda i: mod(*ins), steps, 10, 3) * 1e3
        us_lib = time_loop(torch, lambda i: mm(A, B), steps, 10, 3) * 1e3
        rows.append({"key": key, "tile": node.target.tile.tag(), "us": round(us, 2), "unfused_us": round(us_eager, 2),
                     "library_gemm_alone_us": round(us_lib, 2)})
        log(f"[bench] {key} {rows[-1]}")
        del ins, outs, refs, gm, a, b, A, B
        torch.cuda.empty_cache()
    import math
    tot = {k: round(sum(r[k] for r in rows), 1) for k in ("us", "unfused_us", "library_gemm_alone_us")}
    return {"keys": len(rows), "total_us": tot,
            "geomean_speedup_vs_unfused": round(math.exp(sum(math.log(r["unfused_us"] / r["us"]) for r in rows) / max(len(rows), 1)), 3),
            "slower_than_unfused": [r["key"] for r in rows if r["us"] > r["unfused_us"]],
            "rows": rows}


def cpu_baseline(torch, W, evt_oracle, cfgs, reps=9):
    """PyTorch fp32 eager evaluation of the same subgraphs on the host cores."""
    torch.set_num_threads(min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))))
    flops, secs = 0, 0.0
    for cfg in cfgs:
        wl = W.CONFIGS[cfg]
        inputs = [evt_oracle.widen(t) for t in W.make_inputs(cfg)]
        mod = wl.module()
        with torch.no_grad():
            mod(*inputs)
            ts = []
            for _ in range(reps):
                t0 = time.perf_counter()
                mod(*inputs)
                ts.append(time.perf_counter() - t0)
        ts.sort()
        secs += ts[len(ts) // 2]
        flops += wl.flops
    return flops / secs / 1e12, torch.get_num_threads(), secs


class MfmaProbe:
    """Builds / loads bench_mfma_probe.hip (a register-only MFMA loop, a measurement aid that sits beside this
    script) and runs it on operand data of the caller's choice: what the matrix cores sustain on data like the
    benchmark's, next to the published peak."""

    SOURCE = ROOT / "bench_mfma_probe.hip"

    def __init__(self):
        import hashlib
        from evt_ae_amd import jit
        h = hashlib.sha256((self.SOURCE.read_text() + " ".join(jit.HIPCC_FLAGS)).encode()).hexdigest()[:20]
        self.path = ROOT / "build" / f"bench_mfma_probe_{h}.so"
        self._lib = None

    def build(self, force=False):
        import subprocess
        from evt_ae_amd import jit
        if force or not self.path.exists():
            self.path.parent.mkdir(parents=True, exist_ok=True)
            tmp = self.path.with_suffix(f".tmp{os.getpid()}.so")
            proc = subprocess.run([jit.HIPCC, *jit.HIPCC_FLAGS, str(self.SOURCE), "-o", str(tmp)],
                                  capture_output=True, text=True)
            if proc.returncode != 0:
                raise RuntimeError(f"hipcc failed for {self.SOURCE}:\n{proc.stderr[-4000:]}")
            os.replace(tmp, self.path)
        return self.path

    def run(self, torch, operands, b_operands=None, variant=0, workgroups=256, iters=1 << 15, warm_launches=6):
        """operands (and b_operands, for the B-side registers; default: the same buffer): contiguous CUDA fp16
        tensors of >= 65536 elements.  variant 0: v_mfma_f32_32x32x16_f16, 1: v_mfma_f32_16x16x32_f16.  Returns
        (TFLOP/s, shader MHz) of the last of `warm_launches` + 1 back-to-back launches."""
        import ctypes
        if self._lib is None:
            self.build()
            self._lib = ctypes.CDLL(str(self.path), mode=ctypes.RTLD_LOCAL)
            self._lib.evt_mfma_probe_launch.restype = ctypes.c_int
            self._lib.evt_mfma_probe_launch.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                                        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
        b_operands = operands if b_operands is None else b_operands
        for t in (operands, b_operands):
            if t.dtype != torch.float16 or t.numel() < 65536 or not t.is_contiguous():
                raise ValueError("operands: contiguous fp16 tensors of at least 65536 elements")
        sink = torch.zeros(1024, dtype=torch.float32, device=operands.device)
        clk = torch.zeros(2, dtype=torch.int64, device=operands.device)
        stream = torch.cuda.current_stream().cuda_stream
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for i in range(warm_launches + 1):
            if i == warm_launches:
                e0.record()
            rc = self._lib.evt_mfma_probe_launch(operands.data_ptr(), b_operands.data_ptr(), sink.data_ptr(), clk.data_ptr(),
                                                 workgroups, iters, variant, ctypes.c_void_p(stream))
            if rc != 0:
                raise RuntimeError(f"HIP Error {rc} launching the MFMA probe")
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1)
        cycles, ticks = (int(x) for x in clk.cpu())
        flops = workgroups * 8 * iters * 8 * 32768.0
        return flops / (ms * 1e-3) / 1e12, 100.0 * cycles / max(ticks, 1)

    def run_mix(self, torch, operands, b_operands, lds_reads, transfers, workgroups=256, iters=1 << 14, warm_launches=6):
        """The 32x32x16 loop with `lds_reads` ds_read_b128 and `transfers` global -> LDS transfers (1 KiB per wave
        each) between every 8 MFMAs.  Returns (TFLOP/s, shader MHz)."""
        import ctypes
        self.run(torch, operands, b_operands, iters=64, warm_launches=0)      # loads the library
        fn = self._lib.evt_mfma_probe_launch_mix
        fn.restype = ctypes.c_int
        fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                       ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
        sink = torch.zeros(1024, dtype=torch.float32, device=operands.device)
        clk = torch.zeros(2, dtype=torch.int64, device=operands.device)
        stream = torch.cuda.current_stream().cuda_stream
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for i in range(warm_launches + 1):
            if i == warm_launches:
                e0.record()
            rc = fn(operands.data_ptr(), b_operands.data_ptr(), operands.data_ptr(), sink.data_ptr(), clk.data_ptr(),
                    workgroups, iters, lds_reads, transfers, ctypes.c_void_p(stream))
            if rc != 0:
                raise RuntimeError(f"error {rc} launching the MFMA / traffic mix ({lds_reads}, {transfers})")
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1)
        cycles, ticks = (int(x) for x in clk.cpu())
        flops = workgroups * 8 * iters * 8 * 32768.0
        return flops / (ms * 1e-3) / 1e12, 100.0 * cycles / max(ticks, 1)


def main_loop_traffic(tile):
    """Per k-tile of one workgroup: (MFMAs 32x32x16, KiB read from LDS into fragments, KiB moved global -> LDS)."""
    mfmas = (tile.bm // 32) * (tile.bn // 32) * (tile.bk // 16)
    dma_kib = (tile.bm + tile.bn) * tile.bk * 2 / 1024.0
    lds_kib = tile.wm * tile.wn * (tile.bm // tile.wm + tile.bn // tile.wn) * tile.bk * 2 / 1024.0
    if tile.pipe >= 16:      # k-tiles split between the wave groups: wave tiles of twice the rows, half the depth each
        lds_kib = tile.wm * tile.wn * (2 * tile.bm // tile.wm + tile.bn // tile.wn) * (tile.bk // 2) * 2 / 1024.0
    return mfmas, lds_kib, dma_kib


# ---------------------------------------------------------------------------
# HBM-side traffic of the fused kernels, from rocprofv3 counter runs of this script
# ---------------------------------------------------------------------------
# Two counter runs of this script (`rocprofv3 --pmc FETCH_SIZE`, then `--pmc WRITE_SIZE`, both with
# --copy-calibration) leave one bench_counter_collection.csv each.  `bench.py --traffic-summary FETCH.csv WRITE.csv`
# condenses them into TRAFFIC_FILE: per fused kernel (named by its GemmCfg<...> template arguments and grid size)
# the mean KiB per dispatch of both counters, and the factor each counter needs so that the plain streaming kernel
# of --copy-calibration reads its known size.  A bench run looks the dominant kernel up there; a kernel the file
# does not hold (another tile, no counter run yet) reports "traffic": null.
TRAFFIC_FILE = ROOT / "profiles" / "evt_gemm_kernel_hbm_traffic.txt"
CALIBRATION_KIB = 64 * 4 * 1024      # the streaming kernel reads and writes 64 Mi fp32 values


def kernel_key(source_text):
    """The GemmCfg<...> instantiation a generated module launches, as rocprofv3 prints it in kernel names."""
    import re
    m = re.search(r"using Cfg = (evt::GemmCfg<[^>]*>);", source_text)
    return m.group(1) if m else None


def summarize_traffic(fetch_csv, write_csv, out_path=TRAFFIC_FILE):
    import csv
    import re
    from collections import defaultdict
    sums = {"FETCH_SIZE": defaultdict(list), "WRITE_SIZE": defaultdict(list)}
    for path in (fetch_csv, write_csv):
        with open(path, newline="") as f:
            for r in csv.DictReader(f):
                if r["Counter_Name"] not in sums:
                    continue
                name = r["Kernel_Name"]
                m = re.search(r"evt_gemm_kernel<(evt::GemmCfg<[^>]*>)", name)
                if m:
                    key = (m.group(1), int(r["Grid_Size"]))
                elif "neg_kernel_cuda" in name and int(r["Grid_Size"]) == 64 << 18:
                    key = ("calibration", 0)
                else:
                    continue
                sums[r["Counter_Name"]][key].append(float(r["Counter_Value"]))
    mean = {c: {k: sum(v) / len(v) for k, v in d.items()} for c, d in sums.items()}
    cal = ("calibration", 0)
    if cal not in mean["FETCH_SIZE"] or cal not in mean["WRITE_SIZE"]:
        sys.exit("bench.py: the counter files hold no dispatch of the --copy-calibration kernel")
    lines = ["# written by `bench.py --traffic-summary`; KiB per dispatch, mean over the run's dispatches",
             f"calibration known_kib={CALIBRATION_KIB} fetch_kib={mean['FETCH_SIZE'][cal]:.1f} "
             f"write_kib={mean['WRITE_SIZE'][cal]:.1f} fetch_scale={CALIBRATION_KIB / mean['FETCH_SIZE'][cal]:.4f} "
             f"write_scale={CALIBRATION_KIB / mean['WRITE_SIZE'][cal]:.4f}"]
    for key in sorted(k for k in mean["FETCH_SIZE"] if k != cal and k in mean["WRITE_SIZE"]):
        lines.append(f"kernel {key[0].replace(' ', '')} grid={key[1]} dispatches={len(sums['FETCH_SIZE'][key])} "
                     f"fetch_kib={mean['FETCH_SIZE'][key]:.1f} write_kib={mean['WRITE_SIZE'][key]:.1f}")
    Path(out_path).write_text("\n".join(lines) + "\n")
    return lines


def _short_kernel_name(name):
    import re
    m = re.search(r"evt_gemm_kernel<evt::GemmCfg<([^>]*)>", name)
    if m:
        return "evt_gemm_kernel<" + m.group(1).replace(" ", "") + ">"
    m = re.search(r"evt_row_kernel<evt::RowCfg<([^>]*)>.*?, (\d)>", name)
    if m:
        return "evt_row_kernel<" + m.group(1).replace(" ", "") + ";fast=" + m.group(2) + ">"
    m = re.search(r"(evt_\w+_kernel)", name)
    if m:
        return m.group(1)
    if "neg_kernel" in name:
        return "at::native neg kernel (calibration: 256 MiB in, 256 MiB out)"
    return name[:76]


def summarize_profiles(root):
    """Text summary of the rocprofv3 output folders under `root`: for every sub-folder that holds a
    *_kernel_stats.csv (a --kernel-trace --stats run) the calls and average / minimum / maximum duration of each
    kernel, and for every one that holds a *_counter_collection.csv (a --pmc run) the mean of each counter per
    dispatch of each kernel of this package (and of the calibration kernel).  No GPU work."""
    import csv
    from collections import defaultdict
    out = [f"# written by `bench.py --profile-summary {root}` from the rocprofv3 CSV files under that folder"]
    for sub in sorted(p for p in Path(root).iterdir() if p.is_dir()):
        for stats in sorted(sub.rglob("*_kernel_stats.csv")):
            out += ["", f"[{sub.name}] kernel trace ({stats.relative_to(root)}): calls, average / minimum / maximum duration in us, share of the run's kernel time",
                    f"{'kernel':<92} {'calls':>6} {'avg':>9} {'min':>9} {'max':>9} {'%':>6}"]
            with open(stats, newline="") as f:
                rows = list(csv.DictReader(f))
            for r in rows:
                short = _short_kernel_name(r["Name"])
                if float(r["Percentage"]) < 0.3 and not short.startswith("evt_"):
                    continue
                out.append(f"{short:<92} {r['Calls']:>6} {float(r['AverageNs']) / 1e3:9.2f} {float(r['MinNs']) / 1e3:9.2f} "
                           f"{float(r['MaxNs']) / 1e3:9.2f} {float(r['Percentage']):6.2f}")
        for cc in sorted(sub.rglob("*_counter_collection.csv")):
            vals = defaultdict(list)
            with open(cc, newline="") as f:
                for r in csv.DictReader(f):
                    short = _short_kernel_name(r["Kernel_Name"])
                    if short.startswith("evt_") or short.startswith("at::native neg"):
                        vals[(short, int(r["Grid_Size"]), r["Counter_Name"])].append(float(r["Counter_Value"]))
            out += ["", f"[{sub.name}] counters ({cc.relative_to(root)}): mean per dispatch",
                    f"{'kernel':<92} {'grid':>9} {'counter':<30} {'n':>6} {'mean':>14}"]
            for (short, grid, counter), v in sorted(vals.items()):
                out.append(f"{short:<92} {grid:>9} {counter:<30} {len(v):>6} {sum(v) / len(v):14.6g}")
    return out


def measured_traffic_bytes(key, path=TRAFFIC_FILE):
    """HBM-side bytes per launch of the kernel `key`, scaled by the calibration; None when the file does not hold
    the kernel, or holds it at several grid sizes (then the entry cannot be told apart from here)."""
    if key is None or not Path(path).exists():
        return None
    scale, found = None, []
    for ln in Path(path).read_text().splitlines():
        if ln.startswith("#"):
            continue
        f = dict(kv.split("=", 1) for kv in ln.split()[1:] if "=" in kv)
        if ln.startswith("calibration"):
            scale = (float(f["fetch_scale"]), float(f["write_scale"]))
        elif ln.startswith("kernel") and ln.split()[1] == key.replace(" ", ""):
            found.append((float(f["fetch_kib"]), float(f["write_kib"])))
    if scale is None or len(found) != 1:
        return None
    return int((scale[0] * found[0][0] + scale[1] * found[0][1]) * 1024)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--repeats", type=int, default=5,
                    help="timed regions of --steps launches per config; the median is reported")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-check", action="store_true")
    ap.add_argument("--only-encoder-step", choices=("fused", "eager"), default=None,
                    help="run nothing but the encoder layer's training step, that side only, in a plain loop, and print "
                         "a short JSON line (for rocprofv3 kernel traces of the step)")
    ap.add_argument("--no-encoder-step", dest="encoder_step", action="store_false",
                    help="skip the fused-vs-eager training step of an encoder layer (encoder_layer_step in the output)")
    ap.add_argument("--no-row-anchors", dest="row_anchors", action="store_false",
                    help="skip the bandwidth measurement of the softmax / layer norm anchors (row_anchors in the output)")
    ap.add_argument("--configs", default="1,2,3,4,5")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 256 MiB streaming kernel (torch.neg, known traffic) so HBM counters can be scaled")
    ap.add_argument("--no-clock-probe", dest="clock_probe", action="store_false",
                    help="skip the diagnostic build of each kernel that reports the shader clock it ran at and "
                         "workgroup 0's main-loop / epilogue split (per_config[*].clock_probe, roofline.shader_mhz)")
    ap.add_argument("--reference-keys", nargs="*", metavar="SUBSTRING", default=None,
                    help="run nothing but the GEMM / BMM problems of the reference's tuner caches (all of them, or "
                         "those whose key contains one of the substrings) at their real sizes: fused, unfused and the "
                         "library's GEMM alone; prints one JSON line")
    ap.add_argument("--no-power", dest="power", action="store_false",
                    help="skip the socket-power readings taken while each config and the MFMA probe run for two seconds "
                         "(per_config[*].power, roofline.mfma_only.power)")
    ap.add_argument("--traffic-summary", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"), default=None,
                    help="no GPU work: condense the counter files of two rocprofv3 --pmc runs of this script "
                         f"(FETCH_SIZE, WRITE_SIZE) into {TRAFFIC_FILE.relative_to(ROOT)} and exit")
    ap.add_argument("--profile-summary", metavar="DIR", default=None,
                    help="no GPU work: print a text summary of the rocprofv3 output folders under DIR (kernel statistics "
                         "and per-dispatch counter means) and exit")
    args = ap.parse_args()
    if args.profile_summary:
        print("\n".join(summarize_profiles(args.profile_summary)))
        return
    if args.traffic_summary:
        print("\n".join(summarize_traffic(*args.traffic_summary)))
        return
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU (the fused GEMM+epilogue path has no cross-GPU exchange); "
                 "run with --gpus 1")

    import torch
    from evt_ae_amd import jit, workloads as W
    from oracle import evt_oracle
    fused_nodes = W.fused_nodes

    if not torch.cuda.is_available():
        sys.exit("bench.py: no HIP device available")
    torch.cuda.set_device(0)
    if args.only_encoder_step:
        print(json.dumps({"encoder_layer_step": bench_encoder_step(torch, W, only=args.only_encoder_step)}), flush=True)
        return
    if args.reference_keys is not None:
        print(json.dumps({"reference_keys": bench_reference_keys(torch, only=args.reference_keys or None)}), flush=True)
        return
    cfgs = [int(c) for c in args.configs.split(",")]
    meter = PowerMeter(torch) if args.power else None
    details = {}
    operand_chunks, tiles = {}, {}
    for cfg in cfgs:
        case = Case(cfg, torch, W, fused_nodes)
        wl = case.wl
        # parity first: a number from a kernel that computes something else is void
        parity = normwise = None
        if not args.no_check:
            case.launch(0)
            torch.cuda.synchronize()
            refs = evt_oracle.eval_fp32(wl.module(), case.cpu_inputs)
            errs = []
            for i, (o, r) in enumerate(zip(case.outputs(0), refs)):
                ok, err = evt_oracle.check(o, r, reduction=i in wl.reduction_outputs)
                errs.append(err)
                if not ok:
                    sys.exit(f"bench.py: config {cfg} output {i} fails parity (max rel err {err:.3e})")
            parity = max(errs)
            normwise = max(float((o.detach().cpu().float() - r).abs().max() / r.abs().max().clamp_min(1e-30))
                           for o, r in zip(case.outputs(0), refs))
        ms = time_loop(torch, case.launch, args.steps, args.warmup, args.repeats)
        ms_graph = time_graph(torch, case.launch, args.steps, args.warmup, span=case.nsets * 4)
        ms_unf = time_loop(torch, case.launch_unfused, max(20, args.steps // 4), max(5, args.warmup // 4))
        ms_unf_graph = time_graph(torch, case.launch_unfused, max(20, args.steps // 4), 5, span=case.nsets)
        best = min(x for x in (ms, ms_graph) if x)
        best_unf = min(x for x in (ms_unf, ms_unf_graph) if x)
        ms_unf_lib = None
        if cfg == 1:   # the library-fused form of the same graph: bias folded into the GEMM (addmm), then GELU
            gelu = torch.nn.functional.gelu
            ms_unf_lib = time_loop(torch, lambda i: gelu(torch.addmm(case.sets[i % case.nsets][3][2],
                                                                     case.sets[i % case.nsets][3][0],
                                                                     case.sets[i % case.nsets][3][1]), approximate="tanh"),
                                   max(20, args.steps // 4), 5)
        if ms_unf_lib is not None:
            best_unf = min(best_unf, ms_unf_lib)   # the speed-up is quoted against the fastest unfused form
        details[cfg] = {
            "workload": wl.name, "dims_MNKL": list(wl.dims), "tile": case.op.tile.tag(),
            "us": round(ms * 1e3, 2), "us_graph": None if ms_graph is None else round(ms_graph * 1e3, 2),
            "tflops": round(wl.flops / (best * 1e-3) / 1e12, 1),
            "frac_mfma_peak": round(wl.flops / (best * 1e-3) / 1e12 / PEAK_FP16_TFLOPS, 4),
            "alg_GBps": round(wl.bytes / (best * 1e-3) / 1e9, 1),
            "frac_hbm_peak": round(wl.bytes / (best * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
            "unfused_us": round(ms_unf * 1e3, 2),
            "unfused_us_graph": None if ms_unf_graph is None else round(ms_unf_graph * 1e3, 2),
            "speedup_vs_unfused": round(best_unf / best, 3),
            "max_rel_err": parity, "normwise_err": normwise, "buffer_sets": case.nsets, "_ms": ms, "_best": best,
            "_key": kernel_key(case.op.module.source),
        }
        if ms_unf_lib is not None:
            details[cfg]["unfused_addmm_gelu_us"] = round(ms_unf_lib * 1e3, 2)
        if args.clock_probe:
            details[cfg]["clock_probe"] = case.clock_probe(jit)
        if meter is not None:
            details[cfg]["power"] = meter.under_load(case.launch)
        log(f"[bench] config {cfg} {wl.name}: {details[cfg]}")
        # 64 Ki elements of each anchor operand, for the register-only MFMA loop below
        operand_chunks[cfg] = tuple(t.reshape(-1)[:1 << 16].clone() for t in case.sets[0][1][:2])
        tiles[cfg] = case.op.tile
        del case
        torch.cuda.empty_cache()

    if args.copy_calibration:
        src = torch.empty(64 << 20, dtype=torch.float32, device="cuda").normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.neg(src, out=dst)   # a plain streaming kernel of known traffic: reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst
    vcfgs = [c for c in VALUE_CONFIGS if c in details]
    flops = sum(W.CONFIGS[c].flops for c in vcfgs)
    step_ms = sum(details[c]["_ms"] for c in vcfgs)
    # the dominant kernel of a step: the one with the longest launch
    dom = max(vcfgs, key=lambda c: details[c]["_ms"])
    dom_tflops = W.CONFIGS[dom].flops / (details[dom]["_ms"] * 1e-3) / 1e12
    cpu = None
    if not args.no_cpu_baseline:
        cpu_reps = 9
        v, cores, secs = cpu_baseline(torch, W, evt_oracle, vcfgs, cpu_reps)
        cpu_model = next((ln.split(":", 1)[1].strip() for ln in open("/proc/cpuinfo") if ln.startswith("model name")), "")
        cpu = {"value": round(v, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port", "cpu": cpu_model,
               "sample": f"configs {vcfgs} at full size, PyTorch fp32 eager on CPU, median of {cpu_reps} after 1 warm-up "
                         f"({secs:.2f} s per pass)"}
    # the published peak assumes 2.4 GHz; under this load the part clocks lower, so also relate the kernel to the
    # MFMA rate at the clock it was measured to run at
    clock = {}
    if "clock_probe" in details[dom]:
        mhz = details[dom]["clock_probe"]["shader_mhz"]
        clock = {"shader_mhz": mhz, "peak_at_shader_mhz": round(PEAK_FP16_TFLOPS * mhz / 2400.0, 1),
                 "frac_at_shader_mhz": round(dom_tflops / (PEAK_FP16_TFLOPS * mhz / 2400.0), 4)}
    # what the matrix cores alone sustain (register-only MFMA loop, no memory traffic) on operands distributed
    # like the benchmark's, and on zeros: the first is the practical MFMA ceiling for this data on this part
    mfma_only = None
    if args.clock_probe:
        probe = MfmaProbe()
        g = torch.Generator(device="cpu").manual_seed(0xE7A0)
        rnd = torch.randn(1 << 16, generator=g).half().cuda()
        t_rnd, mhz_rnd = probe.run(torch, rnd)
        t_zero, mhz_zero = probe.run(torch, torch.zeros_like(rnd))
        mfma_only = {"normal_operands_tflops": round(t_rnd, 1), "normal_operands_shader_mhz": round(mhz_rnd),
                     "zero_operands_tflops": round(t_zero, 1), "zero_operands_shader_mhz": round(mhz_zero)}
        if meter is not None:
            # the same loop held for two seconds: what the socket draws with the matrix cores busy on random data,
            # where the clock falls, and on zeros, where it does not
            zeros = torch.zeros_like(rnd)
            mfma_only["power"] = {
                "normal_operands": meter.under_load(lambda i: probe.run(torch, rnd, warm_launches=0), batch=4),
                "zero_operands": meter.under_load(lambda i: probe.run(torch, zeros, warm_launches=0), batch=4)}
        # the same loop on chunks of each config's own operands (A-side registers from its left operand, B-side
        # from its right one: activations ~ N(0, 1) against weights ~ N(0, 0.02)), with the 32x32x16 instruction of
        # the fused kernels and with 16x16x32
        own = {}
        for cfg in sorted(operand_chunks):
            a_chunk, b_chunk = operand_chunks[cfg]
            t32, mhz32 = probe.run(torch, a_chunk, b_chunk, variant=0)
            t16, mhz16 = probe.run(torch, a_chunk, b_chunk, variant=1)
            own[str(cfg)] = {"mfma_32x32x16_tflops": round(t32, 1), "mfma_32x32x16_shader_mhz": round(mhz32),
                             "mfma_16x16x32_tflops": round(t16, 1), "mfma_16x16x32_shader_mhz": round(mhz16)}
            if "clock_probe" in details[cfg]:
                details[cfg]["frac_of_mfma_only_own_operands"] = round(details[cfg]["tflops"] / t32, 4)
        mfma_only["own_operands"] = own
        # What the traffic of a main loop costs next to its MFMAs on this data: the loop with LDS reads and global ->
        # LDS transfers mixed in, on the dominant config's operands; the cost of a KiB of either kind, in units of one
        # MFMA, follows from the rates (the part is power-bound on this data: rate ~ 1 / energy per MFMA).  With them,
        # every config's main loop gets a predicted rate from its tile's traffic, beside the rate it reached.
        a_chunk, b_chunk = operand_chunks[dom]
        mix = {}
        for r_, d_ in ((0, 0), (6, 0), (8, 0), (0, 2), (0, 3), (6, 3)):
            t_, mhz_ = probe.run_mix(torch, a_chunk, b_chunk, r_, d_)
            mix[f"{r_}_reads_{d_}_transfers_per_8_mfma"] = {"tflops": round(t_, 1), "shader_mhz": round(mhz_)}
        base = mix["0_reads_0_transfers_per_8_mfma"]["tflops"]
        e_lds = ((base / mix["8_reads_0_transfers_per_8_mfma"]["tflops"] - 1.0) / 1.0 +
                 (base / mix["6_reads_0_transfers_per_8_mfma"]["tflops"] - 1.0) / 0.75) / 2.0
        e_dma = ((base / mix["0_reads_3_transfers_per_8_mfma"]["tflops"] - 1.0) / 0.375 +
                 (base / mix["0_reads_2_transfers_per_8_mfma"]["tflops"] - 1.0) / 0.25) / 2.0
        both = base / (1.0 + 0.75 * e_lds + 0.375 * e_dma)
        mfma_only["traffic_mix"] = {"rates": mix, "mfma_energies_per_kib_lds_read": round(e_lds, 3),
                                    "mfma_energies_per_kib_global_to_lds": round(e_dma, 3),
                                    "check_6_reads_3_transfers": {"predicted_tflops": round(both, 1),
                                                                  "measured_tflops": mix["6_reads_3_transfers_per_8_mfma"]["tflops"]}}
        for cfg in sorted(operand_chunks):
            if "clock_probe" not in details[cfg]:
                continue
            mfmas, lds_kib, dma_kib = main_loop_traffic(tiles[cfg])
            ceiling = own[str(cfg)]["mfma_32x32x16_tflops"]
            predicted = ceiling / (1.0 + e_lds * lds_kib / mfmas + e_dma * dma_kib / mfmas)
            reached = W.CONFIGS[cfg].flops / (details[cfg]["clock_probe"]["wg0_mainloop_us"] * 1e-6) / 1e12
            details[cfg]["main_loop_model"] = {
                "mfmas_per_k_tile": mfmas, "lds_read_kib_per_k_tile": round(lds_kib, 1), "global_to_lds_kib_per_k_tile": round(dma_kib, 1),
                "mfma_only_tflops_own_operands": ceiling, "predicted_main_loop_tflops": round(predicted, 1),
                "reached_main_loop_tflops": round(reached, 1), "reached_over_predicted": round(reached / predicted, 3)}
        clock["frac_of_mfma_only_normal_operands"] = round(dom_tflops / t_rnd, 4)
        clock["frac_of_mfma_only_own_operands"] = round(dom_tflops / own[str(dom)]["mfma_32x32x16_tflops"], 4)
        log(f"[bench] register-only MFMA loop: {mfma_only}")
    traffic = measured_traffic_bytes(details[dom]["_key"])
    for d in details.values():
        d.pop("_ms"); d.pop("_best"); d.pop("_key")
    line = {
        "metric": "fused GEMM+epilogue TFLOP/s, % MI355X fp16 MFMA peak, speedup vs unfused",
        "value": round(flops / (step_ms * 1e-3) / 1e12, 2), "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "repeats": args.repeats, "ms_per_step": round(step_ms, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "one fused launch each of configs " + ",".join(map(str, vcfgs)) +
                               " (ffn_up_gelu 4096x4096x1024, attn_score_softmax_stats 64x512x512x64, "
                               "out_proj_residual_ln_stats 8192x1024x4096, ffn_backward_dbias 8192x1024x4096)",
                   "frac_mfma_peak": round(flops / (step_ms * 1e-3) / 1e12 / PEAK_FP16_TFLOPS, 4)},
        "roofline": {"bound": "mfma", "achieved": round(dom_tflops, 1), "peak": PEAK_FP16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(dom_tflops / PEAK_FP16_TFLOPS, 4),
                     "traffic": traffic,
                     "kernel": f"config {dom} ({details[dom]['workload']}, tile {details[dom]['tile']})",
                     "us": details[dom]["us"], **clock, "mfma_only": mfma_only},
        "cpu_baseline": cpu,
        "per_config": details,
        "row_anchors": bench_row_anchors(torch, W, max(20, args.steps // 4), 5) if args.row_anchors else None,
        "encoder_layer_step": bench_encoder_step(torch, W) if args.encoder_step else None,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
