#!/usr/bin/env python3
"""Benchmark of the weight-quantised MatMul hot path on one MI355X.

A step is one fused dequant-MatMul call (bias + SiLU epilogue) over one batch of synthetic
activations, with every operand already resident in HBM.  The default workload is the
I4 GEMM of BASELINE.json's configs[1] (K=4096, N=11008) at M=1 (bandwidth-bound GEMV);
`--m 256` selects the matrix-core regime of the same configuration.  Consecutive steps
walk over a ring of distinct weight copies larger than the 256 MB Infinity Cache, so the
reported GB/s is HBM traffic, not cache replay (`--ring 1` gives the warm number).

`--steps` is a minimum: the timed region is whole trips round the ring, never fewer than 20; the headline figure is
over the whole region, the median and minimum are over the trips.  The same line also carries the GEMV at
K = N = 4096 (I8 and I4 weights) and the M = 256 GEMM for I4, I8 and FP8 weights (`gemv_4096`, `gemm_m256`).

Prints ONE JSON line (metric/value/... plus `roofline` and `cpu_baseline`).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = {"f16": 2500.0, "bf16": 2500.0, "i8": 5000.0, "fp8": 5000.0}

WORKLOADS = {
    # name: (dtype name, K, N, bias, act)
    "c1_i8": ("i8", 4096, 4096, False, "none"),
    "c2_i4": ("i4", 4096, 11008, True, "silu"),
    "c3_i4cb": ("i4cb", 4096, 4096, False, "none"),
    "c4_f8_up": ("f8", 2048, 8192, False, "gelu"),
    "c4_f4_up": ("f4", 2048, 8192, False, "gelu"),
    "c4_f8_down": ("f8", 8192, 2048, False, "none"),
    "c4_f4_down": ("f4", 8192, 2048, False, "none"),
    "i4_4096": ("i4", 4096, 4096, False, "none"),
    "f8_4096": ("f8", 4096, 4096, False, "none"),
}


def parsed_options(args, flib):
    """--opt NAME=VALUE items as (name, OPT_* identifier, value)."""
    out = []
    for item in args.opt:
        name, _, value = item.partition("=")
        ident = getattr(flib, "OPT_" + name.strip().upper(), None)
        if ident is None or not value.strip().lstrip("-").isdigit():
            raise ValueError(f"unknown option {item!r}")
        out.append((name.strip().lower(), ident, int(value)))
    return out


# composite configurations: (kind, parameter)
COMPOSITE = {
    "c4_mlp_f8": ("mlp", "f8"), "c4_mlp_f4": ("mlp", "f4"),
    "c5_yolo_b1": ("yolo", 1), "c5_yolo_b16": ("yolo", 16),
    "c5_yolo_graph_b1": ("yolo_graph", 1), "c5_yolo_graph_b16": ("yolo_graph", 16),
}

# YOLOv8n-shaped conv list (width 0.25, depth 0.33, 640x640 input, Detect head excluded): (C_in, H_in, C_out, k, stride);
# every conv is followed by bias + SiLU.  C2f(c1,c2,n) = cv1 1x1 c1->c2, n bottlenecks of two 3x3 c2/2->c2/2, cv2 1x1 (2+n)c2/2->c2.
def yolo_convs():
    L = []
    def conv(c, h, oc, k, s): L.append((c, h, oc, k, s))
    def c2f(c1, c2, n, h):
        conv(c1, h, c2, 1, 1)
        for _ in range(2 * n): conv(c2 // 2, h, c2 // 2, 3, 1)
        conv((2 + n) * c2 // 2, h, c2, 1, 1)
    conv(3, 640, 16, 3, 2); conv(16, 320, 32, 3, 2); c2f(32, 32, 1, 160)
    conv(32, 160, 64, 3, 2); c2f(64, 64, 2, 80)
    conv(64, 80, 128, 3, 2); c2f(128, 128, 2, 40)
    conv(128, 40, 256, 3, 2); c2f(256, 256, 1, 20)
    conv(256, 20, 128, 1, 1); conv(512, 20, 256, 1, 1)            # SPPF cv1, cv2
    c2f(384, 128, 1, 40); c2f(192, 64, 1, 80)
    conv(64, 80, 64, 3, 2); c2f(192, 128, 1, 40)
    conv(128, 40, 128, 3, 2); c2f(384, 256, 1, 20)
    return L


def yolo_graph(batch, rng, size=640):
    """The same network as a graph in the reference's node-dict form (backbone layers 0-9, neck layers 10-21, Detect
    head excluded): Conv + SiLU, C2f with channel Split / residual Add / Concat, SPPF max-pool pyramid, nearest
    2x Resize.  Returns (nodes, params, input shape, output names)."""
    nodes, params = [], {}
    cnt = [0]

    def uid(p):
        cnt[0] += 1
        return f"{p}{cnt[0]}"

    def conv(x, c, oc, k, s):
        w, b, y0, y = uid("w"), uid("b"), uid("c"), uid("s")
        kk = c * k * k
        params[w] = (rng.standard_normal((oc, c, k, k)) * np.sqrt(2.0 / kk)).astype(np.float32)
        params[b] = (rng.standard_normal(oc) * 0.05).astype(np.float32)
        nodes.append({"name": y0, "op_type": "Conv", "inputs": f"[{x}, {w}, {b}]", "outputs": f"[{y0}]", "strides": str(s),
                      "pads": str(k // 2), "group": "1"})
        nodes.append({"name": y, "op_type": "Silu", "inputs": f"[{y0}]", "outputs": f"[{y}]"})
        return y

    def c2f(x, c1, c2, n, shortcut):
        y = conv(x, c1, c2, 1, 1)
        a, b = uid("h"), uid("h")
        nodes.append({"name": a, "op_type": "Split", "inputs": f"[{y}]", "outputs": f"[{a}, {b}]", "axis": "1"})
        parts, last = [a, b], b
        for _ in range(n):
            t = conv(conv(last, c2 // 2, c2 // 2, 3, 1), c2 // 2, c2 // 2, 3, 1)
            if shortcut:
                r = uid("r")
                nodes.append({"name": r, "op_type": "Add", "inputs": f"[{last}, {t}]", "outputs": f"[{r}]"})
                t = r
            parts.append(t)
            last = t
        cat = uid("k")
        nodes.append({"name": cat, "op_type": "Concat", "inputs": "[" + ", ".join(parts) + "]", "outputs": f"[{cat}]", "axis": "1"})
        return conv(cat, (2 + n) * c2 // 2, c2, 1, 1)

    def concat(xs):
        cat = uid("k")
        nodes.append({"name": cat, "op_type": "Concat", "inputs": "[" + ", ".join(xs) + "]", "outputs": f"[{cat}]", "axis": "1"})
        return cat

    def up(x):
        u = uid("u")
        nodes.append({"name": u, "op_type": "Resize", "inputs": f"[{x}]", "outputs": f"[{u}]", "mode": "nearest", "scale_h": "2", "scale_w": "2"})
        return u

    x = conv("x", 3, 16, 3, 2)
    x = conv(x, 16, 32, 3, 2)
    x = c2f(x, 32, 32, 1, True)
    x = conv(x, 32, 64, 3, 2)
    p3 = c2f(x, 64, 64, 2, True)
    x = conv(p3, 64, 128, 3, 2)
    p4 = c2f(x, 128, 128, 2, True)
    x = conv(p4, 128, 256, 3, 2)
    x = c2f(x, 256, 256, 1, True)
    s = conv(x, 256, 128, 1, 1)                                   # SPPF
    pools = [s]
    for _ in range(3):
        m = uid("m")
        nodes.append({"name": m, "op_type": "MaxPool", "inputs": f"[{pools[-1]}]", "outputs": f"[{m}]", "kernel_shape": "5", "strides": "1", "pads": "2"})
        pools.append(m)
    p5 = conv(concat(pools), 512, 256, 1, 1)
    n4 = c2f(concat([up(p5), p4]), 384, 128, 1, False)
    n3 = c2f(concat([up(n4), p3]), 192, 64, 1, False)
    n4b = c2f(concat([conv(n3, 64, 64, 3, 2), n4]), 192, 128, 1, False)
    n5 = c2f(concat([conv(n4b, 128, 128, 3, 2), p5]), 384, 256, 1, False)
    return nodes, params, [batch, 3, size, size], [n3, n4b, n5]


def composite_result(args) -> dict:
    """C4 (FP8 / FP4 MLP stack, 64 tokens) through the plan dispatcher, or C5 (YOLOv8n-shaped I8 conv list / graph)
    through the conv entry point / AotExecutor.  One step = one forward pass over resident inputs."""
    import fastnn_amd
    from fastnn_amd import lib as flib
    kind, par = COMPOSITE[args.workload]
    rng = np.random.default_rng(0)
    steps, warm = min(args.steps, 50), min(args.warmup, 5)
    if kind == "mlp":
        from fastnn_amd.backend import ExecutablePlan, HipBackend, KERNEL_OF, meta_of
        dt = flib.DT_F8 if par == "f8" else flib.DT_F4
        m, d, f, layers = 64, 2048, 8192, 4
        top = [0]
        def take(nb):
            o = top[0]; top[0] += (nb + 63) // 64 * 64; return (o, nb)
        s_x = [take(m * d * 4) for _ in range(layers + 1)]
        s_h, s_y = take(m * f * 4), take(m * d * 4)
        consts = []
        for _ in range(layers):
            w1 = fastnn_amd.quantize_weights(dt, (rng.standard_normal((f, d)) / np.sqrt(d)).astype(np.float32))
            w2 = fastnn_amd.quantize_weights(dt, (rng.standard_normal((d, f)) / np.sqrt(f)).astype(np.float32))
            consts.append((w1, take(w1.words.nbytes), w2, take(w2.words.nbytes)))
        plan = ExecutablePlan(top[0])
        for w1, s1, w2, s2 in consts:
            plan.write_const(s1[0], w1.words).write_const(s2[0], w2.words)
        for i, (w1, s1, w2, s2) in enumerate(consts):
            plan.call_kernel(KERNEL_OF[dt] + "_gelu", [s_x[i], s1], s_h, [m, d, f], meta_of(w1))
            plan.call_kernel(KERNEL_OF[dt], [s_h, s2], s_y, [m, f, d], meta_of(w2))
            plan.call_kernel("add_f32", [s_y, s_x[i]], s_x[i + 1], [m * d])
        be = HipBackend(0)
        for _, ident, value in parsed_options(args, flib):
            be.set_option(ident, value)
        be.allocate_arena(top[0])
        be.write_arena(s_x[0][0], rng.standard_normal((m, d)).astype(np.float32))
        for _ in range(1 + warm):
            be.dispatch(plan)
        t0 = time.perf_counter()
        for _ in range(steps):
            be.dispatch(plan)
        ms = (time.perf_counter() - t0) * 1e3 / steps
        y = be.read_arena(*s_x[layers], np.float32)
        # the same plan with activations rounded to f16 once (stated tolerance 1e-3 instead of 2e-5)
        be.set_kernel_flags(flib.FLAG_ACT_F16_SINGLE)
        for _ in range(2 + warm):
            be.dispatch(plan)
        t0 = time.perf_counter()
        for _ in range(steps):
            be.dispatch(plan)
        ms1 = (time.perf_counter() - t0) * 1e3 / steps
        y1 = be.read_arena(*s_x[layers], np.float32)
        be.set_kernel_flags(0)
        flops = 2.0 * m * d * f * 2 * layers
        wbytes = sum(w1.packed_bytes() + w2.packed_bytes() for w1, _, w2, _ in consts)
        out = {"metric": f"C4 MLP stack forward ({par}, 4x[2048->8192 GELU, 8192->2048 + residual], 64 tokens)",
               "value": round(flops / (ms * 1e-3) / 1e12, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": steps, "warmup": warm,
               "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
               "data": "synthetic", "config": {"workload": args.workload, "launch": "plan dispatch (12 instructions, HIP-graph replay) + sync per step",
                          "residual_adds_inside_the_matmul": plan.residuals_fused, "options": {n: v for n, _, v in parsed_options(args, flib)}},
               "weight_gb_per_s": round(wbytes / (ms * 1e-3) / 1e9, 1), "packed_weight_bytes": wbytes,
               "finite_output": bool(np.isfinite(y).all()),
               "f16x1": {"ms_per_step": round(ms1, 4), "tflop_per_s": round(flops / (ms1 * 1e-3) / 1e12, 2),
                         "max_rel_vs_default": float(np.abs(y1 - y).max() / (np.abs(y).max() + 1e-30))}}
        be.close()
        return out
    if kind == "yolo_graph":
        from fastnn_amd.aot import AotExecutor
        batch = par
        nodes, params, shape, outs = yolo_graph(batch, rng)
        t0 = time.perf_counter()
        ex = AotExecutor(nodes, params, ["x"], outs, {"x": shape}, quantize=8)
        build_s = time.perf_counter() - t0
        for _, ident, value in parsed_options(args, flib):
            ex.set_option(ident, value)
        if args.mode == "eager":   # instruction by instruction instead of one HIP-graph replay (kernel traces)
            ex.set_graph_replay(False)
        ex.write_inputs({"x": rng.uniform(0, 1, shape).astype(np.float32)})
        for _ in range(2 + warm):
            ex.dispatch()
        t0 = time.perf_counter()
        for _ in range(steps):
            ex.dispatch()
        ms = (time.perf_counter() - t0) * 1e3 / steps
        flops = sum(2.0 * batch * ((h + 2 * (k // 2) - k) // s + 1) ** 2 * c * k * k * oc for (c, h, oc, k, s) in yolo_convs())
        y = [ex.read_output(o) for o in outs]
        kinds = {}
        for ins in ex.instructions:
            kinds[ins[0]] = kinds.get(ins[0], 0) + 1
        out = {"metric": f"C5 YOLOv8n-shaped I8 graph forward (backbone + neck as one plan, B={batch})",
               "value": round(batch / (ms * 1e-3), 1), "unit": "images/s", "n_gpus": 1, "steps": steps, "warmup": warm,
               "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "i8/i32",
               "data": "synthetic", "config": {"workload": args.workload, "launch": "AotExecutor plan, " + ("HIP-graph replay" if args.mode == "graph" else "instruction by instruction") + " + sync per step",
                                               "instructions": kinds, "arena_bytes": ex.arena_size,
                                               "options": {n: v for n, _, v in parsed_options(args, flib)}},
               "tops": round(flops / (ms * 1e-3) / 1e12, 2), "replayed": ex.replayed, "convs_with_ranges_from_their_producer": ex.ranges_used, "lowering_s": round(build_s, 2),
               "outputs": [list(t.shape) for t in y], "finite_output": bool(all(np.isfinite(t).all() for t in y))}
        ex.close()
        return out
    batch = par
    ctx = fastnn_amd.HipContext(0)
    for _, ident, value in parsed_options(args, flib):
        ctx.set_option(ident, value)
    layers_ = []
    flops = 0.0
    for (c, h, oc, k, s) in yolo_convs():
        kk = c * k * k
        wt = (rng.standard_normal((oc, kk)) * np.sqrt(2.0 / kk)).astype(np.float32)
        pw = fastnn_amd.quantize_weights(flib.DT_I8, wt)
        pad = k // 2
        ho = (h + 2 * pad - k) // s + 1
        x = ctx.to_device(rng.uniform(0, 1, (batch, c, h, h)).astype(np.float32))
        bias = ctx.to_device((rng.standard_normal(oc) * 0.05).astype(np.float32))
        y = ctx.alloc(batch * oc * ho * ho * 4)
        layers_.append((ctx.register(pw), x, bias, y, c, h, oc, k, s, pad))
        flops += 2.0 * batch * ho * ho * kk * oc
    def fwd():
        for (hd, x, bias, y, c, h, oc, k, s, pad) in layers_:
            rc = ctx.lib.fnn_hip_qconv2d(ctx.handle, hd, x.ptr, batch, c, h, h, k, k, s, pad, 1, 1, bias.ptr, flib.ACT_SILU, y.ptr,
                                         None, flib.FLAG_DEVICE_PTRS)
            if rc:
                raise flib.FnnError(rc, ctx.lib.fnn_hip_last_error(ctx.handle).decode())
    for _ in range(1 + warm):
        fwd()
    ctx.sync()
    graph = None
    if args.mode == "graph":     # the whole forward (5 launches per conv) as one HIP graph
        ctx.graph_begin()
        fwd()
        graph = ctx.graph_end()
        ctx.graph_launch(graph)
        ctx.sync()
    t0 = time.perf_counter()
    ctx.timer_start()
    for _ in range(steps):
        if graph is not None:
            ctx.graph_launch(graph)
        else:
            fwd()
    ev = ctx.timer_stop() / steps
    ms = (time.perf_counter() - t0) * 1e3 / steps
    out = {"metric": f"C5 YOLOv8n-shaped I8 conv list forward ({len(layers_)} convs + bias + SiLU, B={batch})",
           "value": round(batch / (ms * 1e-3), 1), "unit": "images/s", "n_gpus": 1, "steps": steps, "warmup": warm,
           "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "i8/i32",
           "data": "synthetic", "config": {"workload": args.workload, "launch": args.mode + ", each conv on its own resident input",
                                           "options": {n: v for n, _, v in parsed_options(args, flib)}},
           "event_ms_per_step": round(ev, 4), "gop_per_step": round(flops / 1e9, 2), "top_per_s": round(flops / (ms * 1e-3) / 1e12, 2)}
    ctx.close()
    return out


def composite(args) -> int:
    print(json.dumps(composite_result(args)))
    return 0


def synth_weight(name: str, k: int, n: int, rng) -> np.ndarray:
    """[N,K] f32 weights with the distribution the configuration names (seed 0)."""
    if name == "c3_i4cb":
        w = np.where(rng.random((n, k)) < 0.9, rng.laplace(0, 0.02, (n, k)), rng.laplace(0, 0.10, (n, k)))
    elif name.startswith("c4"):
        w = rng.standard_normal((n, k)) / np.sqrt(k)
    else:
        w = rng.standard_normal((n, k)) * 0.02
        if name == "c2_i4":
            idx = rng.choice(n * k, size=(n * k) // 1000, replace=False)
            w.reshape(-1)[idx] *= 8
    return w.astype(np.float32)


def algorithmic_bytes(dt: str, m: int, k: int, n: int, bias: bool) -> int:
    """Every operand read once + output written once; packed weights without the margin."""
    bits = 8 if dt in ("i8", "u8", "f8", "f8r") else 4
    wbytes = n * k * bits // 8
    if dt == "i4cb":
        side = 4 * n * (k // 32) + 64
    elif dt in ("f8", "f8r"):
        side = 4 * n
    else:
        side = 8 * n
    if bias:
        side += 4 * n
    return wbytes + side + 4 * m * k + 4 * m * n


PROBE_SRC = os.path.join(ROOT, "bench_probe.hip")
PROBE_LIB = os.path.join(ROOT, "libbench_probe.so")


def build_probe(force: bool = False) -> str:
    """Compiles bench_probe.hip (plain read / copy / matrix-core / LDS kernels that only this benchmark uses) into
    libbench_probe.so beside it.  hipcc cross-compiles for gfx950 without a GPU."""
    import subprocess
    if force or not os.path.exists(PROBE_LIB) or os.path.getmtime(PROBE_LIB) < os.path.getmtime(PROBE_SRC):
        cmd = ["/opt/rocm/bin/hipcc", "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-shared", PROBE_SRC, "-o", PROBE_LIB]
        r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if r.returncode != 0:
            raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), r.stdout))
    return PROBE_LIB


class Probe:
    """The plain read / copy kernels of libbench_probe.so (this benchmark's own measurement aid, not part of the
    product library), launched on the context's stream so that the context's events time them."""

    def __init__(self, ctx):
        import ctypes as C
        if not os.path.exists(PROBE_LIB):
            build_probe()
        self.lib = C.CDLL(PROBE_LIB)
        self.lib.fnn_probe_stream.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_void_p]
        self.lib.fnn_probe_mfma.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p]
        self.lib.fnn_probe_lds_delivery.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p,
                                                    C.POINTER(C.c_double)]
        self.lib.fnn_probe_gemv_pattern.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_int, C.c_void_p]
        self.ctx = ctx
        self.stream = ctx.stream()
        self.sink = ctx.alloc(256)

    def launch(self, src, dst, nbytes, loads=1, wgs=0):
        rc = self.lib.fnn_probe_stream(self.stream, src, dst or None, nbytes, loads, wgs, self.sink.ptr)
        if rc:
            raise RuntimeError(f"fnn_probe_stream failed: hipError {rc}")

    def ceiling(self, ptrs, nbytes, configs=((1, 0), (4, 0), (8, 0), (4, 2048), (8, 2048), (8, 1024))):
        """Best plain read of `nbytes` per launch over the buffers `ptrs` (eager launches, events on the stream):
        (loads per lane, workgroups; 0 = one per chunk) -> microseconds."""
        out = {}
        for loads, wgs in configs:
            for p in ptrs:
                self.launch(p, 0, nbytes, loads, wgs)
            self.ctx.sync()
            n = max(len(ptrs) * 4, 64)
            self.ctx.timer_start()
            for i in range(n):
                self.launch(ptrs[i % len(ptrs)], 0, nbytes, loads, wgs)
            out[f"{loads}x16B/lane,{'all' if wgs == 0 else wgs}wg"] = round(self.ctx.timer_stop() / n * 1e3, 3)
        return out


    def gemv_pattern(self, ptrs, rows, row_bytes, row_tiles=3):
        """The int8 GEMV kernel's read pattern over rows x row_bytes packed bytes and nothing else (16 rows x 64
        bytes per wave-load, a wave per 256-byte column segment, `row_tiles` * 16 rows per workgroup): microseconds."""
        for p in ptrs:
            self.lib.fnn_probe_gemv_pattern(self.stream, p, rows, row_bytes, row_tiles, self.sink.ptr)
        self.ctx.sync()
        n = max(len(ptrs) * 4, 64)
        self.ctx.timer_start()
        for i in range(n):
            rc = self.lib.fnn_probe_gemv_pattern(self.stream, ptrs[i % len(ptrs)], rows, row_bytes, row_tiles, self.sink.ptr)
            if rc:
                raise RuntimeError(f"fnn_probe_gemv_pattern failed: hipError {rc}")
        return round(self.ctx.timer_stop() / n * 1e3, 3)

    def lds_delivery(self, iters=400):
        """Bytes per microsecond that loops of `global_load_lds_dwordx4` stages deliver into the LDS, by waves per
        CU: 256 / 512 / 768 workgroups of 4 waves, 256 of 8 and of 16; ring of 3 stages (and 6 for 4 and 8 waves)."""
        import ctypes as C
        src = self.ctx.alloc(8 << 20)
        out = {}
        for name, waves, stages, wgs in (("4 waves/CU", 4, 3, 256), ("4 waves/CU, 6 stages", 4, 6, 256), ("2x4 waves/CU", 4, 3, 512),
                                         ("3x4 waves/CU", 4, 3, 768), ("8 waves/CU", 8, 3, 256), ("8 waves/CU, 6 stages", 8, 6, 256),
                                         ("16 waves/CU", 16, 3, 256)):
            nbytes = C.c_double(0.0)
            for _ in range(2):
                rc = self.lib.fnn_probe_lds_delivery(self.stream, src.ptr, waves, stages, wgs, iters, self.sink.ptr, C.byref(nbytes))
                if rc:
                    raise RuntimeError(f"fnn_probe_lds_delivery failed: hipError {rc}")
            self.ctx.sync()
            n = 5
            self.ctx.timer_start()
            for _ in range(n):
                self.lib.fnn_probe_lds_delivery(self.stream, src.ptr, waves, stages, wgs, iters, self.sink.ptr, C.byref(nbytes))
            us = self.ctx.timer_stop() / n * 1e3
            out[name] = {"us": round(us, 1), "tb_per_s": round(nbytes.value / us / 1e6, 2),
                         "bytes_per_us_and_cu": round(nbytes.value / us / 256.0, 0)}
        src.free()
        return out

    def mfma_ceiling(self, target_us=(20.0, 60.0)):
        """What the matrix cores sustain with nothing else in the way: a kernel of MFMAs only (pseudo-random
        register operands, no memory traffic), sized to run about `target_us` per launch, one and two workgroups of
        4 waves per CU and one of 8.  -> {kind: {shape: {us, tops}}}; f16 counts flops, int8 ops."""
        out = {}
        for kind, name, per in ((0, "f16_32x32x16", 32768.0), (1, "i8_32x32x32", 65536.0)):
            res = {}
            for wgs, waves in ((256, 4), (512, 4), (256, 8)):
                for tus in target_us:
                    # 32 clocks per instruction and SIMD at ~2 GHz; waves beyond one per SIMD share the matrix core
                    per_simd = max(1, wgs * waves // 1024)
                    iters = max(8, int(tus * 2000.0 / 32.0 / 4.0 / per_simd))
                    for _ in range(3):
                        rc = self.lib.fnn_probe_mfma(self.stream, kind, wgs, waves, iters, self.sink.ptr)
                        if rc:
                            raise RuntimeError(f"fnn_probe_mfma failed: hipError {rc}")
                    self.ctx.sync()
                    n = 20
                    self.ctx.timer_start()
                    for _ in range(n):
                        self.lib.fnn_probe_mfma(self.stream, kind, wgs, waves, iters, self.sink.ptr)
                    us = self.ctx.timer_stop() / n * 1e3
                    ops = float(wgs) * waves * 4 * iters * per
                    res[f"{wgs}wg x {waves} waves, {iters * 4} mfma/wave"] = {"us": round(us, 2), "tops": round(ops / us / 1e6, 1)}
            out[name] = res
        return out


def make_ring(ctx, fastnn_amd, flib, workload, ring_arg):
    """Quantise the workload's weight once and register `ring` distinct device copies of it (rows rotated by i),
    so that consecutive steps stream from HBM and not from the 256 MB Infinity Cache."""
    dtn, k, n, has_bias, actn = WORKLOADS[workload]
    dt = {"i8": flib.DT_I8, "i4": flib.DT_I4, "i4cb": flib.DT_I4CB, "f8": flib.DT_F8, "f4": flib.DT_F4}[dtn]
    rng = np.random.default_rng(0)
    w = synth_weight(workload, k, n, rng)
    bias = (rng.standard_normal(n) * 0.01).astype(np.float32) if has_bias else None
    t0 = time.time()
    pw = fastnn_amd.quantize_weights(dt, w)
    t_quant = time.time() - t0
    wbytes = pw.packed_bytes()
    ring = ring_arg if ring_arg > 0 else max(2, int(np.ceil(544e6 / wbytes)))
    items = 32 // pw.bit_width
    kp = -(-k // items)
    base_words = pw.words[: n * kp].reshape(n, kp)
    handles = []
    for i in range(ring):
        if i == 0:
            pwi = pw
        else:
            words = np.concatenate([np.roll(base_words, i, axis=0).reshape(-1), np.zeros(16, np.uint32)])
            if dt == flib.DT_I4CB:
                bpr = k // 32
                sc = np.roll(pw.scales.reshape(n, bpr), i, axis=0).reshape(-1).copy()
                zr = pw.zeros
            else:
                sc, zr = np.roll(pw.scales, i).copy(), np.roll(pw.zeros, i).copy()
            pwi = fastnn_amd.PackedWeight(dt, n, k, words, sc, zr, pw.qblock, pw.codebook)
        handles.append(ctx.register(pwi))
    return {"workload": workload, "dtn": dtn, "dt": dt, "k": k, "n": n, "bias": bias, "actn": actn,
            "act": {"none": 0, "relu": 1, "gelu": 2, "silu": 3}[actn], "pw": pw, "wbytes": wbytes, "ring": ring,
            "handles": handles, "dbias": ctx.to_device(bias) if has_bias else None, "quantize_s": t_quant}


def free_ring(ctx, r):
    for h in r["handles"]:
        ctx.release(h)
    if r["dbias"]:
        r["dbias"].free()


def time_i8act(ctx, flib, r, m, calls=200):
    """matmul_i8_i8 / matmul_i4_i8: I8 activation payload x packed weights (quantised once on the host, resident),
    eager launches over the weight ring.  Integer ops 2*M*K*N against the nominal int8 peak."""
    import ctypes as C
    k, n, ring = r["k"], r["n"], r["ring"]
    x = np.random.default_rng(2).standard_normal((m, k)).astype(np.float32)
    payload = ctx.quantize_activations(x)
    dp, dout = ctx.to_device(payload), ctx.alloc(m * n * 4)
    vp = C.c_void_p

    def call(i):
        ctx._check(ctx.lib.fnn_hip_qmatmul_i8act(ctx.handle, r["handles"][i % ring], vp(dp.ptr), m, vp(dout.ptr), None, flib.FLAG_DEVICE_PTRS))

    for i in range(ring):
        call(i)
    ctx.sync()
    ctx.timer_start()
    for i in range(calls):
        call(i)
    us = ctx.timer_stop() * 1e3 / calls
    dp.free()
    dout.free()
    tops = 2.0 * m * k * n / us / 1e6
    return {"us": round(us, 2), "top_per_s": round(tops, 1), "frac": round(tops / MFMA_PEAK_TFLOPS["i8"], 4), "peak": MFMA_PEAK_TFLOPS["i8"], "calls": calls}


def time_matmul(ctx, flib, r, m, steps_min, warmup, mode, flags=0, a_seed=0):
    """`steps_min` or more MatMul calls at M = m over the ring, rounded up to whole trips and to at least 20 of them.
    graph mode: one HIP graph = one trip round the ring.  Returns the continuous figure (events around all trips:
    the headline) and per-trip figures (each trip between its own events: median and minimum per step)."""
    k, n, ring = r["k"], r["n"], r["ring"]
    a = np.random.default_rng(a_seed).standard_normal((m, k)).astype(np.float32)
    da, dout = ctx.to_device(a), ctx.alloc(m * n * 4)
    bias_ptr = r["dbias"].ptr if r["dbias"] else 0

    def step(i):
        ctx.qmatmul_dev(r["handles"][i % ring], da.ptr, m, dout.ptr, bias_ptr, r["act"], flags)

    for i in range(ring):          # first-use side tables and workspace sizes, before any capture
        step(i)
    for i in range(warmup):
        step(i)
    ctx.sync()
    trips = max(20, -(-steps_min // ring))
    steps = trips * ring
    graph = None
    if mode == "graph":
        ctx.graph_begin()
        for i in range(ring):
            step(i)
        graph = ctx.graph_end()
        ctx.graph_launch(graph)
        ctx.sync()

    def trip():
        if graph is not None:
            ctx.graph_launch(graph)
        else:
            for i in range(ring):
                step(i)

    ctx.sync()
    t0 = time.perf_counter()
    ctx.timer_start()
    for _ in range(trips):
        trip()
    ev_ms = ctx.timer_stop()
    ctx.sync()
    wall_s = time.perf_counter() - t0
    per_trip = []
    for _ in range(trips):
        ctx.timer_start()
        trip()
        per_trip.append(ctx.timer_stop() / ring * 1e3)
    # what was timed is checked against a second, independent kernel (the shape-agnostic one) on the weight copy
    # the last step used
    got = dout.download(np.float32, m * n).reshape(m, n)
    chk = ctx.qmatmul(r["handles"][ring - 1], a, n, bias=r["bias"], act=r["act"], flags=flags | flib.FLAG_FORCE_GENERIC)
    res = {"steps": steps, "trips": trips, "kernel_us": ev_ms / steps * 1e3, "wall_ms_per_step": wall_s * 1e3 / steps,
           "event_ms_total": ev_ms, "wall_ms_total": wall_s * 1e3,
           "per_trip_us_median": float(np.median(per_trip)), "per_trip_us_min": float(np.min(per_trip)),
           "self_check_max_rel": float(np.abs(got - chk).max() / (np.abs(chk).max() + 1e-30)), "a": a}
    if graph is not None:
        ctx.graph_destroy(graph)
    da.free()
    dout.free()
    return res


def gemv_summary(r, m, t, probe_us=None):
    abytes = algorithmic_bytes(r["dtn"], m, r["k"], r["n"], r["bias"] is not None)
    ach = abytes / (t["kernel_us"] * 1e-6) / 1e9
    out = {"workload": r["workload"], "m": m, "k": r["k"], "n": r["n"], "steps": t["steps"], "weight_ring": r["ring"],
           "kernel_us": round(t["kernel_us"], 3), "kernel_us_median": round(t["per_trip_us_median"], 3),
           "kernel_us_min": round(t["per_trip_us_min"], 3), "algorithmic_bytes": abytes,
           "gb_per_s": round(ach, 1), "frac_of_hbm_peak": round(ach / HBM_PEAK_GBS, 4),
           "self_check_max_rel": t["self_check_max_rel"]}
    if probe_us:
        best = min(probe_us.values())
        out["plain_read_us"] = best
        out["frac_of_plain_read"] = round(best / t["kernel_us"], 3)
    return out


def matrix_entry(r, m, t):
    """One (configuration, M) pair of the benchmark matrix: time per call, algorithmic bytes and flops, and the
    fraction of the roof that applies (HBM for M <= 64: at most 128 flop per weight byte against a ridge of about 312;
    the nominal dense f16 matrix-core peak above)."""
    abytes = algorithmic_bytes(r["dtn"], m, r["k"], r["n"], r["bias"] is not None)
    flops = 2.0 * m * r["k"] * r["n"]
    sec = t["kernel_us"] * 1e-6
    e = {"us": round(t["kernel_us"], 2), "us_median": round(t["per_trip_us_median"], 2), "us_min": round(t["per_trip_us_min"], 2),
         "algorithmic_bytes": abytes, "flops": flops, "gb_per_s": round(abytes / sec / 1e9, 1),
         "tflop_per_s": round(flops / sec / 1e12, 2), "self_check_max_rel": t["self_check_max_rel"]}
    if m <= 64:
        e["roof"], e["frac"] = "hbm", round(abytes / sec / 1e9 / HBM_PEAK_GBS, 4)
    else:
        e["roof"], e["frac"] = "mfma_f16", round(flops / sec / 1e12 / MFMA_PEAK_TFLOPS["f16"], 4)
    return e


def gemm_summary(r, m, t, peak_name="f16"):
    flops = 2.0 * m * r["k"] * r["n"]
    peak = MFMA_PEAK_TFLOPS[peak_name]
    tf = flops / (t["kernel_us"] * 1e-6) / 1e12
    return {"us": round(t["kernel_us"], 2), "us_median": round(t["per_trip_us_median"], 2), "us_min": round(t["per_trip_us_min"], 2),
            "tflop_per_s": round(tf, 1), "frac": round(tf / peak, 4), "peak": peak, "steps": t["steps"],
            "self_check_max_rel": t["self_check_max_rel"]}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=480, help="timed steps at least (rounded up to whole trips round the weight ring, 20 trips or more)")
    ap.add_argument("--warmup", type=int, default=48)
    ap.add_argument("--workload", default="c2_i4", choices=sorted(WORKLOADS) + sorted(COMPOSITE),
                    help="single quantised MatMul (default: the configuration the metric is quoted on), or one of "
                         "the composite configurations run through the plan dispatcher: " + ", ".join(sorted(COMPOSITE)))
    ap.add_argument("--m", type=int, default=1)
    ap.add_argument("--ring", type=int, default=0, help="distinct weight copies (0: enough for > 512 MB)")
    ap.add_argument("--mode", default="graph", choices=["graph", "eager"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--fast-act16", action="store_true", help="single f16 rounding of activations on the MFMA path")
    ap.add_argument("--act-quant", action="store_true", help="the opt-in activation-quantised mode (FNN_FLAG_ACT_QUANT; I8 / I4 / F8 weights, "
                    "M >= 17): NOT parity with the default MatMul")
    ap.add_argument("--i8act", action="store_true", help="time only matmul_i8_i8 / matmul_i4_i8 (an int8 activation payload, resident) at "
                    "--m on the workload's weights, eager launches (the gemm_m256.c1_i8_i8act leg on its own, for kernel traces)")
    ap.add_argument("--no-extra", "--no-m256", dest="no_extra", action="store_true",
                    help="skip the extra legs (K=N=4096 GEMVs, M=256 GEMMs)")
    ap.add_argument("--opt", action="append", default=[], metavar="NAME=VALUE",
                    help="kernel selection option of the context, e.g. gemv_int8=0 for the f16 matrix-core GEMV "
                         "(names: the FNN_OPT_* of include/fastnn_hip.h, lower case without the prefix)")
    ap.add_argument("--probe", default="", choices=["", "read", "copy", "mfma", "lds"],
                    help="instead of the MatMul, time a plain streaming read / copy of the same number of bytes "
                         "per launch over the same ring (device ceiling; calibration kernel for byte counters)")
    ap.add_argument("--traffic-json", default="", help="JSON file {\"fetch_bytes\": .., \"write_bytes\": ..} with "
                    "counter-derived HBM bytes per launch (see profiles/); copied into roofline.traffic")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path shards over N without changing the "
              "per-GPU kernel); run with --gpus 1", file=sys.stderr)
        return 2

    import fastnn_amd
    from fastnn_amd import lib as flib

    try:
        parsed_options(args, flib)
    except ValueError as e:
        print(f"bench.py: {e}", file=sys.stderr)
        return 2
    if args.workload in COMPOSITE:
        return composite(args)

    m = args.m
    flags = flib.FLAG_ACT_F16_SINGLE if args.fast_act16 else 0
    if args.act_quant:
        flags |= flib.FLAG_ACT_QUANT
    ctx = fastnn_amd.HipContext(0)
    opts = {}
    for name, ident, value in parsed_options(args, flib):
        ctx.set_option(ident, value)
        opts[name] = value
    probe = Probe(ctx)
    if args.probe == "mfma":
        res = probe.mfma_ceiling()
        best = {k: max(v2["tops"] for v2 in v.values()) for k, v in res.items()}
        print(json.dumps({"metric": "matrix-core instructions only (no memory traffic)", "value": best["f16_32x32x16"], "unit": "TFLOP/s",
                          "n_gpus": 1, "higher_is_better": True, "data": "synthetic", "best": best, "all": res,
                          "config": {"workload": "probe mfma"}}))
        return 0
    if args.probe == "lds":
        res = probe.lds_delivery()
        print(json.dumps({"metric": "HBM/L2 -> LDS delivery of global_load_lds loops (no other work)", "value": max(v["tb_per_s"] for v in res.values()),
                          "unit": "TB/s", "n_gpus": 1, "higher_is_better": True, "data": "synthetic", "all": res,
                          "config": {"workload": "probe lds"}}))
        return 0
    r = make_ring(ctx, fastnn_amd, flib, args.workload, args.ring)
    dtn, k, n, wbytes, ring = r["dtn"], r["k"], r["n"], r["wbytes"], r["ring"]
    has_bias = r["bias"] is not None
    src_ptrs = [ctx.alloc(wbytes).ptr for _ in range(ring)]

    if args.probe:
        # same launch count, same ring size, same bytes per launch as the MatMul's packed weights
        dst = ctx.alloc(wbytes).ptr if args.probe == "copy" else 0
        for p in src_ptrs:
            probe.launch(p, dst, wbytes)
        ctx.sync()
        trips = max(20, -(-args.steps // ring))
        ctx.graph_begin()
        for p in src_ptrs:
            probe.launch(p, dst, wbytes)
        graph = ctx.graph_end()
        ctx.graph_launch(graph)
        ctx.sync()
        ctx.timer_start()
        for _ in range(trips):
            ctx.graph_launch(graph)
        us = ctx.timer_stop() / (trips * ring) * 1e3
        nb = wbytes * (2 if args.probe == "copy" else 1)
        print(json.dumps({"metric": f"plain {args.probe} of {wbytes} bytes per launch", "value": round(nb / us / 1e3, 1), "unit": "GB/s",
                          "n_gpus": 1, "steps": trips * ring, "warmup": ring, "ms_per_step": round(us * 1e-3, 6), "higher_is_better": True,
                          "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
                          "config": {"workload": f"probe {args.probe}", "bytes_per_launch": nb, "weight_ring": ring}}))
        ctx.graph_destroy(graph)
        ctx.close()
        return 0

    if args.i8act:
        if dtn not in ("i8", "i4"):
            raise SystemExit("--i8act: the I8-activation MatMul takes I8 and I4 weights")
        t8 = time_i8act(ctx, flib, r, m, max(args.steps, 20))
        print(json.dumps({"metric": f"matmul_{dtn}_i8 at M={m} (int8 activation payload x packed weights, eager launches over the weight ring)",
                          "value": t8["top_per_s"], "unit": "TOP/s", "n_gpus": 1, "steps": t8["calls"], "warmup": ring, "ms_per_step": round(t8["us"] * 1e-3, 6),
                          "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "i8/i32", "data": "synthetic",
                          "config": {"workload": args.workload, "m": m, "k": k, "n": n, "options": opts}, "frac_of_int8_peak": t8["frac"]}))
        free_ring(ctx, r)
        ctx.close()
        return 0

    t = time_matmul(ctx, flib, r, m, args.steps, args.warmup, args.mode, flags)
    steps = t["steps"]
    ms_per_step = t["wall_ms_per_step"]
    kernel_ms = t["kernel_us"] * 1e-3      # HIP events on the launch stream over the timed region
    abytes = algorithmic_bytes(dtn, m, k, n, has_bias)
    flops = 2.0 * m * k * n
    gbs = abytes / (ms_per_step * 1e-3) / 1e9
    tops = flops / (ms_per_step * 1e-3) / 1e12

    # device ceiling for one launch of this size: plain streaming reads of the packed bytes over a ring of buffers
    # of the same size, several launch shapes (loads in flight per lane, all-at-once or walking grid), the best counts
    ceil_us = probe.ceiling(src_ptrs, wbytes)
    best_cfg = min(ceil_us, key=ceil_us.get)

    bandwidth_bound = m <= 32
    if bandwidth_bound:
        achieved = abytes / (kernel_ms * 1e-3) / 1e9
        roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                    "kernel_us": round(kernel_ms * 1e3, 3), "kernel_us_median": round(t["per_trip_us_median"], 3),
                    "kernel_us_min": round(t["per_trip_us_min"], 3), "algorithmic_bytes": abytes}
        metric, value, unit = f"qGEMM GB/s at M={m} ({dtn} K={k} N={n})", gbs, "GB/s"
    else:
        peak = MFMA_PEAK_TFLOPS["f16"]
        achieved = flops / (kernel_ms * 1e-3) / 1e12
        roofline = {"bound": "mfma", "achieved": round(achieved, 2), "peak": peak, "unit": "TFLOP/s",
                    "frac": round(achieved / peak, 4), "traffic": None,
                    "kernel_us": round(kernel_ms * 1e3, 3), "kernel_us_median": round(t["per_trip_us_median"], 3),
                    "kernel_us_min": round(t["per_trip_us_min"], 3), "algorithmic_flops": flops}
        metric, value, unit = f"qGEMM TOPS at M={m} ({dtn} K={k} N={n})", tops, "TFLOP/s"
    roofline["device_stream_read"] = {"gb_per_s": round(wbytes / ceil_us[best_cfg] / 1e3, 1), "us": ceil_us[best_cfg], "bytes": wbytes,
                                      "launch_shape": best_cfg, "all_shapes_us": ceil_us,
                                      "frac_of_this_ceiling": round(ceil_us[best_cfg] / (kernel_ms * 1e3), 3),
                                      "note": "best plain read of the same packed bytes per launch over a ring of buffers of "
                                              "the same size, eager launches, events on the same stream"}
    if bandwidth_bound and wbytes % n == 0 and (wbytes // n) % 2048 == 0:
        # the same bytes read in the GEMV kernel's own order (16 rows x 64 bytes per wave-load) and nothing else
        roofline["device_stream_read"]["gemv_pattern_us"] = {f"{rt}x16 rows/wg": probe.gemv_pattern(src_ptrs, n, wbytes // n, rt) for rt in (1, 2, 3)}
    # counter-derived HBM bytes per launch, recorded under profiles/ for the measured configurations
    tj = args.traffic_json or os.path.join(ROOT, "profiles", f"traffic_{args.workload}_m{m}.json")
    if os.path.exists(tj):
        with open(tj) as f:
            td = json.load(f)
        roofline["traffic"] = td.get("bytes")
        roofline["traffic_detail"] = td

    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline(r["pw"], t["a"], r["bias"], r["act"], abytes, flops, bandwidth_bound, args.cpu_seconds)

    # the other shapes the target is worded on, in the same line: the GEMV at K = N = 4096 (I8 and I4) and the
    # M = 256 GEMM for I4 (this configuration), I8 and FP8
    gemv_4096, gemm_m256, config_matrix = None, None, None
    if not args.no_extra:
        gemm_m256 = {"m": 256, "unit": "TFLOP/s",
                     "note": "algorithmic flops 2*M*K*N over the whole call (activation preparation + GEMM kernels), eager "
                             "launches over the weight ring; 'default' (2e-5 agreement): I8 / I4 weights run on the int8 matrix "
                             "cores over three exact activation digit planes (3x the algorithmic ops at the int8 rate), FP8 on "
                             "the f16 matrix cores with hi+lo f16 activation rows (2x the algorithmic flops); 'f16x1' (1e-3): "
                             "activations rounded to f16 once; frac is of the nominal dense f16 peak (2.5 PFLOP/s); "
                             "matrix_core_only = what a kernel of MFMAs alone (no memory traffic) sustains on this device"}
        mc = probe.mfma_ceiling(target_us=(40.0,))
        gemm_m256["matrix_core_only"] = {"f16_tflop_per_s": max(v["tops"] for v in mc["f16_32x32x16"].values()),
                                         "i8_top_per_s": max(v["tops"] for v in mc["i8_32x32x32"].values())}
        def act_quant_leg(rr):
            peak = "fp8" if rr["dtn"] == "f8" else "i8"
            e = gemm_summary(rr, 256, time_matmul(ctx, flib, rr, 256, 200, rr["ring"], "eager", flib.FLAG_ACT_QUANT, a_seed=1), peak)
            e["note"] = ("FNN_FLAG_ACT_QUANT, NOT parity with matmul_%s: activations quantised on the way in (%s), one plane on the "
                         "%s matrix cores; frac is of the nominal dense %s peak" %
                         (rr["dtn"], "E4M3, one power-of-two scale per row; within 5e-2 of max|ref|" if peak == "fp8" else
                          "the reference's quantize_activations -> matmul_*_i8 chain, integer accumulators bit-exact against it",
                          peak, peak))
            return e

        if m != 256:
            gemm_m256[args.workload] = {
                "default": gemm_summary(r, 256, time_matmul(ctx, flib, r, 256, 200, ring, "eager", 0, a_seed=1)),
                "f16x1": gemm_summary(r, 256, time_matmul(ctx, flib, r, 256, 200, ring, "eager", flib.FLAG_ACT_F16_SINGLE, a_seed=1))}
            if dtn in ("i8", "i4", "f8"):
                gemm_m256[args.workload]["act_quant"] = act_quant_leg(r)
        # every (configuration, M) pair the benchmark configurations name, graph replay over the weight ring
        config_matrix = {"note": "time per call (HIP events on the launch stream, graph replay of whole trips round a weight ring "
                                 "larger than the Infinity Cache), algorithmic bytes / flops, fraction of the applicable roof: "
                                 "8 TB/s HBM for M <= 64, nominal dense f16 matrix-core peak 2.5 PFLOP/s above"}
        matrix_ms = {"c1_i8": (32,), "c2_i4": (16, 128, 256), "c3_i4cb": (1, 64, 256), "c4_f8_up": (64,), "c4_f8_down": (64,),
                     "c4_f4_up": (64,), "c4_f4_down": (64,)}

        def matrix_legs(rr):
            for mm in matrix_ms.get(rr["workload"], ()):
                tt = time_matmul(ctx, flib, rr, mm, 100, 5, "graph", 0, a_seed=1)
                config_matrix.setdefault(rr["workload"], {})[str(mm)] = matrix_entry(rr, mm, tt)

        config_matrix.setdefault(args.workload, {})[str(m)] = matrix_entry(r, m, t)
        matrix_legs(r)
        free_ring(ctx, r)
        gemv_4096 = {}
        for wl in ("c1_i8", "i4_4096", "f8_4096"):
            r2 = make_ring(ctx, fastnn_amd, flib, wl, 0)
            if wl != "f8_4096":
                t2 = time_matmul(ctx, flib, r2, 1, args.steps, r2["ring"], args.mode, flags)
                p2 = [ctx.alloc(r2["wbytes"]) for _ in range(min(r2["ring"], 40))]
                gemv_4096[wl] = gemv_summary(r2, 1, t2, probe.ceiling([b.ptr for b in p2], r2["wbytes"], configs=((1, 0), (8, 0), (8, 2048))))
                for b in p2:
                    b.free()
            if wl != "i4_4096":
                gemm_m256[wl] = {
                    "default": gemm_summary(r2, 256, time_matmul(ctx, flib, r2, 256, 200, r2["ring"], "eager", 0, a_seed=1)),
                    "f16x1": gemm_summary(r2, 256, time_matmul(ctx, flib, r2, 256, 200, r2["ring"], "eager", flib.FLAG_ACT_F16_SINGLE, a_seed=1)),
                    "act_quant": act_quant_leg(r2)}
            if wl == "c1_i8":
                gemm_m256["c1_i8_i8act"] = time_i8act(ctx, flib, r2, 256)
                config_matrix.setdefault(wl, {})["1"] = matrix_entry(r2, 1, t2)
                if args.workload != wl:
                    matrix_legs(r2)
            free_ring(ctx, r2)
        for wl in ("c3_i4cb", "c4_f8_up", "c4_f8_down", "c4_f4_up", "c4_f4_down"):
            if wl == args.workload:
                continue
            r2 = make_ring(ctx, fastnn_amd, flib, wl, 0)
            matrix_legs(r2)
            free_ring(ctx, r2)

    # the composite configurations (conv list, conv plan, MLP stack), each its own short run: ms per forward
    composites = None
    if not args.no_extra:
        import copy
        composites = {}
        ctx.close()
        ctx = None
        for wl in ("c5_yolo_b1", "c5_yolo_b16", "c5_yolo_graph_b1", "c5_yolo_graph_b16", "c4_mlp_f8", "c4_mlp_f4"):
            a2 = copy.copy(args)
            a2.workload, a2.steps, a2.warmup, a2.mode, a2.opt = wl, 30, 3, "graph", []
            try:
                res = composite_result(a2)
                composites[wl] = {k2: res[k2] for k2 in ("metric", "ms_per_step", "value", "unit") if k2 in res}
            except Exception as e:   # the headline stands on its own
                composites[wl] = {"error": str(e)[:200]}

    out = {
        "metric": metric, "value": round(value, 2), "unit": unit, "n_gpus": 1, "steps": steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 6), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"{args.workload}: {dtn} weights [N={n},K={k}] per-channel, f32 activations "
                               f"[M={m},K={k}] ~N(0,1), bias={has_bias}, act={r['actn']}, seed 0",
                   "m": m, "k": k, "n": n, "weight_ring": ring, "ring_bytes": ring * wbytes, "trips": t["trips"],
                   "launch": args.mode, "act_rounding": "act_quant (not parity)" if args.act_quant else ("f16x1" if args.fast_act16 else "default"),
                   **({"options": opts} if opts else {})},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "gemv_4096": gemv_4096,
        "gemm_m256": gemm_m256,
        "config_matrix": config_matrix,
        "composites": composites,
        "gb_per_s": round(gbs, 1), "tflop_per_s": round(tops, 3),
        "event_ms_total": round(t["event_ms_total"], 4), "wall_ms_total": round(t["wall_ms_total"], 4),
        "quantize_host_s": round(r["quantize_s"], 3), "self_check_max_rel": t["self_check_max_rel"],
    }
    print(json.dumps(out))
    if ctx is not None:
        ctx.close()
    return 0


def cpu_baseline(pw, a, bias, act, abytes, flops, bandwidth_bound, budget_s):
    """fastnn's CPU path beside the GPU figure, timed on this host on the same workload: the tuned port
    (oracle/fnn_cpu_baseline.c: AVX2 unpack + FMA dots as gemm_batch_packed_simd does them) on one thread, which is
    how the reference runs M = 1 today, and with the weight rows over the host's cores, which is how its published
    GEMV rows were measured.  Weight types the tuned port does not cover fall back to the oracle's scalar restatement
    on a row sample."""
    from oracle import oracle
    po = oracle.Packed(pw.dtype, pw.rows, pw.inner, pw.words, pw.scales, pw.zeros, pw.qblock, pw.codebook)
    m, n = a.shape[0], pw.rows
    published = ("published by the reference (CHANGELOG.md:628-635, GEMV 4096x4096, Ryzen 7 3700X, 8 threads): "
                 "U8x4 0.76 ms, U4x8 0.55 ms")
    cores = max(1, min(16, len(os.sched_getaffinity(0))))

    def run(fn, seconds):
        fn()
        times = []
        t_end = time.perf_counter() + seconds
        while (time.perf_counter() < t_end and len(times) < 400) or len(times) < 3:
            t0 = time.perf_counter()
            fn()
            times.append(time.perf_counter() - t0)
        return float(np.median(times)), float(np.min(times)), len(times)

    def rate(sec, frac=1.0):
        return (abytes * frac / sec / 1e9, "GB/s") if bandwidth_bound else (flops * frac / sec / 1e12, "TFLOP/s")

    if pw.dtype in (0, 1):
        med1, min1, n1 = run(lambda: oracle.cpu_qgemm(po, a, bias=bias, act=act, threads=1), budget_s / 2)
        medc, minc, nc = run(lambda: oracle.cpu_qgemm(po, a, bias=bias, act=act, threads=cores), budget_s / 2)
        value, unit = rate(medc)
        return {"value": round(value, 3), "unit": unit, "cores": cores, "kind": "port",
                "median_ms": round(medc * 1e3, 3), "min_ms": round(minc * 1e3, 3),
                "single_thread": {"value": round(rate(med1)[0], 3), "unit": unit, "median_ms": round(med1 * 1e3, 3),
                                  "min_ms": round(min1 * 1e3, 3), "calls": n1},
                "sample": f"{nc} calls of the whole workload (N={n}, M={m}) through oracle/fnn_cpu_baseline.c (gcc -O3 -mavx2 -mfma, "
                          f"AVX2 unpack + FMA dot per weight row, rows over {cores} threads; host shows "
                          f"{os.cpu_count()} logical CPUs, {len(os.sched_getaffinity(0))} usable); single_thread = the same on one "
                          f"thread, as the reference runs M=1 today; {published}"}
    # other weight types: the scalar restatement of gemm_batch_packed_simd on a bounded row sample
    rows = n
    est = 2e-9 * m * pw.inner * n + 4e-9 * pw.inner * n   # rough seconds per call
    if est > budget_s / 4:
        rows = max(64, int(n * (budget_s / 4) / est))
    if rows < n:
        items = 32 // pw.bit_width
        kp = -(-pw.inner // items)
        words = np.concatenate([pw.words[: rows * kp], np.zeros(16, np.uint32)])
        if pw.dtype == 7:
            bpr = pw.inner // pw.qblock
            po = oracle.Packed(pw.dtype, rows, pw.inner, words, pw.scales[: rows * bpr], pw.zeros, pw.qblock, pw.codebook)
        else:
            po = oracle.Packed(pw.dtype, rows, pw.inner, words, pw.scales[:rows], pw.zeros[:rows])
        bias = None if bias is None else bias[:rows]
    med, mn, cnt = run(lambda: oracle.qmatmul(po, a, order=1, bias=bias, act=act), budget_s)
    value, unit = rate(med, rows / n)
    return {"value": round(value, 4), "unit": unit, "cores": 1, "kind": "port", "median_ms": round(med * 1e3, 3),
            "min_ms": round(mn * 1e3, 3),
            "sample": f"{cnt} calls of the C restatement of gemm_batch_packed_simd (scalar unpack, AVX2 dot order, one "
                      f"thread) on {rows}/{n} weight rows, M={m}; {published}"}


if __name__ == "__main__":
    sys.exit(main())
