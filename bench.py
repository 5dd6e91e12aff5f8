#!/usr/bin/env python3
"""Benchmark of the low-bit GEMM/GEMV hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--no-extra]

A "step" is one pass of the decode-shape sweep of the benchmark configuration: the four fp16 x int4
(g128) M = 1 linear layers of a Llama-7B-like block -- (N,K) = (12288,4096) fused QKV, (4096,4096)
O-proj, (22016,4096) gate+up, (4096,11008) down -- one launch each, through the C ABI.  To keep the
figure an HBM figure, the weights of `layers` independent layers (same distributions, > 600 MB in
total, more than the 256 MB last-level cache) are resident and step i uses layer i mod layers, as a
decoder walks its layers.  Inputs are resident in HBM before the timed region; the timed region is K
steps captured in one HIP graph (launch-bound otherwise: each kernel runs for a few microseconds),
bracketed by synchronisation.

Prints ONE JSON line.  `value` = algorithmic bytes of a step (every operand read once, output written
once) / time per step.  `roofline` covers the kernel that dominates the step; `cpu_baseline` times the
same sweep on the host cores with the reference's CPU GEMM (MLAS built from the reference tree, or the
oracle's own port when that library is absent) on fp32 weights dequantised beforehand.  `extra` holds
the other configurations (prefill GEMM, W8A8, fused MLP), each measured for a few iterations.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

COLD_FOOTPRINT_BYTES = 600 * 1000 * 1000  # buffers walked by a timing loop: more than the last-level cache holds
HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
MFMA_F16_PEAK_TFLOPS = 2500.0  # dense fp16 MFMA
MFMA_I8_PEAK_TOPS = 5000.0     # dense int8 MFMA

DECODE_SHAPES = [(12288, 4096), (4096, 4096), (22016, 4096), (4096, 11008)]  # (N, K), M = 1
GROUP = 128
PROBE_BYTES = 1 << 30  # size of the calibration copy of --pmc-probe
# HBM bytes per launch of the K = 4096 row-streaming kernel (mean over its three launches of a step), from two
# rocprofv3 --pmc runs of `bench.py --pmc-probe`: FETCH_SIZE 13268.7 KiB x 2.000 (the factor by which the
# counter under-reports the 1 GiB calibration copy) + WRITE_SIZE 27.3 KiB x 1.000.  Algorithmic: 27 067 392.
ROWS_K4096_TRAFFIC_BYTES = int((13268.7 * 2.0 + 27.3) * 1024)


def w4a16_bytes(m, n, k):
    """Algorithmic bytes: int4 weights + fp16 group scales + fp16 activations + fp16 output."""
    return n * k // 2 + n * (k // GROUP) * 2 + m * k * 2 + m * n * 2


def w8a8_bytes(m, n, k):
    return n * k + n * 4 + m * k + m * 4 + m * n * 2


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1200)
    ap.add_argument("--warmup", type=int, default=24)
    ap.add_argument("--layers", type=int, default=6, help="independent weight sets walked by the steps")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true")
    ap.add_argument("--pmc-probe", action="store_true",
                    help="for hardware-counter runs: a plain copy of known size, then the sweep launched eagerly; "
                         "no timing, no JSON")
    ap.add_argument("--mfma-probe", action="store_true",
                    help="print the MFMA-only rates (no memory traffic) for different operand values and exit")
    ap.add_argument("--gemm-probe", action="store_true",
                    help="for hardware-counter runs: the fp16 x int4 and the W8A8 GEMM at M=4096, N=K=8192, twelve "
                         "launches each; prints their event-timed means, no JSON line of the benchmark")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU (no sharding, no collectives); use --gpus 1")

    import numpy as np
    import torch

    from nnfusion_amd import _lib, datagen, ops

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = torch.device("cuda:0")
    lib = _lib.kernels()

    def dev_t(a):
        return torch.from_numpy(np.ascontiguousarray(a)).to(dev)

    if args.gemm_probe:
        print(json.dumps(run_gemm_probe(torch, dev, datagen, ops)))
        return

    # ---- resident inputs ------------------------------------------------------------------------
    layers = []
    host_layer0 = []
    for layer in range(args.layers):
        shapes = []
        for (n, k) in DECODE_SHAPES:
            a, wq, s = datagen.w4a16_case(layer, 1, n, k)  # seed = layer index; layer 0 is "seed 0"
            if layer == 0:
                host_layer0.append((a, wq, s))
            shapes.append((dev_t(a), dev_t(wq), dev_t(s), torch.empty((1, n), dtype=torch.float16, device=dev)))
        layers.append(shapes)
    ws = torch.empty(1 << 20, dtype=torch.uint8, device=dev)

    def launch(shape_tensors):
        a, wq, s, y = shape_tensors
        n, k = wq.shape[0], a.shape[1]
        # the current stream: torch's capture stream while a graph is being recorded
        st = lib.nnf_w4a16_gemm(torch.cuda.current_stream().cuda_stream, a.data_ptr(), wq.data_ptr(), s.data_ptr(), y.data_ptr(),
                                1, n, k, GROUP, 8, ws.data_ptr(), ws.numel())
        if st != 0:
            raise RuntimeError(f"nnf_w4a16_gemm failed: {st} {lib.nnf_status_string(st).decode()}")

    def step(i):
        for sh in layers[i % args.layers]:
            launch(sh)

    def timed_graph(fn_list, reps):
        """Capture fn_list (callables that enqueue launches) into one graph; return mean microseconds of
        one replay over `reps` replays, measured with events on the launch stream."""
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for fn in fn_list:
                fn()
        g.replay()
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            g.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1000.0 / reps

    if args.mfma_probe:
        print(json.dumps(run_mfma_probe(torch, lib)))
        return

    if args.pmc_probe:
        # Calibration for FETCH_SIZE / WRITE_SIZE: a device-to-device copy that reads and writes exactly
        # PROBE_BYTES, larger than the last-level cache, followed by the sweep over every resident layer.
        src = torch.empty(PROBE_BYTES // 4, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        for _ in range(4):
            dst.copy_(src)
        torch.cuda.synchronize()
        for i in range(2 * args.layers):
            step(i)
        torch.cuda.synchronize()
        # the same weights with 16 activation rows (the row-streaming MFMA kernel; K = 11008: three ranges of K
        # and the reduction pass), over every resident layer
        ws16 = torch.empty(16 << 20, dtype=torch.uint8, device=dev)
        for shapes in layers:
            for (_, wq, s, _) in shapes:
                a16 = torch.empty((16, wq.shape[1] * 2), dtype=torch.float16, device=dev).normal_()
                ops.w4a16_gemm(a16, wq, s, workspace=ws16)
        torch.cuda.synchronize()
        print(f"pmc probe: copy of {PROBE_BYTES} bytes x4, then {2 * args.layers} sweeps, then {args.layers} sweeps with 16 rows", flush=True)
        return

    # ---- warm-up (untimed), then exactly K steps in the timed region ------------------------------
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for i in range(args.steps):
            step(i)
    g.replay()  # graph upload, untimed
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    g.replay()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1000.0
    ms_per_step = e0.elapsed_time(e1) / args.steps
    step_bytes = sum(w4a16_bytes(1, n, k) for (n, k) in DECODE_SHAPES)
    value = step_bytes / (ms_per_step * 1e-3) / 1e9

    # ---- per-shape launch durations -------------------------------------------------------------
    # Events around a graph of one shape walking enough copies of its weights (device-side clones of the
    # layers) that no launch finds them in the last-level cache, as in the timed region above.
    per_shape = []
    for si, (n, k) in enumerate(DECODE_SHAPES):
        n_copies = max(args.layers, -(-COLD_FOOTPRINT_BYTES // w4a16_bytes(1, n, k)))
        copies = []
        for c in range(n_copies):
            a, wq, s, y = layers[c % args.layers][si]
            copies.append((a, wq, s, y) if c < args.layers else (a, wq.clone(), s.clone(), y))
        fns = [(lambda t=t: launch(t)) for t in copies]
        us = timed_graph(fns, 4) / len(fns)
        del copies
        per_shape.append({"N": n, "K": k, "us": round(us, 3), "GB/s": round(w4a16_bytes(1, n, k) / us / 1e3, 1),
                          "frac_hbm": round(w4a16_bytes(1, n, k) / us / 1e3 / HBM_PEAK_GBS, 4)})
    if not args.no_extra:
        run_read_probe(torch, dev, lib, args.layers, per_shape, timed_graph)
    # dominant kernel: the K = 4096 instantiations of the row-streaming kernel serve three of the four launches
    k4096 = [p for p in per_shape if p["K"] == 4096]
    dom_us = sum(p["us"] for p in k4096) / len(k4096)
    dom_bytes = sum(w4a16_bytes(1, p["N"], p["K"]) for p in k4096) / len(k4096)
    roofline = {
        "bound": "hbm",
        "kernel": "nnf::w4a16_gemv_rows_kernel<2, D, 8> (K=4096: two KiB per row; mean over its three launches per step)",
        "achieved": round(dom_bytes / dom_us / 1e3, 1),
        "peak": HBM_PEAK_GBS,
        "unit": "GB/s",
        "frac": round(dom_bytes / dom_us / 1e3 / HBM_PEAK_GBS, 4),
        "traffic": ROWS_K4096_TRAFFIC_BYTES,
        "bytes_per_launch": int(dom_bytes),
        "us_per_launch": round(dom_us, 3),
    }

    extra = {}
    if not args.no_extra:
        extra = run_extra(torch, np, dev, lib, datagen, ops)

    cpu_baseline = None
    if not args.no_cpu_baseline:
        cpu_baseline = run_cpu_baseline(np, host_layer0, step_bytes)

    out = {
        "metric": "fp16xint4 g128 decode GEMV sweep, HBM GB/s (algorithmic bytes / time), M=1, 1 MI355X",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {
            "workload": "configs[1]: decode-shape sweep M=1, (N,K) in (12288,4096),(4096,4096),(22016,4096),"
                        "(4096,11008), fp16 x int4 g128 zp8",
            "layers_resident": args.layers,
            "bytes_per_step": step_bytes,
            "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
            "timed_region_wall_ms": round(wall_ms, 3),
        },
        "per_shape": per_shape,
        "roofline": roofline,
        "cpu_baseline": cpu_baseline,
        "extra": extra,
    }
    print(json.dumps(out))


def run_read_probe(torch, dev, lib, n_layers, per_shape, timed_graph):
    """What a launch costs that does nothing but read the same number of bytes once: plain 128-bit loads, one
    workgroup per CU, three depths of loads in flight (the best is kept as plain_read_us); the same bytes in the
    M <= 16 kernel's tile order; and in plain order but through LDS.  Timed exactly like the GEMV launches, over
    as many distinct buffers (nothing is found in the last-level cache)."""
    import ctypes

    fn = lib.nnf_internal_read_probe
    fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_longlong, ctypes.c_int, ctypes.c_int]
    fn.restype = ctypes.c_int
    num_cu = torch.cuda.get_device_properties(0).multi_processor_count
    for entry in per_shape:
        nbytes = (w4a16_bytes(1, entry["N"], entry["K"]) + 15) // 16 * 16
        n_bufs = max(n_layers, -(-COLD_FOOTPRINT_BYTES // nbytes))
        bufs = [torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device=dev) for _ in range(n_bufs)]
        best = None
        by_variant = []
        for variant in range(5):
            def make(buf, variant=variant):
                def call():
                    st = fn(torch.cuda.current_stream().cuda_stream, buf.data_ptr(), nbytes, variant, num_cu)
                    if st != 0:
                        raise RuntimeError(f"nnf_internal_read_probe failed: {st}")
                return call
            fns = [make(b) for b in bufs]
            fns[0]()
            torch.cuda.synchronize()
            us = timed_graph(fns, 4) / len(fns)
            if variant < 3:
                best = us if best is None else min(best, us)
            by_variant.append(round(us, 3))
        entry["plain_read_us"] = round(best, 3)
        entry["plain_read_us_32_64_128KiB_in_flight_per_cu"] = by_variant[:3]
        entry["read_us_in_tile_order"] = by_variant[3]
        entry["read_us_through_lds"] = by_variant[4]
        entry["gemv_time_over_plain_read"] = round(entry["us"] / best, 3)
        del bufs


def run_gemm_probe(torch, dev, datagen, ops, m=4096, n=8192, k=8192, launches=12):
    """The two compute-bound GEMMs of the extra configurations on their own (what a counter run looks at)."""
    ws = torch.empty(256 << 20, dtype=torch.uint8, device=dev)

    def timed(fn):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(launches):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1000.0 / launches

    a, wq, s = datagen.w4a16_case(0, m, n, k)
    ta, tw, ts = (torch.from_numpy(x).to(dev) for x in (a, wq, s))
    y = torch.empty((m, n), dtype=torch.float16, device=dev)
    us16 = timed(lambda: ops.w4a16_gemm(ta, tw, ts, out=y, workspace=ws))
    _, _, w8, s_ch = datagen.w8a8_case(0, 1, n, k)
    tw8, tsch = torch.from_numpy(w8).to(dev), torch.from_numpy(s_ch).to(dev)
    a8 = torch.from_numpy(datagen.uniform_i8(0, datagen.S_A8, (m, k))).to(dev)
    st = torch.from_numpy(datagen.uniform_f32(0, datagen.S_STOK, (m,), 0.001, 0.01)).to(dev)
    us8 = timed(lambda: ops.w8a8_gemm(a8, st, tw8, tsch, out=y, workspace=ws))
    ops_total = 2.0 * m * n * k
    return {"shape": [m, n, k], "launches": launches,
            "w4a16_us": round(us16, 1), "w4a16_tflops": round(ops_total / us16 / 1e6, 1),
            "w8a8_us": round(us8, 1), "w8a8_tops": round(ops_total / us8 / 1e6, 1)}


def run_mfma_probe(torch, lib):
    """MFMA-only loops (operands in registers, two wavefronts per SIMD, eight accumulators each): the rate the
    matrix cores sustain depends on the operand values, because the chip is power managed."""
    import ctypes

    fn = lib.nnf_internal_mfma_probe
    fn.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_double),
                   ctypes.POINTER(ctypes.c_double)]
    fn.restype = ctypes.c_int
    num_cu = torch.cuda.get_device_properties(0).multi_processor_count
    out = {"num_cu": num_cu, "unit": "Tera-op/s", "note": "published dense peaks: fp16 2500, int8 5000"}
    for kind, kname in ((0, "f16_32x32x16"), (1, "i8_32x32x32")):
        for mode, mname in ((0, "all_ones"), (1, "normal_or_uniform_random"), (2, "small_integers")):
            tops, mhz = ctypes.c_double(0.0), ctypes.c_double(0.0)
            st = fn(kind, mode, 60000, num_cu, ctypes.byref(tops), ctypes.byref(mhz))
            if st != 0:
                raise RuntimeError(f"nnf_internal_mfma_probe failed: {st}")
            out[f"{kname}.{mname}"] = {"tops": round(tops.value, 1), "shader_mhz": round(mhz.value)}
    return out


def run_extra(torch, np, dev, lib, datagen, ops):
    """The other benchmark configurations, a few iterations each (not part of `value`).  Rows with M <= 128 are
    memory-bound: they are timed over copies of the weights that miss the last-level cache."""

    def dev_t(a):
        return torch.from_numpy(np.ascontiguousarray(a)).to(dev)

    def time_us(fn, iters):
        for _ in range(10):
            fn()
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1000.0 / iters

    def time_cold_us(make_fn, weight_sets):
        """Launches walking device-side copies of the weights (more than the last-level cache holds), captured in
        one graph: for the rows whose time is a memory time."""
        fns = [make_fn(*w) for w in weight_sets]
        fns[0]()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for f in fns:
                f()
        # untimed replays first: after the host-side preparation of a row the first replays run 5-13 % slow
        for _ in range(6):
            g.replay()
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(6):
            g.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1000.0 / (6 * len(fns))

    def copies_of(*tensors):
        nbytes = sum(t.numel() * t.element_size() for t in tensors)
        return [tensors] + [tuple(t.clone() for t in tensors) for _ in range(-(-COLD_FOOTPRINT_BYTES // nbytes))]

    res = {}
    # configs[2]: fp16 x int4 GEMM, N = K = 8192
    n = k = 8192
    _, wq, s = datagen.w4a16_case(0, 1, n, k)
    twq, ts = dev_t(wq), dev_t(s)
    rows = []
    for m in (16, 128, 1024, 4096):
        a = dev_t(datagen.normal_f16(0, datagen.S_ACT, (m, k)))
        y = torch.empty((m, n), dtype=torch.float16, device=dev)
        ws = torch.empty(max(lib.nnf_w4a16_gemm_workspace_bytes(m, n, k, GROUP), 256), dtype=torch.uint8, device=dev)
        if m <= 128:
            sets = copies_of(twq, ts)
            us = time_cold_us(lambda w, sc: (lambda: ops.w4a16_gemm(a, w, sc, out=y, workspace=ws)), sets)
            del sets
        else:
            us = time_us(lambda: ops.w4a16_gemm(a, twq, ts, out=y, workspace=ws), 20)
        fl = 2.0 * m * n * k
        rows.append({"M": m, "us": round(us, 2), "TFLOP/s": round(fl / us / 1e6, 1),
                     "frac_mfma_f16": round(fl / us / 1e6 / MFMA_F16_PEAK_TFLOPS, 4),
                     "GB/s": round(w4a16_bytes(m, n, k) / us / 1e3, 1)})
    res["w4a16_gemm_N8192_K8192"] = rows
    del twq, ts
    # the decode sweep's shapes with a handful of rows (batched decode; not one of the benchmark's configurations):
    # cold weights, the time of the whole sweep per batch size
    rows = []
    shapes = [(12288, 4096), (4096, 4096), (22016, 4096), (4096, 11008)]
    weights = []
    for (sn, sk) in shapes:
        _, wq, s = datagen.w4a16_case(0, 1, sn, sk)
        weights.append((dev_t(wq), dev_t(s)))
    for m in (2, 4, 8, 16):
        total_us, total_bytes = 0.0, 0
        for (sn, sk), (twq, ts) in zip(shapes, weights):
            a = dev_t(datagen.normal_f16(0, datagen.S_ACT, (m, sk)))
            y = torch.empty((m, sn), dtype=torch.float16, device=dev)
            ws = torch.empty(max(lib.nnf_w4a16_gemm_workspace_bytes(m, sn, sk, GROUP), 256), dtype=torch.uint8, device=dev)
            sets = copies_of(twq, ts)
            total_us += time_cold_us(lambda w, sc: (lambda: ops.w4a16_gemm(a, w, sc, out=y, workspace=ws)), sets)
            total_bytes += w4a16_bytes(m, sn, sk)
            del sets
        rows.append({"M": m, "us_per_sweep": round(total_us, 2), "GB/s": round(total_bytes / total_us / 1e3, 1)})
    res["w4a16_decode_sweep_small_batches"] = rows
    del weights
    # configs[3]: W8A8, N = K = 8192
    _, _, w8, s_ch = datagen.w8a8_case(0, 1, n, k)
    tw8, tsch = dev_t(w8), dev_t(s_ch)
    rows = []
    for m in (1, 32, 512, 4096):
        a8 = dev_t(datagen.uniform_i8(0, datagen.S_A8, (m, k)))
        st = dev_t(datagen.uniform_f32(0, datagen.S_STOK, (m,), 0.001, 0.01))
        y = torch.empty((m, n), dtype=torch.float16, device=dev)
        ws = torch.empty(max(lib.nnf_w8a8_gemm_workspace_bytes(m, n, k), 256), dtype=torch.uint8, device=dev)
        if m <= 128:
            sets = copies_of(tw8)
            us = time_cold_us(lambda w: (lambda: ops.w8a8_gemm(a8, st, w, tsch, out=y, workspace=ws)), sets)
            del sets
        else:
            us = time_us(lambda: ops.w8a8_gemm(a8, st, tw8, tsch, out=y, workspace=ws), 20)
        op = 2.0 * m * n * k
        rows.append({"M": m, "us": round(us, 2), "TOP/s": round(op / us / 1e6, 1),
                     "frac_mfma_i8": round(op / us / 1e6 / MFMA_I8_PEAK_TOPS, 4),
                     "GB/s": round(w8a8_bytes(m, n, k) / us / 1e3, 1)})
    res["w8a8_gemm_N8192_K8192"] = rows
    del tw8, tsch
    # configs[4]: fused MLP block, M = 256
    m, h, i = 256, 4096, 11008
    tens = [dev_t(t) for t in datagen.mlp_case(0, m, h, i)]
    out = torch.empty((m, h), dtype=torch.float16, device=dev)
    wsz = lib.nnf_fused_mlp_w4a16_workspace_bytes(m, h, i, GROUP)
    wsm = torch.empty(wsz, dtype=torch.uint8, device=dev)
    us = time_us(lambda: ops.fused_mlp_w4a16(*tens, out=out, workspace=wsm), 20)
    fl = 2.0 * m * (2 * i) * h + 2.0 * m * h * i
    res["fused_mlp_M256_4096_11008"] = {"us": round(us, 2), "TFLOP/s": round(fl / us / 1e6, 1),
                                        "frac_mfma_f16": round(fl / us / 1e6 / MFMA_F16_PEAK_TFLOPS, 4)}
    del tens, out, wsm
    # For scale only: the vendor library's unquantized GEMMs on the same box and value distributions (fp16 weights,
    # four times the bytes, no unpacking; int8 x int8 -> int32 without the scaling epilogue), M = 4096, N = K = 8192.
    try:
        m, n, k = 4096, 8192, 8192
        a = torch.randn(m, k, device=dev, dtype=torch.float16)
        w = torch.randn(n, k, device=dev, dtype=torch.float16)
        y = torch.empty(m, n, device=dev, dtype=torch.float16)
        us16 = time_us(lambda: torch.matmul(a, w.t(), out=y), 20)
        a8 = torch.randint(-127, 128, (m, k), device=dev, dtype=torch.int8)
        w8 = torch.randint(-127, 128, (n, k), device=dev, dtype=torch.int8)
        us8 = time_us(lambda: torch._int_mm(a8, w8.t()), 20)
        res["vendor_library_for_scale_M4096"] = {"fp16_matmul_us": round(us16, 1), "fp16_TFLOP/s": round(2.0 * m * n * k / us16 / 1e6, 1),
                                                 "int8_mm_us": round(us8, 1), "int8_TOP/s": round(2.0 * m * n * k / us8 / 1e6, 1)}
    except Exception as e:  # a yardstick, not part of the benchmark
        res["vendor_library_for_scale_M4096"] = {"error": str(e)[:200]}
    return res


def run_cpu_baseline(np, host_layer0, step_bytes):
    """The reference's CPU path for the same sweep, on this host's cores: fp32 GEMM on weights
    dequantised once beforehand (constants are folded at init in the reference), 5 warm-ups + 100
    timed calls per shape (the loop of the generated CPU main_test)."""
    import oracle

    use_ref = oracle.mlas_ref() is not None
    total_ms = 0.0
    detail = []
    for (a, wq, s) in host_layer0:
        wd = oracle.dequantize_w4(wq, s)
        a32 = oracle.f16_to_f32(a)
        if use_ref:
            mean_ms, min_ms = oracle.mlas_time_sgemm_nt(a32, wd, warmup=5, iters=100)
        else:
            mean_ms, min_ms = oracle.time_dot_f32(a32, wd, warmup=5, iters=100, threads=16)
        total_ms += mean_ms
        detail.append({"N": int(wq.shape[0]), "K": int(a.shape[1]), "mean_ms": round(mean_ms, 4),
                       "min_ms": round(min_ms, 4)})
        del wd
    cores = os.cpu_count() or 1
    threads = min(16, cores)  # MLAS caps its own partitioning at 16 threads
    return {
        "value": round(step_bytes / (total_ms * 1e-3) / 1e9, 3),
        "unit": "GB/s",
        "cores": threads,
        "kind": "reference" if use_ref else "port",
        "sample": "the whole sweep (4 shapes, layer 0): 5 warm-up + 100 timed fp32 GEMM calls per shape on "
                  "weights dequantised once (untimed); value = int4-path algorithmic bytes / summed mean time",
        "ms_per_step": round(total_ms, 4),
        "host_cpus": cores,
        "per_shape": detail,
    }


if __name__ == "__main__":
    main()
