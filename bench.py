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

Before anything is timed, every configuration that will be timed is run once and compared with the CPU
oracle (the sweep on whole outputs; the large configurations on sampled output columns / token rows);
a mismatch aborts the run with a non-zero exit status and no JSON line.

Prints ONE JSON line.  `value` = algorithmic bytes of a step (every operand read once, output written
once) / time per step.  `roofline` covers the kernel that dominates the step; `roofline_extra` holds the
same figures for every other configuration (prefill GEMM, batched decode, W8A8, fused MLP), each
measured for a few iterations (`extra` has their plain timings); `traffic` fields are HBM bytes per launch
from hardware-counter runs, read from the summaries under profiles/ (null where none is recorded).
`cpu_baseline` times the sweep on the host cores with the reference's CPU GEMM (MLAS built from the
reference tree, or the oracle's own port when that library is absent) on fp32 weights dequantised
beforehand.
"""
import argparse
import ctypes
import glob
import json
import os
import sys
import time
import warnings

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

COLD_FOOTPRINT_BYTES = 600 * 1000 * 1000  # buffers walked by a timing loop: more than the last-level cache holds
HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
MFMA_F16_PEAK_TFLOPS = 2500.0  # dense fp16 MFMA
MFMA_I8_PEAK_TOPS = 5000.0     # dense int8 MFMA

DECODE_SHAPES = [(12288, 4096), (4096, 4096), (22016, 4096), (4096, 11008)]  # (N, K), M = 1
GROUP = 128
PROBE_BYTES = 1 << 30  # size of the calibration copy of --pmc-probe and of the large plain read
W4A16_TOL = 1e-2       # max |y - y_ref| <= W4A16_TOL * RMS(y_ref): the tolerance of the fp16 x int4 path
PROBES_SO = os.path.join(ROOT, "nnfusion_amd", "lib", "libnnf_bench_probes.so")
PROFILES_DIR = os.path.join(ROOT, "profiles")

GEMM_NK = 8192
GEMM_MS = (16, 128, 1024, 4096)       # configs[2]
W8A8_MS = (1, 32, 512, 4096)          # configs[3]
SMALL_BATCHES = (2, 4, 8, 16)         # the sweep's shapes with a few rows
# the fp16 x int-N product with other block parameters (bits, group, zero point per (row, group)?) than the benchmark's,
# on the two plain kernels that serve them, at N = K = GEMM_NK
WNA16_CASES = ((8, 128, False), (4, 64, True))
WNA16_MS = (1, 16, 4096)
MLP_HI = (4096, 11008)                # configs[4]: hidden and intermediate size
MLP_MS = (1, 16, 256)                 # ... at M = 256; the same block at decode sizes beside it

def load_row_kernels():
    """The kernels each configuration row launches, as a kernel trace of `bench.py --pmc-probe` shows them: the last
    column of the rows of profiles/bench_configurations_hbm_traffic.txt (`<row key> <five numbers>  <kernels>`)."""
    out = {}
    path = os.path.join(PROFILES_DIR, "bench_configurations_hbm_traffic.txt")
    if not os.path.exists(path):
        return out
    with open(path) as f:
        for line in f:
            parts = line.split(None, 6)
            if len(parts) == 7 and parts[0] != "row":
                try:
                    [float(x) for x in parts[1:6]]
                except ValueError:
                    continue
                out[parts[0]] = parts[6].strip()
    return out


def wna16_key(bits, group, zp_tensor, n, k, m):
    return f"wna16_b{bits}_g{group}_{'zp_tensor' if zp_tensor else 'zp_scalar'}_N{n}_K{k}.M{m}"


def w4a16_bytes(m, n, k):
    """Algorithmic bytes: int4 weights + fp16 group scales + fp16 activations + fp16 output."""
    return n * k // 2 + n * (k // GROUP) * 2 + m * k * 2 + m * n * 2


def wna16_bytes(m, n, k, bits, group, zp_tensor):
    """Weights of `bits` bits + fp16 scales (+ one zero point of `bits` bits) per group + fp16 activations and output."""
    g = k // group
    return n * k * bits // 8 + n * g * 2 + (n * ((g * bits + 7) // 8) if zp_tensor else 0) + m * k * 2 + m * n * 2


def w8a8_bytes(m, n, k):
    return n * k + n * 4 + m * k + m * 4 + m * n * 2


def mlp_bytes(m, h, i):
    """x, gamma, both weight matrices with scales, h written and read once (it is a tensor of the block), out."""
    return m * h * 2 + h * 2 + (2 * i * h // 2 + 2 * i * (h // GROUP) * 2) + (h * i // 2 + h * (i // GROUP) * 2) + \
        2 * m * i * 2 + m * h * 2


def load_traffic():
    """`traffic_bytes_per_launch <row key> <bytes>` lines of the hardware-counter summaries under profiles/."""
    out = {}
    for path in sorted(glob.glob(os.path.join(PROFILES_DIR, "*.txt"))):
        with open(path) as f:
            for line in f:
                parts = line.split()
                if len(parts) == 3 and parts[0] == "traffic_bytes_per_launch":
                    try:
                        out[parts[1]] = int(parts[2])
                    except ValueError:
                        pass
    return out


def load_probes():
    if not os.path.exists(PROBES_SO):
        sys.exit(f"bench.py: {PROBES_SO} is not built (make -C nnfusion_amd/csrc)")
    lib = ctypes.CDLL(PROBES_SO)
    lib.nnf_probe_read.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_longlong, ctypes.c_int, ctypes.c_int]
    lib.nnf_probe_read.restype = ctypes.c_int
    lib.nnf_probe_mfma.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_double),
                                   ctypes.POINTER(ctypes.c_double)]
    lib.nnf_probe_mfma.restype = ctypes.c_int
    vp, ci = ctypes.c_void_p, ctypes.c_int
    lib.nnf_probe_gemv_timeline.argtypes = [vp] * 5 + [ci, ci, vp, ci]
    lib.nnf_probe_gemv_timeline.restype = ci
    lib.nnf_probe_gemm_timeline.argtypes = [vp] * 5 + [ci] * 4 + [vp, ctypes.c_size_t, vp, ctypes.c_size_t, vp, ci]
    lib.nnf_probe_gemm_timeline.restype = ci
    return lib


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1200)
    ap.add_argument("--warmup", type=int, default=24)
    ap.add_argument("--layers", type=int, default=6, help="independent weight sets walked by the steps")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true")
    ap.add_argument("--pmc-probe", action="store_true",
                    help="for hardware-counter runs: a plain copy of known size, then every configuration launched "
                         "eagerly, a marker launch ahead of each; prints the order of the rows, no timing")
    ap.add_argument("--mfma-probe", action="store_true",
                    help="print the MFMA-only rates (no memory traffic) for different operand values and exit")
    ap.add_argument("--gemm-probe", action="store_true",
                    help="for hardware-counter runs: the fp16 x int4 and the W8A8 GEMM at M=4096, N=K=8192, twelve "
                         "launches each; prints their event-timed means, no JSON line of the benchmark")
    ap.add_argument("--timeline", action="store_true",
                    help="time stamps from inside the kernels (the probe library's builds of the single-row GEMV and of "
                         "the tile GEMM in its one-launch form): prints a table per shape, no JSON line of the benchmark")
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
    env = Env(torch, np, dev, lib, datagen, ops)

    if args.gemm_probe:
        print(json.dumps(run_gemm_probe(env)))
        return
    if args.mfma_probe:
        print(json.dumps(run_mfma_probe(env, load_probes())))
        return
    if args.timeline:
        run_timeline(env, load_probes())
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
            shapes.append((env.dev_t(a), env.dev_t(wq), env.dev_t(s), torch.empty((1, n), dtype=torch.float16, device=dev)))
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

    if args.pmc_probe:
        run_pmc_probe(env, load_probes(), layers, step, args.layers)
        return

    # ---- parity gate: nothing is timed unless the results are the oracle's ----------------------------
    import oracle

    parity = {}
    step(0)
    torch.cuda.synchronize()
    for (a, wq, s), (_, _, _, y) in zip(host_layer0, layers[0]):
        ref = oracle.w4a16_gemm(a, wq, s, f32_out=True)
        check_w4a16(np, parity, f"decode_sweep.N{wq.shape[0]}_K{a.shape[1]}", y.cpu().numpy(), ref)
    if not args.no_extra:
        parity_extra(env, oracle, parity)

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
    traffic = load_traffic()
    per_shape = []
    for si, (n, k) in enumerate(DECODE_SHAPES):
        n_copies = max(args.layers, -(-COLD_FOOTPRINT_BYTES // w4a16_bytes(1, n, k)))
        copies = []
        for c in range(n_copies):
            a, wq, s, y = layers[c % args.layers][si]
            copies.append((a, wq, s, y) if c < args.layers else (a, wq.clone(), s.clone(), y))
        fns = [(lambda t=t: launch(t)) for t in copies]
        us = env.timed_graph(fns, 4) / len(fns)
        del copies
        per_shape.append({"N": n, "K": k, "us": round(us, 3), "GB/s": round(w4a16_bytes(1, n, k) / us / 1e3, 1),
                          "frac_hbm": round(w4a16_bytes(1, n, k) / us / 1e3 / HBM_PEAK_GBS, 4),
                          "traffic": traffic.get(f"decode_sweep.N{n}_K{k}")})
    plain_read = None
    if not args.no_extra:
        probes = load_probes()
        run_read_probe(env, probes, args.layers, per_shape)
        plain_read = run_large_read_probe(env, probes)
    # dominant kernel: the K = 4096 instantiations of the row-streaming kernel serve three of the four launches
    k4096 = [p for p in per_shape if p["K"] == 4096]
    dom_us = sum(p["us"] for p in k4096) / len(k4096)
    dom_bytes = sum(w4a16_bytes(1, p["N"], p["K"]) for p in k4096) / len(k4096)
    dom_traffic = [p["traffic"] for p in k4096]
    roofline = {
        "bound": "hbm",
        # (as the kernel trace behind profiles/bench_configurations_hbm_traffic.txt names it)
        "kernel": " | ".join(sorted({load_row_kernels().get(f"decode_sweep.N{p['N']}_K{p['K']}", "?") for p in k4096})) +
                  " (the K=4096 launches: two KiB per weight row; mean over the three of them in a step)",
        "achieved": round(dom_bytes / dom_us / 1e3, 1),
        "peak": HBM_PEAK_GBS,
        "unit": "GB/s",
        "frac": round(dom_bytes / dom_us / 1e3 / HBM_PEAK_GBS, 4),
        "traffic": None if any(t is None for t in dom_traffic) else int(sum(dom_traffic) / len(dom_traffic)),
        "bytes_per_launch": int(dom_bytes),
        "us_per_launch": round(dom_us, 3),
    }
    if plain_read is not None:
        roofline["frac_of_plain_read_1GiB"] = round(dom_bytes / dom_us / 1e3 / plain_read, 4)

    extra, roofline_extra = {}, []
    if not args.no_extra:
        extra, roofline_extra = run_extra(env, traffic)

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
        "parity": parity,
        "plain_read_1GiB_GB/s": plain_read,
        "per_shape": per_shape,
        "roofline": roofline,
        "roofline_extra": roofline_extra,
        "cpu_baseline": cpu_baseline,
        "extra": extra,
    }
    print(json.dumps(out))


class Env:
    """What the measuring functions share: modules, the device, the library and the timers."""

    def __init__(self, torch, np, dev, lib, datagen, ops):
        self.torch, self.np, self.dev, self.lib, self.datagen, self.ops = torch, np, dev, lib, datagen, ops
        # nnf_plan::sync_flags: cleared once here, left clear by every call; what an emitted function's persistent,
        # zero-initialised tensor is.  With it the tile GEMM adds up the tiles its workgroups share inside its one launch.
        self.sync = ops.sync_flags(dev)

    def dev_t(self, a):
        return self.torch.from_numpy(self.np.ascontiguousarray(a)).to(self.dev)

    def timed_graph(self, fn_list, reps):
        """Capture fn_list (callables that enqueue launches) into one graph; return mean microseconds of
        one replay over `reps` replays, measured with events on the launch stream."""
        torch = self.torch
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

    def time_us(self, fn, iters):
        """Mean microseconds per call in a sustained run: the compute-bound rows run 10-15 % slower for the first tens of
        milliseconds after the chip has been idle (vendor library included), so about 40 ms of untimed calls go ahead
        of at least `iters` timed ones (at least 20 ms of them)."""
        torch = self.torch

        def run(n):
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(n):
                fn()
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) * 1000.0 / n

        first = run(5)
        run(max(5, min(2000, int(40e3 / max(first, 1.0)))))
        return run(max(iters, min(2000, int(20e3 / max(first, 1.0)))))

    def time_span_us(self, fn, span_us):
        """Mean microseconds per call over about `span_us` of back-to-back calls (no warm-up of its own)."""
        torch = self.torch
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        torch.cuda.synchronize()
        n = max(3, min(2000, int(span_us / max(e0.elapsed_time(e1) * 1000.0, 1.0))))
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1000.0 / n

    def time_cold_us(self, make_fn, weight_sets):
        """Launches walking device-side copies of the weights (more than the last-level cache holds), captured in
        one graph: for the rows whose time is a memory time."""
        torch = self.torch
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

    def copies_of(self, *tensors):
        nbytes = sum(t.numel() * t.element_size() for t in tensors)
        return [tensors] + [tuple(t.clone() for t in tensors) for _ in range(-(-COLD_FOOTPRINT_BYTES // nbytes))]

    def workspace(self, nbytes):
        return self.torch.empty(max(int(nbytes), 256), dtype=self.torch.uint8, device=self.dev)


# ---- parity gate ----------------------------------------------------------------------------------------
def parity_fail(name, detail):
    sys.stderr.write(f"bench.py: PARITY FAILURE in {name}: {detail}; nothing was timed\n")
    sys.exit(1)


def check_w4a16(np, parity, name, y, ref, tol=W4A16_TOL):
    rms = float(np.sqrt(np.mean(ref.astype(np.float64) ** 2)))
    err = float(np.abs(y.astype(np.float32) - ref.astype(np.float32)).max())
    if not (err <= tol * max(rms, 1e-6)):
        parity_fail(name, f"max |y - oracle| = {err:.4g} > {tol} x RMS(oracle) = {tol * rms:.4g}")
    parity[name] = {"max_err_over_rms": round(err / max(rms, 1e-30), 6), "tol": tol}


def parity_extra(env, oracle, parity):
    """The configurations of run_extra, each run once and compared with the oracle: the GEMMs on sampled output
    columns (the oracle computes those columns from the same weight rows), W8A8 bit for bit, the MLP block on its
    first token rows (rows are independent)."""
    np, torch, ops, datagen = env.np, env.torch, env.ops, env.datagen
    n = k = GEMM_NK
    rng = np.random.default_rng(0)
    cols = np.sort(rng.choice(n, 96, replace=False))
    _, wq, s = datagen.w4a16_case(0, 1, n, k)
    twq, ts = env.dev_t(wq), env.dev_t(s)
    for m in GEMM_MS:
        a = datagen.normal_f16(0, datagen.S_ACT, (m, k))
        y = ops.w4a16_gemm_variant(env.dev_t(a), twq, ts, "auto", sync=env.sync)
        torch.cuda.synchronize()
        ref = oracle.w4a16_gemm(a, wq[cols], s[cols], f32_out=True)
        check_w4a16(np, parity, f"w4a16_gemm_N{n}_K{k}.M{m}", y.cpu().numpy()[:, cols], ref)
    del twq, ts
    for (sn, sk) in DECODE_SHAPES:
        _, wq, s = datagen.w4a16_case(0, 1, sn, sk)
        twq, ts = env.dev_t(wq), env.dev_t(s)
        scols = np.sort(rng.choice(sn, 96, replace=False))
        for m in SMALL_BATCHES:
            a = datagen.normal_f16(0, datagen.S_ACT, (m, sk))
            y = ops.w4a16_gemm(env.dev_t(a), twq, ts)
            torch.cuda.synchronize()
            ref = oracle.w4a16_gemm(a, wq[scols], s[scols], f32_out=True)
            check_w4a16(np, parity, f"decode_sweep_M{m}.N{sn}_K{sk}", y.cpu().numpy()[:, scols], ref)
        del twq, ts
    _, _, w8, s_ch = datagen.w8a8_case(0, 1, n, k)
    tw8, tsch = env.dev_t(w8), env.dev_t(s_ch)
    cols8 = np.sort(rng.choice(n, 64, replace=False))
    for m in W8A8_MS:
        a8 = datagen.uniform_i8(0, datagen.S_A8, (m, k))
        st = datagen.uniform_f32(0, datagen.S_STOK, (m,), 0.001, 0.01)
        y = ops.w8a8_gemm(env.dev_t(a8), env.dev_t(st), tw8, tsch)
        torch.cuda.synchronize()
        acc = oracle.w8a8_acc(a8, w8[cols8])
        ref = oracle.w8a8_epilogue(acc, st, s_ch[cols8])
        name = f"w8a8_gemm_N{n}_K{k}.M{m}"
        if not np.array_equal(y.cpu().numpy()[:, cols8].view(np.uint16), ref.view(np.uint16)):
            parity_fail(name, "fp16 outputs differ from the oracle's (the bar is bit-exact)")
        parity[name] = {"bit_exact_columns": int(len(cols8))}
    del tw8, tsch
    for bits, group, zpt in WNA16_CASES:
        _, wq, s, z = datagen.wna16_case(0, 1, n, k, bits, group, zpt)
        tw, tsc, tz = env.dev_t(wq), env.dev_t(s), (env.dev_t(z) if zpt else None)
        for m in WNA16_MS:
            a = datagen.normal_f16(0, datagen.S_ACT, (m, k))
            y = ops.wna16_gemm(env.dev_t(a), tw, tsc, bits=bits, group=group, zp=1 << (bits - 1), zero_points=tz)
            torch.cuda.synchronize()
            ref = oracle.wna16_gemm(a, wq[cols], s[cols], bits, group, zp=1 << (bits - 1),
                                    zero_points=None if z is None else z[cols], f32_out=True)
            check_w4a16(np, parity, wna16_key(bits, group, zpt, n, k, m), y.cpu().numpy()[:, cols], ref)
        del tw, tsc, tz
    h, i = MLP_HI
    for m in MLP_MS:
        x, gamma, wgu, sgu, wd, sd = datagen.mlp_case(0, m, h, i)
        out = ops.fused_mlp_w4a16(*[env.dev_t(t) for t in (x, gamma, wgu, sgu, wd, sd)], sync=env.sync)
        torch.cuda.synchronize()
        rows = min(m, 8)
        ref = oracle.fused_mlp_w4a16(x[:rows].copy(), gamma, wgu, sgu, wd, sd)
        check_w4a16(np, parity, f"fused_mlp_M{m}_{h}_{i}.rows0-{rows - 1}", out.cpu().numpy()[:rows], ref)


# ---- probes ---------------------------------------------------------------------------------------------
def run_read_probe(env, probes, n_layers, per_shape):
    """What a launch costs that does nothing but read the same number of bytes once: plain 128-bit loads, one
    workgroup per CU, three depths of loads in flight (the best is kept as plain_read_us); the same bytes in the
    M <= 16 kernel's tile order; and in plain order but through LDS.  Timed exactly like the GEMV launches, over
    as many distinct buffers (nothing is found in the last-level cache)."""
    torch = env.torch
    fn = probes.nnf_probe_read
    num_cu = torch.cuda.get_device_properties(0).multi_processor_count
    for entry in per_shape:
        nbytes = (w4a16_bytes(1, entry["N"], entry["K"]) + 15) // 16 * 16
        n_bufs = max(n_layers, -(-COLD_FOOTPRINT_BYTES // nbytes))
        bufs = [torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device=env.dev) for _ in range(n_bufs)]
        best = None
        by_variant = []
        for variant in range(5):
            def make(buf, variant=variant):
                def call():
                    st = fn(torch.cuda.current_stream().cuda_stream, buf.data_ptr(), nbytes, variant, num_cu)
                    if st != 0:
                        raise RuntimeError(f"nnf_probe_read failed: {st}")
                return call
            fns = [make(b) for b in bufs]
            fns[0]()
            torch.cuda.synchronize()
            us = env.timed_graph(fns, 4) / len(fns)
            if variant < 3:
                best = us if best is None else min(best, us)
            by_variant.append(round(us, 3))
        entry["plain_read_us"] = round(best, 3)
        entry["plain_read_us_32_64_128KiB_in_flight_per_cu"] = by_variant[:3]
        entry["read_us_in_tile_order"] = by_variant[3]
        entry["read_us_through_lds"] = by_variant[4]
        entry["gemv_time_over_plain_read"] = round(entry["us"] / best, 3)
        del bufs


def run_large_read_probe(env, probes):
    """GB/s of one launch that reads 1 GiB once with plain 128-bit loads (the best of the three depths of loads in
    flight): the rate this box's HBM gives a kernel that does nothing else, next to the published 8 TB/s."""
    torch = env.torch
    fn = probes.nnf_probe_read
    num_cu = torch.cuda.get_device_properties(0).multi_processor_count
    buf = torch.randint(0, 255, (PROBE_BYTES,), dtype=torch.uint8, device=env.dev)
    best = None
    for variant in range(3):
        def call(variant=variant):
            st = fn(torch.cuda.current_stream().cuda_stream, buf.data_ptr(), PROBE_BYTES, variant, num_cu)
            if st != 0:
                raise RuntimeError(f"nnf_probe_read failed: {st}")
        us = env.time_us(call, 10)
        best = us if best is None else min(best, us)
    del buf
    return round(PROBE_BYTES / best / 1e3, 1)


def run_gemm_probe(env, m=4096, n=8192, k=8192, launches=12):
    """The two compute-bound GEMMs of the extra configurations on their own (what a counter run looks at)."""
    torch, datagen, ops, dev = env.torch, env.datagen, env.ops, env.dev
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


def run_timeline(env, probes):
    """Where a launch spends its time, from stamps of the 100 MHz clock taken inside the kernels (the probe library compiles
    the product's kernel bodies once more with the stamps).  Every launch reads weights that no cache holds (copies walked
    in turn), alone on the device; per stamp: the earliest, the mean and the latest workgroup, in us since the first
    workgroup of the launch started, means over ten launches."""
    torch, np, datagen, dev = env.torch, env.np, env.datagen, env.dev
    stream = torch.cuda.current_stream().cuda_stream
    num_cu = torch.cuda.get_device_properties(dev).multi_processor_count

    def table(title, names, launch, per_wg, n_copies):
        trace = torch.zeros(1024 * per_wg, dtype=torch.int64, device=dev)
        rows, spans = [], []
        for it in range(12):
            trace.zero_()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            grid = launch(it % n_copies, trace)
            e1.record()
            torch.cuda.synchronize()
            if grid <= 0:
                sys.exit(f"bench.py: the timeline probe does not cover {title}")
            if it < 2:
                continue
            tr = trace.cpu().numpy().reshape(-1, per_wg)[:grid].astype(np.float64)
            rel = (tr - tr[:, 0].min()) / 100.0
            rel[tr == 0] = np.nan
            rows.append(rel)
            spans.append(e0.elapsed_time(e1) * 1e3)
        with np.errstate(all="ignore"), warnings.catch_warnings():
            warnings.simplefilter("ignore", RuntimeWarning)  # (stamps that a kernel does not take: columns of NaN)
            rel = np.nanmean(np.stack(rows), axis=0)
        print(f"{title}: grid {grid}; events around the launch (eager, launch overhead included): {sum(spans) / len(spans):.1f} us")
        print(f"    {'stamp':<58} {'first':>8} {'mean':>8} {'last':>8}")
        for i, name in names:
            col = rel[:, i]
            if not np.all(np.isnan(col)):
                print(f"    {name:<58} {np.nanmin(col):>8.2f} {np.nanmean(col):>8.2f} {np.nanmax(col):>8.2f}")
        print()

    gemv_names = [(0, "workgroup starts"), (1, "activations and scales arrived (first wavefront)"),
                  (2, "activations prepared by every wavefront"), (3, "first row's weights arrived"),
                  (4, "first wavefront's last row added up"), (5, "every wavefront's last row added up"), (7, "outputs written, end")]
    for (n, k) in DECODE_SHAPES:
        a, wq, s = datagen.w4a16_case(0, 1, n, k)
        ta = env.dev_t(a)
        copies = [(env.dev_t(wq), env.dev_t(s)) for _ in range(max(2, -(-COLD_FOOTPRINT_BYTES // wq.nbytes)))]
        y = torch.empty((1, n), dtype=torch.float16, device=dev)
        us = w4a16_bytes(1, n, k) / 8e3 / 1e3

        def launch(c, trace, ta=ta, copies=copies, y=y, n=n, k=k):
            return probes.nnf_probe_gemv_timeline(stream, ta.data_ptr(), copies[c][0].data_ptr(), copies[c][1].data_ptr(), y.data_ptr(),
                                                  n, k, trace.data_ptr(), num_cu)

        table(f"single-row GEMV N={n} K={k} ({w4a16_bytes(1, n, k)} bytes: {us:.2f} us at 8 TB/s)", gemv_names, launch, 8, len(copies))
        del copies

    gemm_names = [(0, "workgroup starts"), (1, "first operands arrived"), (10, "(two segments) K loop of the first over"),
                  (11, "(two segments) its part parked and counted in"), (12, "(two segments) first operands of the last arrived"),
                  (2, "K loop of its last segment over"), (3, "its part parked"),
                  (4, "... and counted in"), (5, "waits for the other workgroups of its shared tiles over"),
                  (6, "its share of those tiles finished"), (9, "end")]
    ws = env.workspace(256 << 20)
    for (m, n, k, cols) in ((128, 8192, 8192, 128), (256, 2 * MLP_HI[1], MLP_HI[0], 256), (256, MLP_HI[0], MLP_HI[1], 128)):
        if k % 256:
            continue
        _, wq, s = datagen.w4a16_case(0, 1, n, k)
        ta = env.dev_t(datagen.normal_f16(0, datagen.S_ACT, (m, k)))
        copies = [(env.dev_t(wq), env.dev_t(s)) for _ in range(max(2, -(-COLD_FOOTPRINT_BYTES // wq.nbytes)))]
        y = torch.empty((m, n), dtype=torch.float16, device=dev)

        def launch(c, trace, ta=ta, copies=copies, y=y, m=m, n=n, k=k, cols=cols):
            return probes.nnf_probe_gemm_timeline(stream, ta.data_ptr(), copies[c][0].data_ptr(), copies[c][1].data_ptr(), y.data_ptr(),
                                                  m, n, k, cols, ws.data_ptr(), ws.numel(), env.sync.data_ptr(), env.sync.numel(),
                                                  trace.data_ptr(), num_cu)

        table(f"tile GEMM (one launch, 128 x {cols} tiles) M={m} N={n} K={k}", gemm_names, launch, 16, len(copies))
        del copies


def run_mfma_probe(env, probes):
    """MFMA-only loops (operands in registers, two wavefronts per SIMD, eight accumulators each): the rate the
    matrix cores sustain depends on the operand values, because the chip is power managed."""
    fn = probes.nnf_probe_mfma
    num_cu = env.torch.cuda.get_device_properties(0).multi_processor_count
    out = {"num_cu": num_cu, "unit": "Tera-op/s", "note": "published dense peaks: fp16 2500, int8 5000"}
    for kind, kname in ((0, "f16_32x32x16"), (1, "i8_32x32x32")):
        for mode, mname in ((0, "all_ones"), (1, "normal_or_uniform_random"), (2, "small_integers")):
            tops, mhz = ctypes.c_double(0.0), ctypes.c_double(0.0)
            st = fn(kind, mode, 60000, num_cu, ctypes.byref(tops), ctypes.byref(mhz))
            if st != 0:
                raise RuntimeError(f"nnf_probe_mfma failed: {st}")
            out[f"{kname}.{mname}"] = {"tops": round(tops.value, 1), "shader_mhz": round(mhz.value)}
    return out


def extra_rows(env):
    """The configurations beside the sweep as (row key, algorithmic bytes, operations, callable factory, weight
    tensors): the factory takes (copies of) the weights and returns the callable that enqueues the row once."""
    torch, datagen, ops, lib, dev = env.torch, env.datagen, env.ops, env.lib, env.dev
    n = k = GEMM_NK
    rows = []
    _, wq, s = datagen.w4a16_case(0, 1, n, k)
    twq, ts = env.dev_t(wq), env.dev_t(s)
    for m in GEMM_MS:
        a = env.dev_t(datagen.normal_f16(0, datagen.S_ACT, (m, k)))
        y = torch.empty((m, n), dtype=torch.float16, device=dev)
        ws = env.workspace(lib.nnf_w4a16_gemm_workspace_bytes(m, n, k, GROUP))
        rows.append({"key": f"w4a16_gemm_N{n}_K{k}.M{m}", "group": f"w4a16_gemm_N{n}_K{k}", "M": m,
                     "bytes": w4a16_bytes(m, n, k), "ops": 2.0 * m * n * k, "int8": False, "weights": (twq, ts),
                     "make": (lambda w, sc, a=a, y=y, ws=ws: (lambda: ops.w4a16_gemm_variant(a, w, sc, "auto", out=y, workspace=ws,
                                                                                            sync=env.sync)))})
    _, _, w8, s_ch = datagen.w8a8_case(0, 1, n, k)
    tw8, tsch = env.dev_t(w8), env.dev_t(s_ch)
    for m in W8A8_MS:
        a8 = env.dev_t(datagen.uniform_i8(0, datagen.S_A8, (m, k)))
        st = env.dev_t(datagen.uniform_f32(0, datagen.S_STOK, (m,), 0.001, 0.01))
        y = torch.empty((m, n), dtype=torch.float16, device=dev)
        ws = env.workspace(lib.nnf_w8a8_gemm_workspace_bytes(m, n, k))
        rows.append({"key": f"w8a8_gemm_N{n}_K{k}.M{m}", "group": f"w8a8_gemm_N{n}_K{k}", "M": m,
                     "bytes": w8a8_bytes(m, n, k), "ops": 2.0 * m * n * k, "int8": True, "weights": (tw8,),
                     "make": (lambda w, a8=a8, st=st, y=y, ws=ws: (lambda: ops.w8a8_gemm(a8, st, w, tsch, out=y, workspace=ws, sync=env.sync)))})
    for bits, group, zpt in WNA16_CASES:
        _, wq, s, z = datagen.wna16_case(0, 1, n, k, bits, group, zpt)
        tw, tsc, tz = env.dev_t(wq), env.dev_t(s), (env.dev_t(z) if zpt else None)
        for m in WNA16_MS:
            a = env.dev_t(datagen.normal_f16(0, datagen.S_ACT, (m, k)))
            y = torch.empty((m, n), dtype=torch.float16, device=dev)
            wsq = env.workspace(ops.wna16_workspace_bytes(m, n, k, bits, group, tz))
            rows.append({"key": wna16_key(bits, group, zpt, n, k, m), "group": None, "M": m,
                         "bytes": wna16_bytes(m, n, k, bits, group, zpt), "ops": 2.0 * m * n * k, "int8": False,
                         "weights": (tw, tsc) + ((tz,) if zpt else ()),
                         "make": (lambda w, sc, zz=None, a=a, y=y, bits=bits, group=group, wsq=wsq:
                                  (lambda: ops.wna16_gemm(a, w, sc, bits=bits, group=group, zp=1 << (bits - 1), zero_points=zz,
                                                          out=y, workspace=wsq)))})
    h, i = MLP_HI
    _, gamma, wgu, sgu, wd, sd = [env.dev_t(t) for t in datagen.mlp_case(0, 1, h, i)]  # the weights do not depend on M
    for m in MLP_MS:
        x = env.dev_t(datagen.mlp_case(0, m, h, i)[0])
        out = torch.empty((m, h), dtype=torch.float16, device=dev)
        wsm = env.workspace(lib.nnf_fused_mlp_w4a16_workspace_bytes(m, h, i, GROUP))
        rows.append({"key": f"fused_mlp_M{m}_{h}_{i}", "group": None, "M": m, "bytes": mlp_bytes(m, h, i),
                     "ops": 2.0 * m * (2 * i) * h + 2.0 * m * h * i, "int8": False, "weights": (wgu, sgu, wd, sd),
                     "make": (lambda a, b, c, d, x=x, out=out, wsm=wsm:
                              (lambda: ops.fused_mlp_w4a16(x, gamma, a, b, c, d, out=out, workspace=wsm, sync=env.sync)))})
    return rows


def small_batch_rows(env):
    """The decode sweep's shapes with a handful of rows (batched decode), per batch size: a list of
    (bytes, factory, weights) per shape."""
    torch, datagen, ops, lib, dev = env.torch, env.datagen, env.ops, env.lib, env.dev
    weights = []
    for (sn, sk) in DECODE_SHAPES:
        _, wq, s = datagen.w4a16_case(0, 1, sn, sk)
        weights.append((env.dev_t(wq), env.dev_t(s)))
    out = []
    for m in SMALL_BATCHES:
        shapes = []
        for (sn, sk), (twq, ts) in zip(DECODE_SHAPES, weights):
            a = env.dev_t(datagen.normal_f16(0, datagen.S_ACT, (m, sk)))
            y = torch.empty((m, sn), dtype=torch.float16, device=dev)
            ws = env.workspace(lib.nnf_w4a16_gemm_workspace_bytes(m, sn, sk, GROUP))
            shapes.append({"key": f"decode_sweep_M{m}.N{sn}_K{sk}", "bytes": w4a16_bytes(m, sn, sk), "weights": (twq, ts),
                           "make": (lambda w, sc, a=a, y=y, ws=ws: (lambda: ops.w4a16_gemm_variant(a, w, sc, "auto", out=y, workspace=ws,
                                                                                                  sync=env.sync)))})
        out.append((m, shapes))
    return out


def run_extra(env, traffic):
    """The other benchmark configurations, a few iterations each (not part of `value`).  Rows with M <= 128 are
    memory-bound: they are timed over copies of the weights that miss the last-level cache.  Returns the plain
    timings and, per row, the roofline figures: the ceiling is the matrix cores' when the row's operations per
    algorithmic byte exceed peak operations / peak bandwidth, else HBM's."""
    torch = env.torch
    res, roofs = {}, []
    row_kernels = load_row_kernels()
    for row in extra_rows(env):
        if row["M"] <= 128:
            sets = env.copies_of(*row["weights"])
            us = env.time_cold_us(row["make"], sets)
            del sets
        else:
            us = env.time_us(row["make"](*row["weights"]), 20)
        peak_ops = MFMA_I8_PEAK_TOPS if row["int8"] else MFMA_F16_PEAK_TFLOPS
        rate = row["ops"] / us / 1e6  # Tera-op/s
        gbs = row["bytes"] / us / 1e3
        unit_ops = "TOP/s" if row["int8"] else "TFLOP/s"
        entry = {"M": row["M"], "us": round(us, 2), unit_ops: round(rate, 1),
                 ("frac_mfma_i8" if row["int8"] else "frac_mfma_f16"): round(rate / peak_ops, 4), "GB/s": round(gbs, 1)}
        if row["group"]:
            res.setdefault(row["group"], []).append(entry)
        else:
            entry.pop("M")
            res[row["key"]] = entry
        mfma_bound = row["ops"] / row["bytes"] > peak_ops * 1e12 / (HBM_PEAK_GBS * 1e9)
        roofs.append({"row": row["key"], "kernel": row_kernels.get(row["key"]),
                      "bound": "mfma" if mfma_bound else "hbm",
                      "achieved": round(rate if mfma_bound else gbs, 1),
                      "peak": peak_ops if mfma_bound else HBM_PEAK_GBS,
                      "unit": unit_ops if mfma_bound else "GB/s",
                      "frac": round(rate / peak_ops if mfma_bound else gbs / HBM_PEAK_GBS, 4),
                      "traffic": traffic.get(row["key"]), "algorithmic_bytes": int(row["bytes"]),
                      "us_per_launch": round(us, 2)})
    sweep = []
    for m, shapes in small_batch_rows(env):
        total_us, total_bytes, total_traffic = 0.0, 0, 0
        for sh in shapes:
            sets = env.copies_of(*sh["weights"])
            total_us += env.time_cold_us(sh["make"], sets)
            total_bytes += sh["bytes"]
            t = traffic.get(sh["key"])
            total_traffic = None if (t is None or total_traffic is None) else total_traffic + t
            del sets
        sweep.append({"M": m, "us_per_sweep": round(total_us, 2), "GB/s": round(total_bytes / total_us / 1e3, 1)})
        roofs.append({"row": f"decode_sweep_M{m}", "kernel": " | ".join(sorted({row_kernels.get(sh["key"], "?") for sh in shapes})),
                      "bound": "hbm", "achieved": round(total_bytes / total_us / 1e3, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                      "frac": round(total_bytes / total_us / 1e3 / HBM_PEAK_GBS, 4), "traffic": total_traffic,
                      "algorithmic_bytes": int(total_bytes), "us_per_launch": round(total_us, 2)})
    res["w4a16_decode_sweep_small_batches"] = sweep
    # For scale only: the vendor library's unquantized GEMMs on the same box and value distributions (fp16 weights, four
    # times the bytes, no unpacking; int8 x int8 -> int32 without the scaling epilogue) at the shapes of the compute-bound
    # rows: N = K = 8192 at M = 128 .. 4096, and the two products of the MLP block at M = 256.  The clock a kernel gets
    # depends on what ran in the seconds before it, so each shape is timed in turns -- this library's kernel, the vendor's,
    # three times over, about 20 ms each, same operands every launch (hot caches for both) -- and both means are
    # reported (nnf_*: this library in the same loop; its rows above walk cold copies of the weights).
    vendor = {}
    try:
        dev = env.dev

        def in_turns(fns, rounds=3):
            sums = [0.0] * len(fns)
            for f in fns:
                env.time_us(f, 5)
            for _ in range(rounds):
                for i, f in enumerate(fns):
                    sums[i] += env.time_span_us(f, 20e3)
            return [x / rounds for x in sums]

        for (m, n, k, int8_too) in ((128, 8192, 8192, False), (512, 8192, 8192, True), (1024, 8192, 8192, False),
                                    (4096, 8192, 8192, True), (256, 2 * MLP_HI[1], MLP_HI[0], False), (256, MLP_HI[0], MLP_HI[1], False)):
            a = torch.randn(m, k, device=dev, dtype=torch.float16)
            w = torch.randn(n, k, device=dev, dtype=torch.float16)
            y = torch.empty(m, n, device=dev, dtype=torch.float16)
            _, wq, s = env.datagen.w4a16_case(0, 1, n, k)
            tq, tsc = env.dev_t(wq), env.dev_t(s)
            ws = env.workspace(env.lib.nnf_w4a16_gemm_workspace_bytes(m, n, k, GROUP))
            y4 = torch.empty(m, n, device=dev, dtype=torch.float16)
            ours, theirs = in_turns([lambda: env.ops.w4a16_gemm_variant(a, tq, tsc, "auto", out=y4, workspace=ws, sync=env.sync),
                                     lambda: torch.matmul(a, w.t(), out=y)])
            entry = {"fp16_matmul_us": round(theirs, 1), "fp16_TFLOP/s": round(2.0 * m * n * k / theirs / 1e6, 1),
                     "nnf_w4a16_us": round(ours, 1), "nnf_w4a16_TFLOP/s": round(2.0 * m * n * k / ours / 1e6, 1)}
            del a, w, y, tq, tsc, y4, ws
            if int8_too:
                a8 = torch.randint(-127, 128, (m, k), device=dev, dtype=torch.int8)
                w8 = torch.randint(-127, 128, (n, k), device=dev, dtype=torch.int8)
                st = env.dev_t(env.datagen.uniform_f32(0, env.datagen.S_STOK, (m,), 0.001, 0.01))
                sch = env.dev_t(env.datagen.uniform_f32(1, env.datagen.S_STOK, (n,), 0.001, 0.01))
                y8 = torch.empty(m, n, device=dev, dtype=torch.float16)
                ws8 = env.workspace(env.lib.nnf_w8a8_gemm_workspace_bytes(m, n, k))
                ours8, theirs8 = in_turns([lambda: env.ops.w8a8_gemm(a8, st, w8, sch, out=y8, workspace=ws8), lambda: torch._int_mm(a8, w8.t())])
                entry.update({"int8_mm_us": round(theirs8, 1), "int8_TOP/s": round(2.0 * m * n * k / theirs8 / 1e6, 1),
                              "nnf_w8a8_us": round(ours8, 1), "nnf_w8a8_TOP/s": round(2.0 * m * n * k / ours8 / 1e6, 1)})
                del a8, w8, y8, ws8
            vendor[f"M{m}_N{n}_K{k}"] = entry
    except Exception as e:  # a yardstick, not part of the benchmark
        vendor["error"] = str(e)[:200]
    res["vendor_library_for_scale"] = vendor
    return res, roofs


def run_pmc_probe(env, probes, layers, step, n_layers):
    """For FETCH_SIZE / WRITE_SIZE runs.  Calibration: a device-to-device copy that reads and writes exactly
    PROBE_BYTES, larger than the last-level cache.  Then every configuration row, launched eagerly a few times, each
    behind one marker launch (the read probe on 16 x (row index + 1) bytes) by which a reader of the counter file
    tells the rows apart.  Prints the rows in launch order with their algorithmic bytes."""
    torch = env.torch
    num_cu = torch.cuda.get_device_properties(0).multi_processor_count
    src = torch.empty(PROBE_BYTES // 4, dtype=torch.float32, device=env.dev).normal_()
    dst = torch.empty_like(src)
    marker_buf = torch.zeros(4096, dtype=torch.uint8, device=env.dev)
    torch.cuda.synchronize()
    for _ in range(4):
        dst.copy_(src)
    torch.cuda.synchronize()
    del src, dst
    order = []

    def marker():
        st = probes.nnf_probe_read(torch.cuda.current_stream().cuda_stream, marker_buf.data_ptr(), 16 * (len(order) + 1), 0, num_cu)
        if st != 0:
            raise RuntimeError(f"nnf_probe_read failed: {st}")

    # the sweep, shape by shape over every resident layer
    for si, (n, k) in enumerate(DECODE_SHAPES):
        marker()
        for layer in layers:
            a, wq, s, y = layer[si]
            st = env.lib.nnf_w4a16_gemm(torch.cuda.current_stream().cuda_stream, a.data_ptr(), wq.data_ptr(), s.data_ptr(),
                                        y.data_ptr(), 1, n, k, GROUP, 8, None, 0)
            if st != 0:
                raise RuntimeError(f"nnf_w4a16_gemm failed: {st}")
        order.append({"row": f"decode_sweep.N{n}_K{k}", "launches": n_layers, "algorithmic_bytes": w4a16_bytes(1, n, k)})
    torch.cuda.synchronize()
    for m, shapes in small_batch_rows(env):
        for sh in shapes:
            marker()
            fn = sh["make"](*sh["weights"])
            for _ in range(3):
                fn()
            order.append({"row": sh["key"], "launches": 3, "algorithmic_bytes": sh["bytes"]})
        torch.cuda.synchronize()
    for row in extra_rows(env):
        marker()
        fn = row["make"](*row["weights"])
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        order.append({"row": row["key"], "launches": 3, "algorithmic_bytes": int(row["bytes"])})
    print(json.dumps({"pmc_probe": {"calibration_copy_bytes": PROBE_BYTES, "calibration_copies": 4, "rows": order}}), flush=True)


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
