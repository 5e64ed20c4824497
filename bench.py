#!/usr/bin/env python3
"""Benchmark of the TOSA hot path on one MI355X.

A "step" is one pass of the hot path over one batch of synthetic input, inputs resident in HBM:
BASELINE config 1, the fused int8 MATMUL + RESCALE (8 x 512x1024 . 8 x 1024x1024, a_zp=2, b_zp=-1, per-tensor
multiplier 1518500250 / shift 39, double round), one launch of the MFMA contraction kernel.  The same JSON line
also reports the MobileNetV2-shaped int8 graph at batch 32 (BASELINE config 3) executed through the host-side
GraphPipeline, the roofline position of the dominant kernel and a CPU baseline (the oracle on the host cores).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only LEG] [--layer N]

`--only` restricts the run to one leg (profiling runs: one kernel family per trace): `config0` (fused CONV2D + RESCALE,
1x56x56x64), `config1`, `config2` (the inverted-residual block), `mobilenetv2` (config 3), `encoder` (config 4),
`gemm_large` (the config 1 operator at 4096^3 and 8192^3), `layer --layer N` (the N-th launch of the fused MobileNetV2
graph 200 times back to back and nothing else, so that counters of a single layer can be collected), `standalone`
(the bandwidth-bound operators as stand-alone launches on config 2's and on config 3's largest tensors), `copy` (the
plain copy kernel over grid and size: the measured HBM ceiling), `extra` (data-movement operators outside the
benchmark graphs), `vendor` (the GPU vendor's matrix library through torch on the products timed here, as a calibration
of the box; nothing of the product runs in that leg), `issue` (what a lone wavefront issues while its matrix
instructions run: the instruction mixes of a contraction loop alone, behind and between the matrix instructions).  `ms_per_step` is the median over at least 10 rounds of `--steps` launches; the whole-graph legs
report the median over rounds that hold at least 50 graphs.
"""
import re
import argparse
import ctypes as C
import importlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
PKG = "ai-ml-emulation-layer-for-vulkan_amd"

INT8_MFMA_PEAK_TOPS = 5000.0  # MI355X published dense int8 peak, TOP/s
HBM_PEAK_GBS = 8000.0         # MI355X published HBM3E bandwidth, GB/s


def device_peaks(info):
    """The published peaks next to what the device's own properties give: matrix cores = compute units x 4 SIMDs x
    1024 int8 multiply-adds per clock x 2 ops x the reported shader clock; HBM = reported memory clock x 4 transfers
    per clock (HBM3E at 8 Gbit/s per pin reports 2000 MHz) x bus width.  The roofline fractions of this file use the
    published figures."""
    cus, clk = info["compute_units"], info["clock_khz"] * 1e3
    return {"int8_mfma_published_tops": INT8_MFMA_PEAK_TOPS,
            "int8_mfma_from_device_tops": cus * 4 * 1024 * 2 * clk / 1e12,
            "fp16_mfma_from_device_tflops": cus * 4 * 512 * 2 * clk / 1e12,
            "hbm_published_gbs": HBM_PEAK_GBS,
            "hbm_from_device_properties_gbs": info["mem_clock_khz"] * 1e3 * 4 * info["bus_width_bits"] / 8 / 1e9,
            "compute_units": cus, "clock_mhz": info["clock_khz"] / 1e3, "mem_clock_mhz": info["mem_clock_khz"] / 1e3,
            "bus_width_bits": info["bus_width_bits"]}


def reference_layer_probe():
    """Looks for what a run of the reference layer itself would need on this host -- a Vulkan loader, the lavapipe
    ICD manifest and the layer's manifest (VK_LAYER_ML_Graph_Emulation) -- without installing or loading anything.
    With all three the CPU baseline could be the reference on lavapipe; without them it is the oracle (kind "port")."""
    import ctypes.util
    import glob
    loader = ctypes.util.find_library("vulkan")
    roots = ["/usr/share/vulkan", "/usr/local/share/vulkan", "/etc/vulkan", os.path.expanduser("~/.local/share/vulkan")]
    layer_dirs = [os.path.join(r, d) for r in roots for d in ("explicit_layer.d", "implicit_layer.d")]
    for var in ("VK_LAYER_PATH", "VK_ADD_LAYER_PATH"):
        layer_dirs += [d for d in os.environ.get(var, "").split(os.pathsep) if d]
    layer = None
    for d in layer_dirs:
        for f in sorted(glob.glob(os.path.join(d, "*.json"))):
            try:
                if "VK_LAYER_ML_Graph_Emulation" in open(f, errors="replace").read():
                    layer = f
            except OSError:
                pass
    icds = [f for r in roots for f in glob.glob(os.path.join(r, "icd.d", "lvp_icd*.json"))]
    icds += [f for f in os.environ.get("VK_ICD_FILENAMES", "").split(os.pathsep) if "lvp" in f and os.path.exists(f)]
    return {"vulkan_loader": loader, "lavapipe_icd": icds[0] if icds else None, "layer_manifest": layer,
            "reference_layer_found": bool(loader and icds and layer)}

CONFIG1_KERNEL = "gemm_i8_kernel<128,128,2,2,X_PLAIN_DL,W_KMAJOR_DL,SUMS,Q8>"
CONFIG1_PROFILE = os.path.join(ROOT, "profiles", "gemm_i8_kernel_config1_matmul_rescale.md")


def config1_traffic_bytes():
    """HBM bytes per launch of the config 1 kernel as the committed counter summary states them (two rocprofv3 --pmc
    runs, FETCH_SIZE and WRITE_SIZE, each scaled by what it reads for the 256 MiB copy kernel): the line
    `traffic_bytes_per_launch = N` of the profile of this kernel, or None when the summary is missing or is of another
    kernel."""
    try:
        text = open(CONFIG1_PROFILE).read()
    except OSError:
        return None
    m = re.search(r"traffic_bytes_per_launch\s*=\s*(\d+)", text)
    k = re.search(r"traffic_kernel\s*=\s*(\S+)", text)
    if not m or not k or k.group(1).strip("`") != CONFIG1_KERNEL:
        return None
    return int(m.group(1))


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def config1_inputs():
    rng = np.random.default_rng(1001)
    a = rng.integers(-128, 127, (8, 512, 1024), endpoint=True).astype(np.int8)
    b = rng.integers(-128, 127, (8, 1024, 1024), endpoint=True).astype(np.int8)
    return a, b, np.array([1518500250], np.int32), np.array([39], np.int8)


def bench_config1(dev, abi, steps, warmup, in_flight_counts=(2, 4), rounds=10):
    a, b, mult, shift = config1_inputs()
    ta, tb, tm, ts = dev.from_numpy(a), dev.from_numpy(b), dev.from_numpy(mult), dev.from_numpy(shift)
    to = dev.tensor(abi.I8, (8, 512, 1024))
    attr = abi.MatmulAttr(2, -1)
    epi = dev.epilogue(tm, ts, abi.rescale_attr(0, 0, True, True, False))
    stream = dev.new_stream()
    dev.stream = stream

    def step():
        dev.op("matmul_rescale", to.ref, ta.ref, tb.ref, C.byref(attr), C.byref(epi))

    for _ in range(warmup):
        step()
    dev.sync()
    ev0, ev1 = dev.event(), dev.event()
    walls, kernels = [], []
    for _ in range(rounds):  # every round: `steps` launches between two events and two host time stamps
        t0 = time.perf_counter()
        dev.record(ev0)
        for _ in range(steps):
            step()
        dev.record(ev1)
        dev.sync()
        walls.append((time.perf_counter() - t0) / steps)
        kernels.append(dev.elapsed_ms(ev0, ev1) / steps)  # back-to-back launches of the one kernel on its own stream
    wall, kernel_ms = float(np.median(walls)), float(np.median(kernels))
    ops = 2.0 * 8 * 512 * 1024 * 1024
    res = {
        "ms_per_step": wall * 1e3,
        "tops": ops / wall / 1e12,
        "kernel_ms": kernel_ms,
        "kernel_tops": ops / (kernel_ms * 1e-3) / 1e12,
        "rounds": rounds,
        "ms_per_step_min_max": [min(walls) * 1e3, max(walls) * 1e3],
        "algorithmic_bytes": 8 * (512 * 1024 + 1024 * 1024 + 512 * 1024) + 5,
        "ops": ops,
    }
    out = to.download()
    # The same launches with two and four of them in flight (a stream and an output tensor each): what the kernel
    # delivers when its fixed latency (launch, first fetch, last store) is hidden behind another launch's loop.
    # Reported beside the one-stream figures, which stay the step time and the roofline of the JSON line.
    in_flight = []
    for count in in_flight_counts:
        streams = importlib.import_module(PKG + ".graphs").in_flight_streams(dev, count)
        outs = [dev.tensor(abi.I8, (8, 512, 1024)) for _ in range(count)]
        n = count * max(steps // count, 10)
        for rep in range(2):  # the first round warms up
            dev._check(dev.lib.mlel_hip_sync(dev.ctx, None))
            t0 = time.perf_counter()
            for k in range(n):
                dev.stream = streams[k % count]
                dev.op("matmul_rescale", outs[k % count].ref, ta.ref, tb.ref, C.byref(attr), C.byref(epi))
            dev._check(dev.lib.mlel_hip_sync(dev.ctx, None))
            per = (time.perf_counter() - t0) / n
        same = all(np.array_equal(t.download(), out) for t in outs)
        in_flight.append({"streams": count, "launches_timed": n, "us_per_launch": per * 1e6, "tops": ops / per / 1e12,
                          "frac_of_int8_peak": ops / per / 1e12 / 5000.0, "outputs_equal": bool(same)})
        for t in outs:
            t.free()
    res["launches_in_flight"] = in_flight
    dev.stream = None
    # the same step when the caller hands over host buffers: upload A and B, launch, download the result
    t0 = time.perf_counter()
    for _ in range(3):
        ta.upload(a)
        tb.upload(b)
        step()
        to.download()
    res["host_buffers_ms_per_step"] = (time.perf_counter() - t0) * 1e3 / 3
    return res, (a, b, mult, shift, out)


def _median_us(dev, fn, reps, rounds=5, warm=3):
    """Microseconds per call of `fn`: `reps` back-to-back calls between two events on the launch stream, the median of
    `rounds` such measurements."""
    for _ in range(warm):
        fn()
    ev0, ev1 = dev.event(), dev.event()
    got = []
    for _ in range(rounds):
        dev.record(ev0)
        for _ in range(reps):
            fn()
        dev.record(ev1)
        dev.sync()
        got.append(dev.elapsed_ms(ev0, ev1) / reps * 1e3)
    return float(np.median(got))


def bench_config0(dev, abi, steps, warmup, check=True):
    """BASELINE config 0: CONV2D 3x3 (1x56x56x64 -> 64 channels, stride 1, pad 1, input_zp -5) + per-channel RESCALE
    (double round, output_zp 3) to int8, one fused launch."""
    rng = np.random.default_rng(1000)
    x = rng.integers(-128, 127, (1, 56, 56, 64), endpoint=True).astype(np.int8)
    w = rng.integers(-127, 127, (64, 3, 3, 64), endpoint=True).astype(np.int8)
    b = rng.integers(-2 ** 15, 2 ** 15, (64,), endpoint=True).astype(np.int32)
    mult = rng.integers(2 ** 30, 2 ** 31 - 1, (64,), endpoint=True).astype(np.int32)
    shift = rng.integers(30, 38, (64,), endpoint=True).astype(np.int8)
    attr = abi.conv2d_attr((1, 1, 1, 1), (1, 1), (1, 1), -5, 0)
    rattr = abi.rescale_attr(0, 3, True, True, True)
    tx, tw, tb, tm, ts = (dev.from_numpy(v) for v in (x, w, b, mult, shift))
    to = dev.tensor(abi.I8, (1, 56, 56, 64))
    epi = dev.epilogue(tm, ts, rattr)
    fn = lambda: dev.op("conv2d_rescale_clamp", to.ref, tx.ref, tw.ref, tb.ref, C.byref(attr), C.byref(epi))
    us = _median_us(dev, fn, max(steps, 20), rounds=10, warm=max(warmup, 3))
    ops = 2.0 * 56 * 56 * 64 * 9 * 64
    nbytes = x.size + w.size + 9 * 64 + x.size
    res = {"us_per_launch": us, "launches_timed": 10 * max(steps, 20), "tops": ops / (us * 1e-6) / 1e12, "ops": ops,
           "algorithmic_bytes": nbytes,
           "roofline": {"mfma_frac": ops / (us * 1e-6) / 1e12 / INT8_MFMA_PEAK_TOPS,
                        "hbm_frac": nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS,
                        "note": "0.23 GOP and 0.44 MB: a launch of this size is bound by its own latency"}}
    if check:
        oracle = importlib.import_module("oracle.mlel_oracle")
        exp = oracle.rescale(oracle.conv2d(x, w, b, (1, 56, 56, 64), abi.I32, attr), mult, shift, abi.I8, rattr)
        res["bit_exact_vs_oracle"] = bool(np.array_equal(to.download(), exp))
    for t in (tx, tw, tb, tm, ts, to):
        t.free()
    return res


def bench_gemm_large(dev, abi, sizes=(4096, 8192), check=True):
    """The config 1 operator (int8 MATMUL, a_zp 2, b_zp -1, + per-tensor RESCALE to int8, one fused launch) on square
    problems large enough to fill the machine for many tile rounds: what the contraction kernel reaches when launch
    latency, prologue and epilogue are a small share."""
    out = []
    for n in sizes:
        rng = np.random.default_rng(n)
        a = rng.integers(-128, 127, (1, n, n), endpoint=True).astype(np.int8)
        b = rng.integers(-128, 127, (1, n, n), endpoint=True).astype(np.int8)
        ta, tb = dev.from_numpy(a), dev.from_numpy(b)
        tm, ts = dev.from_numpy(np.array([1518500250], np.int32)), dev.from_numpy(np.array([39], np.int8))
        to = dev.tensor(abi.I8, (1, n, n))
        attr = abi.MatmulAttr(2, -1)
        rattr = abi.rescale_attr(0, 0, True, True, False)
        epi = dev.epilogue(tm, ts, rattr)
        fn = lambda: dev.op("matmul_rescale", to.ref, ta.ref, tb.ref, C.byref(attr), C.byref(epi))
        us = _median_us(dev, fn, 10, rounds=5, warm=2)
        ops = 2.0 * n * n * n
        rec = {"shape": [n, n, n], "us_per_launch": us, "launches_timed": 50, "tops": ops / (us * 1e-6) / 1e12,
               "frac_of_int8_peak": ops / (us * 1e-6) / 1e12 / INT8_MFMA_PEAK_TOPS, "algorithmic_bytes": 3 * n * n + 5}
        if check:  # a band of rows against the oracle
            oracle = importlib.import_module("oracle.mlel_oracle")
            rows = slice(n - 24, n - 8)
            exp = oracle.rescale(oracle.matmul(a[:, rows], b, abi.I32, 2, -1), np.array([1518500250], np.int32),
                                 np.array([39], np.int8), abi.I8, rattr)
            rec["rows_checked_vs_oracle"] = 16
            rec["bit_exact_vs_oracle"] = bool(np.array_equal(to.download()[:, rows], exp))
        out.append(rec)
        for t in (ta, tb, tm, ts, to):
            t.free()
    return out


def bench_copy_sweep(dev, info):
    """The plain copy kernel over grid size, 16-byte pieces in flight per thread and temporal / non-temporal accesses,
    on 1 GiB (beyond the 256 MiB last-level cache) and on 64 MiB (inside it), plus a read-only and a write-only pass:
    what the memory system of this part delivers to the simplest streaming kernel, i.e. the ceiling every
    bandwidth-bound kernel here is to be read against."""
    cus = info["compute_units"]
    rows = []
    for nbytes in (1 << 30, 64 << 20):
        src, dst = dev.alloc(nbytes), dev.alloc(nbytes)
        for mode, name, moved in ((0, "copy", 2.0), (1, "read", 1.0), (2, "write", 1.0)):
            for nt in (0, 1):
                for u in (1, 2, 4, 8):
                    for blocks in (0, cus * 4, cus * 8, cus * 16, cus * 32):
                        if mode != 0 and (blocks not in (0, cus * 8) or u not in (1, 4)):
                            continue
                        fn = lambda: dev._check(dev.lib.mlel_hip_copy_kernel_variant(
                            dev.ctx, dev.stream, C.c_void_p(dst), C.c_void_p(src), nbytes, blocks, u, nt, mode))
                        us = _median_us(dev, fn, 5, rounds=3, warm=1)
                        rows.append({"bytes": nbytes, "mode": name, "non_temporal": nt, "pieces_in_flight": u,
                                     "blocks": blocks, "us": round(us, 1),
                                     "gbs": round(moved * nbytes / (us * 1e-6) / 1e9, 1)})
        dev.free(src)
        dev.free(dst)
    best = {}
    for r in rows:
        key = f"{r['mode']}_{r['bytes'] >> 20}MiB"
        if key not in best or r["gbs"] > best[key]["gbs"]:
            best[key] = r
    return {"rows": rows, "best": best,
            "hbm_ceiling_gbs": best["copy_1024MiB"]["gbs"], "hbm_ceiling_frac_of_published": best["copy_1024MiB"]["gbs"] / HBM_PEAK_GBS}


def bench_mfma_rate(dev, info):
    """The int8 matrix cores with operands in registers (no memory, no LDS in the loop), two resident blocks per compute
    unit: TOP/s with all-zero operands and with random bytes.  The sustained rate of this part depends on the operand
    data; the random-data figure is what a contraction over real tensors can at most approach."""
    cus = info["compute_units"]
    blocks, iters = cus * 2, 4000
    out = dev.alloc(blocks * 256 * 4)
    res = {}
    for name, data in (("zeros", np.zeros(65536, np.uint8)),
                       ("random", np.random.default_rng(7).integers(0, 255, 65536, endpoint=True).astype(np.uint8))):
        t = dev.from_numpy(data)
        fn = lambda: dev._check(dev.lib.mlel_hip_mfma_rate_probe(dev.ctx, dev.stream, C.c_void_p(t.ptr), C.c_void_p(out),
                                                                 blocks, iters))
        us = _median_us(dev, fn, 3, rounds=5, warm=2)
        ops = 2.0 * 32 * 32 * 32 * 8 * iters * blocks * 4
        res[name] = {"us": round(us, 1), "tops": round(ops / (us * 1e-6) / 1e12, 1),
                     "frac_of_published_peak": round(ops / (us * 1e-6) / 1e12 / INT8_MFMA_PEAK_TOPS, 4)}
        t.free()
    dev.free(out)
    return res


ISSUE_MODES = [
    (0, "4 x v_mfma_i32_32x32x32_i8"),
    (1, "16 x v_dot4"), (2, "4 matrix instructions, then 16 x v_dot4"), (3, "matrix instruction + 4 x v_dot4, four times"),
    (4, "16 x v_add_u32"), (5, "4 matrix instructions, then 16 x v_add_u32"), (6, "matrix instruction + 4 x v_add_u32, four times"),
    (7, "matrix instruction + 4 x v_sad_u8, four times"),
    (8, "6 x ds_read_b128 + wait"), (9, "4 matrix instructions, then 6 x ds_read_b128 + wait"),
    (10, "matrix instruction + 2 reads, three times, matrix instruction, wait"),
    (11, "4 x buffer_load_dwordx4 ... lds"), (12, "4 matrix instructions, then 4 loads to LDS"),
    (13, "matrix instruction + load to LDS, four times"),
    (14, "matrix instruction + v_mfma_i32_16x16x64_i8, four times"),
]


def bench_issue_probe(dev, info, iters=512):
    """What a wavefront alone on its SIMD issues in the shadow of its matrix instructions (mlel_hip_issue_probe): clocks
    per round of every instruction mix, one block of four wavefronts per compute unit, random operand bytes."""
    data = np.random.default_rng(11).integers(0, 255, 65536, endpoint=True).astype(np.uint8)
    t = dev.from_numpy(data)
    n_out = 2 + 256 * info["compute_units"]
    out = dev.tensor(importlib.import_module(PKG + ".abi").I32, (n_out,))
    rows = []
    for mode, name in ISSUE_MODES:
        for _ in range(2):  # the second launch is the one that counts (code and operands are then resident)
            dev._check(dev.lib.mlel_hip_issue_probe(dev.ctx, dev.stream, C.c_void_p(t.ptr), C.c_void_p(out.ptr), mode, iters))
        dev.sync()
        w = out.download().view(np.uint32)
        clocks = int(w[0]) | (int(w[1]) << 32)
        rows.append({"mode": mode, "instructions": name, "clocks_per_round": round(clocks / iters, 1)})
        log("issue probe:", rows[-1])
    t.free()
    out.free()
    return rows


def measure_copy(dev, nbytes, reps=5):
    src, dst = dev.alloc(nbytes), dev.alloc(nbytes)
    best = 0.0
    for _ in range(reps):
        e0, e1 = dev.event(), dev.event()
        dev.record(e0)
        dev._check(dev.lib.mlel_hip_copy_kernel(dev.ctx, dev.stream, C.c_void_p(dst), C.c_void_p(src), nbytes))
        dev.record(e1)
        dev.sync()
        best = max(best, 2.0 * nbytes / (dev.elapsed_ms(e0, e1) * 1e-3) / 1e9)
    dev.free(src)
    dev.free(dst)
    return best


def cpu_baseline_config1(abi, inputs, gpu_out):
    """The oracle (a port of the reference shaders, not the reference binary) on the host cores: one batch of the
    eight (512x1024x1024) per repetition, repeated for about ten seconds; also re-checks the GPU result."""
    oracle = importlib.import_module("oracle.mlel_oracle")
    a, b, mult, shift, _ = inputs
    rattr = abi.rescale_attr(0, 0, True, True, False)
    reps, spent = 0, 0.0
    ok = True
    while spent < 10.0 and reps < 4096:
        i = reps % 8
        t0 = time.perf_counter()
        acc = oracle.matmul(a[i:i + 1], b[i:i + 1], abi.I32, 2, -1)
        ref = oracle.rescale(acc, mult, shift, abi.I8, rattr)
        spent += time.perf_counter() - t0
        if reps < 8:
            ok = ok and bool(np.array_equal(ref[0], gpu_out[i]))
        reps += 1
    ops = 2.0 * 512 * 1024 * 1024 * reps
    return {"value": ops / spent / 1e12, "unit": "TOPS", "cores": oracle.num_threads(), "kind": "port",
            "sample": f"{reps} x one batch (512x1024 . 1024x1024 int8 MATMUL + RESCALE) of config 1, "
                      f"{spent:.1f} s of CPU work, OpenMP"}, ok


def cpu_baseline_mobilenetv2(abi, budget_s=10.0):
    """The oracle executing the unfused MobileNetV2-shaped graph (183 operators) on the host cores, batch 4 per pass
    (one eighth of config 3's batch; every operator is independent across the batch), repeated for about ten seconds."""
    oracle = importlib.import_module("oracle.mlel_oracle")
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from oracle_graph import run_spec
    graphs = importlib.import_module(PKG + ".graphs")
    batch = 4
    spec = graphs.mobilenetv2_spec(batch=batch)
    x = np.random.default_rng(1003).integers(-128, 127, spec.inputs[0][2], endpoint=True).astype(np.int8)
    reps, spent = 0, 0.0
    while spent < budget_s and reps < 64:
        t0 = time.perf_counter()
        run_spec(oracle, spec, {"input": x})
        spent += time.perf_counter() - t0
        reps += 1
    return {"value": batch * reps / spent, "unit": "img/s", "cores": oracle.num_threads(), "kind": "port",
            "sample": f"{reps} x the unfused graph at batch {batch} (of config 3's 32), {spent:.1f} s of CPU work, OpenMP"}


def run_layer(dev, abi, index, reps=200):
    """One launch of the fused config 3 graph (position `index` among its launches), `reps` times back to back (for
    counter collection)."""
    graphs = importlib.import_module(PKG + ".graphs")
    spec = graphs.mobilenetv2_spec(batch=32)
    g = graphs.build(dev, spec, fuse=True)
    g.set_input("input", np.random.default_rng(1003).integers(-128, 127, spec.inputs[0][2], endpoint=True).astype(np.int8))
    g.dispatch()
    dev.sync()
    ms = graphs.time_operators(dev, g, reps=reps, only=[index])[index]
    launches = graphs.launch_layers(g, spec)
    if launches is None:
        raise SystemExit("bench.py: the fused graph's launches do not line up with the layers of its specification")
    layer = launches[index]
    res = {"layer": index, "name": g.op_name(index), "kind": layer["kind"], "in": list(layer["in"]),
           "out": list(layer["out"]), "us": ms * 1e3, "launches": reps + 3 + 1,
           "tops": 2.0 * layer["macs"] / (ms * 1e-3) / 1e12, "algorithmic_bytes": layer["bytes"],
           "gbs": layer["bytes"] / (ms * 1e-3) / 1e9}
    g.close()
    return res


def bench_standalone(dev, abi, shape=(16, 56, 56, 144), reps=100):
    """The bandwidth-bound operators of an UNFUSED int8 graph as stand-alone launches: on config 2's tensor sizes
    (16 x 56 x 56 x 144 int32 accumulators / int8 activations, 7 - 36 MB per tensor, where the launch floor is a third
    of the time) and on config 3's largest tensor (32 x 112 x 112 x 96: 38.5 MB as int8, 154 MB as int32, beyond what
    the last-level cache holds for a three-tensor operator).  Microseconds per launch and algorithmic GB/s (input +
    output bytes once) of the packed 128-bit kernels, `reps` back-to-back launches each between two events."""
    rng = np.random.default_rng(1005)
    n = int(np.prod(shape))
    ch = shape[3]
    acc = rng.integers(-2 ** 22, 2 ** 22, shape).astype(np.int32)
    acc2 = rng.integers(-2 ** 22, 2 ** 22, shape).astype(np.int32)
    x8 = rng.integers(-128, 127, shape, endpoint=True).astype(np.int8)
    mult = rng.integers(2 ** 30, 2 ** 31 - 1, (ch,), endpoint=True).astype(np.int32)
    shift = rng.integers(30, 38, (ch,), endpoint=True).astype(np.int8)
    tab = rng.integers(-128, 127, (256,), endpoint=True).astype(np.int8)
    t_acc, t_acc2, t_x8 = dev.from_numpy(acc), dev.from_numpy(acc2), dev.from_numpy(x8)
    t_m, t_s, t_tab = dev.from_numpy(mult), dev.from_numpy(shift), dev.from_numpy(tab)
    o8, o32 = dev.tensor(abi.I8, shape), dev.tensor(abi.I32, shape)
    o_pool = dev.tensor(abi.I8, (shape[0], shape[1] // 2, shape[2] // 2, ch))
    held = [t_acc, t_acc2, t_x8, t_m, t_s, t_tab, o8, o32, o_pool]
    # reduced-precision storage: bf16 values as the upper halves of fp32 numbers, fp32 values inside e4m3's range
    f32 = (rng.standard_normal(shape) * 20).astype(np.float32)
    bf = (f32.view(np.uint32) >> 16).astype(np.uint16)
    t_bf1, t_bf2, t_f32 = dev.from_numpy(bf, abi.BF16), dev.from_numpy(bf[::-1].copy(), abi.BF16), dev.from_numpy(f32)
    o_bf, o_f8 = dev.tensor(abi.BF16, shape), dev.tensor(abi.F8E4M3, shape)
    held += [t_bf1, t_bf2, t_f32, o_bf, o_f8]
    r_down = abi.rescale_attr(0, 3, True, True, True)
    r_up = abi.rescale_attr(-5, 0, True, True, True)
    clamp = abi.ClampAttr(0.0, 96.0, int(abi.NAN_PROPAGATE))
    pool = abi.pool2d_attr((3, 3), (2, 2), (0, 1, 0, 1))
    cases = [
        ("RESCALE int32->int8 per channel", 5 * n,
         lambda: dev.op("rescale", o8.ref, t_acc.ref, t_m.ref, t_s.ref, C.byref(r_down))),
        ("RESCALE int8->int32 per channel", 5 * n,
         lambda: dev.op("rescale", o32.ref, t_x8.ref, t_m.ref, t_s.ref, C.byref(r_up))),
        ("CLAMP int8", 2 * n, lambda: dev.op("clamp", o8.ref, t_x8.ref, C.byref(clamp))),
        ("ADD int32", 12 * n, lambda: dev.op("elementwise_binary", abi.BIN["ADD"], o32.ref, t_acc.ref, t_acc2.ref,
                                             int(abi.NAN_PROPAGATE))),
        ("TABLE int8", 2 * n, lambda: dev.op("table", o8.ref, t_x8.ref, t_tab.ref)),
        ("MAX_POOL2D int8 3x3 stride 2", n + n // 4, lambda: dev.op("max_pool2d", o_pool.ref, t_x8.ref, C.byref(pool))),
        ("ADD bf16", 6 * n, lambda: dev.op("elementwise_binary", abi.BIN["ADD"], o_bf.ref, t_bf1.ref, t_bf2.ref,
                                           int(abi.NAN_PROPAGATE))),
        ("CAST fp32->fp8 e4m3", 5 * n, lambda: dev.op("cast", o_f8.ref, t_f32.ref)),
    ]
    out = []
    ev0, ev1 = dev.event(), dev.event()
    for name, nbytes, fn in cases:
        for _ in range(5):
            fn()
        dev.record(ev0)
        for _ in range(reps):
            fn()
        dev.record(ev1)
        dev.sync()
        us = dev.elapsed_ms(ev0, ev1) / reps * 1e3
        out.append({"operator": name, "shape": list(shape), "us": round(us, 2), "algorithmic_bytes": nbytes,
                    "gbs": round(nbytes / (us * 1e-6) / 1e9, 1), "hbm_frac": round(nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)})
    for t in held:
        t.free()
    return out


def bench_extra(dev, abi, reps=50):
    """Data-movement operators outside the benchmark graphs (SLICE, CONCAT, PAD, TILE, REVERSE, GATHER) on dense int8
    tensors of config 3's 56 x 56 stage (32 x 56 x 56 x 144, 14.5 MB): microseconds and algorithmic GB/s (bytes read
    once + bytes written once)."""
    rng = np.random.default_rng(1006)
    n, h, w, c = 32, 56, 56, 144
    x = rng.integers(-128, 127, (n, h, w, c), endpoint=True).astype(np.int8)
    tx = dev.from_numpy(x)
    held = [tx]

    def new(shape, dtype=abi.I8, loose=False):
        # loose: 64 bytes between the batch elements, which sends the operator to the one-thread-per-element kernel
        strides = None
        if loose:
            strides = list(abi.packed_strides(shape, abi.DTYPE_SIZE[dtype]))
            first = 0 if shape[0] > 1 else 1  # an extent of one has no stride to speak of
            for i in range(first + 1):
                strides[i] += 64
        t = dev.tensor(dtype, shape, strides)
        held.append(t)
        return t

    u32 = lambda v: (C.c_uint32 * abi.MAX_RANK)(*[int(p) for p in v])
    o_slice = new((n, h - 2, w - 2, c))
    start = u32((0, 1, 1, 0))
    half = dev.from_numpy(x[..., : c // 2].copy())
    held.append(half)
    o_cat = new((n, h, w, c))
    o_pad = new((n, h + 2, w + 2, c))
    t_pad = dev.from_numpy(np.array([0, 0, 1, 1, 1, 1, 0, 0], np.int32))
    held.append(t_pad)
    small = dev.from_numpy(x[: n // 2].copy())
    held.append(small)
    o_tile = new((n, h, w, c))
    o_rev = new((n, h, w, c))
    vals = dev.from_numpy(x.reshape(n, h * w, c))
    idx = dev.from_numpy(np.stack([rng.permutation(h * w) for _ in range(n)]).astype(np.int32))
    held += [vals, idx]
    o_gather = new((n, h * w, c))
    size = x.size
    l_slice, l_cat, l_pad = new(o_slice.shape, loose=True), new(o_cat.shape, loose=True), new(o_pad.shape, loose=True)
    l_tile, l_rev, l_gather = new(o_tile.shape, loose=True), new(o_rev.shape, loose=True), new(o_gather.shape, loose=True)
    cases = [
        ("SLICE crop of one pixel all round", o_slice.nbytes * 2,
         lambda o=o_slice: dev.op("slice", o.ref, tx.ref, start), l_slice),
        ("CONCAT of two halves along the channels", size * 2,
         lambda o=o_cat: (dev.op("concat", o.ref, half.ref, 3, 0), dev.op("concat", o.ref, half.ref, 3, c // 2)), l_cat),
        ("PAD of one pixel all round", size + o_pad.nbytes,
         lambda o=o_pad: dev.op("pad", o.ref, tx.ref, t_pad.ref, 0.0, 0), l_pad),
        ("TILE of the batch, twice", size // 2 + size, lambda o=o_tile: dev.op("tile", o.ref, small.ref), l_tile),
        ("REVERSE along the width", size * 2, lambda o=o_rev: dev.op("reverse", o.ref, tx.ref, 2), l_rev),
        ("GATHER of every pixel row, permuted", size * 2 + idx.nbytes,
         lambda o=o_gather: dev.op("gather", o.ref, vals.ref, idx.ref), l_gather),
    ]
    out = []
    for name, nbytes, fn, loose in cases:
        us = _median_us(dev, fn, reps, rounds=5, warm=3)
        # the same operator into an output whose batch elements lie 64 bytes apart: the element-wise kernel takes it
        us_elem = _median_us(dev, lambda: fn(loose), max(reps // 5, 3), rounds=3, warm=1)
        out.append({"operator": name, "shape": [n, h, w, c], "us": round(us, 2), "algorithmic_bytes": int(nbytes),
                    "gbs": round(nbytes / (us * 1e-6) / 1e9, 1), "hbm_frac": round(nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
                    "us_one_thread_per_element": round(us_elem, 2)})
    # CONV3D 3x3x3, 16 -> 32 channels over 16 x 56 x 56: as one CONV2D on the matrix cores (depth taps laid along the
    # channels of a temporary: the call allocates and synchronises) against the one-thread-per-output kernel, which an
    # output with loose batch strides gets
    d3, h3, c3, oc3 = 16, 56, 16, 32
    x3 = dev.from_numpy(rng.integers(-128, 127, (1, d3, h3, h3, c3), endpoint=True).astype(np.int8))
    w3 = dev.from_numpy(rng.integers(-128, 127, (oc3, 3, 3, 3, c3), endpoint=True).astype(np.int8))
    b3 = dev.from_numpy(rng.integers(-1000, 1000, (oc3,)).astype(np.int32))
    o3 = new((1, d3, h3, h3, oc3), abi.I32)
    l3 = new((1, d3, h3, h3, oc3), abi.I32, loose=True)
    held += [x3, w3, b3]
    attr3 = abi.conv3d_attr((1, 1, 1, 1, 1, 1), (1, 1, 1), (1, 1, 1), -3, 0)
    fn3 = lambda o=o3: dev.op("conv3d", o.ref, x3.ref, w3.ref, b3.ref, C.byref(attr3))
    us = _median_us(dev, fn3, 10, rounds=3, warm=1)
    us_elem = _median_us(dev, lambda: fn3(l3), 2, rounds=2, warm=1)
    macs = d3 * h3 * h3 * oc3 * 27 * c3
    out.append({"operator": "CONV3D 3x3x3 16->32 on 1x16x56x56, int8 -> int32",
                "shape": [1, d3, h3, h3, c3], "us": round(us, 1), "tops": round(2.0 * macs / (us * 1e-6) / 1e12, 2),
                "us_one_thread_per_output": round(us_elem, 1)})
    for t in held:
        t.free()
    return out


def bench_vendor_library():
    """The GPU vendor's matrix library (through torch._int_mm / torch.matmul) on the shapes this file times, on the same
    box: a calibration of what the hardware gives a tuned library, not part of the product (which links no BLAS).  The
    int8 product there is plain: int32 result, no zero points, no RESCALE."""
    import torch

    def med_us(fn, n, rounds=5):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        t = []
        for _ in range(rounds):
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
            for _ in range(n):
                fn()
            e.record()
            torch.cuda.synchronize()
            t.append(s.elapsed_time(e) / n * 1e3)
        return sorted(t)[len(t) // 2]

    rows = []
    dev = "cuda:0"
    for m, k, n, reps in ((4096, 1024, 1024, 200), (4096, 4096, 4096, 10), (8192, 8192, 8192, 5)):
        a = torch.randint(-128, 128, (m, k), dtype=torch.int8, device=dev)
        b = torch.randint(-128, 128, (k, n), dtype=torch.int8, device=dev)
        for layout, bb in (("B [K][N]", b), ("B [N][K]", b.t().contiguous().t())):
            try:
                us = med_us(lambda: torch._int_mm(a, bb), reps)
                rows.append({"product": f"int8 {m}x{k}x{n}", "layout": layout, "us": round(us, 2),
                             "tops": round(2.0 * m * k * n / us / 1e6, 1)})
            except Exception as e:
                rows.append({"product": f"int8 {m}x{k}x{n}", "layout": layout, "error": repr(e)[:160]})
            log("vendor:", rows[-1])
    for m, k, n in ((4096, 768, 768), (4096, 768, 2304), (4096, 768, 3072), (4096, 3072, 768), (8192, 8192, 8192)):
        a = torch.randn(m, k, dtype=torch.float16, device=dev)
        b = torch.randn(k, n, dtype=torch.float16, device=dev)
        for layout, bb in (("B [K][N]", b), ("B [N][K]", b.t().contiguous().t())):
            us = med_us(lambda: torch.matmul(a, bb), 20 if m < 8192 else 5)
            rows.append({"product": f"fp16 {m}x{k}x{n}", "layout": layout, "us": round(us, 2),
                         "tflops": round(2.0 * m * k * n / us / 1e6, 1)})
            log("vendor:", rows[-1])
    q = torch.randn(96, 512, 64, dtype=torch.float16, device=dev)
    kt = torch.randn(96, 64, 512, dtype=torch.float16, device=dev)
    rows.append({"product": "fp16 scores only, 96 heads x (512x64 . 64x512)", "layout": "batched",
                 "us": round(med_us(lambda: torch.bmm(q, kt), 20), 2)})
    log("vendor:", rows[-1])
    return rows


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--skip-cpu", action="store_true", help="omit the CPU baseline legs (profiling runs)")
    ap.add_argument("--one-stream", action="store_true",
                    help="omit the legs with several launches / sessions in flight (profiling runs: one kernel at a time)")
    ap.add_argument("--skip-graph", action="store_true", help="omit the MobileNetV2 and encoder graph legs")
    ap.add_argument("--only", choices=["all", "config0", "config1", "config2", "mobilenetv2", "encoder", "gemm_large",
                                       "layer", "standalone", "copy", "extra", "vendor", "issue"], default="all")
    ap.add_argument("--layer", type=int, default=3, help="with --only layer: position in the fused config 3 graph")
    ap.add_argument("--gemm-size", type=int, default=0, help="with --only gemm_large: this one size instead of 4096 and 8192")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    if args.only == "vendor":
        print(json.dumps({"only": "vendor", "library": "torch._int_mm / torch.matmul / torch.bmm",
                          "products": bench_vendor_library()}), flush=True)
        return

    abi = importlib.import_module(PKG + ".abi")
    hb = importlib.import_module(PKG + ".hip_backend")
    dev = hb.Device(0)
    info = dev.info()
    log("device:", info)

    if args.only == "layer":
        print(json.dumps(run_layer(dev, abi, args.layer)), flush=True)
        dev.close()
        return

    if args.only == "standalone":
        print(json.dumps({"only": "standalone", "operators": bench_standalone(dev, abi) +
                          bench_standalone(dev, abi, (32, 112, 112, 96), reps=30)}), flush=True)
        dev.close()
        return

    if args.only == "copy":
        print(json.dumps(dict({"only": "copy", "mfma_rate": bench_mfma_rate(dev, info)}, **bench_copy_sweep(dev, info))),
              flush=True)
        dev.close()
        return

    if args.only == "issue":
        print(json.dumps({"only": "issue", "rounds": bench_issue_probe(dev, info)}), flush=True)
        dev.close()
        return

    if args.only == "extra":
        print(json.dumps({"only": "extra", "operators": bench_extra(dev, abi)}), flush=True)
        dev.close()
        return

    want = lambda leg: args.only in ("all", leg)
    graph_steps = max(20, args.steps // 10)

    # one plain 256 MiB device-to-device copy: the kernel of known traffic that calibrates the FETCH_SIZE / WRITE_SIZE
    # counters in profiling runs, and a measured HBM ceiling
    copy_gbs = measure_copy(dev, 256 << 20)
    log(f"copy kernel: {copy_gbs:.0f} GB/s (read + write)")

    c1, inputs = (None, None)
    if want("config1"):
        c1, inputs = bench_config1(dev, abi, args.steps, args.warmup, () if args.one_stream else (2, 4))
        log("config 1:", c1)

    extra = {}
    graphs = importlib.import_module(PKG + ".graphs")
    if want("config0"):
        extra["config0_conv2d_rescale_1x56x56x64"] = bench_config0(dev, abi, args.steps, args.warmup, not args.skip_cpu)
        log("config 0:", extra["config0_conv2d_rescale_1x56x56x64"])
    if want("config2") and not args.skip_graph:
        extra.update(graphs.bench_inverted_residual(dev, steps=graph_steps, warmup=max(3, args.warmup // 10)))
        log("config 2:", extra["config2_inverted_residual_b16"])
    if want("gemm_large"):
        extra["gemm_large"] = bench_gemm_large(dev, abi, sizes=(args.gemm_size,) if args.gemm_size > 0 else (4096, 8192),
                                               check=not args.skip_cpu)
        log("large products:", extra["gemm_large"])
    if want("mobilenetv2") and not args.skip_graph:
        try:
            extra.update(graphs.bench_mobilenetv2(dev, steps=graph_steps, warmup=max(3, args.warmup // 10),
                                                  in_flight=() if args.one_stream else (2, 3, 4)))
            log("config 3:", {k: v for k, v in extra["mobilenetv2_b32"].items() if k != "layers"})
        except Exception as e:  # the line below still reports config 1; the failure is visible
            log("config 3 leg failed:", repr(e))
            extra["mobilenetv2_b32"] = {"error": repr(e)}
    if want("encoder") and not args.skip_graph:
        try:
            extra.update(graphs.bench_transformer(dev, steps=graph_steps, warmup=max(3, args.warmup // 10),
                                                  in_flight=() if args.one_stream else (2, 3, 4)))
            log("config 4:", extra["transformer_b8_s512_d768"])
        except Exception as e:
            log("config 4 leg failed:", repr(e))
            extra["transformer_b8_s512_d768"] = {"error": repr(e)}

    cpu = None
    parity_ok = None
    if not args.skip_cpu and c1 is not None:
        cpu, parity_ok = cpu_baseline_config1(abi, inputs, inputs[4])
        cpu.update(reference_layer_probe())
        log("cpu baseline:", cpu, "gpu==oracle:", parity_ok)
    if not args.skip_cpu and "mobilenetv2_b32" in extra and "error" not in extra["mobilenetv2_b32"]:
        extra["mobilenetv2_b32"]["cpu_baseline"] = cpu_baseline_mobilenetv2(abi)
        log("cpu baseline (config 3):", extra["mobilenetv2_b32"]["cpu_baseline"])

    if c1 is None:  # a single graph leg: its own record, no config 1 fields to report
        print(json.dumps(dict({"only": args.only, "copy_kernel_gbs": copy_gbs, "peaks": device_peaks(info)}, **extra)),
              flush=True)
        dev.close()
        return

    line = {
        "metric": "int8 TOPS (config 1: MATMUL 8x512x1024x1024 + RESCALE, fused) + MobileNetV2-shape b32 img/s",
        "value": c1["tops"],
        "unit": "TOPS",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": c1["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "i8",
        "data": "synthetic",
        "config": {"workload": "BASELINE configs[1]: int8 MATMUL 8x(512x1024 . 1024x1024), a_zp=2 b_zp=-1, "
                               "+ per-tensor RESCALE (1518500250, 39, double_round) -> int8, one fused launch",
                   "device": info["name"], "compute_units": info["compute_units"]},
        "roofline": {"bound": "mfma", "achieved": c1["kernel_tops"], "peak": INT8_MFMA_PEAK_TOPS / 1.0,
                     "unit": "TFLOP/s", "ops_are": "int8 multiply and add counted as 2 ops", "frac": c1["kernel_tops"] / INT8_MFMA_PEAK_TOPS,
                     "frac_of_peak_from_device_properties": c1["kernel_tops"] / device_peaks(info)["int8_mfma_from_device_tops"],
                     "traffic": config1_traffic_bytes(),
                     "kernel": CONFIG1_KERNEL, "kernel_ms": c1["kernel_ms"],
                     "algorithmic_bytes": c1["algorithmic_bytes"],
                     "hbm_frac_if_bandwidth_bound": c1["algorithmic_bytes"] / (c1["kernel_ms"] * 1e-3) / 1e9 /
                     HBM_PEAK_GBS},
        "cpu_baseline": cpu,
        "peaks": device_peaks(info),
        "timing": f"ms_per_step: median of {c1['rounds']} rounds of {args.steps} launches "
                  f"(min {c1['ms_per_step_min_max'][0]:.5f}, max {c1['ms_per_step_min_max'][1]:.5f} ms)",
        "bit_exact_vs_oracle": parity_ok,
        "copy_kernel_gbs": copy_gbs,
        "host_buffers_ms_per_step": c1["host_buffers_ms_per_step"],
        "launches_in_flight": c1["launches_in_flight"],
    }
    line.update(extra)
    print(json.dumps(line), flush=True)
    dev.close()


if __name__ == "__main__":
    main()
