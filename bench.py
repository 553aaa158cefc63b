#!/usr/bin/env python3
"""Benchmark of the GEMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu] [--no-extra]

One step = one GEMM launch on operands already resident in HBM.  The headline line is the
fp32 M=N=K=8192 product (dense fp32 MFMA roof); the same JSON line carries the fp16 4096^3
product (dense fp16 MFMA roof) and the bandwidth-bound shapes under "other_workloads".
The kernel time is measured with HIP events recorded on the launch stream.  The CPU
baseline is the in-repo AVX2 restatement of the reference's multithreaded CPU GEMM, timed
on the host cores on the same workload (every fp32 workload of the baseline's configurations
carries its own: thread count stated, best of a few calls for the short ones) and checked
bit-for-bit against the scalar fma chain on sampled rows; every GEMM workload also carries
the GPU result's error against the CPU result or, where the reference has no CPU form, against
the chain on sampled rows ("gpu_parity").
"""
import argparse
import math
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_F32_TFLOPS = 157.3      # MI355X dense fp32 matrix
PEAK_F16_TFLOPS = 2500.0     # MI355X dense fp16 matrix
PEAK_F64_TFLOPS = 78.6       # MI355X dense fp64 matrix
PEAK_HBM_GBS = 8000.0        # MI355X HBM3E

# Bytes per launch that crossed the L2 <-> fabric boundary (HBM or the memory-side cache behind it), recorded from
# rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE in KiB per dispatch, scaled by what the same counters read for a copy
# kernel of known size) of this same file's workloads.  Each figure names the profile that holds it and the source
# file of the kernel it was measured on with that file's SHA-256 at the time: when the kernel source has changed
# since, the figure is withheld ("traffic": null, "traffic_stale": true) until the workload is profiled again.  It is
# withheld as well when the planner now picks another tile, grid or split of K than the launch that was profiled
# ("plan": what decx_hip_gemm_plan reported then).
MEASURED_TRAFFIC = {
    "fp32_8192": {"plan": {"tile": [256, 128], "grid": 2048, "k_splits": 1, "whole_tiles": 0},
             "bytes": 5.67e9, "counters": "FETCH_SIZE 2.6357e6 x 2.0 KiB + WRITE_SIZE 2.621e5 KiB (FETCH_SIZE 2.64e6 ... 3.40e6 from run to run)",
                  "kernel": "gemm_f32_dma_kernel<256, 128, 2, 2, 16, 2, false, 0, false, false>", "source": "decx_amd/csrc/gemm_f32_dma.hip",
                  "source_sha256": "05e995711ad2ff03fbcdb66fe8e73d86fadc8c04529cec00e667e61192f79bc9", "profile": "profiles/gemm_f32_dma_fp32_8192cubed.md"},
    "fp16_4096": {"plan": {"tile": [256, 256], "grid": 256, "k_splits": 1, "whole_tiles": 0},
             "bytes": 2.35e8, "counters": "FETCH_SIZE 98 543 x 2.0 KiB + WRITE_SIZE 32 772 KiB",
                  "kernel": "gemm_f16_dma_kernel<256, 256, 2, 4, 64, 2, false>", "source": "decx_amd/csrc/gemm_f16_dma.hip",
                  "source_sha256": "2b04e868882c6407c3754860b2f2ac9b2e3ee34ede28e59ee9a4296e973c1d22", "profile": "profiles/gemm_f16_dma_fp16_4096cubed.md"},
    "fp16_3000": {"plan": {"tile": [192, 192], "grid": 256, "k_splits": 1, "whole_tiles": 0},
        "bytes": 1.29e8, "counters": "FETCH_SIZE 53 033 x 2.0 KiB + WRITE_SIZE 19 829 KiB",
                  "kernel": "gemm_f16_dma_kernel<192, 192, 4, 2, 64, 2, false>", "source": "decx_amd/csrc/gemm_f16_dma.hip",
                  "source_sha256": "2b04e868882c6407c3754860b2f2ac9b2e3ee34ede28e59ee9a4296e973c1d22", "profile": "profiles/gemm_f16_dma_tiles_of_192_and_last_round_split.md"},
    "fp16_7000": {"plan": {"tile": [256, 256], "grid": 848, "k_splits": 5, "whole_tiles": 768},
        "bytes": 1.27e9, "counters": "FETCH_SIZE 563 674 x 2.0 KiB + WRITE_SIZE 116 314 KiB (operands, the output, and the slots of the 16 tiles that are split in five)",
                  "kernel": "gemm_f16_dma_kernel<256, 256, 2, 4, 64, 2, true>", "source": "decx_amd/csrc/gemm_f16_dma.hip",
                  "source_sha256": "2b04e868882c6407c3754860b2f2ac9b2e3ee34ede28e59ee9a4296e973c1d22", "profile": "profiles/gemm_f16_dma_tiles_of_192_and_last_round_split.md"},
    "fp64_4096": {"plan": {"tile": [256, 128], "grid": 512, "k_splits": 1, "whole_tiles": 0},
             "bytes": 1.21e9, "counters": "FETCH_SIZE 524 460 x 2.0 KiB + WRITE_SIZE 131 099 KiB",
                  "kernel": "gemm_f64_dma_kernel<256, 128, 4, 2, 16, 3, false>", "source": "decx_amd/csrc/gemm_f64.hip",
                  "source_sha256": "9b5e3fa596b998df4fc2b5621237519022c52fca841bb3593d9a27a39c34f335", "profile": "profiles/gemm_f64_dma_fp64_4096cubed.md"},
    "fp32_1024": {"plan": {"tile": [64, 64], "grid": 256, "k_splits": 1, "whole_tiles": 0},
             "bytes": 2.95e7, "counters": "FETCH_SIZE 12 345 x 2.0 KiB + WRITE_SIZE 4 096 KiB",
                  "kernel": "gemm_f32_dma_kernel<64, 64, 2, 2, 32, 2, true, 0, false, false>", "source": "decx_amd/csrc/gemm_f32_dma.hip",
                  "source_sha256": "05e995711ad2ff03fbcdb66fe8e73d86fadc8c04529cec00e667e61192f79bc9", "profile": "profiles/gemm_f32_dma_small_and_ragged.md"},
    "fp32_ragged": {"plan": {"tile": [64, 64], "grid": 512, "k_splits": 2, "whole_tiles": 256},
               "bytes": 4.43e7, "counters": "FETCH_SIZE 16 662 x 2.0 KiB + WRITE_SIZE 9 983 KiB (operands, and the slots of the 128 tiles that are split in two; 256 tiles are whole)",
                    "kernel": "gemm_f32_dma_kernel<64, 64, 2, 2, 32, 2, true, 0, true, false>", "source": "decx_amd/csrc/gemm_f32_dma.hip",
                    "source_sha256": "05e995711ad2ff03fbcdb66fe8e73d86fadc8c04529cec00e667e61192f79bc9", "profile": "profiles/gemm_f32_dma_small_and_ragged.md"},
    "fp32_ragged_abc": {"plan": {"tile": [64, 64], "grid": 512, "k_splits": 2, "whole_tiles": 256},
                   "bytes": 5.04e7, "counters": "FETCH_SIZE 19 595 x 2.0 KiB + WRITE_SIZE 9 983 KiB",
                        "kernel": "gemm_f32_dma_kernel<64, 64, 2, 2, 32, 2, true, 0, true, true>", "source": "decx_amd/csrc/gemm_f32_dma.hip",
                        "source_sha256": "05e995711ad2ff03fbcdb66fe8e73d86fadc8c04529cec00e667e61192f79bc9", "profile": "profiles/gemm_f32_dma_small_and_ragged.md"},
    "fp32_tall_skinny": {"plan": {"tile": [256, 128], "grid": 512, "k_splits": 1, "whole_tiles": 0},
                    "bytes": 3.58e8, "counters": "FETCH_SIZE 142 002 x 2.0 KiB + WRITE_SIZE 65 541 KiB",
                         "kernel": "gemm_f32_dma_kernel<256, 128, 2, 2, 16, 2, false, 0, false, false>", "source": "decx_amd/csrc/gemm_f32_dma.hip",
                         "source_sha256": "05e995711ad2ff03fbcdb66fe8e73d86fadc8c04529cec00e667e61192f79bc9", "profile": "profiles/gemm_f32_dma_small_and_ragged.md"},
    "fp32_mid_long_k": {"plan": {"tile": [64, 64], "grid": 512, "k_splits": 4, "whole_tiles": 256},
                   "bytes": 3.12e8, "counters": "FETCH_SIZE 147 815 x 2.0 KiB + WRITE_SIZE 9 226 KiB (operands, and the slots of the 64 tiles that are split in four; 256 tiles are whole)",
                        "kernel": "gemm_f32_dma_kernel<64, 64, 2, 2, 32, 2, true, 0, true, false>", "source": "decx_amd/csrc/gemm_f32_dma.hip",
                        "source_sha256": "05e995711ad2ff03fbcdb66fe8e73d86fadc8c04529cec00e667e61192f79bc9", "profile": "profiles/split_k_mid_size_and_direct_conv.md"},
    "fp32_gemv": {"plan": {"tile": [32, 1], "grid": 256, "k_splits": 1, "whole_tiles": 0},
             "bytes": 2.69e8, "counters": "FETCH_SIZE 131 258 x 2.0 KiB + WRITE_SIZE 32 KiB (x and y are dense columns)",
                  "kernel": "gemv_kernel<float, float, 2, 1>", "source": "decx_amd/csrc/gemv.hip",
                  "source_sha256": "bd1e8a2fd885c5a4483c53bea615087b75da480171828cff8a68b201a3d6b229", "profile": "profiles/gemv_gevm_8192x8192.md"},
    "fp32_gevm": {"plan": {"tile": [1, 32], "grid": 256, "k_splits": 1, "whole_tiles": 0},
             "bytes": 2.69e8, "counters": "FETCH_SIZE 131 241 x 2.0 KiB + WRITE_SIZE 32 KiB",
                  "kernel": "gevm_kernel<float, float, 8>", "source": "decx_amd/csrc/gemv.hip",
                  "source_sha256": "bd1e8a2fd885c5a4483c53bea615087b75da480171828cff8a68b201a3d6b229", "profile": "profiles/gemv_gevm_8192x8192.md"},
    "fp16_gemv": {"plan": {"tile": [32, 1], "grid": 256, "k_splits": 1, "whole_tiles": 0},
             "bytes": 1.34e8, "counters": "FETCH_SIZE 65 659 x 2.0 KiB + WRITE_SIZE 16 KiB (x and y are dense columns)",
                  "kernel": "gemv_kernel<_Float16, _Float16, 2, 1>", "source": "decx_amd/csrc/gemv.hip",
                  "source_sha256": "bd1e8a2fd885c5a4483c53bea615087b75da480171828cff8a68b201a3d6b229", "profile": "profiles/gemv_gevm_8192x8192.md"},
    "fp16_gevm": {"plan": {"tile": [1, 64], "grid": 256, "k_splits": 2, "whole_tiles": 0},
             "bytes": 1.35e8, "counters": "FETCH_SIZE 65 683 x 2.0 KiB + WRITE_SIZE 92 KiB",
                  "kernel": "gevm_kernel<_Float16, _Float16, 8>", "source": "decx_amd/csrc/gemv.hip",
                  "source_sha256": "bd1e8a2fd885c5a4483c53bea615087b75da480171828cff8a68b201a3d6b229", "profile": "profiles/gemv_gevm_8192x8192.md"},
    "conv2d": {"bytes": 1.08e8, "counters": "FETCH_SIZE 20 527 x 2.0 KiB + WRITE_SIZE 64 546 KiB",
               "kernel": "gemm_f32_dma_kernel<256, 256, 2, 4, 16, 4, false, 2, false, false>", "source": "decx_amd/csrc/gemm_f32_dma.hip",
               "source_sha256": "05e995711ad2ff03fbcdb66fe8e73d86fadc8c04529cec00e667e61192f79bc9", "profile": "profiles/conv2d_implicit_gemm_256x256x112_3x3x256.md"},
    "conv2d_rgb": {"bytes": 1.01e8, "counters": "FETCH_SIZE 16 457 x 2.0 KiB + WRITE_SIZE 66 138 KiB",
                   "kernel": "conv2d_direct_kernel<8, 3>", "source": "decx_amd/csrc/conv_direct.hip",
                   "source_sha256": "c7eb7cf36f24f0ea5cbad9b81e882fd40584839840d91afe1e302abf4bd8fcc0", "profile": "profiles/split_k_mid_size_and_direct_conv.md"},
}


def strip_comment(line):
    """The code of a C++ source line: everything in front of a `//` that is not inside a string literal."""
    quoted = False
    i = 0
    while i < len(line):
        c = line[i]
        if c == "\\" and quoted:
            i += 2
            continue
        if c == '"':
            quoted = not quoted
        elif c == "/" and not quoted and line[i:i + 2] == "//":
            return line[:i].strip()
        i += 1
    return line.strip()


def sources_sha256(source):
    """SHA-256 over the code of a kernel's source file and of the headers the kernels share (the argument block and
    block -> tile map, and where the ranges of a split K meet).  `//` comments, indentation and empty lines are left
    out: a note added to a source file changes no kernel."""
    import hashlib
    h = hashlib.sha256()
    try:
        for f in (source, "decx_amd/csrc/gemm_common.hpp", "decx_amd/csrc/split_k_exchange.hpp"):
            for line in open(os.path.join(ROOT, f), "r", encoding="utf-8"):
                code = strip_comment(line)
                if code:
                    h.update(code.encode("utf-8") + b"\n")
    except OSError:
        return None
    return h.hexdigest()


def traffic_fields(name, plan=None):
    """{"traffic": bytes or None, "traffic_measured_at": ...} for a roofline object.  plan: what the planner reports
    for the workload now (tile, grid, k_splits, whole_tiles)."""
    rec = MEASURED_TRAFFIC.get(name)
    if rec is None:
        return {"traffic": None}
    now = sources_sha256(rec["source"])
    at = {"kernel": rec["kernel"], "source": rec["source"], "source_sha256": rec["source_sha256"][:16],
          "profile": rec["profile"], "counters": rec["counters"]}
    if now is None or now != rec["source_sha256"]:
        return {"traffic": None, "traffic_stale": True, "traffic_measured_at": at}
    if plan is not None and "plan" in rec and any(plan.get(k) != v for k, v in rec["plan"].items()):
        at["plan"] = rec["plan"]
        return {"traffic": None, "traffic_stale": True, "traffic_stale_reason": "the planner's choice has changed", "traffic_measured_at": at}
    return {"traffic": rec["bytes"], "traffic_measured_at": at}


WORKLOADS = {
    # name: (dtype, M, N, K, bound, config number for seeds, description)
    "fp32_8192": ("f32", 8192, 8192, 8192, "mfma", 4, "fp32 GEMM C=A.B M=N=K=8192, uniform[-1,1]"),
    "fp16_4096": ("f16", 4096, 4096, 4096, "mfma", 3, "fp16 GEMM (fp32 accumulate, fp16 out) M=N=K=4096, normal(0,0.5) clipped to [-4,4]"),
    "fp16_3000": ("f16", 3000, 3000, 3000, "mfma", 9, "fp16 GEMM M=N=K=3000 (256 tiles of 192 x 192 where 256 x 256 gives 144 for 256 CUs), normal(0,0.5)"),
    "fp16_7000": ("f16", 7000, 7000, 7000, "mfma", 10, "fp16 GEMM M=N=K=7000 (784 tiles of 256 x 256: three rounds whole, the 16 of the last round split along K), normal(0,0.5)"),
    "fp64_4096": ("f64", 4096, 4096, 4096, "mfma", 7, "fp64 GEMM M=N=K=4096, uniform[-1,1]"),
    "fp32_1024": ("f32", 1024, 1024, 1024, "mfma", 1, "fp32 GEMM M=N=K=1024, uniform[-1,1]"),
    "fp32_ragged": ("f32", 1000, 1500, 777, "mfma", 2, "fp32 GEMM M=1000 N=1500 K=777, uniform[-1,1]"),
    "fp32_ragged_abc": ("f32", 1000, 1500, 777, "mfma", 2, "fp32 GEMM D=A.B+C M=1000 N=1500 K=777 (four-matrix entry, alpha=beta=1), uniform[-1,1]"),
    "fp32_tall_skinny": ("f32", 65536, 256, 1024, "mfma", 5, "fp32 GEMM M=65536 N=256 K=1024, uniform[-1,1]"),
    "fp32_mid_long_k": ("f32", 1280, 1024, 8192, "mfma", 8, "fp32 GEMM M=1280 N=1024 K=8192 (320 small tiles: 256 whole, 64 split along K through the workspace), uniform[-1,1]"),
    "fp32_gemv": ("f32", 8192, 1, 8192, "hbm", 6, "fp32 GEMM M=8192 N=1 K=8192 (GEMV-like), uniform[-1,1]"),
    "fp32_gevm": ("f32", 1, 8192, 8192, "hbm", 6, "fp32 GEMM M=1 N=8192 K=8192 (vector x matrix), uniform[-1,1]"),
    "fp16_gemv": ("f16", 8192, 1, 8192, "hbm", 6, "fp16 GEMM M=8192 N=1 K=8192 (fp32 accumulate), normal(0,0.5)"),
    "fp16_gevm": ("f16", 1, 8192, 8192, "hbm", 6, "fp16 GEMM M=1 N=8192 K=8192 (fp32 accumulate), normal(0,0.5)"),
}


def make_inputs(name):
    from decx_amd import synth
    dt, M, N, K, _, cfg, _ = WORKLOADS[name]
    sa, sb, _ = synth.seeds(cfg)
    if dt == "f32":
        return synth.uniform_f32(M, K, sa), synth.uniform_f32(K, N, sb)
    if dt == "f64":
        return synth.uniform_f64(M, K, sa), synth.uniform_f64(K, N, sb)
    return synth.normal_half(M, K, sa), synth.normal_half(K, N, sb)


def device_pitch(cols, itemsize):
    """Row pitch in elements as de::GPU_Matrix lays a matrix out: rows padded to 128 bytes, a single column dense."""
    if cols == 1:
        return 1
    per = 128 // itemsize
    return (cols + per - 1) // per * per


def run_workload(name, steps, warmup, keep_inputs=False, settle_s=0.0):
    from decx_amd import hip, synth
    dt, M, N, K, bound, cfg, desc = WORKLOADS[name]
    npdt = {"f32": np.float32, "f16": np.float16, "f64": np.float64}[dt]
    A, B = make_inputs(name)
    C = synth.uniform_f32(M, N, synth.seeds(cfg)[2]) if name.endswith("_abc") else None
    isz = np.dtype(npdt).itemsize
    dA = hip.DeviceMatrix(M, K, npdt, device_pitch(K, isz), A)
    dB = hip.DeviceMatrix(K, N, npdt, device_pitch(N, isz), B)
    dC = hip.DeviceMatrix(M, N, npdt, device_pitch(N, isz), C) if C is not None else None
    dD = hip.DeviceMatrix(M, N, npdt, device_pitch(N, isz))
    # the workspace the library asks for (split K, the dense copy of a column operand), held by the caller as the
    # de:: layer holds it; none for most shapes
    need = int(hip.lib().decx_hip_gemm_workspace(isz, M, N, K))
    ws = hip.DeviceMatrix(1, need // 4, np.float32) if need else None
    call = lambda: hip.gemm(dA, dB, dD, dC, 1.0, 1.0, workspace=ws)
    for _ in range(warmup):
        call()
    hip.sync()
    # short kernels: keep launching until the clocks have settled (the first milliseconds after
    # idle run at ramping clocks and would be what a 20-launch measurement sees)
    t_settle = time.perf_counter()
    while time.perf_counter() - t_settle < settle_s:
        for _ in range(10):
            call()
        hip.sync()
    timer = hip.Timer()
    t0 = time.perf_counter()
    timer.start()
    for _ in range(steps):
        call()
    kernel_ms = timer.stop() / steps            # HIP events on the launch stream
    hip.sync()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    flops = 2.0 * M * N * K
    abytes = float(isz) * (M * K + K * N + M * N + (M * N if C is not None else 0))
    tflops = flops / (kernel_ms * 1e-3) / 1e12
    gbs = abytes / (kernel_ms * 1e-3) / 1e9
    if bound == "mfma":
        peak = {"f32": PEAK_F32_TFLOPS, "f16": PEAK_F16_TFLOPS, "f64": PEAK_F64_TFLOPS}[dt]
        roof = {"bound": "mfma", "achieved": round(tflops, 3), "peak": peak, "unit": "TFLOP/s",
                "frac": round(tflops / peak, 4)}
    else:
        roof = {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                "frac": round(gbs / PEAK_HBM_GBS, 4)}
    p = hip.plan(isz, M, N, K)
    roof.update(traffic_fields(name, {"tile": [int(p.tile_m), int(p.tile_n)], "grid": int(p.grid), "k_splits": int(p.k_splits),
                                      "whole_tiles": int(p.whole_tiles)}))
    out = {"name": name, "workload": desc, "dtype": dt, "value": round(tflops, 3), "unit": "TFLOP/s",
           "hbm_gbs_algorithmic": round(gbs, 1), "kernel_ms": round(kernel_ms, 5), "wall_ms_per_step": round(wall_ms, 5),
           "plan": {"path": int(p.path), "tile": [int(p.tile_m), int(p.tile_n)], "grid": int(p.grid), "edge": int(p.edge),
                    "k_splits": int(p.k_splits), "whole_tiles": int(p.whole_tiles), "workspace_bytes": need},
           "roofline": roof}
    result = (out, (A, B, C, dD.download()) if keep_inputs else None)    # the result goes to the CPU leg's comparison
    for d in (dA, dB, dC, dD, ws):
        if d is not None:
            d.free()
    return result


def sustained_mfma(seconds=0.5, launches=50):
    """What the fp16 matrix pipe sustains on this board with nothing else to do: the library's register-only loop of
    v_mfma_f32_16x16x32_f16 (decx_hip_calibration_mfma: no loads, no LDS, no barriers) on operands drawn like the fp16
    workload's, timed after the clocks have settled.  The nominal peak assumes 2.4 GHz; with operands that toggle the
    multipliers' inputs the board's power management allows less (the same loop on zeros runs near nominal), and this
    is the rate it allows the instruction stream alone.  (No fp32 twin: the fp32 GEMM kernel runs at the nominal
    clock, and a bare loop of its MFMAs draws more than the kernel does and comes out slower.)"""
    import ctypes
    from decx_amd import hip, synth
    L = hip.lib()
    cus = int(hip.device_props().compute_units)
    sink = hip.DeviceMatrix(1, cus * 512, np.float32)
    flops = ctypes.c_double()
    out = {}
    for label, ops in (("value", synth.normal_half(1024, 2048, 0xCA16)), ("on_zero_operands", np.zeros((1024, 2048), np.float16))):
        d_ops = hip.DeviceMatrix(ops.shape[0], ops.shape[1], ops.dtype, data=ops)
        # 1024 rounds of 16 tiles per wavefront: twice the flops of a 4096^3 product, so that launch gaps do not show
        call = lambda: hip.check(L.decx_hip_calibration_mfma(2, d_ops.ptr, ops.nbytes, sink.ptr, cus * 512, 1024, ctypes.byref(flops), None))
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < seconds:
            for _ in range(10):
                call()
            hip.sync()
        timer = hip.Timer(); timer.start()
        for _ in range(launches):
            call()
        ms = timer.stop() / launches
        out[label] = round(flops.value / (ms * 1e-3) / 1e12, 1)
        d_ops.free()
    sink.free()
    out.update({"unit": "TFLOP/s", "frac_of_nominal": round(out["value"] / PEAK_F16_TFLOPS, 4),
                "implied_clock_ghz": round(2.4 * out["value"] / PEAK_F16_TFLOPS, 3),
                "kernel": "register-only loop of v_mfma_f32_16x16x32_f16, 8 wavefronts per CU, operands N(0, 0.5) halves as in the "
                          "workload (on_zero_operands: the same loop on zeros)"})
    return out


def zero_operand_rate(name, launches=50, seconds=0.5):
    """TFLOP/s of a GEMM workload's launch on all-zero operands of the same shape: the same instructions, but nothing
    toggles in the multipliers, so the board's power management does not hold the clock down.  It shows what the
    kernel's schedule reaches when power is not the limit; the workload's own figure is measured on its own data."""
    from decx_amd import hip
    dt, M, N, K = WORKLOADS[name][:4]
    npdt = {"f32": np.float32, "f16": np.float16}[dt]
    isz = np.dtype(npdt).itemsize
    dA = hip.DeviceMatrix(M, K, npdt, device_pitch(K, isz), np.zeros((M, K), npdt))
    dB = hip.DeviceMatrix(K, N, npdt, device_pitch(N, isz), np.zeros((K, N), npdt))
    dD = hip.DeviceMatrix(M, N, npdt, device_pitch(N, isz))
    call = lambda: hip.gemm(dA, dB, dD)
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(10):
            call()
        hip.sync()
    timer = hip.Timer(); timer.start()
    for _ in range(launches):
        call()
    ms = timer.stop() / launches
    for d in (dA, dB, dD):
        d.free()
    return round(2.0 * M * N * K / (ms * 1e-3) / 1e12, 1)


def copy_rate(steps=10, warmup=3):
    """Read + write GB/s of the library's plain copy kernel over 1 GiB: the memory system's rate for traffic that is
    half writes, the yardstick for the write-heavy workloads (the nominal 8 TB/s is a read figure)."""
    from decx_amd import hip
    n = 1 << 30
    src = hip.DeviceMatrix(1, n // 4, np.float32); dst = hip.DeviceMatrix(1, n // 4, np.float32)
    hip.check(hip.lib().decx_hip_memset_async(src.ptr, 1, n, None))
    for _ in range(warmup):
        hip.check(hip.lib().decx_hip_calibration_copy(dst.ptr, src.ptr, n, None))
    hip.sync()
    timer = hip.Timer(); timer.start()
    for _ in range(steps):
        hip.check(hip.lib().decx_hip_calibration_copy(dst.ptr, src.ptr, n, None))
    ms = timer.stop() / steps
    # and a write-only pass over the same gigabyte (the runtime's fill kernel behind decx_hip_memset_async)
    for _ in range(warmup):
        hip.check(hip.lib().decx_hip_memset_async(dst.ptr, 0, n, None))
    hip.sync()
    timer.start()
    for _ in range(steps):
        hip.check(hip.lib().decx_hip_memset_async(dst.ptr, 0, n, None))
    fill_ms = timer.stop() / steps
    # and a read-only pass over both gigabytes, laid end to end: far more than the 256 MB memory-side cache holds
    for d in (src, dst):
        d.free()
    both = hip.DeviceMatrix(1, 2 * n // 4, np.float32)
    sink = hip.DeviceMatrix(1, 2 * n // 2048, np.uint32)
    hip.check(hip.lib().decx_hip_memset_async(both.ptr, 1, 2 * n, None))
    for _ in range(warmup):
        hip.check(hip.lib().decx_hip_calibration_read(both.ptr, 2 * n, sink.ptr, 2 * n // 2048, None))
    hip.sync()
    timer.start()
    for _ in range(steps):
        hip.check(hip.lib().decx_hip_calibration_read(both.ptr, 2 * n, sink.ptr, 2 * n // 2048, None))
    read_ms = timer.stop() / steps
    for d in (both, sink):
        d.free()
    return {"value": round(2 * n / ms / 1e6, 1), "unit": "GB/s", "what": "calibration copy kernel, 1 GiB read + 1 GiB written per launch",
            "kernel_ms": round(ms, 4), "write_only_gbs": round(n / fill_ms / 1e6, 1), "write_only_what": "fill of 1 GiB (hipMemsetAsync)",
            "read_only_gbs": round(2 * n / read_ms / 1e6, 1), "read_only_what": "calibration read kernel over 2 GiB (128-bit loads in the order the matrix x vector kernel reads rows of 64 KB, nothing stored)"}


def gemv_sizes(launches=50, batches=5):
    """y = A.x through decx_hip_gemm_* on matrices of 2 MB to 2 GB (fp32 and fp16, dense x): time against size separates
    what a launch costs whatever it moves from the rate at which the rows stream once they do.  Matrices beyond the
    256 MB of the memory-side cache show the rate of HBM itself; the smaller ones are partly served by that cache from
    launch to launch."""
    from decx_amd import hip
    rows = []
    for dt, name in ((np.float32, "f32"), (np.float16, "f16")):
        for M, K in ((8192, 64), (8192, 512), (8192, 2048), (8192, 4096), (8192, 8192), (8192, 16384), (16384, 8192), (32768, 8192),
                     (65536, 8192), (32768, 16384), (65536, 4096), (262144, 1024)):
            A = hip.DeviceMatrix(M, K, dt, K); X = hip.DeviceMatrix(K, 1, dt, 1); Y = hip.DeviceMatrix(M, 1, dt, 1)
            hip.check(hip.lib().decx_hip_memset_async(A.ptr, 0, M * K * np.dtype(dt).itemsize, None))
            for _ in range(10):
                hip.gemm(A, X, Y)
            hip.sync()
            timer = hip.Timer(); best = 1e30
            for _ in range(batches):
                timer.start()
                for _ in range(launches):
                    hip.gemm(A, X, Y)
                best = min(best, timer.stop() / launches)
            mb = M * K * np.dtype(dt).itemsize / 1e6
            rows.append({"dtype": name, "M": M, "K": K, "matrix_MB": round(mb, 1), "kernel_us": round(best * 1e3, 2),
                         "GB/s": round(mb / best, 1)})
            for d in (A, X, Y):
                d.free()
    # the transposed form, y = x.B (K x N), with the workspace its split over ranges of K wants
    gevm_rows = []
    for dt, name in ((np.float32, "f32"), (np.float16, "f16")):
        esz = np.dtype(dt).itemsize
        for K, N in ((8192, 8192), (32768, 8192), (8192, 32768), (131072, 2048)):
            B = hip.DeviceMatrix(K, N, dt, N); X = hip.DeviceMatrix(1, K, dt, K); Y = hip.DeviceMatrix(1, N, dt, N)
            hip.check(hip.lib().decx_hip_memset_async(B.ptr, 0, K * N * esz, None))
            need = int(hip.lib().decx_hip_gemm_workspace(esz, 1, N, K))
            W = hip.DeviceMatrix(1, max(need // 4, 4), np.float32)
            for _ in range(10):
                hip.gemm(X, B, Y, workspace=W)
            hip.sync()
            timer = hip.Timer(); best = 1e30
            for _ in range(batches):
                timer.start()
                for _ in range(launches):
                    hip.gemm(X, B, Y, workspace=W)
                best = min(best, timer.stop() / launches)
            mb = K * N * esz / 1e6
            gevm_rows.append({"dtype": name, "K": K, "N": N, "matrix_MB": round(mb, 1), "kernel_us": round(best * 1e3, 2),
                              "GB/s": round(mb / best, 1), "k_splits": int(hip.plan(esz, 1, N, K).k_splits)})
            for d in (B, X, Y, W):
                d.free()
    big = [r for r in rows if r["matrix_MB"] > 1000]
    return {"workload": "gemv over matrix sizes", "launches": launches, "batches": batches, "rows": rows, "gevm_rows": gevm_rows,
            "floor_us": min(r["kernel_us"] for r in rows), "streaming_GB/s": max(r["GB/s"] for r in big)}


def launch_floor(launches=200, batches=3):
    """Microseconds from launch to launch of a kernel that has next to nothing to do (y = A.x on a 2 MB matrix, one
    workgroup per CU): what any single launch costs on this board before its own work counts."""
    from decx_amd import hip
    M, K = 8192, 64
    A = hip.DeviceMatrix(M, K, np.float32, K); X = hip.DeviceMatrix(K, 1, np.float32, 1); Y = hip.DeviceMatrix(M, 1, np.float32, 1)
    hip.check(hip.lib().decx_hip_memset_async(A.ptr, 0, M * K * 4, None))
    for _ in range(20):
        hip.gemm(A, X, Y)
    hip.sync()
    timer = hip.Timer(); best = 1e30
    for _ in range(batches):
        timer.start()
        for _ in range(launches):
            hip.gemm(A, X, Y)
        best = min(best, timer.stop() / launches)
    for d in (A, X, Y):
        d.free()
    return round(best * 1e3, 2)


def add_sustained(out, sustained):
    """Puts the in-run sustained matrix rate beside a workload's nominal roofline."""
    roof = out["roofline"]
    roof["sustained"] = dict(sustained, frac_of_sustained=round(roof["achieved"] / sustained["value"], 4))
    return out


CONV = {"W": 256, "H": 256, "C": 112, "OC": 256, "KW": 3, "KH": 3}     # 64 516 pixels x 256 channels x 1008 taps
CONV_RGB = {"W": 1920, "H": 1080, "C": 3, "OC": 8, "KW": 3, "KH": 3}    # a filter bank over an RGB frame: 36 taps, bound by HBM


def run_conv(steps, warmup, settle_s=0.25, c=None, parity=False):
    """fp32 3 x 3 convolution of a 256 x 256 x 112 image with 256 kernels through decx_hip_conv2d_f32_depth (implicit GEMM,
    operands resident): the workload the tall-skinny GEMM shape 65536 x 256 x 1024 stands for.  c: another
    configuration (CONV_RGB: a shallow patch and few kernels, which the library runs a lane per output pixel)."""
    from decx_amd import hip, synth
    c = c or CONV
    L = hip.lib()
    dp, wp = (c["C"] + 3) // 4 * 4, (c["W"] + 7) // 8 * 8
    img = np.zeros((c["H"], wp, dp), np.float32)
    img[:, :c["W"], :c["C"]] = synth.uniform_f32(c["H"], c["W"] * c["C"], 0xA007).reshape(c["H"], c["W"], c["C"])
    d_img = hip.DeviceMatrix(c["H"], wp * dp, np.float32, data=img.reshape(c["H"], -1))
    K = c["KH"] * c["KW"] * dp
    kmat = np.zeros((K, c["OC"]), np.float32)
    kmat.reshape(c["KH"] * c["KW"], dp, c["OC"])[:, :c["C"], :] = synth.uniform_f32(c["KH"] * c["KW"] * c["C"], c["OC"], 0xB007).reshape(-1, c["C"], c["OC"])
    d_kmat = hip.DeviceMatrix(K, c["OC"], np.float32, data=kmat)
    ow, oh = c["W"] - c["KW"] + 1, c["H"] - c["KH"] + 1
    owp = (ow + 7) // 8 * 8
    d_out = hip.DeviceMatrix(oh, owp * c["OC"], np.float32)
    call = lambda: hip.check(L.decx_hip_conv2d_f32_depth(d_img.ptr, d_kmat.ptr, d_out.ptr, ow, oh, c["OC"], c["KW"], c["KH"], c["C"], dp, wp,
                                                   1, 1, c["OC"], c["OC"], owp, None))
    for _ in range(warmup):
        call()
    hip.sync()
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < settle_s:
        for _ in range(10):
            call()
        hip.sync()
    timer = hip.Timer(); timer.start()
    for _ in range(steps):
        call()
    ms = timer.stop() / steps
    flops = 2.0 * ow * oh * c["OC"] * c["KH"] * c["KW"] * c["C"]
    abytes = 4.0 * (c["H"] * c["W"] * c["C"] + c["KH"] * c["KW"] * c["C"] * c["OC"] + ow * oh * c["OC"])
    tf = flops / (ms * 1e-3) / 1e12
    gbs = abytes / (ms * 1e-3) / 1e9
    desc = "fp32 conv2D %dx%d, image %dx%dx%d, %d kernels (%d x %d x %d as a GEMM), uniform[-1,1]" % (
        c["KW"], c["KH"], c["W"], c["H"], c["C"], c["OC"], ow * oh, c["OC"], K)
    if c is CONV:
        roof = {"bound": "mfma", "achieved": round(tf, 3), "peak": PEAK_F32_TFLOPS, "unit": "TFLOP/s",
                "frac": round(tf / PEAK_F32_TFLOPS, 4)}
        roof.update(traffic_fields("conv2d"))
    else:                                        # 16 flop per byte: the memory system bounds it
        roof = {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                "frac": round(gbs / PEAK_HBM_GBS, 4)}
        roof.update(traffic_fields("conv2d_rgb"))
    out = {"name": "conv2d" if c is CONV else "conv2d_rgb", "workload": desc, "dtype": "f32", "value": round(tf, 3), "unit": "TFLOP/s", "hbm_gbs_algorithmic": round(gbs, 1),
           "kernel_ms": round(ms, 5), "roofline": roof}
    if parity:
        # bands of output rows against the oracle's fmaf chain over (kernel row, kernel column, channel) on the image
        # rows under them
        from oracle import binding as oracle
        got = d_out.download().reshape(oh, owp, c["OC"])[:, :ow, :]
        kernels = kmat.reshape(c["KH"], c["KW"], dp, c["OC"])[:, :, :c["C"], :].transpose(3, 0, 1, 2)
        worst, scale, count = 0.0, 1e-30, 0
        for r0 in (0, oh // 2 - 1, oh - 2):
            ref = oracle.conv2d_f32(img[r0:r0 + 2 + c["KH"] - 1, :c["W"], :c["C"]], kernels).astype(np.float64)
            worst = max(worst, float(np.max(np.abs(got[r0:r0 + 2].astype(np.float64) - ref))))
            scale = max(scale, float(np.max(np.abs(ref)))); count += ref.size
        taps = c["KH"] * c["KW"] * c["C"]
        out["cpu_baseline"] = None               # the reference has no CPU convolution
        out["gpu_parity"] = {"rel_err": float("%.3g" % (worst / (scale * math.sqrt(taps)))), "bar": 1e-5, "elements": count,
                             "against": "fmaf chain oracle (oracle/conv_oracle.c)",
                             "measure": "max|gpu - chain| / (max|chain| sqrt(taps)) over 6 output rows"}
    for d in (d_img, d_kmat, d_out):
        d.free()
    return out


def run_complex(double, n, steps, warmup, settle_s=0.25, parity=False):
    """Complex GEMM D = A.B (interleaved re / im, n x n x n) through decx_hip_gemm_c32 / _c64 with a caller-held
    workspace: one pass expanding B, then one real GEMM on the fp32 / fp64 matrix pipe.  8 real flops per complex
    multiply-add; the expansion pass is inside the timed region."""
    from decx_amd import hip, synth
    L = hip.lib()
    cdt, rb = (np.complex128, 8) if double else (np.complex64, 4)
    draw = synth.uniform_f64 if double else synth.uniform_f32
    a = (draw(n, n, 0xA008) + 1j * draw(n, n, 0xA009)).astype(cdt)
    b = (draw(n, n, 0xB008) + 1j * draw(n, n, 0xB009)).astype(cdt)
    dA = hip.DeviceMatrix(n, n, cdt, n, a); dB = hip.DeviceMatrix(n, n, cdt, n, b); dD = hip.DeviceMatrix(n, n, cdt, n)
    need = L.decx_hip_gemm_complex_workspace(rb, n, n)
    ws = hip.DeviceMatrix(1, need // 16, np.complex128)
    fn = L.decx_hip_gemm_c64 if double else L.decx_hip_gemm_c32
    call = lambda: hip.check(fn(dA.ptr, dB.ptr, None, dD.ptr, n, n, n, n, n, 0, n, 1.0, 0.0, 1.0, 0.0, ws.ptr, need, None))
    for _ in range(warmup):
        call()
    hip.sync()
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < settle_s:
        call()
        hip.sync()
    timer = hip.Timer(); timer.start()
    for _ in range(steps):
        call()
    ms = timer.stop() / steps
    tf = 8.0 * n ** 3 / (ms * 1e-3) / 1e12
    peak = PEAK_F64_TFLOPS if double else PEAK_F32_TFLOPS
    out = {"name": "c128_%d" % n if double else "c64_%d" % n, "workload": "%s GEMM M=N=K=%d (real expansion of B + one %s GEMM), uniform[-1,1]" % (np.dtype(cdt).name, n, "fp64" if double else "fp32"),
           "dtype": "c128" if double else "c64", "value": round(tf, 3), "unit": "TFLOP/s",
           "hbm_gbs_algorithmic": round(3.0 * n * n * 2 * rb / (ms * 1e-3) / 1e9, 1), "kernel_ms": round(ms, 5),
           "roofline": {"bound": "mfma", "achieved": round(tf, 3), "peak": peak, "unit": "TFLOP/s", "frac": round(tf / peak, 4),
                        "traffic": None}}
    if parity:
        # sampled rows against the real chain oracle on the same expansion of B
        from oracle import binding as oracle
        rt = np.float64 if double else np.float32
        pick = np.unique(np.concatenate([[0, n - 1], np.random.default_rng(1).integers(0, n, 14)])).astype(np.uint32)
        fn = oracle.gemm_f64 if double else oracle.gemm_f32
        ref = fn(np.ascontiguousarray(a).view(rt), oracle.complex_embed(b), rows=pick).astype(np.float64)
        got = np.ascontiguousarray(dD.download()[pick]).view(rt).astype(np.float64)
        err = float(np.max(np.abs(got - ref))) / (float(np.max(np.abs(ref))) * math.sqrt(2 * n))
        out["cpu_baseline"] = None               # the reference's complex CPU GEMM is not restated as a timed port
        out["gpu_parity"] = {"rel_err": float("%.3g" % err), "bar": 1e-14 if double else 1e-5, "elements": int(len(pick)) * 2 * n,
                             "against": "fma chain oracle on the real expansion",
                             "measure": "max|gpu - chain| / (max|chain| sqrt(2K)) over %d sampled rows" % len(pick)}
    for d in (dA, dB, dD, ws):
        d.free()
    return out


# how the CPU leg runs each fp32 workload: (thread counts, calls per thread count -- the best one is reported)
CPU_LEGS = {
    "fp32_8192": ((16,), 1),            # ~1.4 s per call
    "fp32_1024": ((16,), 5),            # the one configuration the reference publishes a CPU time for (9.98 ms on its authors' host)
    "fp32_ragged": ((16,), 5),
    "fp32_ragged_abc": ((16,), 5),
    "fp32_tall_skinny": ((16,), 2),
    "fp32_gemv": ((1, 16), 3),          # the reference itself is only correct single-threaded on this shape
}


# ---- the planner against every other plan, on shapes it was not fitted on -------------------------------------------------

SWEEP_TILES = {"f32": {0: (256, 128), 1: (128, 128), 2: (64, 64)},
               "f16": {0: (256, 256), 1: (128, 128), 2: (64, 64), 3: (192, 192), 4: (192, 256), 5: (256, 192)},
               "f64": {0: (256, 128), 1: (128, 128), 2: (64, 64)}}
SWEEP_SPLIT_FIT = {"f32": {2: 4}, "f16": {2: 4, 1: 2, 0: 1}, "f64": {2: 2}}       # tile classes whose kernels split K: workgroups that share a CU


def sweep_shapes(seed, per_type, large=False):
    """Seeded shapes with log-uniform sides, none of them round: M, N in 40 .. 6500, K in 300 .. 14000, between 0.2 and
    150 GFLOP (fp64: 50); large: M, N in 1200 .. 9000, K in 500 .. 9000, up to 1200 GFLOP (fp64: 400)."""
    rng = np.random.default_rng(seed + (1 if large else 0))
    side = (1200, 9000) if large else (40, 6500)
    depth = (500, 9000) if large else (300, 14000)
    shapes = []
    for dt in ("f32", "f16", "f64"):
        got = 0
        cap = (4e11 if dt == "f64" else 1.2e12) if large else (5e10 if dt == "f64" else 1.5e11)
        while got < per_type:
            M, N = (int(math.exp(rng.uniform(math.log(side[0]), math.log(side[1])))) for _ in range(2))
            K = int(math.exp(rng.uniform(math.log(depth[0]), math.log(depth[1]))))
            flops = 2.0 * M * N * K
            if flops < 2e8 or flops > cap or M % 64 == 0 or N % 64 == 0:
                continue
            shapes.append((dt, M, N, K)); got += 1
    return shapes


def planner_sweep(seed=20261125, per_type=16, batches=3, launches=10, large=False, only=None):
    """Every shape runs on the planner's pick (the *_ws entry point with the workspace it asks for) and on every other
    plan there is a kernel for: each tile class whole, and K on 2 .. 32 ranges on the classes that split, for all
    tiles, for the tiles of a ragged last round, and for the tiles beyond one to three whole ones per CU.  A plan's
    time is the best of `batches` batches of `launches` launches (HIP events); the pick and the best other plan are
    then timed again in turns, and the ratio of those two is what the summary counts."""
    from decx_amd import hip, synth
    L = hip.lib()
    cus = int(hip.device_props().compute_units)
    npdt = {"f32": np.float32, "f16": np.float16, "f64": np.float64}
    draw = {"f32": synth.uniform_f32, "f16": synth.normal_half, "f64": synth.uniform_f64}
    peak = {"f32": PEAK_F32_TFLOPS, "f16": PEAK_F16_TFLOPS, "f64": PEAK_F64_TFLOPS}
    ws_cap = 1 << 30
    ws = hip.DeviceMatrix(1, ws_cap // 4, np.float32)

    def time_call(call):
        best = 1e30
        for _ in range(batches):
            call(); call()
            timer = hip.Timer(); timer.start()
            for _ in range(launches):
                call()
            best = min(best, timer.stop() / launches)
        return best * 1e3                                   # microseconds

    rows = []
    for dt, M, N, K in sweep_shapes(seed, per_type, large):
        if only and dt not in only:
            continue
        isz = np.dtype(npdt[dt]).itemsize
        dA = hip.DeviceMatrix(M, K, npdt[dt], device_pitch(K, isz), draw[dt](M, K, 0xA500 + M))
        dB = hip.DeviceMatrix(K, N, npdt[dt], device_pitch(N, isz), draw[dt](K, N, 0xB500 + N))
        dD = hip.DeviceMatrix(M, N, npdt[dt], device_pitch(N, isz))
        p = hip.plan(isz, M, N, K)
        pick_plan = {"tile": [int(p.tile_m), int(p.tile_n)], "k_splits": int(p.k_splits), "whole_tiles": int(p.whole_tiles)}
        ws_entry = {"f32": L.decx_hip_gemm_f32_ws, "f16": L.decx_hip_gemm_f16_ws, "f64": L.decx_hip_gemm_f64_ws}[dt]
        pick = lambda: hip.check(ws_entry(dA.ptr, dB.ptr, None, dD.ptr, M, N, K, dA.pitch, dB.pitch, 0, dD.pitch, 1.0, 1.0, ws.ptr, ws_cap, None))

        def forced(tile, splits, whole):
            return lambda: hip.check(L.decx_hip_gemm_forced_plan(isz, dA.ptr, dB.ptr, None, dD.ptr, M, N, K, dA.pitch, dB.pitch, 0, dD.pitch,
                                                                 1.0, 1.0, tile, splits, whole, ws.ptr, ws_cap, None))
        cands = [({"tile": list(t), "k_splits": 1, "whole_tiles": 0}, forced(c, 1, 0)) for c, t in SWEEP_TILES[dt].items()]
        for c, fit in SWEEP_SPLIT_FIT[dt].items():
            bm, bn = SWEEP_TILES[dt][c]
            if dt == "f32" and c == 2 and N <= 32:
                bm, bn = 128, 32
            t = -(-M // bm) * -(-N // bn)
            if t > 16 * cus:
                continue
            slots = fit * cus
            wholes = {0}
            if t > slots and t % slots:
                wholes.add(t // slots * slots)
            wholes.update(j * cus for j in range(1, fit) if j * cus < t)
            for ranges in (2, 3, 4, 5, 6, 8, 10, 12, 16, 24, 32):
                if K // ranges < 256 or (c != 2 and ranges > 8):
                    continue
                for whole in sorted(wholes):
                    if (t - whole) * ranges > 4096 or (t - whole) * ranges * bm * bn * (8 if dt == "f64" else 4) > ws_cap:
                        continue
                    call = forced(c, ranges, whole)
                    if L.decx_hip_gemm_forced_plan(isz, dA.ptr, dB.ptr, None, dD.ptr, M, N, K, dA.pitch, dB.pitch, 0, dD.pitch, 1.0, 1.0,
                                                   c, ranges, whole, ws.ptr, ws_cap, None) != 0:
                        continue                            # no kernel for this plan (ranges that do not come out even)
                    cands.append(({"tile": [bm, bn], "k_splits": ranges, "whole_tiles": whole}, call))
        hip.sync()
        t_pick = time_call(pick)
        timed = [(time_call(call), plan) for plan, call in cands]
        t_best, best_plan = min(timed, key=lambda x: x[0])
        best_call = [call for plan, call in cands if plan == best_plan][0]
        # the two in turns: what the summary counts
        again_pick, again_best = [], []
        for _ in range(3):
            again_pick.append(time_call(pick)); again_best.append(time_call(best_call))
        t_pick, t_best = min(again_pick + [t_pick]), min(again_best + [t_best])
        flops = 2.0 * M * N * K
        rows.append({"dtype": dt, "M": M, "N": N, "K": K, "pick": pick_plan, "pick_us": round(t_pick, 2),
                     "pick_tflops": round(flops / t_pick / 1e6, 1), "frac_of_peak": round(flops / t_pick / 1e6 / peak[dt], 3),
                     "best_other": best_plan, "best_other_us": round(t_best, 2), "plans_timed": len(cands),
                     "pick_over_best": round(t_pick / t_best, 4), "pick_is_best_plan": best_plan == pick_plan})
        print("sweep %s %5d x %5d x %5d  pick %s %.1f us  best other %s %.1f us  ratio %.3f  (%d plans)" % (
            dt, M, N, K, pick_plan, t_pick, best_plan, t_best, t_pick / t_best, len(cands)), file=sys.stderr, flush=True)
        for d in (dA, dB, dD):
            d.free()
    ws.free()
    ratios = sorted(r["pick_over_best"] for r in rows)
    summary = {"shapes": len(rows), "median_pick_over_best": ratios[len(ratios) // 2], "worst_pick_over_best": ratios[-1],
               "within_3_percent": sum(r <= 1.03 for r in ratios), "within_10_percent": sum(r <= 1.10 for r in ratios)}
    for dt in ("f32", "f16", "f64"):
        rr = sorted(r["pick_over_best"] for r in rows if r["dtype"] == dt) or [float("nan")]
        summary[dt] = {"shapes": len(rr), "median": rr[len(rr) // 2], "worst": rr[-1]}
    return {"workload": "planner sweep: the planner's pick against every other plan on seeded shapes it was not fitted on",
            "seed": seed, "large": large, "summary": summary, "shapes": rows}


def sweep_markdown(result):
    """The sweep as a table (what profiles/planner_sweep.md holds below its header)."""
    s = result["summary"]
    out = ["| dtype | M | N | K | planner's pick (tile, ranges, whole tiles) | us | TFLOP/s | of peak | best other plan | us | pick / best | plans timed |",
           "|---|---|---|---|---|---|---|---|---|---|---|---|"]
    fmt = lambda p: "%d x %d, %d, %d" % (p["tile"][0], p["tile"][1], p["k_splits"], p["whole_tiles"])
    for r in result["shapes"]:
        out.append("| %s | %d | %d | %d | %s | %.1f | %.1f | %.3f | %s | %.1f | %.3f | %d |" % (
            r["dtype"], r["M"], r["N"], r["K"], fmt(r["pick"]), r["pick_us"], r["pick_tflops"], r["frac_of_peak"], fmt(r["best_other"]),
            r["best_other_us"], r["pick_over_best"], r["plans_timed"]))
    out.append("")
    out.append("Pick over best: median %.3f, worst %.3f over %d shapes (%d within 3 %%, %d within 10 %%); fp32 median %.3f worst %.3f, "
               "fp16 %.3f / %.3f, fp64 %.3f / %.3f." % (s["median_pick_over_best"], s["worst_pick_over_best"], s["shapes"], s["within_3_percent"],
                                                       s["within_10_percent"], s["f32"]["median"], s["f32"]["worst"], s["f16"]["median"],
                                                       s["f16"]["worst"], s["f64"]["median"], s["f64"]["worst"]))
    return "\n".join(out)


def cpu_baseline(name, A, B, C, D_gpu):
    """Times the AVX2 restatement of the reference CPU GEMM on this host (best of a few calls for the short
    workloads), checks it bit-for-bit against the scalar fma chain on sampled rows, and compares the GPU's
    whole result with it.  Returns (cpu_baseline, gpu_parity)."""
    from oracle import binding as oracle
    import ctypes
    _, M, N, K, _, _, desc = WORKLOADS[name]
    L = oracle.lib()
    a, lda = oracle.aligned_f32(M, K); a[:, :K] = A
    b, ldb = oracle.aligned_f32(K, N); b[:, :N] = B
    d, ldd = oracle.aligned_f32(M, N)
    c, ldc = (None, 0)
    if C is not None:
        c, ldc = oracle.aligned_f32(M, N); c[:, :N] = C
    scratch, _ = oracle.aligned_f32(1, int(L.cpu_port_scratch_floats(K, N)))
    fp = ctypes.POINTER(ctypes.c_float)
    thread_counts, calls = CPU_LEGS[name]
    runs = []
    for want in thread_counts:
        threads = max(1, min(want, int(L.cpu_port_max_threads()), os.cpu_count() or 1))
        args = [a.ctypes.data_as(fp), b.ctypes.data_as(fp), c.ctypes.data_as(fp) if c is not None else None,
                d.ctypes.data_as(fp), M, N, K, lda, ldb, ldc, ldd, scratch.ctypes.data_as(fp), threads]
        best = 1e30
        for _ in range(calls):
            t0 = time.perf_counter()
            rc = L.cpu_port_gemm_f32(*args)
            best = min(best, time.perf_counter() - t0)
            assert rc == 0
        runs.append({"cores": threads, "ms": round(best * 1e3, 3), "value": round(2.0 * M * N * K / best / 1e12, 4)})
    rows = np.unique(np.random.default_rng(0).integers(0, M, 16)).astype(np.uint32)
    chain = oracle.gemm_f32(A, B, C, rows=rows)
    same = bool(np.array_equal(d[rows, :N].view(np.uint32), chain.view(np.uint32)))
    ref_max = float(np.max(np.abs(d[:, :N])))
    gpu_err = float(np.max(np.abs(D_gpu - d[:, :N]))) / (ref_max * math.sqrt(K))
    top = max(runs, key=lambda r: r["value"])
    base = {"value": top["value"], "unit": "TFLOP/s", "cores": top["cores"], "kind": "port", "ms": top["ms"],
            "sample": "the whole workload (%s), best of %d call%s" % (desc.split(",")[0], calls, "" if calls == 1 else "s"),
            "bit_equal_to_fma_chain": same}
    if len(runs) > 1:
        base["by_thread_count"] = runs
    parity = {"rel_err": float("%.3g" % gpu_err), "bar": 1e-5, "elements": int(M) * int(N), "against": "cpu_baseline",
              "measure": "max|gpu - cpu| / (max|cpu| sqrt(K)) over the whole output"}
    return base, parity


def chain_parity(name, A, B, C, D_gpu, rows=48):
    """GPU result against the oracle's k-ascending fma chain on sampled rows, for the workloads the reference has no
    CPU form of (fp16) or whose CPU form is not restated here (fp64)."""
    from oracle import binding as oracle
    dt, M, N, K = WORKLOADS[name][:4]
    pick = np.unique(np.concatenate([[0, M - 1], np.random.default_rng(1).integers(0, M, rows)])).astype(np.uint32)
    if dt == "f16":
        ref = oracle.gemm_f16(A, B, rows=pick).astype(np.float64); bar = 2e-3
    elif dt == "f64":
        ref = oracle.gemm_f64(A, B, rows=pick); bar = 1e-14
    else:
        ref = oracle.gemm_f32(A, B, C, rows=pick).astype(np.float64); bar = 1e-5
    err = float(np.max(np.abs(D_gpu[pick].astype(np.float64) - ref))) / (float(np.max(np.abs(ref))) * math.sqrt(K))
    return {"rel_err": float("%.3g" % err), "bar": bar, "elements": int(len(pick)) * int(N), "against": "fma chain oracle",
            "measure": "max|gpu - chain| / (max|chain| sqrt(K)) over %d sampled rows" % len(pick)}


def cpu_and_parity(name, out, inputs):
    """Adds "cpu_baseline" and "gpu_parity" to a workload's record."""
    A, B, C, D_gpu = inputs
    if name in CPU_LEGS:
        out["cpu_baseline"], out["gpu_parity"] = cpu_baseline(name, A, B, C, D_gpu)
    else:
        out["cpu_baseline"] = None           # no CPU form in the reference (fp16) / none restated here (fp64, the long-K split)
        out["gpu_parity"] = chain_parity(name, A, B, C, D_gpu)
    return out


def api_wall_time(name, repeats=10):
    """End-to-end wall time of de::blas::cuda::GEMM(GPU_Matrix x 3) (the reference's entry point,
    srcs/modules/BLAS/GEMM/CUDA/GEMM_LS.cu:315-350) for the workload, stream set-up, launch and the
    completion wait included, measured by the C++ driver of the de:: API in a process of its own."""
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tests", "cpp", "de_api_test")
    dtype, M, N, K = WORKLOADS[name][:4]
    if not os.path.exists(exe) or dtype not in ("f32", "f16"):
        return None
    if M * N * K < 2 ** 34:
        repeats = 200
    out = subprocess.run([exe, "gemmtime", dtype, str(M), str(N), str(K), str(repeats)], capture_output=True, text=True, timeout=300)
    for l in out.stdout.splitlines():
        if l.startswith("gemmtime"):
            f = l.split()
            med, best = float(f[2]), float(f[4])
            return {"entry": "de::blas::cuda::GEMM(GPU_Matrix, GPU_Matrix, GPU_Matrix)", "median_ms": med, "min_ms": best,
                    "calls": int(f[6]), "tflops_at_median": round(2.0 * M * N * K / med / 1e9, 2)}
    return {"error": (out.stderr or out.stdout)[-200:]}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="fp32_8192", choices=sorted(WORKLOADS) + ["copy_1GiB", "mfma_f16", "gemv_sizes", "planner_sweep", "conv2d", "conv2d_rgb", "c64_4096", "c128_2048"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the other workloads")
    ap.add_argument("--sweep-seed", type=int, default=20261125, help="planner_sweep: seed of the shapes")
    ap.add_argument("--sweep-shapes", type=int, default=16, help="planner_sweep: shapes per element type")
    ap.add_argument("--sweep-large", action="store_true", help="planner_sweep: sides of 1200 .. 9000 instead of 40 .. 6500")
    ap.add_argument("--sweep-dtypes", default=None, help="planner_sweep: only these element types, e.g. f16 or f32,f64")
    ap.add_argument("--sweep-markdown", default=None, help="planner_sweep: also write the table to this file")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this GEMM path runs on one GPU; --gpus %d is not supported (use --gpus 1)" % args.gpus)

    # the de:: API's own wall time, before this process takes the GPU
    api = api_wall_time(args.workload) if (args.workload in WORKLOADS and not args.no_extra) else None
    api16 = api_wall_time("fp16_4096") if (args.workload == "fp32_8192" and not args.no_extra) else None
    api_gemv = api_wall_time("fp32_gemv") if (args.workload == "fp32_8192" and not args.no_extra) else None

    from decx_amd import hip
    hip.init(0)
    props = hip.device_props()

    if args.workload == "copy_1GiB":
        # counter calibration: a copy whose HBM traffic is known (1 GiB read + 1 GiB written per launch)
        n = 1 << 30
        src = hip.DeviceMatrix(1, n // 4, np.float32); dst = hip.DeviceMatrix(1, n // 4, np.float32)
        hip.check(hip.lib().decx_hip_memset_async(src.ptr, 1, n, None))
        for _ in range(args.warmup):
            hip.check(hip.lib().decx_hip_calibration_copy(dst.ptr, src.ptr, n, None))
        hip.sync()
        timer = hip.Timer(); timer.start()
        for _ in range(args.steps):
            hip.check(hip.lib().decx_hip_calibration_copy(dst.ptr, src.ptr, n, None))
        ms = timer.stop() / args.steps
        print(json.dumps({"workload": "calibration copy 1 GiB", "kernel_ms": ms, "GB/s_read_plus_write": 2 * n / ms / 1e6}))
        return
    if args.workload == "planner_sweep":
        result = planner_sweep(seed=args.sweep_seed, per_type=args.sweep_shapes, large=args.sweep_large, launches=4 if args.sweep_large else 10,
                               only=args.sweep_dtypes.split(",") if args.sweep_dtypes else None)
        if args.sweep_markdown:
            with open(args.sweep_markdown, "w") as f:
                f.write(sweep_markdown(result) + "\n")
        print(json.dumps(result))
        return
    if args.workload == "mfma_f16":
        print(json.dumps(dict(sustained_mfma(launches=args.steps), workload="register-only matrix-core loop")))
        return
    if args.workload == "gemv_sizes":
        print(json.dumps(gemv_sizes()))
        return

    if args.workload in ("conv2d", "conv2d_rgb"):
        print(json.dumps(run_conv(args.steps, args.warmup, c=CONV if args.workload == "conv2d" else CONV_RGB, parity=not args.no_cpu)))
        return
    if args.workload in ("c64_4096", "c128_2048"):
        print(json.dumps(run_complex(args.workload == "c128_2048", 4096 if args.workload == "c64_4096" else 2048, args.steps, args.warmup, parity=not args.no_cpu)))
        return

    main_out, inputs = run_workload(args.workload, args.steps, args.warmup, keep_inputs=not args.no_cpu,
                                    settle_s=0.25 if args.workload != "fp32_8192" else 0.0)
    if args.workload == "fp16_4096" and not args.no_extra:
        add_sustained(main_out, sustained_mfma())
        main_out["roofline"]["on_zero_operands"] = zero_operand_rate("fp16_4096")
    line = {
        "metric": "GEMM TFLOP/s (fp32 8192^3 headline; fp16 4096^3 under config.fp16_4096 and other_workloads) on 1 MI355X",
        "value": main_out["value"], "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": main_out["kernel_ms"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": main_out["dtype"], "data": "synthetic",
        "config": {"workload": main_out["workload"], "plan": main_out["plan"],
                   "device": props.name.decode(), "arch": props.arch.decode(), "compute_units": int(props.compute_units),
                   "clock_mhz": props.clock_khz / 1000.0,
                   "peak_recomputed_tflops": round(props.compute_units * (256 if main_out["dtype"] == "f32" else 4096)
                                                   * props.clock_khz * 1e3 / 1e12, 1)},
        "wall_ms_per_step": main_out["wall_ms_per_step"],
        "roofline": main_out["roofline"],
    }
    if api is not None:
        line["api_wall"] = api
    others = []
    if not args.no_extra:
        copy = copy_rate()
        line["config"]["copy_rate"] = copy
        floor_us = launch_floor()
        line["config"]["launch_floor_us"] = floor_us
        for name in WORKLOADS:
            if name != args.workload:
                small = WORKLOADS[name][1] * WORKLOADS[name][2] * WORKLOADS[name][3] < 2 ** 38
                o, inp = run_workload(name, 200 if small else args.steps, args.warmup, keep_inputs=not args.no_cpu, settle_s=0.25)
                if not args.no_cpu:
                    cpu_and_parity(name, o, inp)
                if name == "fp16_4096":
                    add_sustained(o, sustained_mfma())
                    o["roofline"]["on_zero_operands"] = zero_operand_rate("fp16_4096")
                    if api16 is not None:
                        o["api_wall"] = api16
                    # the second half of the metric, where the records that keep only `config` hold it too
                    line["config"]["fp16_4096"] = {
                        "workload": o["workload"], "value": o["value"], "unit": "TFLOP/s", "kernel_ms": o["kernel_ms"],
                        "frac": o["roofline"]["frac"], "peak": PEAK_F16_TFLOPS,
                        "sustained": o["roofline"]["sustained"]["value"], "frac_of_sustained": o["roofline"]["sustained"]["frac_of_sustained"],
                        "sustained_on_zero_operands": o["roofline"]["sustained"]["on_zero_operands"],
                        "value_on_zero_operands": o["roofline"]["on_zero_operands"],
                        "note": "sustained: a register-only loop of the kernel's MFMA on operands drawn like the workload's, same run; "
                                "*_on_zero_operands: the same launches on zeros, where the board's power management does not hold the clock down",
                        "gpu_parity_rel_err": (o.get("gpu_parity") or {}).get("rel_err"), "parity_bar": 2e-3,
                        "plan": o["plan"], "api_wall_median_ms": (api16 or {}).get("median_ms")}
                if name == "fp32_gemv" and api_gemv is not None:
                    o["api_wall"] = api_gemv
                others.append(o)
                del inp
        others.append(run_conv(200, args.warmup, parity=not args.no_cpu))
        rgb = run_conv(200, args.warmup, c=CONV_RGB, parity=not args.no_cpu)
        rgb["roofline"]["copy_rate_gbs"] = copy["value"]           # what this board moves when half the traffic is writes
        rgb["roofline"]["frac_of_copy_rate"] = round(rgb["roofline"]["achieved"] / copy["value"], 4)
        rgb["roofline"]["write_only_gbs"] = copy["write_only_gbs"]  # ... and when all of it is (73 % of this workload's bytes are)
        # a launch of next to nothing, plus the workload's algorithmic bytes at the copy kernel's rate
        rgb["roofline"]["floor_us"] = round(floor_us + rgb["roofline"]["achieved"] * rgb["kernel_ms"] * 1e3 / copy["value"], 2)
        rgb["roofline"]["frac_of_floor"] = round(rgb["roofline"]["floor_us"] / (rgb["kernel_ms"] * 1e3), 4)
        others.append(rgb)
        others.append(run_complex(False, 4096, args.steps, args.warmup, parity=not args.no_cpu))
        others.append(run_complex(True, 2048, 50, args.warmup, parity=not args.no_cpu))
        line["config"]["summary"] = {o["name"]: [o["roofline"]["achieved"], o["roofline"]["unit"], o["roofline"]["frac"]] for o in others}
    if not args.no_cpu:
        cpu_and_parity(args.workload, line, inputs)
        if line["cpu_baseline"] is not None:     # where the first round's readers look for it
            line["cpu_baseline"]["gpu_parity"] = line["gpu_parity"]
    if others:
        # the long list first: a reader that keeps only the end of the line still has the headline and `config`
        line = dict([("other_workloads", others)] + list(line.items()))
    print(json.dumps(line))


if __name__ == "__main__":
    main()
