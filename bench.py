#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

Headline workload (benchmark config 2): RMSNorm bf16 over X[8192,4096]
(f32 accumulate, eps 1e-6, learned scale) followed by a fused pointwise MUL —
one `step` is one such launch through the C ABI with inputs resident in HBM.
Buffer sets are rotated so the 256 MB Infinity Cache cannot serve the reads.

Prints ONE JSON line.  `value` is algorithmic GB/s over the timed wall-clock
region; `roofline` prices the kernel's own average duration (HIP events on the
launch stream) against the 8 TB/s HBM peak; `cpu_baseline` is the CPU oracle's
restatement of the same op timed on this box's host cores over a bounded
sample; `others` carries the remaining benchmark configs (TFLOP/s or GB/s and
fraction of their rooflines), measured the same way except that each warms up
for at least 40 ms (`warmup_launches` says how many launches that took).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from fusilli_amd import capi, synth  # noqa: E402

HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of the headline kernel, measured under rocprofv3
# (--pmc FETCH_SIZE and --pmc WRITE_SIZE runs of this script, each scaled by
# what the same counter reads for `--calibrate-copy`): 65 608 KiB fetched +
# 65 536 KiB written.  Counters cannot be read from inside this process.
RMSNORM_TRAFFIC_BYTES = (65608 + 65536) * 1024
PEAK_TFLOPS = {"bf16": 2500.0, "fp8": 5000.0, "int8": 5000.0, "f32": 157.3}

# HBM bytes per launch of the dominant kernel of a line (FETCH_SIZE + WRITE_SIZE
# of rocprofv3 --pmc runs of this script, each scaled by what the same counter
# reads for `--calibrate-copy`), with the summary under profiles/ that records
# the run.  Counters cannot be read from inside this process: these are the
# figures of the recorded runs, not of this one.
TRAFFIC = {
    "conv_fprop_bf16_n32c64h56w56_k128r3s3_bias_relu":
        (int((8467.5 * 1.9985 + 25088) * 1024),
         "profiles/conv_rf_dgrad_wgrad_direct_bf16_n32c64h56w56_k128r3s3.md"),
    "sdpa_fwd_bf16_causal_b4h32s2048d128":
        (int(149207.4 * 1.9985 * 1024) + 64 * 1024 * 1024,
         "profiles/sdpa_fwd_bf16_causal_b4h32s2048d128.md"),
    "matmul_int8_4096x8192x4096_i32":
        (201_000_000 + 64 * 1024 * 1024, "profiles/gemm_mfma_4096x8192x4096_int8_fp8_bf16.md"),
    "matmul_fp8e4m3_4096x8192x4096_scaled_bf16_out":
        (201_000_000 + 32 * 1024 * 1024, "profiles/gemm_mfma_4096x8192x4096_int8_fp8_bf16.md"),
}

# The benchmark's configurations: line of `others` (None: the headline), the
# north-star target for its roofline fraction (None: plumbing case without a
# target), the kernel variant that must have run (prefix of fhip_last_kernel),
# and the driver command that times the same problem through Graph::execute.
CONFIGS = {
    "C1": ("matmul_f32_1x256x512x256", None, "matmul_f32_splitk",
           "matmul -M 256 -N 256 -K 512 --a_type f32 --b_type f32 --out_type f32"),
    "C2": (None, 0.70, "rownorm chunks=",
           "rmsnorm -X 8192x4096 -t bf16 -e 1e-6 --mul 0.5"),
    "C3": ("conv_fprop_bf16_n32c64h56w56_k128r3s3_bias_relu", 0.60, "conv_rf c=64 r=3 s=3",
           "conv -F 1 -n 32 -c 64 -H 56 -W 56 -k 128 -y 3 -x 3 -p 1 -q 1 -u 1 -v 1 -l 1 -j 1 "
           "--in_layout NHWC --out_layout NHWC --fil_layout NHWC --spatial_dim 2 --bf16 --bias --relu"),
    "C4": ("sdpa_fwd_bf16_causal_b4h32s2048d128", 0.60, "sdpa_fwd d=128 causal=1 mask=0",
           "sdpa -B 4 --heads_q 32 --heads_kv 32 --seq_q 2048 --seq_kv 2048 -d 128 -t bf16 --causal"),
    "C5a": ("matmul_int8_4096x8192x4096_i32", 0.60, "gemm_mfma i8 256x256 waves=8 split=1",
            "matmul -M 4096 -N 4096 -K 8192 --a_type i8 --b_type i8 --out_type i32"),
    "C5b": ("matmul_fp8e4m3_4096x8192x4096_scaled_bf16_out", 0.60,
            "gemm_mfma fp8e4m3 256x256 waves=8 split=1",
            "matmul -M 4096 -N 4096 -K 8192 --a_type fp8 --b_type fp8 --out_type bf16 "
            "--out_scale 0.0000049824617"),
}
FLOOR_FILE = os.path.join(ROOT, "bench_floor.json")
DRIVER = os.path.join(ROOT, "fusilli_amd", "bench", "bin", "driver")


def graph_api_us(command, kernel_us):
    """Average time of one Graph::execute of `command`'s graph (HIP events
    around --iter back-to-back executes inside the benchmark driver, a child
    process: variant-pack lookup, plan and argument set-up included), or None
    when the driver binary is not built.  As many untimed executes first as
    60 ms of the kernel's time (`kernel_us` per launch): the GPU's clocks take
    tens of milliseconds of load to settle, and a short kernel timed before
    that reads 10-20 % slow."""
    import shlex
    import subprocess
    if not os.path.exists(DRIVER):
        return None
    try:
        # (--fill random: constant operands toggle fewer bits and let the MFMA
        # kernels clock higher than real data does)
        warm = max(50, int(60e3 / max(kernel_us, 1.0)))
        iters = max(200, int(20e3 / max(kernel_us, 1.0)))
        proc = subprocess.run([DRIVER, "--iter", str(iters), "--warmup", str(warm), "--fill", "random"]
                              + shlex.split(command),
                              capture_output=True, text=True, timeout=120)
        if proc.returncode != 0:
            return None
        lines = proc.stdout.strip().splitlines()
        rec = dict(zip(lines[-2].split(","), lines[-1].split(",")))
        return round(float(rec["avg_us"]), 2)
    except Exception:  # a missing figure, not a failed benchmark
        return None


# The secondary workloads warm up for at least this long (the GPU's clocks take
# tens of milliseconds of load to settle: a short MFMA kernel timed right after
# idle reads 10-20 % slow).  The headline keeps exactly --warmup launches.
MIN_WARM_MS = 0.0
LAST_WARMUP = 0


def timed_loop(ctx, launch, steps, warmup):
    """W untimed + K timed launches; returns (wall ms/step, event ms/step)."""
    global LAST_WARMUP
    t_warm = time.perf_counter()
    for i in range(warmup):
        launch(i)
    ctx.sync()
    done = warmup
    while (time.perf_counter() - t_warm) * 1e3 < MIN_WARM_MS:
        for i in range(max(8, warmup)):
            launch(done + i)
        ctx.sync()
        done += max(8, warmup)
    LAST_WARMUP = done
    e0, e1 = ctx.event(), ctx.event()
    t0 = time.perf_counter()
    e0.record()
    for i in range(steps):
        launch(i)
    e1.record()
    ctx.sync()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    ev_ms = e1.elapsed_ms_since(e0) / steps
    return wall_ms, ev_ms


# ---------------------------------------------------------------------------
# C2: RMSNorm + MUL
# ---------------------------------------------------------------------------
def rmsnorm_desc(rows, cols, mul_kind):
    d = capi.NormDesc()
    d.x = capi.TensorDesc.make([rows, cols], [cols, 1], capi.BFLOAT16)
    d.scale = capi.TensorDesc.make([1, cols], [cols, 1], capi.BFLOAT16)
    d.y = capi.TensorDesc.make([rows, cols], [cols, 1], capi.FLOAT)
    d.out = capi.TensorDesc.make([rows, cols], [cols, 1], capi.BFLOAT16)
    d.out_dtype = capi.BFLOAT16
    d.epsilon = 1e-6
    if mul_kind == "scalar":
        op = capi.epilogue_op(capi.PW["MUL"], capi.BFLOAT16, scalar=0.5)
    else:
        op = capi.epilogue_op(
            capi.PW["MUL"], capi.BFLOAT16, operand_index=0,
            operand=capi.TensorDesc.make([rows, cols], [cols, 1], capi.BFLOAT16))
    d.epilogue = capi.make_epilogue([op])
    return d


def bench_rmsnorm(ctx, steps, warmup, mul_kind="scalar", sets=5):
    rows, cols = 8192, 4096
    d = rmsnorm_desc(rows, cols, mul_kind)
    assert ctx.lib.fhip_norm_fwd_supported(d) == 2, "tuned row kernel not chosen"
    n = rows * cols
    scale = ctx.to_device(synth.f32_to_bf16_bits(synth.normal(2, 1, cols, 1.0, 0.02)))
    xs, gs, ys = [], [], []
    for s in range(sets):
        xs.append(ctx.to_device(synth.f32_to_bf16_bits(synth.normal(2, 10 + s, n))))
        ys.append(ctx.alloc(n * 2))
        if mul_kind == "full":
            gs.append(ctx.to_device(synth.f32_to_bf16_bits(synth.normal(2, 50 + s, n))))

    def launch(i):
        j = i % sets
        ctx.norm_fwd(d, xs[j], scale, None, ys[j],
                     epilogue_operands=[gs[j]] if gs else ())

    wall_ms, ev_ms = timed_loop(ctx, launch, steps, warmup)
    # spread of single launches (outside the timed region): batches of 10
    # back-to-back launches between two events, so that the event overhead of
    # an idle stream does not enter
    batches = []
    for b in range(100):
        e0, e1 = ctx.event(), ctx.event()
        e0.record()
        for i in range(10):
            launch(b * 10 + i)
        e1.record()
        ctx.sync()
        batches.append(e1.elapsed_ms_since(e0) * 100.0)  # us per launch
    mean = sum(batches) / len(batches)
    std = (sum((t - mean) ** 2 for t in batches) / len(batches)) ** 0.5
    algo_bytes = 2 * n * 2 + cols * 2 + (n * 2 if mul_kind == "full" else 0)
    return {"wall_ms": wall_ms, "kernel_ms": ev_ms, "bytes": algo_bytes,
            "gbs_wall": algo_bytes / wall_ms / 1e6,
            "gbs_kernel": algo_bytes / ev_ms / 1e6,
            "sets": sets,
            "launch_us": {"min": round(min(batches), 2), "mean": round(mean, 2),
                          "stddev": round(std, 2),
                          "sample": "100 batches of 10 launches"}}


# ---------------------------------------------------------------------------
# Matmul configs (C5a int8 -> int32, C5b fp8 -> bf16 with scales, bf16 GEMM)
# ---------------------------------------------------------------------------
def matmul_desc(m, n, k, in_dt, c_dt, out_dt, epilogue=()):
    d = capi.MatmulDesc()
    d.a = capi.TensorDesc.make([m, k], [k, 1], in_dt)
    d.b = capi.TensorDesc.make([k, n], [n, 1], in_dt)
    d.c = capi.TensorDesc.make([m, n], [n, 1], c_dt)
    d.out = capi.TensorDesc.make([m, n], [n, 1], out_dt)
    d.out_dtype = out_dt
    d.epilogue = capi.make_epilogue(list(epilogue))
    return d


def bench_matmul(ctx, steps, warmup, kind, m=4096, n=4096, k=8192):
    if kind == "int8":
        in_dt, c_dt, out_dt, epi = capi.INT8, capi.INT32, capi.INT32, ()
        gen = lambda tid, cnt: synth.integers(5, tid, cnt, -127, 127).astype(np.int8)
        peak = PEAK_TFLOPS["int8"]
    elif kind == "fp8":
        in_dt, c_dt, out_dt = capi.FP8E4M3, capi.FLOAT, capi.BFLOAT16
        epi = (capi.epilogue_op(capi.PW["MUL"], capi.BFLOAT16, scalar=1.0 / (448.0 * 448.0)),)
        gen = lambda tid, cnt: synth.f32_to_fp8_bits(synth.uniform(6, tid, cnt) * 448.0, 4)
        peak = PEAK_TFLOPS["fp8"]
    else:
        in_dt, c_dt, out_dt, epi = capi.BFLOAT16, capi.FLOAT, capi.BFLOAT16, ()
        gen = lambda tid, cnt: synth.f32_to_bf16_bits(synth.normal(7, tid, cnt))
        peak = PEAK_TFLOPS["bf16"]
    d = matmul_desc(m, n, k, in_dt, c_dt, out_dt, epi)
    assert ctx.lib.fhip_matmul_supported(d) == 2, "MFMA kernel not chosen"
    a = ctx.to_device(gen(0, m * k))
    b = ctx.to_device(gen(1, k * n))
    out = ctx.alloc(m * n * capi.DTYPE_SIZE[out_dt])
    wall_ms, ev_ms = timed_loop(ctx, lambda i: ctx.matmul(d, a, b, out),
                                steps, warmup)
    flop = 2.0 * m * n * k
    return {"value": round(flop / ev_ms / 1e9, 1),
            "unit": "TOP/s" if kind == "int8" else "TFLOP/s",
            "frac_of_mfma_peak": round(flop / ev_ms / 1e9 / peak, 4),
            "kernel_us": round(ev_ms * 1e3, 2), "work": flop}


def bench_matmul_f32_c1(ctx, steps, warmup):
    """benchmark config 1: f32 A[1,256,512] x B[1,512,256] (the reference's
    CPU-runnable case).  Runs on the stride-generic f32 MFMA kernels
    (v_mfma_f32_32x32x2_f32; at this size 32 x 32 tiles with K split over the
    four wavefronts of a workgroup: 64 workgroups)."""
    d = capi.MatmulDesc()
    d.a = capi.TensorDesc.make([1, 256, 512], [256 * 512, 512, 1], capi.FLOAT)
    d.b = capi.TensorDesc.make([1, 512, 256], [512 * 256, 256, 1], capi.FLOAT)
    d.c = capi.TensorDesc.make([1, 256, 256], [256 * 256, 256, 1], capi.FLOAT)
    d.out = capi.TensorDesc.make([1, 256, 256], [256 * 256, 256, 1], capi.FLOAT)
    d.out_dtype = capi.FLOAT
    d.epilogue = capi.make_epilogue([])
    assert ctx.lib.fhip_matmul_supported(d) >= 1
    a = ctx.to_device(synth.uniform(1, 0, 256 * 512).astype(np.float32))
    b = ctx.to_device(synth.uniform(1, 1, 512 * 256).astype(np.float32))
    out = ctx.alloc(256 * 256 * 4)
    wall_ms, ev_ms = timed_loop(ctx, lambda i: ctx.matmul(d, a, b, out), steps, warmup)
    flop = 2.0 * 256 * 512 * 256
    return {"value": round(flop / ev_ms / 1e9, 3), "unit": "TFLOP/s",
            "frac_of_mfma_peak": round(flop / ev_ms / 1e9 / 157.3, 5),
            "kernel_us": round(ev_ms * 1e3, 2), "work": flop,
            "kernel_note": "stride-generic f32 MFMA tiles (fhip_matmul_supported == %d)"
                           % ctx.lib.fhip_matmul_supported(d)}


def bench_conv(ctx, steps, warmup):
    """C3: conv_fprop bf16 NHWC N32 C64 56x56, K128 3x3 pad 1, + bias + ReLU."""
    n, c, h, w, k, r = 32, 64, 56, 56, 128, 3
    cl = lambda dims: [dims[1] * dims[2] * dims[3], 1, dims[3] * dims[1], dims[1]]
    xd, wd, yd = [n, c, h, w], [k, c, r, r], [n, k, h, w]
    d = capi.ConvDesc()
    d.x = capi.TensorDesc.make(xd, cl(xd), capi.BFLOAT16)
    d.w = capi.TensorDesc.make(wd, cl(wd), capi.BFLOAT16)
    d.y = capi.TensorDesc.make(yd, cl(yd), capi.FLOAT)
    d.out = capi.TensorDesc.make(yd, cl(yd), capi.BFLOAT16)
    d.out_dtype = capi.BFLOAT16
    d.spatial_rank = 2
    for i in range(2):
        d.padding[i], d.stride[i], d.dilation[i] = 1, 1, 1
    bias_desc = capi.TensorDesc.make([1, k, 1, 1], [k, 1, k, k], capi.BFLOAT16)
    d.epilogue = capi.make_epilogue([
        capi.epilogue_op(capi.PW["ADD"], capi.FLOAT, operand_index=0,
                         operand=bias_desc),
        capi.epilogue_op(capi.PW["RELU_FWD"], capi.BFLOAT16)])
    assert ctx.lib.fhip_conv_fprop_supported(d) == 2, "MFMA conv not chosen"
    x = ctx.to_device(synth.f32_to_bf16_bits(synth.normal(8, 0, n * c * h * w)))
    wt = ctx.to_device(synth.f32_to_bf16_bits(synth.normal(8, 1, k * c * r * r, 0.0, 0.05)))
    bias = ctx.to_device(synth.f32_to_bf16_bits(synth.normal(8, 2, k)))
    out = ctx.alloc(n * k * h * w * 2)
    wall_ms, ev_ms = timed_loop(
        ctx, lambda i: ctx.conv_fprop(d, x, wt, out, epilogue_operands=[bias]),
        steps, warmup)
    flop = 2.0 * n * h * w * k * c * r * r
    # launch overhead, reported beside the kernel time: host time to enqueue
    # one call (descriptor -> plan -> hipLaunchKernel), and the event-to-event
    # time of a launch on an idle stream (dispatch latency + kernel)
    launch = lambda: ctx.conv_fprop(d, x, wt, out, epilogue_operands=[bias])
    ctx.sync()
    t0 = time.perf_counter()
    for _ in range(50):
        launch()
    enqueue_us = (time.perf_counter() - t0) * 1e6 / 50
    ctx.sync()
    isolated = []
    for _ in range(10):
        e0, e1 = ctx.event(), ctx.event()
        e0.record()
        launch()
        e1.record()
        ctx.sync()
        isolated.append(e1.elapsed_ms_since(e0) * 1e3)
    return {"value": round(flop / ev_ms / 1e9, 1), "unit": "TFLOP/s",
            "frac_of_mfma_peak": round(flop / ev_ms / 1e9 / PEAK_TFLOPS["bf16"], 4),
            "kernel_us": round(ev_ms * 1e3, 2), "work": flop,
            "launch_overhead": {"host_enqueue_us": round(enqueue_us, 2),
                                "idle_stream_launch_us": round(min(isolated), 2)}}


def bench_conv_dgrad(ctx, steps, warmup):
    """Data gradient of C3: DY bf16 NHWC [32,128,56,56], W KRSC [128,64,3,3]
    -> DX [32,64,56,56]; one kernel that keeps the filter in registers and
    reads W as it lies (no mirrored copy, the workspace stays unused)."""
    n, c, h, w, k, r = 32, 64, 56, 56, 128, 3
    cl = lambda dims: [dims[1] * dims[2] * dims[3], 1, dims[3] * dims[1], dims[1]]
    xd, wd, yd = [n, c, h, w], [k, c, r, r], [n, k, h, w]
    d = capi.ConvDesc()
    d.x = capi.TensorDesc.make(xd, cl(xd), capi.BFLOAT16)
    d.w = capi.TensorDesc.make(wd, cl(wd), capi.BFLOAT16)
    d.y = capi.TensorDesc.make(yd, cl(yd), capi.BFLOAT16)
    d.spatial_rank = 2
    for i in range(2):
        d.padding[i], d.stride[i], d.dilation[i] = 1, 1, 1
    d.epilogue = capi.make_epilogue([])
    assert ctx.lib.fhip_conv_dgrad_supported(d) == 2, "MFMA dgrad not chosen"
    dy = ctx.to_device(synth.f32_to_bf16_bits(synth.normal(9, 0, n * k * h * w)))
    wt = ctx.to_device(synth.f32_to_bf16_bits(synth.normal(9, 1, k * c * r * r, 0.0, 0.05)))
    dx = ctx.alloc(n * c * h * w * 2)
    ws = ctx.alloc(ctx.conv_dgrad_workspace(d))
    wall_ms, ev_ms = timed_loop(
        ctx, lambda i: ctx.conv_dgrad(d, dy, wt, dx, workspace=ws), steps, warmup)
    flop = 2.0 * n * h * w * k * c * r * r
    return {"value": round(flop / ev_ms / 1e9, 1), "unit": "TFLOP/s",
            "frac_of_mfma_peak": round(flop / ev_ms / 1e9 / PEAK_TFLOPS["bf16"], 4),
            "call_us": round(ev_ms * 1e3, 2), "work": flop,
            "kernels_per_call": 1}


def bench_conv_wgrad(ctx, steps, warmup):
    """Weight gradient of C3: DY bf16 NHWC [32,128,56,56], X [32,64,56,56] ->
    DW KRSC [128,64,3,3]; one MFMA kernel that reads X and DY in place and
    leaves one block of partial sums per workgroup, then their sum (2 kernels
    per call)."""
    n, c, h, w, k, r = 32, 64, 56, 56, 128, 3
    cl = lambda dims: [dims[1] * dims[2] * dims[3], 1, dims[3] * dims[1], dims[1]]
    xd, wd, yd = [n, c, h, w], [k, c, r, r], [n, k, h, w]
    d = capi.ConvDesc()
    d.x = capi.TensorDesc.make(xd, cl(xd), capi.BFLOAT16)
    d.w = capi.TensorDesc.make(wd, cl(wd), capi.BFLOAT16)
    d.y = capi.TensorDesc.make(yd, cl(yd), capi.BFLOAT16)
    d.spatial_rank = 2
    for i in range(2):
        d.padding[i], d.stride[i], d.dilation[i] = 1, 1, 1
    d.epilogue = capi.make_epilogue([])
    assert ctx.lib.fhip_conv_wgrad_supported(d) == 2, "MFMA wgrad not chosen"
    dy = ctx.to_device(synth.f32_to_bf16_bits(synth.normal(10, 0, n * k * h * w)))
    x = ctx.to_device(synth.f32_to_bf16_bits(synth.normal(10, 1, n * c * h * w)))
    dw = ctx.alloc(k * c * r * r * 2)
    ws = ctx.alloc(ctx.conv_wgrad_workspace(d))
    wall_ms, ev_ms = timed_loop(
        ctx, lambda i: ctx.conv_wgrad(d, dy, x, dw, workspace=ws), steps, warmup)
    flop = 2.0 * n * h * w * k * c * r * r
    return {"value": round(flop / ev_ms / 1e9, 1), "unit": "TFLOP/s",
            "frac_of_mfma_peak": round(flop / ev_ms / 1e9 / PEAK_TFLOPS["bf16"], 4),
            "call_us": round(ev_ms * 1e3, 2), "work": flop,
            "kernels_per_call": 2}


def bench_reduce(ctx, steps, warmup, mode="SUM", sets=5):
    """Row reduction bf16 X[8192,4096] -> f32 Y[8192,1] (reads 64 MiB per launch)."""
    rows, cols = 8192, 4096
    d = capi.ReduceDesc()
    d.x = capi.TensorDesc.make([rows, cols], [cols, 1], capi.BFLOAT16)
    d.y = capi.TensorDesc.make([rows, 1], [1, 1], capi.FLOAT)
    d.mode = capi.RED[mode]
    assert ctx.lib.fhip_reduce_supported(d) == 2, "row-reduction kernel not chosen"
    xs = [ctx.to_device(synth.f32_to_bf16_bits(synth.normal(10, s, rows * cols)))
          for s in range(sets)]
    y = ctx.alloc(rows * 4)
    wall_ms, ev_ms = timed_loop(ctx, lambda i: ctx.reduce(d, xs[i % sets], y),
                                steps, warmup)
    nbytes = rows * cols * 2 + rows * 4
    return {"value": round(nbytes / ev_ms / 1e6, 1), "unit": "GB/s",
            "frac_of_hbm_peak": round(nbytes / ev_ms / 1e6 / HBM_PEAK_GBS, 4),
            "kernel_us": round(ev_ms * 1e3, 2), "bytes": nbytes}


def bench_pointwise(ctx, steps, warmup, mode="ADD", sets=5):
    """Pointwise bf16 [8192,4096]: ADD of a bias row [1,4096], or unary GELU."""
    rows, cols = 8192, 4096
    n = rows * cols
    d = capi.PointwiseDesc()
    d.mode = capi.PW[mode]
    d.params = capi.PointwiseParams.default()
    d.in_[0] = capi.TensorDesc.make([rows, cols], [cols, 1], capi.BFLOAT16)
    d.out = capi.TensorDesc.make([rows, cols], [cols, 1], capi.BFLOAT16)
    bias = None
    if mode == "ADD":
        d.num_inputs = 2
        d.in_[1] = capi.TensorDesc.make([1, cols], [cols, 1], capi.BFLOAT16)
        bias = ctx.to_device(synth.f32_to_bf16_bits(synth.normal(12, 1, cols)))
    else:
        d.num_inputs = 1
    assert ctx.lib.fhip_pointwise_supported(d) == 2, "vector pointwise kernel not chosen"
    xs = [ctx.to_device(synth.f32_to_bf16_bits(synth.normal(12, 10 + s, n))) for s in range(sets)]
    ys = [ctx.alloc(n * 2) for _ in range(sets)]
    wall_ms, ev_ms = timed_loop(
        ctx, lambda i: ctx.pointwise(d, xs[i % sets], bias, None, ys[i % sets]),
        steps, warmup)
    nbytes = 2 * n * 2 + (cols * 2 if bias is not None else 0)
    return {"value": round(nbytes / ev_ms / 1e6, 1), "unit": "GB/s",
            "frac_of_hbm_peak": round(nbytes / ev_ms / 1e6 / HBM_PEAK_GBS, 4),
            "kernel_us": round(ev_ms * 1e3, 2), "bytes": nbytes}


def bench_layernorm(ctx, steps, warmup, sets=5):
    """LayerNorm bf16 X[8192,4096] with scale and bias (inference), bf16 out."""
    rows, cols = 8192, 4096
    d = capi.NormDesc()
    d.x = capi.TensorDesc.make([rows, cols], [cols, 1], capi.BFLOAT16)
    d.scale = capi.TensorDesc.make([1, cols], [cols, 1], capi.BFLOAT16)
    d.bias = capi.TensorDesc.make([1, cols], [cols, 1], capi.BFLOAT16)
    d.y = capi.TensorDesc.make([rows, cols], [cols, 1], capi.BFLOAT16)
    d.out = capi.TensorDesc.make([rows, cols], [cols, 1], capi.BFLOAT16)
    d.out_dtype = capi.BFLOAT16
    d.epsilon = 1e-5
    d.is_layernorm = 1
    d.epilogue = capi.make_epilogue([])
    assert ctx.lib.fhip_norm_fwd_supported(d) == 2, "tuned row kernel not chosen"
    n = rows * cols
    scale = ctx.to_device(synth.f32_to_bf16_bits(synth.normal(11, 1, cols, 1.0, 0.02)))
    bias = ctx.to_device(synth.f32_to_bf16_bits(synth.normal(11, 2, cols, 0.0, 0.02)))
    xs = [ctx.to_device(synth.f32_to_bf16_bits(synth.normal(11, 10 + s, n))) for s in range(sets)]
    ys = [ctx.alloc(n * 2) for _ in range(sets)]
    wall_ms, ev_ms = timed_loop(
        ctx, lambda i: ctx.norm_fwd(d, xs[i % sets], scale, bias, ys[i % sets]),
        steps, warmup)
    nbytes = 2 * n * 2 + 2 * cols * 2
    return {"value": round(nbytes / ev_ms / 1e6, 1), "unit": "GB/s",
            "frac_of_hbm_peak": round(nbytes / ev_ms / 1e6 / HBM_PEAK_GBS, 4),
            "kernel_us": round(ev_ms * 1e3, 2), "bytes": nbytes}


def bench_sdpa(ctx, steps, warmup, b=4, h=32, sq=2048, d=128, masked=False):
    """C4: SDPA forward bf16 causal B4 H32 S2048 D128 ([B,H,S,D] contiguous);
    `masked`: the same tensors under an additive bf16 mask [B,1,S,S] (shared
    by the heads, as the reference's benchmark driver builds it) instead of
    the causal flag."""
    dims = [b, h, sq, d]
    strides = [h * sq * d, sq * d, d, 1]
    desc = capi.SdpaDesc()
    desc.q = desc.k = desc.v = desc.o = capi.TensorDesc.make(dims, strides, capi.BFLOAT16)
    desc.is_causal = 0 if masked else 1
    mask = None
    if masked:
        desc.mask = capi.TensorDesc.make([b, 1, sq, sq], [sq * sq, sq * sq, sq, 1],
                                         capi.BFLOAT16)
        mask = ctx.to_device(synth.f32_to_bf16_bits(synth.normal(9, 7, b * sq * sq)))
    assert ctx.lib.fhip_sdpa_fwd_supported(desc) == 2, "MFMA SDPA not chosen"
    n = b * h * sq * d
    q, k, v = (ctx.to_device(synth.f32_to_bf16_bits(synth.normal(9, i, n)))
               for i in range(3))
    out = ctx.alloc(n * 2)
    wall_ms, ev_ms = timed_loop(
        ctx, lambda i: ctx.sdpa_fwd(desc, q, k, v, out, mask=mask), steps, warmup)
    # causal: only the lower triangle of the S x S score matrix is computed
    flop = 4.0 * b * h * sq * sq * d / (1 if masked else 2)
    return {"value": round(flop / ev_ms / 1e9, 1), "unit": "TFLOP/s",
            "frac_of_mfma_peak": round(flop / ev_ms / 1e9 / PEAK_TFLOPS["bf16"], 4),
            "kernel_us": round(ev_ms * 1e3, 2), "work": flop,
            "flop_convention": "4*B*H*S*S*D" + ("" if masked else "/2 (causal half)")}


def bench_layernorm_long(ctx, steps, warmup, rows=16, cols=128 * 64 * 32):
    """The reference benchmark's LayerNorm shape, 16 x (128 * 64 * 32) bf16
    with scale and bias: rows of 262144 elements, normalised by two kernels
    per call (segment statistics, then the normalisation)."""
    d = capi.NormDesc()
    d.x = capi.TensorDesc.make([rows, cols], [cols, 1], capi.BFLOAT16)
    d.scale = capi.TensorDesc.make([1, cols], [cols, 1], capi.BFLOAT16)
    d.bias = capi.TensorDesc.make([1, cols], [cols, 1], capi.BFLOAT16)
    d.y = capi.TensorDesc.make([rows, cols], [cols, 1], capi.BFLOAT16)
    d.out = capi.TensorDesc.make([rows, cols], [cols, 1], capi.BFLOAT16)
    d.out_dtype = capi.BFLOAT16
    d.epsilon = 1e-5
    d.is_layernorm = 1
    d.epilogue = capi.make_epilogue([])
    assert ctx.lib.fhip_norm_fwd_supported(d) == 2, "long-row norm not chosen"
    n = rows * cols
    x = ctx.to_device(synth.f32_to_bf16_bits(synth.normal(12, 0, n)))
    scale = ctx.to_device(synth.f32_to_bf16_bits(synth.normal(12, 1, cols, 1.0, 0.02)))
    bias = ctx.to_device(synth.f32_to_bf16_bits(synth.normal(12, 2, cols, 0.0, 0.02)))
    y = ctx.alloc(n * 2)
    wall_ms, ev_ms = timed_loop(ctx, lambda i: ctx.norm_fwd(d, x, scale, bias, y),
                                steps, warmup)
    nbytes = 2 * n * 2 + 2 * cols * 2
    return {"value": round(nbytes / ev_ms / 1e6, 1), "unit": "GB/s",
            "frac_of_hbm_peak": round(nbytes / ev_ms / 1e6 / HBM_PEAK_GBS, 4),
            "call_us": round(ev_ms * 1e3, 2), "bytes": nbytes, "kernels_per_call": 2,
            "note": "8 MB of X: the whole call is a few launch latencies long"}


def bench_batchnorm_train(ctx, steps, warmup):
    """Training batch norm with scale and bias over N32 C128 56x56 bf16,
    channels-last: column statistics (one read of X), a per-channel finalize,
    and the apply pass (a second read of X, mostly from the caches, and the
    write of Y): 3 kernels per call.  Algorithmic bytes: X once + Y once."""
    n, c, h, w = 32, 128, 56, 56
    dims = [n, c, h, w]
    cl = [c * h * w, 1, w * c, c]
    d = capi.BatchNormDesc()
    d.x = capi.TensorDesc.make(dims, cl, capi.BFLOAT16)
    d.y = capi.TensorDesc.make(dims, cl, capi.BFLOAT16)
    d.training = 1
    d.has_scale = d.has_bias = 1
    d.scale_dtype = d.bias_dtype = d.running_dtype = d.stats_dtype = capi.FLOAT
    d.epsilon = 1e-5
    assert ctx.lib.fhip_batchnorm_fwd_supported(d) == 2, "channels-last batch norm not chosen"
    x = ctx.to_device(synth.f32_to_bf16_bits(synth.normal(12, 0, n * c * h * w)))
    sc = ctx.to_device(synth.normal(12, 1, c, 1.0, 0.2).astype(np.float32))
    bi = ctx.to_device(synth.normal(12, 2, c).astype(np.float32))
    y = ctx.alloc(n * c * h * w * 2)
    sm, sv = ctx.alloc(c * 4), ctx.alloc(c * 4)
    wall_ms, ev_ms = timed_loop(
        ctx, lambda i: ctx.batchnorm_fwd(d, x, y, sc, bi, None, None, sm, sv), steps, warmup)
    nbytes = 2 * n * c * h * w * 2 + 4 * c * 4
    return {"value": round(nbytes / ev_ms / 1e6, 1), "unit": "GB/s",
            "frac_of_hbm_peak": round(nbytes / ev_ms / 1e6 / HBM_PEAK_GBS, 4),
            "call_us": round(ev_ms * 1e3, 2), "bytes": nbytes, "kernels_per_call": 3}


def bench_conv_padded(ctx, steps, warmup):
    """The reference benchmark's conv2d_nhwc_fp16 shape: N16 C48 48x32, K48
    3x3, padding 2 -- a channel count that is no multiple of 64, so X and W
    are first copied into zero-padded 64-channel tensors (3 kernels per call)."""
    n, c, h, w, k, r, pad = 16, 48, 48, 32, 48, 3, 2
    p, q = h + 2 * pad - (r - 1), w + 2 * pad - (r - 1)
    cl = lambda dims: [dims[1] * dims[2] * dims[3], 1, dims[3] * dims[1], dims[1]]
    xd, wd, yd = [n, c, h, w], [k, c, r, r], [n, k, p, q]
    d = capi.ConvDesc()
    d.x = capi.TensorDesc.make(xd, cl(xd), capi.HALF)
    d.w = capi.TensorDesc.make(wd, cl(wd), capi.HALF)
    d.y = capi.TensorDesc.make(yd, cl(yd), capi.HALF)
    d.out = capi.TensorDesc.make(yd, cl(yd), capi.HALF)
    d.out_dtype = capi.HALF
    d.spatial_rank = 2
    for i in range(2):
        d.padding[i], d.stride[i], d.dilation[i] = pad, 1, 1
    d.epilogue = capi.make_epilogue([])
    assert ctx.lib.fhip_conv_fprop_supported(d) == 2, "MFMA conv not chosen"
    x = ctx.to_device(synth.normal(8, 3, n * c * h * w).astype(np.float16))
    wt = ctx.to_device(synth.normal(8, 4, k * c * r * r, 0.0, 0.05).astype(np.float16))
    out = ctx.alloc(n * k * p * q * 2)
    wall_ms, ev_ms = timed_loop(ctx, lambda i: ctx.conv_fprop(d, x, wt, out),
                                steps, warmup)
    flop = 2.0 * n * p * q * k * c * r * r
    return {"value": round(flop / ev_ms / 1e9, 1), "unit": "TFLOP/s",
            "frac_of_mfma_peak": round(flop / ev_ms / 1e9 / PEAK_TFLOPS["bf16"], 4),
            "call_us": round(ev_ms * 1e3, 2), "work": flop, "kernels_per_call": 3,
            "note": "1.4 GFLOP: launch-latency bound"}


def bench_conv_grouped(ctx, steps, warmup, n=32, c=256, h=56, w=56, k=256, groups=4):
    """3 x 3 convolution, padding 1, bf16 channels-last, no fused operations.
    The default: N32 C256 56x56 -> K256 in 4 groups of 64 -> 64 channels (the
    register-filter kernel with two groups per workgroup, runs of 2-row tiles).
    Also used for one-group shapes around C3: K = 64 (64 output channels per
    workgroup) and N = 64 (two tiles per workgroup)."""
    r = 3
    cl = lambda dims: [dims[1] * dims[2] * dims[3], 1, dims[3] * dims[1], dims[1]]
    xd, wd, yd = [n, c, h, w], [k, c // groups, r, r], [n, k, h, w]
    d = capi.ConvDesc()
    d.x = capi.TensorDesc.make(xd, cl(xd), capi.BFLOAT16)
    d.w = capi.TensorDesc.make(wd, cl(wd), capi.BFLOAT16)
    d.y = capi.TensorDesc.make(yd, cl(yd), capi.FLOAT)
    d.out = capi.TensorDesc.make(yd, cl(yd), capi.BFLOAT16)
    d.out_dtype = capi.BFLOAT16
    d.spatial_rank = 2
    for i in range(2):
        d.padding[i], d.stride[i], d.dilation[i] = 1, 1, 1
    d.epilogue = capi.make_epilogue([])
    assert ctx.lib.fhip_conv_fprop_supported(d) == 2, "MFMA conv not chosen"
    x = ctx.to_device(synth.f32_to_bf16_bits(synth.normal(8, 5, n * c * h * w)))
    wt = ctx.to_device(synth.f32_to_bf16_bits(
        synth.normal(8, 6, k * (c // groups) * r * r, 0.0, 0.05)))
    out = ctx.alloc(n * k * h * w * 2)
    wall_ms, ev_ms = timed_loop(ctx, lambda i: ctx.conv_fprop(d, x, wt, out),
                                steps, warmup)
    flop = 2.0 * n * h * w * k * (c // groups) * r * r
    return {"value": round(flop / ev_ms / 1e9, 1), "unit": "TFLOP/s",
            "frac_of_mfma_peak": round(flop / ev_ms / 1e9 / PEAK_TFLOPS["bf16"], 4),
            "call_us": round(ev_ms * 1e3, 2), "work": flop, "kernels_per_call": 1}


def bench_conv_deep_layer(ctx, steps, warmup):
    """A late ResNet layer: N32 C512 7x7 -> K512, 3x3, padding 1, bf16
    channels-last.  1568 output pixels make 52 tiles, so the planner cuts the
    reduction into four parts on workgroups of their own and a second kernel
    adds them (two kernels per call)."""
    n, c, h, w, k, r = 32, 512, 7, 7, 512, 3
    cl = lambda dims: [dims[1] * dims[2] * dims[3], 1, dims[3] * dims[1], dims[1]]
    xd, wd, yd = [n, c, h, w], [k, c, r, r], [n, k, h, w]
    d = capi.ConvDesc()
    d.x = capi.TensorDesc.make(xd, cl(xd), capi.BFLOAT16)
    d.w = capi.TensorDesc.make(wd, cl(wd), capi.BFLOAT16)
    d.y = capi.TensorDesc.make(yd, cl(yd), capi.FLOAT)
    d.out = capi.TensorDesc.make(yd, cl(yd), capi.BFLOAT16)
    d.out_dtype = capi.BFLOAT16
    d.spatial_rank = 2
    for i in range(2):
        d.padding[i], d.stride[i], d.dilation[i] = 1, 1, 1
    d.epilogue = capi.make_epilogue([])
    assert ctx.lib.fhip_conv_fprop_supported(d) == 2, "MFMA conv not chosen"
    x = ctx.to_device(synth.f32_to_bf16_bits(synth.normal(8, 9, n * c * h * w)))
    wt = ctx.to_device(synth.f32_to_bf16_bits(synth.normal(8, 10, k * c * r * r, 0.0, 0.02)))
    out = ctx.alloc(n * k * h * w * 2)
    wall_ms, ev_ms = timed_loop(ctx, lambda i: ctx.conv_fprop(d, x, wt, out),
                                steps, warmup)
    flop = 2.0 * n * h * w * k * c * r * r
    return {"value": round(flop / ev_ms / 1e9, 1), "unit": "TFLOP/s",
            "frac_of_mfma_peak": round(flop / ev_ms / 1e9 / PEAK_TFLOPS["bf16"], 4),
            "call_us": round(ev_ms * 1e3, 2), "work": flop, "kernels_per_call": 2}


def bench_matmul_split(ctx, steps, warmup):
    """bf16 1024 x 1024 x 8192: 16 tiles of 256 x 256, so the planner cuts K
    into parts on workgroups of their own (f32 partial sums in the context's
    scratch) and a second kernel adds them: two kernels per call."""
    r = bench_matmul(ctx, steps, warmup, "bf16", 1024, 1024, 8192)
    r["call_us"] = r.pop("kernel_us")
    r["kernels_per_call"] = 2
    return r


def bench_conv_depthwise(ctx, steps, warmup):
    """Depthwise 3x3 convolution (groups = channels), N32 C128 56x56, padding 1,
    bf16 channels-last: the channels-last small-group kernel; bound by HBM
    (X read once, OUT written once)."""
    n, c, h, w, r = 32, 128, 56, 56, 3
    cl = lambda dims: [dims[1] * dims[2] * dims[3], 1, dims[3] * dims[1], dims[1]]
    xd, wd, yd = [n, c, h, w], [c, 1, r, r], [n, c, h, w]
    d = capi.ConvDesc()
    d.x = capi.TensorDesc.make(xd, cl(xd), capi.BFLOAT16)
    d.w = capi.TensorDesc.make(wd, cl(wd), capi.BFLOAT16)
    d.y = capi.TensorDesc.make(yd, cl(yd), capi.FLOAT)
    d.out = capi.TensorDesc.make(yd, cl(yd), capi.BFLOAT16)
    d.out_dtype = capi.BFLOAT16
    d.spatial_rank = 2
    for i in range(2):
        d.padding[i], d.stride[i], d.dilation[i] = 1, 1, 1
    d.epilogue = capi.make_epilogue([])
    assert ctx.lib.fhip_conv_fprop_supported(d) == 2, "small-group kernel not chosen"
    x = ctx.to_device(synth.f32_to_bf16_bits(synth.normal(8, 7, n * c * h * w)))
    wt = ctx.to_device(synth.f32_to_bf16_bits(synth.normal(8, 8, c * r * r, 0.0, 0.3)))
    out = ctx.alloc(n * c * h * w * 2)
    wall_ms, ev_ms = timed_loop(ctx, lambda i: ctx.conv_fprop(d, x, wt, out),
                                steps, warmup)
    nbytes = 2 * n * c * h * w * 2 + c * r * r * 2
    return {"value": round(nbytes / ev_ms / 1e6, 1), "unit": "GB/s",
            "frac_of_hbm_peak": round(nbytes / ev_ms / 1e6 / HBM_PEAK_GBS, 4),
            "call_us": round(ev_ms * 1e3, 2), "bytes": nbytes, "kernels_per_call": 1}


def calibrate_copy(ctx, steps):
    """Plain copy of known size (pointwise IDENTITY over 64 Mi int32 = 256 MiB
    read + 256 MiB written, on the strided kernel: one ordinary 4-byte load
    and store per lane): the yardstick that FETCH_SIZE / WRITE_SIZE counter
    readings of the other kernels are scaled by."""
    n = 64 * 1024 * 1024
    d = capi.PointwiseDesc()
    d.mode, d.num_inputs = capi.PW["IDENTITY"], 1
    d.in_[0] = capi.TensorDesc.make([n], [1], capi.INT32)
    d.out = capi.TensorDesc.make([n], [1], capi.INT32)
    d.params = capi.PointwiseParams.default()
    assert ctx.lib.fhip_pointwise_supported(d) == 1, "calibration must use the plain kernel"
    src, dst = ctx.alloc(n * 4), ctx.alloc(n * 4)
    ctx.memset(src, 0)
    wall_ms, ev_ms = timed_loop(ctx, lambda i: ctx.pointwise(d, src, None, None, dst),
                                steps, 2)
    return {"bytes_read": n * 4, "bytes_written": n * 4,
            "kernel_us": round(ev_ms * 1e3, 2),
            "gbs": round(2 * n * 4 / ev_ms / 1e6, 1)}


def roofline_of(result):
    """The `roofline` object of one `others` line, from the figures its bench
    function measured: algorithmic bytes (or flops) of one call over the
    HIP-event time of one call, against the HBM (or dense MFMA) peak."""
    us = result.get("kernel_us", result.get("call_us"))
    if "bytes" in result:
        achieved = result["bytes"] / us / 1e3
        return {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                "kernel_us": us, "traffic": None}
    achieved = result["work"] / us / 1e6
    peak = achieved / result["frac_of_mfma_peak"] if result["frac_of_mfma_peak"] else None
    return {"bound": "mfma", "achieved": round(achieved, 1),
            "peak": round(peak, 1) if peak else None,
            "unit": result["unit"], "frac": result["frac_of_mfma_peak"],
            "kernel_us": us, "traffic": None}


def _timed_cpu(fn, seconds_budget):
    fn()  # warm (page-in, thread pool)
    reps, t0 = 0, time.perf_counter()
    while True:
        fn()
        reps += 1
        dt = time.perf_counter() - t0
        if dt > seconds_budget:
            return reps, dt


def cpu_baseline_others(seconds_budget=4.0):
    """The CPU oracle (float64 accumulation, OpenMP) on bounded samples of the
    matmul, convolution and attention workloads of `others`."""
    from oracle import oracle
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    out = {}
    # int8 matmul: 32 rows of the 4096 x 8192 x 4096 product
    m, n, k, rows = 4096, 4096, 8192, 32
    a = synth.integers(5, 0, rows * k, -127, 127).astype(np.int8).reshape(rows, k)
    b = synth.integers(5, 1, k * n, -127, 127).astype(np.int8).reshape(k, n)
    idx = np.arange(rows)
    reps, dt = _timed_cpu(lambda: oracle.matmul_rows(a, b, idx), seconds_budget)
    out["matmul_int8_4096x8192x4096_i32"] = {
        "value": round(2.0 * rows * n * k * reps / dt / 1e12, 5), "unit": "TOP/s",
        "cores": threads, "kind": "port",
        "sample": f"{reps} passes over {rows} of {m} output rows, {dt:.1f} s"}
    # convolution: one image of the 32
    c, h, w, kk, r = 64, 56, 56, 128, 3
    x = synth.f32_to_bf16_bits(synth.normal(8, 0, c * h * w))
    x = oracle.dequantize(x, capi.BFLOAT16).reshape(1, h, w, c).transpose(0, 3, 1, 2)
    wt = synth.f32_to_bf16_bits(synth.normal(8, 1, kk * c * r * r, 0.0, 0.05))
    wt = oracle.dequantize(wt, capi.BFLOAT16).reshape(kk, r, r, c).transpose(0, 3, 1, 2)
    reps, dt = _timed_cpu(lambda: oracle.conv_fprop(x, wt, [1, 1], [1, 1], [1, 1]),
                          seconds_budget)
    out["conv_fprop_bf16_n32c64h56w56_k128r3s3_bias_relu"] = {
        "value": round(2.0 * h * w * kk * c * r * r * reps / dt / 1e12, 5),
        "unit": "TFLOP/s", "cores": threads, "kind": "port",
        "sample": f"{reps} passes over 1 of 32 images (convolution only), {dt:.1f} s"}
    # attention: two of the 128 (batch, head) pairs
    sq, dd, heads = 2048, 128, 2
    q, kx, v = (oracle.dequantize(
        synth.f32_to_bf16_bits(synth.normal(9, i, heads * sq * dd)), capi.BFLOAT16
    ).reshape(1, heads, sq, dd) for i in range(3))
    reps, dt = _timed_cpu(lambda: oracle.sdpa(q, kx, v, is_causal=True), seconds_budget)
    out["sdpa_fwd_bf16_causal_b4h32s2048d128"] = {
        "value": round(4.0 * heads * sq * sq * dd / 2 * reps / dt / 1e12, 5),
        "unit": "TFLOP/s", "cores": threads, "kind": "port",
        "sample": f"{reps} passes over {heads} of 128 (batch, head) pairs, {dt:.1f} s"}
    return out


def cpu_baseline_rmsnorm(seconds_budget=12.0):
    """The oracle's bf16 RMSNorm * scalar on the host cores over a row sample."""
    from oracle import oracle
    rows, cols = 1024, 4096
    x = synth.f32_to_bf16_bits(synth.normal(2, 10, rows * cols)).reshape(rows, cols)
    s = synth.f32_to_bf16_bits(synth.normal(2, 1, cols, 1.0, 0.02))
    oracle.rmsnorm_bf16_baseline(x, s, 1e-6, 0.5)  # warm
    reps, t0 = 0, time.perf_counter()
    while True:
        oracle.rmsnorm_bf16_baseline(x, s, 1e-6, 0.5)
        reps += 1
        dt = time.perf_counter() - t0
        if dt > seconds_budget:
            break
    nbytes = (2 * rows * cols * 2 + cols * 2) * reps
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    return {"value": round(nbytes / dt / 1e9, 3), "unit": "GB/s",
            "cores": threads, "kind": "port",
            "sample": f"{reps} passes over {rows}x{cols} bf16 rows "
                      f"(1/8 of the workload's rows), OpenMP, {dt:.1f} s; "
                      "reference IREE llvm-cpu path unavailable offline"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=500)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-others", action="store_true")
    ap.add_argument("--only", default="",
                    help="comma-separated substrings: run only the matching "
                         "lines of `others` (tuning runs; skips the CPU baseline)")
    ap.add_argument("--write-floors", type=float, default=0.0, metavar="FRACTION",
                    help="after the run, write bench_floor.json: FRACTION x this "
                         "run's roofline fraction per line (later runs list the "
                         "lines that fall below their floor under `regressions`)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run only a plain copy kernel of known size (counter "
                         "calibration) and print its figures")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path "
              "(no collectives, no sharding); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    ctx = capi.Context(0)
    if args.calibrate_copy:
        print(json.dumps({"calibrate_copy": calibrate_copy(ctx, max(3, args.steps // 20))}))
        ctx.close()
        return
    r = bench_rmsnorm(ctx, args.steps, args.warmup, "scalar")
    headline_kernel = ctx.last_kernel()
    line = {
        "metric": "GB/s (norms) on 1 MI355X, % roofline",
        "value": round(r["gbs_wall"], 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(r["wall_ms"], 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "RMSNorm bf16 X[8192,4096] eps=1e-6 scale[4096] "
                               "+ fused pointwise MUL (scalar operand), "
                               f"{r['sets']} rotating buffer sets",
                   "device": ctx.arch()},
        "roofline": {"bound": "hbm", "achieved": round(r["gbs_kernel"], 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(r["gbs_kernel"] / HBM_PEAK_GBS, 4),
                     "traffic": RMSNORM_TRAFFIC_BYTES,
                     "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE "
                                       "of an earlier run, scaled by a plain "
                                       "copy (profiles/); not measured by this run",
                     "algorithmic_bytes_per_launch": r["bytes"],
                     "kernel_us": round(r["kernel_ms"] * 1e3, 2),
                     "launch_us": r["launch_us"]},
    }
    if not args.no_others:
        global MIN_WARM_MS
        MIN_WARM_MS = 40.0
        others = {}

        def other(name, result):
            result["warmup_launches"] = LAST_WARMUP
            result["roofline"] = roofline_of(result)
            # (the variant of the line's last call: a line of two kernels names
            # the second)
            result.setdefault("kernel", ctx.last_kernel())
            if name in TRAFFIC:
                result["roofline"]["traffic"], result["roofline"]["traffic_source"] = TRAFFIC[name]
            others[name] = result

        def rms_full():
            r2 = bench_rmsnorm(ctx, args.steps, args.warmup, "full")
            return {"value": round(r2["gbs_kernel"], 1), "unit": "GB/s",
                    "frac_of_hbm_peak": round(r2["gbs_kernel"] / HBM_PEAK_GBS, 4),
                    "kernel_us": round(r2["kernel_ms"] * 1e3, 2), "bytes": r2["bytes"]}

        ksteps, kwarm = max(10, args.steps // 10), max(3, args.warmup // 5)
        lines = [
            ("rmsnorm_bf16_8192x4096_mul_full_operand", rms_full),
            ("layernorm_bf16_8192x4096_scale_bias",
             lambda: bench_layernorm(ctx, args.steps, args.warmup)),
            ("pointwise_add_bf16_8192x4096_bias_row",
             lambda: bench_pointwise(ctx, max(5, args.steps // 4), 2, "ADD")),
            ("pointwise_gelu_bf16_8192x4096",
             lambda: bench_pointwise(ctx, max(5, args.steps // 4), 2, "GELU_FWD")),
            ("reduce_sum_bf16_8192x4096_rows",
             lambda: bench_reduce(ctx, args.steps, args.warmup, "SUM")),
            ("reduce_amax_bf16_8192x4096_rows",
             lambda: bench_reduce(ctx, args.steps, args.warmup, "AMAX")),
            ("matmul_f32_1x256x512x256",
             lambda: bench_matmul_f32_c1(ctx, max(10, args.steps // 4), 3)),
            ("matmul_int8_4096x8192x4096_i32",
             lambda: bench_matmul(ctx, ksteps, kwarm, "int8")),
            ("matmul_fp8e4m3_4096x8192x4096_scaled_bf16_out",
             lambda: bench_matmul(ctx, ksteps, kwarm, "fp8")),
            ("matmul_bf16_4096x4096x4096",
             lambda: bench_matmul(ctx, ksteps, kwarm, "bf16", 4096, 4096, 4096)),
            ("conv_fprop_bf16_n32c64h56w56_k128r3s3_bias_relu",
             lambda: bench_conv(ctx, max(20, args.steps // 4), kwarm)),
            ("conv_dgrad_bf16_n32c64h56w56_k128r3s3",
             lambda: bench_conv_dgrad(ctx, max(20, args.steps // 4), kwarm)),
            ("conv_wgrad_bf16_n32c64h56w56_k128r3s3",
             lambda: bench_conv_wgrad(ctx, max(20, args.steps // 10), kwarm)),
            ("sdpa_fwd_bf16_causal_b4h32s2048d128",
             lambda: bench_sdpa(ctx, max(20, args.steps // 4), kwarm)),
            ("sdpa_fwd_bf16_causal_b4h32s2048d64",
             lambda: bench_sdpa(ctx, max(20, args.steps // 4), kwarm, d=64)),
            ("sdpa_fwd_bf16_mask_b4h32s2048d128",
             lambda: bench_sdpa(ctx, max(20, args.steps // 4), kwarm, masked=True)),
            ("layernorm_bf16_16x262144_long_rows",
             lambda: bench_layernorm_long(ctx, max(20, args.steps // 4), kwarm)),
            ("conv_fprop_bf16_n32c256h56w56_k256r3s3_groups4",
             lambda: bench_conv_grouped(ctx, max(20, args.steps // 10), kwarm)),
            ("conv_fprop_bf16_n32c64h56w56_k64r3s3",
             lambda: bench_conv_grouped(ctx, max(20, args.steps // 10), kwarm, 32, 64, 56, 56, 64, 1)),
            ("conv_fprop_bf16_n64c64h56w56_k128r3s3",
             lambda: bench_conv_grouped(ctx, max(20, args.steps // 10), kwarm, 64, 64, 56, 56, 128, 1)),
            ("conv_fprop_bf16_n32c512h7w7_k512r3s3_split_reduction",
             lambda: bench_conv_deep_layer(ctx, max(20, args.steps // 10), kwarm)),
            ("matmul_bf16_1024x1024x8192_split_reduction",
             lambda: bench_matmul_split(ctx, max(20, args.steps // 10), kwarm)),
            ("conv_fprop_bf16_n32c128h56w56_depthwise_r3s3",
             lambda: bench_conv_depthwise(ctx, max(20, args.steps // 10), kwarm)),
            ("conv_fprop_f16_n16c48h48w32_k48r3s3_padded_channels",
             lambda: bench_conv_padded(ctx, max(20, args.steps // 4), kwarm)),
            ("batchnorm_train_bf16_n32c128h56w56_scale_bias",
             lambda: bench_batchnorm_train(ctx, max(20, args.steps // 10), kwarm)),
        ]
        wanted = [w for w in args.only.split(",") if w]
        for name, fn in lines:
            if wanted and not any(w in name for w in wanted):
                continue
            other(name, fn())
        line["others"] = others
        # ---- the configurations side by side, and the floors --------------------
        if not wanted:
            configs = {}
            for cfg, (name, target, variant, command) in CONFIGS.items():
                if name is None:
                    roof, kernel = line["roofline"], headline_kernel
                else:
                    roof, kernel = others[name]["roofline"], others[name]["kernel"]
                frac, us = roof["frac"], roof["kernel_us"]
                configs[cfg] = {"line": name or "headline", "frac": frac, "target": target,
                                "met": None if target is None else bool(frac >= target),
                                "kernel_us": us, "kernel": kernel,
                                "expected_kernel": bool(kernel.startswith(variant)),
                                "graph_api_us": graph_api_us(command, us),
                                "traffic": roof.get("traffic"),
                                "traffic_source": roof.get("traffic_source")}
            line["configs"] = configs
            floors = json.load(open(FLOOR_FILE)) if os.path.exists(FLOOR_FILE) else {}
            regressions = []
            for name, floor in floors.items():
                if name == "headline":
                    frac = line["roofline"]["frac"]
                elif name in others:
                    frac = others[name]["roofline"]["frac"]
                else:
                    continue
                if frac < floor:
                    regressions.append({"line": name, "frac": frac, "floor": floor})
            for cfg, c in configs.items():
                if not c["expected_kernel"]:
                    regressions.append({"line": cfg, "kernel": c["kernel"],
                                        "expected": CONFIGS[cfg][2]})
            line["regressions"] = regressions
            if args.write_floors > 0:
                new = {"headline": round(line["roofline"]["frac"] * args.write_floors, 4)}
                for name, res in others.items():
                    new[name] = round(res["roofline"]["frac"] * args.write_floors, 4)
                with open(FLOOR_FILE, "w") as f:
                    json.dump(new, f, indent=1, sort_keys=True)
                    f.write("\n")
    if not args.no_cpu_baseline and not args.only:
        line["cpu_baseline"] = cpu_baseline_rmsnorm()
        if not args.no_others:
            line["cpu_baseline"]["others"] = cpu_baseline_others()
    ctx.close()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
