"""Times the vendor libraries (through PyTorch-ROCm: hipBLASLt / rocBLAS,
MIOpen, the flash attention that torch ships) on the benchmark's headline
problems, on random operands, as a yardstick beside bench.py's figures.

    python fusilli_amd/bench/vendor_yardstick.py [--iters 300]

One line per problem: average microseconds per call (HIP events around
`iters` back-to-back calls after at least 50 ms of warm-up) and the rate in
the unit bench.py uses for the same problem.  A problem the installed torch
cannot run prints the error instead of a figure.  Nothing here is used by the
library, the tests or bench.py.
"""
import argparse
import sys

import torch


def timed(fn, iters):
    fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    # warm-up: clocks settle after tens of milliseconds of load
    start.record()
    n = 0
    while True:
        for _ in range(20):
            fn()
        n += 20
        stop.record()
        stop.synchronize()
        if start.elapsed_time(stop) >= 50.0 or n >= 5000:
            break
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) * 1e3 / iters


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--iters", type=int, default=300)
    args = ap.parse_args()
    if not torch.cuda.is_available():
        sys.exit("vendor_yardstick.py needs a GPU")
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev)
    g.manual_seed(7)
    rnd = lambda *shape: torch.randn(*shape, device=dev, generator=g)
    import torch.nn.functional as F

    problems = []

    # C1: f32 matmul 1 x 256 x 512 x 256
    a1, b1 = rnd(1, 256, 512), rnd(1, 512, 256)
    problems.append(("matmul_f32_1x256x512x256", lambda: torch.matmul(a1, b1),
                     2.0 * 256 * 512 * 256, "TFLOP/s"))
    # C2: bf16 RMSNorm 8192 x 4096 with a scale
    x2 = rnd(8192, 4096).bfloat16()
    s2 = rnd(4096).bfloat16()
    problems.append(("rmsnorm_bf16_8192x4096", lambda: F.rms_norm(x2, (4096,), s2, 1e-6),
                     2.0 * 8192 * 4096 * 2, "GB/s"))
    # C3: bf16 conv N32 C64 56x56 -> K128 3x3 pad 1, channels-last, + bias + ReLU
    x3 = rnd(32, 64, 56, 56).bfloat16().contiguous(memory_format=torch.channels_last)
    w3 = (rnd(128, 64, 3, 3) * 0.05).bfloat16().contiguous(memory_format=torch.channels_last)
    b3 = rnd(128).bfloat16()
    problems.append(("conv_fprop_bf16_n32c64h56w56_k128r3s3_bias_relu",
                     lambda: F.relu(F.conv2d(x3, w3, b3, padding=1)),
                     2.0 * 32 * 56 * 56 * 128 * 576, "TFLOP/s"))
    # C4: bf16 causal SDPA B4 H32 S2048 D128
    q4, k4, v4 = (rnd(4, 32, 2048, 128).bfloat16() for _ in range(3))
    problems.append(("sdpa_fwd_bf16_causal_b4h32s2048d128",
                     lambda: F.scaled_dot_product_attention(q4, k4, v4, is_causal=True),
                     4.0 * 4 * 32 * 2048 * 2048 * 128 / 2, "TFLOP/s"))
    # bf16 GEMM 4096^3
    a5, b5 = rnd(4096, 4096).bfloat16(), rnd(4096, 4096).bfloat16()
    problems.append(("matmul_bf16_4096x4096x4096", lambda: torch.matmul(a5, b5),
                     2.0 * 4096 ** 3, "TFLOP/s"))
    # C5a: int8 x int8 -> int32, 4096 x 8192 x 4096
    a6 = torch.randint(-127, 128, (4096, 8192), device=dev, dtype=torch.int8, generator=g)
    b6 = torch.randint(-127, 128, (8192, 4096), device=dev, dtype=torch.int8, generator=g)
    problems.append(("matmul_int8_4096x8192x4096_i32", lambda: torch._int_mm(a6, b6),
                     2.0 * 4096 * 8192 * 4096, "TOP/s"))
    # C5b: fp8 e4m3 x e4m3 -> bf16 with scales (B given column-major, as
    # torch._scaled_mm asks)
    try:
        f8 = torch.float8_e4m3fn
        a7 = (torch.rand(4096, 8192, device=dev, generator=g) * 2 - 1).mul(448.0).to(f8)
        b7 = (torch.rand(4096, 8192, device=dev, generator=g) * 2 - 1).mul(448.0).to(f8).t()
        one = torch.ones((), device=dev)
        problems.append(("matmul_fp8e4m3_4096x8192x4096_scaled_bf16_out",
                         lambda: torch._scaled_mm(a7, b7, scale_a=one, scale_b=one,
                                                  out_dtype=torch.bfloat16),
                         2.0 * 4096 * 8192 * 4096, "TFLOP/s"))
    except Exception as e:  # dtype not in this torch build
        print(f"matmul_fp8e4m3_4096x8192x4096_scaled_bf16_out: not run ({e})")

    print(f"torch {torch.__version__}, {torch.cuda.get_device_name(0)}")
    for name, fn, work, unit in problems:
        try:
            with torch.no_grad():
                us = timed(fn, args.iters)
            rate = work / us / 1e6 if unit != "GB/s" else work / us / 1e3
            print(f"{name:58s} {us:10.2f} us  {rate:10.1f} {unit}", flush=True)
        except Exception as e:  # an op this torch / device combination lacks
            print(f"{name:58s} not run: {type(e).__name__}: {str(e)[:160]}", flush=True)


if __name__ == "__main__":
    main()
