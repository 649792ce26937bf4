// MFMA GEMM kernels for fp8e4m3 operands.
#include "gemm_kernel.h"

int gemm_launch_fp8e4m3(fhip_ctx *ctx, const GemmPlan &p, const GemmArgs &g) {
  return gemm_launch_kind<GK_FP8E4M3>(ctx, p, g);
}
