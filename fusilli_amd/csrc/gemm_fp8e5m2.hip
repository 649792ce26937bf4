// MFMA GEMM kernels for fp8e5m2 operands.
#include "gemm_kernel.h"

int gemm_launch_fp8e5m2(fhip_ctx *ctx, const GemmPlan &p, const GemmArgs &g) {
  return gemm_launch_kind<GK_FP8E5M2>(ctx, p, g);
}
