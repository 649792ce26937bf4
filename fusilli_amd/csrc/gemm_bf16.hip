// MFMA GEMM kernels for bf16 operands.
#include "gemm_kernel.h"

int gemm_launch_bf16(fhip_ctx *ctx, const GemmPlan &p, const GemmArgs &g) {
  return gemm_launch_kind<GK_BF16>(ctx, p, g);
}
