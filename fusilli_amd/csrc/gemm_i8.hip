// MFMA GEMM kernels for i8 operands.
#include "gemm_kernel.h"

int gemm_launch_i8(fhip_ctx *ctx, const GemmPlan &p, const GemmArgs &g) {
  return gemm_launch_kind<GK_I8>(ctx, p, g);
}
