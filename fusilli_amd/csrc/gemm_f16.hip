// MFMA GEMM kernels for f16 operands.
#include "gemm_kernel.h"

int gemm_launch_f16(fhip_ctx *ctx, const GemmPlan &p, const GemmArgs &g) {
  return gemm_launch_kind<GK_F16>(ctx, p, g);
}
