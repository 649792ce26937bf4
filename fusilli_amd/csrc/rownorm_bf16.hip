// Row-normalisation kernels for bf16 rows.
#include "rownorm_kernel.h"

bool rownorm_launch_bf16(int chunks, int wpr, int variant, int64_t rows,
                        int num_cus, hipStream_t s, const RowNormArgs &g) {
  return rownorm_launch_typed<__bf16>(chunks, wpr, variant, rows, num_cus, s, g);
}
