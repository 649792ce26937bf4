// Row-normalisation kernels for bf16 rows.
#include "rownorm_kernel.h"

void rownorm_launch_bf16(int chunks, int wpr, int64_t rows, hipStream_t s,
                         const RowNormArgs &g) {
  rownorm_launch_typed<__bf16>(chunks, wpr, rows, s, g);
}
