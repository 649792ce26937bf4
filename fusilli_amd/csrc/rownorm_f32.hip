// Row-normalisation kernels for f32 rows.
#include "rownorm_kernel.h"

void rownorm_launch_f32(int chunks, int wpr, int64_t rows, hipStream_t s,
                         const RowNormArgs &g) {
  rownorm_launch_typed<float>(chunks, wpr, rows, s, g);
}
