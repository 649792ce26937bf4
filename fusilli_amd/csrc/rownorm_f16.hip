// Row-normalisation kernels for f16 rows.
#include "rownorm_kernel.h"

void rownorm_launch_f16(int chunks, int wpr, int64_t rows, hipStream_t s,
                         const RowNormArgs &g) {
  rownorm_launch_typed<_Float16>(chunks, wpr, rows, s, g);
}
