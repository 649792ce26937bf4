// Register-resident row-normalisation kernel (RMSNorm / LayerNorm forward) and
// its launch helpers; instantiated once per element type in rownorm_<type>.hip.
#ifndef FUSILLI_AMD_CSRC_ROWNORM_KERNEL_H
#define FUSILLI_AMD_CSRC_ROWNORM_KERNEL_H

#include "common.h"

#include <type_traits>


struct FastEpiOp {
  int32_t mode, kind, acc_is_in1, result_dtype, operand_dtype;
  int32_t col_unit; // operand varies along the row (stride 1) or not (0)
  float scalar;
  fhip_pointwise_params params;
  const void *ptr;
  int64_t row_stride;
};

struct RowNormArgs {
  const void *x;
  const void *scale;
  const void *bias;
  void *out;
  void *mean;
  void *rstd;
  int64_t rows, inner;
  int64_t x_row_stride, out_row_stride;
  int32_t scale_dt, bias_dt, y_dt, stats_dt;
  int32_t is_layernorm, emit_stats;
  float eps;
  int32_t epi_count;
  FastEpiOp epi[FHIP_MAX_EPILOGUE];
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct VecOf {
  static constexpr int kVec = 16 / sizeof(T);
};

template <typename T, int VEC>
__device__ __forceinline__ void unpack16(const u32x4 &raw, float *out) {
  const T *p = reinterpret_cast<const T *>(&raw);
#pragma unroll
  for (int i = 0; i < VEC; ++i)
    out[i] = (float)p[i];
}

// Loads VEC consecutive elements starting at element offset `off` as floats.
// The operand has the row's own element type or is f32.
template <typename T, int VEC>
__device__ __forceinline__ void load_vec_as_float(const void *base, int dt,
                                                  int dt_of_T, int64_t off,
                                                  float *out) {
  if (dt == dt_of_T) {
    const u32x4 raw = *reinterpret_cast<const u32x4 *>((const T *)base + off);
    unpack16<T, VEC>(raw, out);
  } else { // FHIP_FLOAT (the predicate admits no third type)
#pragma unroll
    for (int i = 0; i < VEC / 4; ++i) {
      const float4 f =
          *reinterpret_cast<const float4 *>((const float *)base + off + 4 * i);
      out[4 * i + 0] = f.x;
      out[4 * i + 1] = f.y;
      out[4 * i + 2] = f.z;
      out[4 * i + 3] = f.w;
    }
  }
}

template <typename T> struct DtypeOf;
template <> struct DtypeOf<__bf16> {
  static constexpr int value = FHIP_BFLOAT16;
};
template <> struct DtypeOf<_Float16> {
  static constexpr int value = FHIP_HALF;
};
template <> struct DtypeOf<float> {
  static constexpr int value = FHIP_FLOAT;
};

__device__ __forceinline__ float wave_sum64(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1)
    v += __shfl_xor(v, o, 64);
  return v;
}

template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
  if constexpr (N > 0) {
    static_for<N - 1>(f);
    f(std::integral_constant<int, N - 1>{});
  }
}

// WPR = wavefronts cooperating on one row (1 or 4); a 256-thread workgroup
// therefore covers 4 / WPR rows.  CHUNKS = 16-byte loads per lane.  The row
// stays packed in registers (4 VGPRs per chunk) between the statistics pass
// and the apply pass.
template <typename T, int CHUNKS, int WPR, bool EPI>
__global__ __launch_bounds__(256) void rownorm_kernel(RowNormArgs g) {
  constexpr int VEC = VecOf<T>::kVec;
  constexpr int DT = DtypeOf<T>::value;
  constexpr int ROWS_PER_WG = 4 / WPR;
  __shared__ float lds[4];

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wave_in_row = wave % WPR;
  const int64_t row = (int64_t)blockIdx.x * ROWS_PER_WG + wave / WPR;
  const bool row_ok = row < g.rows;
  const T *xrow = (const T *)g.x + (row_ok ? row : 0) * g.x_row_stride;
  const int col0 = (wave_in_row * 64 + lane) * VEC;
  constexpr int COL_STEP = WPR * 64 * VEC;
  const int inner = (int)g.inner;

  u32x4 raw[CHUNKS];
  static_for<CHUNKS>([&](auto ci) {
    constexpr int c = decltype(ci)::value;
    const int col = col0 + c * COL_STEP;
    if (row_ok && col < inner)
      raw[c] = __builtin_nontemporal_load(
          reinterpret_cast<const u32x4 *>(xrow + col));
    else
      raw[c] = u32x4{0, 0, 0, 0};
  });

  const float inv_n = 1.0f / (float)inner;
  float mean = 0.f;
  if (g.is_layernorm) {
    float s = 0.f;
    static_for<CHUNKS>([&](auto ci) {
      constexpr int c = decltype(ci)::value;
      float v[VEC];
      unpack16<T, VEC>(raw[c], v);
#pragma unroll
      for (int i = 0; i < VEC; ++i)
        s += v[i];
    });
    s = wave_sum64(s);
    if (WPR > 1) {
      if (lane == 0)
        lds[wave] = s;
      __syncthreads();
      s = lds[0] + lds[1] + lds[2] + lds[3];
      __syncthreads();
    }
    mean = s * inv_n;
  }
  float ss = 0.f;
  static_for<CHUNKS>([&](auto ci) {
    constexpr int c = decltype(ci)::value;
    const bool live = col0 + c * COL_STEP < inner;
    float v[VEC];
    unpack16<T, VEC>(raw[c], v);
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const float d = live ? v[i] - mean : 0.f;
      ss += d * d;
    }
  });
  ss = wave_sum64(ss);
  if (WPR > 1) {
    if (lane == 0)
      lds[wave] = ss;
    __syncthreads();
    ss = lds[0] + lds[1] + lds[2] + lds[3];
  }
  const float rstd = 1.0f / sqrtf(ss * inv_n + g.eps);
  if (!row_ok)
    return;
  if (g.emit_stats && lane == 0 && wave_in_row == 0) {
    if (g.stats_dt == FHIP_FLOAT) {
      ((float *)g.mean)[row] = mean;
      ((float *)g.rstd)[row] = rstd;
    } else if (g.stats_dt == FHIP_BFLOAT16) {
      ((__bf16 *)g.mean)[row] = (__bf16)mean;
      ((__bf16 *)g.rstd)[row] = (__bf16)rstd;
    } else {
      ((_Float16 *)g.mean)[row] = (_Float16)mean;
      ((_Float16 *)g.rstd)[row] = (_Float16)rstd;
    }
  }

  T *orow = (T *)g.out + row * g.out_row_stride;
  static_for<CHUNKS>([&](auto ci) {
    constexpr int c = decltype(ci)::value;
    const int col = col0 + c * COL_STEP;
    if (col >= inner)
      return;
    float y[VEC];
    unpack16<T, VEC>(raw[c], y);
#pragma unroll
    for (int i = 0; i < VEC; ++i)
      y[i] = (y[i] - mean) * rstd;
    if (g.scale) {
      float s[VEC];
      load_vec_as_float<T, VEC>(g.scale, g.scale_dt, DT, col, s);
#pragma unroll
      for (int i = 0; i < VEC; ++i)
        y[i] *= s[i];
    }
    if (g.bias) {
      float b[VEC];
      load_vec_as_float<T, VEC>(g.bias, g.bias_dt, DT, col, b);
#pragma unroll
      for (int i = 0; i < VEC; ++i)
        y[i] += b[i];
    }
    if (g.y_dt != FHIP_FLOAT) {
#pragma unroll
      for (int i = 0; i < VEC; ++i)
        y[i] = fhip_round_fast(g.y_dt, y[i]);
    }
    for (int e = 0; EPI && e < g.epi_count; ++e) {
      const FastEpiOp &o = g.epi[e];
      if (o.kind == FHIP_OPERAND_NONE) {
#pragma unroll
        for (int i = 0; i < VEC; ++i)
          y[i] = fhip_pw_fast_unary<false>(o.mode, y[i], o.params.swish_beta);
      } else {
        float other[VEC];
        if (o.kind == FHIP_OPERAND_SCALAR) {
#pragma unroll
          for (int i = 0; i < VEC; ++i)
            other[i] = o.scalar;
        } else if (o.col_unit) {
          load_vec_as_float<T, VEC>(o.ptr, o.operand_dtype, DT,
                                    row * o.row_stride + col, other);
        } else {
          const float s =
              o.operand_dtype == DT
                  ? (float)((const T *)o.ptr)[row * o.row_stride]
                  : ((const float *)o.ptr)[row * o.row_stride];
#pragma unroll
          for (int i = 0; i < VEC; ++i)
            other[i] = s;
        }
#pragma unroll
        for (int i = 0; i < VEC; ++i)
          y[i] = o.acc_is_in1 ? fhip_pw_fast_binary(o.mode, other[i], y[i])
                              : fhip_pw_fast_binary(o.mode, y[i], other[i]);
      }
      if (o.result_dtype != FHIP_FLOAT) {
#pragma unroll
        for (int i = 0; i < VEC; ++i)
          y[i] = fhip_round_fast(o.result_dtype, y[i]);
      }
    }
    u32x4 packed;
    T *pp = reinterpret_cast<T *>(&packed);
#pragma unroll
    for (int i = 0; i < VEC; ++i)
      pp[i] = (T)y[i];
    __builtin_nontemporal_store(packed, reinterpret_cast<u32x4 *>(orow + col));
  });
}


template <typename T, int WPR, bool EPI>
void launch_chunks(int chunks, dim3 grid, hipStream_t s, const RowNormArgs &g) {
  switch (chunks) {
  case 1:
    if constexpr (WPR == 1)
      hipLaunchKernelGGL((rownorm_kernel<T, 1, WPR, EPI>), grid, dim3(256), 0, s, g);
    else
      hipLaunchKernelGGL((rownorm_kernel<T, 4, WPR, EPI>), grid, dim3(256), 0, s, g);
    break;
  case 2:
    if constexpr (WPR == 1)
      hipLaunchKernelGGL((rownorm_kernel<T, 2, WPR, EPI>), grid, dim3(256), 0, s, g);
    else
      hipLaunchKernelGGL((rownorm_kernel<T, 4, WPR, EPI>), grid, dim3(256), 0, s, g);
    break;
  case 4:
    hipLaunchKernelGGL((rownorm_kernel<T, 4, WPR, EPI>), grid, dim3(256), 0, s, g);
    break;
  case 8:
    hipLaunchKernelGGL((rownorm_kernel<T, 8, WPR, EPI>), grid, dim3(256), 0, s, g);
    break;
  default:
    if constexpr (WPR == 4)
      hipLaunchKernelGGL((rownorm_kernel<T, 16, WPR, EPI>), grid, dim3(256), 0, s, g);
    break;
  }
}

template <typename T>
void rownorm_launch_typed(int chunks, int wpr, int64_t rows, hipStream_t s,
                          const RowNormArgs &g) {
  const dim3 grid1((unsigned)((rows + 3) / 4)), grid4((unsigned)rows);
  if (g.epi_count == 0) {
    if (wpr == 1)
      launch_chunks<T, 1, false>(chunks, grid1, s, g);
    else
      launch_chunks<T, 4, false>(chunks, grid4, s, g);
  } else {
    if (wpr == 1)
      launch_chunks<T, 1, true>(chunks, grid1, s, g);
    else
      launch_chunks<T, 4, true>(chunks, grid4, s, g);
  }
}


void rownorm_launch_bf16(int chunks, int wpr, int64_t rows, hipStream_t s,
                         const RowNormArgs &g);
void rownorm_launch_f16(int chunks, int wpr, int64_t rows, hipStream_t s,
                        const RowNormArgs &g);
void rownorm_launch_f32(int chunks, int wpr, int64_t rows, hipStream_t s,
                        const RowNormArgs &g);

#endif // FUSILLI_AMD_CSRC_ROWNORM_KERNEL_H
