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

// Compile-time specialisations of the per-row work.  Everything a variant
// fixes is resolved at compile time so the hot loop is straight-line code; the
// general variant decides the same things with wavefront-uniform branches.
enum RowNormVariant {
  RN_GENERAL = 0,        // any combination the predicate admits
  RN_RMS_SCALE = 1,      // RMSNorm, scale of the row's type, no epilogue
  RN_RMS_SCALE_MULS = 2, // ... followed by one MUL with a scalar
  RN_RMS_SCALE_MULT = 3, // ... followed by one MUL with a full-size tensor
                         //     of the row's type
  RN_LN_SCALE_BIAS = 4,  // LayerNorm, scale and bias of the row's type
  RN_VARIANT_COUNT = 5
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct VecOf {
  static constexpr int kVec = 16 / sizeof(T);
};

template <typename T, int VEC>
__device__ __forceinline__ void unpack16(const u32x4 &raw, float (&out)[VEC]) {
  const T *p = reinterpret_cast<const T *>(&raw);
#pragma unroll
  for (int i = 0; i < VEC; ++i)
    out[i] = (float)p[i];
}

template <typename T, int VEC>
__device__ __forceinline__ void load_vec_same(const void *base, int64_t off,
                                              float (&out)[VEC]) {
  const u32x4 raw = *reinterpret_cast<const u32x4 *>((const T *)base + off);
  unpack16<T, VEC>(raw, out);
}

// Loads VEC consecutive elements starting at element offset `off` as floats.
// The operand has the row's own element type or is f32.
template <typename T, int VEC>
__device__ __forceinline__ void load_vec_as_float(const void *base, int dt,
                                                  int dt_of_T, int64_t off,
                                                  float (&out)[VEC]) {
  if (dt == dt_of_T) {
    load_vec_same<T, VEC>(base, off, out);
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

// Sum over the 64 lanes, result in every lane.  DPP row operations (no LDS
// crossbar traffic) reduce each row of 16 lanes; the four row sums are then
// read through scalar registers.
__device__ __forceinline__ float wave_sum64(float v) {
  auto dpp_add = [](float x, auto ctrl) {
    constexpr int kCtrl = decltype(ctrl)::value;
    const int moved = __builtin_amdgcn_update_dpp(
        0, __builtin_bit_cast(int, x), kCtrl, 0xF, 0xF, false);
    return x + __builtin_bit_cast(float, moved);
  };
  v = dpp_add(v, std::integral_constant<int, 0xB1>{});  // quad_perm [1,0,3,2]
  v = dpp_add(v, std::integral_constant<int, 0x4E>{});  // quad_perm [2,3,0,1]
  v = dpp_add(v, std::integral_constant<int, 0x124>{}); // row_ror 4
  v = dpp_add(v, std::integral_constant<int, 0x128>{}); // row_ror 8
  const int bits = __builtin_bit_cast(int, v);
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 0)) +
         __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 16)) +
         __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 32)) +
         __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 48));
}

template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
  if constexpr (N > 0) {
    static_for<N - 1>(f);
    f(std::integral_constant<int, N - 1>{});
  }
}

// WPR = wavefronts cooperating on one row (1, 2, 4, 8 or 16); a workgroup has
// max(4, WPR) wavefronts and covers max(1, 4 / WPR) rows.  CHUNKS = 16-byte
// loads per lane.  Few chunks per lane and many resident wavefronts is what
// saturates HBM on this part: occupancy, not per-lane instruction-level
// parallelism, hides the memory latency.
template <int WPR> struct RowNormGeom {
  static constexpr int kWaves = WPR < 4 ? 4 : WPR;
  static constexpr int kThreads = 64 * kWaves;
  static constexpr int kRowsPerWg = kWaves / WPR;
};

template <int WPR>
__device__ __forceinline__ float row_sum(float v, float *lds, int wave,
                                         int lane) {
  v = wave_sum64(v);
  if constexpr (WPR > 1) {
    __syncthreads(); // previous use of lds is complete
    if (lane == 0)
      lds[wave] = v;
    __syncthreads();
    const int first = (wave / WPR) * WPR;
    v = 0.f;
#pragma unroll
    for (int i = 0; i < WPR; ++i)
      v += lds[first + i];
  }
  return v;
}

// Two sums at once (same barriers as one).
template <int WPR>
__device__ __forceinline__ void row_sum2(float &a, float &b, float *lds,
                                         int wave, int lane) {
  a = wave_sum64(a);
  b = wave_sum64(b);
  if constexpr (WPR > 1) {
    constexpr int W = RowNormGeom<WPR>::kWaves;
    __syncthreads(); // previous use of lds is complete
    if (lane == 0) {
      lds[wave] = a;
      lds[W + wave] = b;
    }
    __syncthreads();
    const int first = (wave / WPR) * WPR;
    a = 0.f;
    b = 0.f;
#pragma unroll
    for (int i = 0; i < WPR; ++i) {
      a += lds[first + i];
      b += lds[W + first + i];
    }
  }
}

// One workgroup pass: the whole row is loaded with one 16-byte load per lane
// per chunk and stays packed in registers (4 VGPRs per chunk) between the
// statistics pass and the apply pass.
template <typename T, int CHUNKS, int WPR, int VARIANT>
__global__ __launch_bounds__(RowNormGeom<WPR>::kThreads) void rownorm_kernel(
    RowNormArgs g) {
  constexpr int VEC = VecOf<T>::kVec;
  constexpr int DT = DtypeOf<T>::value;
  constexpr int ROWS_PER_WG = RowNormGeom<WPR>::kRowsPerWg;
  constexpr bool GENERAL = VARIANT == RN_GENERAL;
  constexpr bool LAYERNORM_FIXED = VARIANT == RN_LN_SCALE_BIAS;
  __shared__ float lds[2 * RowNormGeom<WPR>::kWaves];

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wave_in_row = wave % WPR;
  const int col0 = (wave_in_row * 64 + lane) * VEC;
  constexpr int COL_STEP = WPR * 64 * VEC;
  const int inner = (int)g.inner;

  // The specialised variants fetch everything the apply pass needs ahead of the
  // reduction.  A lane owns the same columns in every row, so the per-column
  // parameters (scale, bias) are loaded once per workgroup and the workgroup
  // walks rows blockIdx.x, blockIdx.x + gridDim.x, ...
  constexpr bool PREFETCH = !GENERAL && CHUNKS <= 4;
  constexpr int PF = PREFETCH ? CHUNKS : 1;
  u32x4 scale_raw[PF], bias_raw[PF], mult_raw[PF];
  if constexpr (PREFETCH) {
    static_for<CHUNKS>([&](auto ci) {
      constexpr int c = decltype(ci)::value;
      const int col = col0 + c * COL_STEP;
      if (col < inner) {
        scale_raw[c] =
            *reinterpret_cast<const u32x4 *>((const T *)g.scale + col);
        if constexpr (VARIANT == RN_LN_SCALE_BIAS)
          bias_raw[c] =
              *reinterpret_cast<const u32x4 *>((const T *)g.bias + col);
      }
    });
  }

  const int64_t row_blocks = (g.rows + ROWS_PER_WG - 1) / ROWS_PER_WG;
  for (int64_t rb = blockIdx.x; rb < row_blocks; rb += gridDim.x) {
  const int64_t row = rb * ROWS_PER_WG + wave / WPR;
  const bool row_ok = row < g.rows;
  const T *xrow = (const T *)g.x + (row_ok ? row : 0) * g.x_row_stride;

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
  if constexpr (PREFETCH && VARIANT == RN_RMS_SCALE_MULT) {
    static_for<CHUNKS>([&](auto ci) {
      constexpr int c = decltype(ci)::value;
      const int col = col0 + c * COL_STEP;
      if (row_ok && col < inner)
        mult_raw[c] = __builtin_nontemporal_load(
            reinterpret_cast<const u32x4 *>((const T *)g.epi[0].ptr +
                                            row * g.epi[0].row_stride + col));
    });
  }

  const bool layernorm = GENERAL ? g.is_layernorm != 0 : LAYERNORM_FIXED;
  const float inv_n = 1.0f / (float)inner;
  float mean = 0.f;
  float ss = 0.f;
  if (layernorm) {
    // One pass, one reduction: sums of (x - p) and (x - p)^2 about a pivot p
    // taken from the row itself (its first element, read by every lane from
    // one cache line), so the variance does not cancel for rows far from 0:
    //   mean = p + S1/n,  var = S2/n - (S1/n)^2.
    const float p = row_ok ? (float)xrow[0] : 0.f;
    float s1 = 0.f, s2 = 0.f;
    static_for<CHUNKS>([&](auto ci) {
      constexpr int c = decltype(ci)::value;
      float v[VEC];
      unpack16<T, VEC>(raw[c], v);
      const bool live = col0 + c * COL_STEP < inner;
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const float d = live ? v[i] - p : 0.f;
        s1 += d;
        s2 += d * d;
      }
    });
    row_sum2<WPR>(s1, s2, lds, wave, lane);
    const float m1 = s1 * inv_n;
    mean = p + m1;
    const float var = s2 * inv_n - m1 * m1;
    ss = (var > 0.f ? var : 0.f) * (float)inner;
  } else {
    static_for<CHUNKS>([&](auto ci) {
      constexpr int c = decltype(ci)::value;
      float v[VEC];
      unpack16<T, VEC>(raw[c], v);
      // padding chunks hold zeros
#pragma unroll
      for (int i = 0; i < VEC; ++i)
        ss += v[i] * v[i];
    });
    ss = row_sum<WPR>(ss, lds, wave, lane);
  }
  const float rstd = 1.0f / sqrtf(ss * inv_n + g.eps);
  if (!row_ok)
    continue;
  if ((GENERAL || LAYERNORM_FIXED) && g.emit_stats && lane == 0 &&
      wave_in_row == 0) {
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
    if (layernorm) {
#pragma unroll
      for (int i = 0; i < VEC; ++i)
        y[i] = (y[i] - mean) * rstd;
    } else {
#pragma unroll
      for (int i = 0; i < VEC; ++i)
        y[i] *= rstd;
    }

    if constexpr (GENERAL) {
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
    } else {
      float s[VEC];
      if constexpr (PREFETCH)
        unpack16<T, VEC>(scale_raw[c], s);
      else
        load_vec_same<T, VEC>(g.scale, col, s);
#pragma unroll
      for (int i = 0; i < VEC; ++i)
        y[i] *= s[i];
      if constexpr (VARIANT == RN_LN_SCALE_BIAS) {
        float b[VEC];
        if constexpr (PREFETCH)
          unpack16<T, VEC>(bias_raw[c], b);
        else
          load_vec_same<T, VEC>(g.bias, col, b);
#pragma unroll
        for (int i = 0; i < VEC; ++i)
          y[i] += b[i];
      }
    }
    // A value that is stored next is rounded by the store's conversion: rounding
    // it to the same type first would only repeat the work.
    constexpr bool Y_IS_LAST = VARIANT == RN_RMS_SCALE || VARIANT == RN_LN_SCALE_BIAS;
    if (!(Y_IS_LAST && g.y_dt == DT))
      fhip_round_fast_vec<VEC>(g.y_dt, y);

    if constexpr (VARIANT == RN_RMS_SCALE_MULS) {
      const float m = g.epi[0].scalar;
#pragma unroll
      for (int i = 0; i < VEC; ++i)
        y[i] *= m;
      if (g.epi[0].result_dtype != DT)
        fhip_round_fast_vec<VEC>(g.epi[0].result_dtype, y);
    } else if constexpr (VARIANT == RN_RMS_SCALE_MULT) {
      float o[VEC];
      if constexpr (PREFETCH)
        unpack16<T, VEC>(mult_raw[c], o);
      else
        load_vec_same<T, VEC>(g.epi[0].ptr, row * g.epi[0].row_stride + col, o);
#pragma unroll
      for (int i = 0; i < VEC; ++i)
        y[i] *= o[i];
      if (g.epi[0].result_dtype != DT)
        fhip_round_fast_vec<VEC>(g.epi[0].result_dtype, y);
    } else if constexpr (GENERAL) {
      for (int e = 0; e < g.epi_count; ++e) {
        const FastEpiOp &o = g.epi[e];
        if (o.kind == FHIP_OPERAND_NONE) {
          fhip_pw_fast_unary_vec<false, VEC>(o.mode, y, o.params.swish_beta);
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
          fhip_pw_fast_binary_vec<VEC>(o.mode, o.acc_is_in1 != 0, y, other);
        }
        fhip_round_fast_vec<VEC>(o.result_dtype, y);
      }
    }
    u32x4 packed;
    T *pp = reinterpret_cast<T *>(&packed);
#pragma unroll
    for (int i = 0; i < VEC; ++i)
      pp[i] = (T)y[i];
    __builtin_nontemporal_store(packed, reinterpret_cast<u32x4 *>(orow + col));
  });
  } // rows of this workgroup
}

// (wavefronts per row, chunks per lane) pairs that are instantiated.  A row of
// N 16-byte-per-lane wavefront-chunks uses the first pair whose product
// covers N.
struct RowNormShape {
  int wpr, chunks;
};
constexpr RowNormShape kRowNormShapes[] = {
    {1, 1}, {1, 2}, {2, 2}, {4, 2}, {8, 2}, {16, 2}, {16, 4}, {16, 8}, {16, 16},
};

template <typename T, int WPR, int CHUNKS>
void rownorm_launch_one(int variant, int64_t rows, int num_cus, hipStream_t s,
                        const RowNormArgs &g) {
  constexpr int rpw = RowNormGeom<WPR>::kRowsPerWg;
  // Workgroups walk the row-blocks with the per-column parameters in
  // registers.  The grid is capped at a number of workgroups per compute unit
  // that leaves them UNEVEN shares of a large tensor (1 or 2 row-blocks each on
  // 8192 rows), which staggers their read and write bursts; measured on
  // 8192 x 4096 bf16, workgroups per CU -> us: LayerNorm 32: 25.0, 16: 24.3,
  // 20: 23.95; RMSNorm + MUL 32: 23.5, 20: 23.2, 24: 23.05.
  // FUSILLI_HIP_ROWNORM_WGS_PER_CU overrides it (0: one row-block each).
  int64_t blocks = (rows + rpw - 1) / rpw;
  int per_cu = variant == RN_LN_SCALE_BIAS ? 20 : 24;
  if (fhip_knobs().has_rownorm_wgs)
    per_cu = fhip_knobs().rownorm_wgs_per_cu;
  const int64_t cus = num_cus > 0 ? num_cus : 256;
  if (per_cu > 0 && blocks > cus * per_cu)
    blocks = cus * per_cu;
  const dim3 grid((unsigned)blocks);
  const dim3 block(RowNormGeom<WPR>::kThreads);
  switch (variant) {
  case RN_RMS_SCALE:
    hipLaunchKernelGGL((rownorm_kernel<T, CHUNKS, WPR, RN_RMS_SCALE>), grid,
                       block, 0, s, g);
    break;
  case RN_RMS_SCALE_MULS:
    hipLaunchKernelGGL((rownorm_kernel<T, CHUNKS, WPR, RN_RMS_SCALE_MULS>),
                       grid, block, 0, s, g);
    break;
  case RN_RMS_SCALE_MULT:
    hipLaunchKernelGGL((rownorm_kernel<T, CHUNKS, WPR, RN_RMS_SCALE_MULT>),
                       grid, block, 0, s, g);
    break;
  case RN_LN_SCALE_BIAS:
    hipLaunchKernelGGL((rownorm_kernel<T, CHUNKS, WPR, RN_LN_SCALE_BIAS>), grid,
                       block, 0, s, g);
    break;
  default:
    hipLaunchKernelGGL((rownorm_kernel<T, CHUNKS, WPR, RN_GENERAL>), grid,
                       block, 0, s, g);
    break;
  }
}

// Returns false when (wpr, chunks) is not an instantiated pair.
template <typename T>
bool rownorm_launch_typed(int chunks, int wpr, int variant, int64_t rows,
                          int num_cus, hipStream_t s, const RowNormArgs &g) {
#define FHIP_ROWNORM_CASE(W, C)                                                \
  if (wpr == W && chunks == C) {                                               \
    rownorm_launch_one<T, W, C>(variant, rows, num_cus, s, g);                          \
    return true;                                                               \
  }
  FHIP_ROWNORM_CASE(1, 1)
  FHIP_ROWNORM_CASE(1, 2)
  FHIP_ROWNORM_CASE(2, 2)
  FHIP_ROWNORM_CASE(4, 2)
  FHIP_ROWNORM_CASE(8, 2)
  FHIP_ROWNORM_CASE(16, 2)
  FHIP_ROWNORM_CASE(16, 4)
  FHIP_ROWNORM_CASE(16, 8)
  FHIP_ROWNORM_CASE(16, 16)
#undef FHIP_ROWNORM_CASE
  return false;
}

bool rownorm_launch_bf16(int chunks, int wpr, int variant, int64_t rows,
                        int num_cus, hipStream_t s, const RowNormArgs &g);
bool rownorm_launch_f16(int chunks, int wpr, int variant, int64_t rows,
                        int num_cus, hipStream_t s, const RowNormArgs &g);
bool rownorm_launch_f32(int chunks, int wpr, int variant, int64_t rows,
                        int num_cus, hipStream_t s, const RowNormArgs &g);

#endif // FUSILLI_AMD_CSRC_ROWNORM_KERNEL_H
