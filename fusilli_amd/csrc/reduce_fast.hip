// Bandwidth-bound keep-dim reductions over the trailing (contiguous) dims of a
// dense row-major tensor: X viewed as [rows, cols] -> Y[rows].
//
// TPR lanes share a row (16, 64 or 256 by row length), each streaming 16-byte
// non-temporal loads into an f32 accumulator; the map (abs / square / zero->1)
// and the combine (add / mul / min / max) are compile-time, so the inner loop
// has no mode dispatch; lanes are combined with wavefront shuffles (+ one LDS
// hop for 256-lane rows).
//
// Reference semantics: node/reduction_node.h:47-56 (a dim is reduced where
// Y == 1 < X), support/asm_emitter.h:2165-2322 (SUM/ADD, MUL, MIN, MAX, AMAX,
// AVG, NORM1, NORM2, MUL_NO_ZEROS).
#include "common.h"
#include "fast_paths.h"

#include <type_traits>

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
#define RF_AS1 __attribute__((address_space(1)))

enum { M_NONE = 0, M_ABS, M_SQUARE, M_ZERO_TO_ONE };
enum { C_ADD = 0, C_MUL, C_MIN, C_MAX };
enum { P_NONE = 0, P_MEAN, P_SQRT };

template <int MAP> __device__ __forceinline__ float rf_map(float v) {
  if constexpr (MAP == M_ABS)
    return fabsf(v);
  else if constexpr (MAP == M_SQUARE)
    return v * v;
  else if constexpr (MAP == M_ZERO_TO_ONE)
    return v == 0.f ? 1.f : v;
  else
    return v;
}

// min / max here ignore NaN (one instruction); NaN propagation (aten.amin /
// amax, and the generic kernel) is restored from `Acc::mag`, the largest
// |x| bit pattern seen: any NaN's pattern exceeds infinity's.
template <int COMB> __device__ __forceinline__ float rf_comb(float a, float b) {
  if constexpr (COMB == C_MUL)
    return a * b;
  else if constexpr (COMB == C_MIN)
    return fminf(a, b);
  else if constexpr (COMB == C_MAX)
    return fmaxf(a, b);
  else
    return a + b;
}

struct Acc {
  float v;      // running combine
  uint32_t mag; // min / max modes: largest magnitude bit pattern (f32 bits, or
                // two 16-bit patterns for the packed AMAX of 16-bit inputs)
};

template <int COMB> __device__ __forceinline__ float rf_identity() {
  if constexpr (COMB == C_MUL)
    return 1.f;
  else if constexpr (COMB == C_MIN)
    return INFINITY;
  else if constexpr (COMB == C_MAX)
    return -INFINITY;
  else
    return 0.f;
}

template <int MAP, int COMB> constexpr bool rf_is_amax() {
  return MAP == M_ABS && COMB == C_MAX;
}
template <int COMB> constexpr bool rf_tracks_nan() {
  return COMB == C_MIN || COMB == C_MAX;
}

template <typename T, int MAP, int COMB>
__device__ __forceinline__ void rf_chunk(const u32x4 v, Acc &a) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
  if constexpr (rf_is_amax<MAP, COMB>()) {
    // max |x| on the bit patterns: unsigned compare orders magnitudes and
    // puts NaN above everything; 16-bit inputs two per instruction
    if constexpr (std::is_same<T, float>::value) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t m = w[i] & 0x7fffffffu;
        a.mag = a.mag > m ? a.mag : m;
      }
    } else {
      typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const u16x2 m = __builtin_bit_cast(u16x2, w[i] & 0x7fff7fffu);
        const u16x2 c = __builtin_bit_cast(u16x2, a.mag);
        a.mag = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(c, m));
      }
    }
  } else if constexpr (std::is_same<T, float>::value) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      a.v = rf_comb<COMB>(a.v, rf_map<MAP>(__builtin_bit_cast(float, w[i])));
      if constexpr (rf_tracks_nan<COMB>()) {
        const uint32_t m = w[i] & 0x7fffffffu;
        a.mag = a.mag > m ? a.mag : m;
      }
    }
  } else {
    typedef T tx8 __attribute__((ext_vector_type(8)));
    const tx8 e = __builtin_bit_cast(tx8, v);
#pragma unroll
    for (int i = 0; i < 8; ++i)
      a.v = rf_comb<COMB>(a.v, rf_map<MAP>((float)e[i]));
    if constexpr (rf_tracks_nan<COMB>()) {
      typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const u16x2 m = __builtin_bit_cast(u16x2, w[i] & 0x7fff7fffu);
        const u16x2 c = __builtin_bit_cast(u16x2, a.mag);
        a.mag = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(c, m));
      }
    }
  }
}

// Folds the two accumulators of a lane / two lanes; `mag` as 16-bit pairs for
// 16-bit inputs, as one f32 pattern otherwise.
template <typename T, int COMB>
__device__ __forceinline__ Acc rf_merge(const Acc &a, const Acc &b) {
  Acc r;
  r.v = rf_comb<COMB>(a.v, b.v);
  if constexpr (std::is_same<T, float>::value) {
    r.mag = a.mag > b.mag ? a.mag : b.mag;
  } else {
    typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
    r.mag = __builtin_bit_cast(
        uint32_t, __builtin_elementwise_max(__builtin_bit_cast(u16x2, a.mag),
                                            __builtin_bit_cast(u16x2, b.mag)));
  }
  return r;
}

// Final value of a row from the merged accumulator.
template <typename T, int MAP, int COMB>
__device__ __forceinline__ float rf_finish(const Acc &a) {
  if constexpr (!rf_tracks_nan<COMB>()) {
    return a.v;
  } else {
    uint32_t mag; // as f32 bits
    if constexpr (std::is_same<T, float>::value) {
      mag = a.mag;
    } else {
      const uint32_t lo = a.mag & 0xffffu, hi = a.mag >> 16;
      const uint32_t m16 = lo > hi ? lo : hi;
      if constexpr (std::is_same<T, __bf16>::value) {
        mag = m16 << 16;
      } else {
        typedef _Float16 h1 __attribute__((ext_vector_type(1)));
        const unsigned short hs = (unsigned short)m16;
        mag = __builtin_bit_cast(uint32_t, (float)__builtin_bit_cast(_Float16, hs));
      }
    }
    const float magf = __builtin_bit_cast(float, mag);
    if (magf != magf)
      return magf; // a NaN was seen
    return rf_is_amax<MAP, COMB>() ? magf : a.v;
  }
}

struct ReduceRowsArgs {
  const char *x;
  void *y;
  int64_t rows;
  int64_t chunks; // 16-byte chunks per row
  int32_t y_dt, post;
  float inv_count;
};

template <typename T, int MAP, int COMB, int TPR>
__global__ __launch_bounds__(256) void reduce_rows_kernel(ReduceRowsArgs g) {
  constexpr int RPW = 256 / TPR; // rows per workgroup
  const int lane = threadIdx.x % TPR;
  const int64_t row = (int64_t)blockIdx.x * RPW + threadIdx.x / TPR;
  const bool live = row < g.rows;
  const RF_AS1 u32x4 *src =
      (const RF_AS1 u32x4 *)(g.x) + (live ? row : 0) * g.chunks;
  // two accumulators: two independent loads in flight per lane
  Acc a0{rf_identity<COMB>(), 0u}, a1{rf_identity<COMB>(), 0u};
  int64_t c = lane;
  if (live) {
    for (; c + TPR < g.chunks; c += 2 * TPR) {
      const u32x4 v0 = __builtin_nontemporal_load(src + c);
      const u32x4 v1 = __builtin_nontemporal_load(src + c + TPR);
      rf_chunk<T, MAP, COMB>(v0, a0);
      rf_chunk<T, MAP, COMB>(v1, a1);
    }
    if (c < g.chunks)
      rf_chunk<T, MAP, COMB>(__builtin_nontemporal_load(src + c), a0);
  }
  Acc a = rf_merge<T, COMB>(a0, a1);
  // combine the lanes of a row (rows never straddle a wavefront for TPR <= 64)
  constexpr int WIDTH = TPR < 64 ? TPR : 64;
#pragma unroll
  for (int s = WIDTH / 2; s > 0; s >>= 1) {
    Acc o;
    o.v = __shfl_xor(a.v, s, 64);
    o.mag = (uint32_t)__shfl_xor((int)a.mag, s, 64);
    a = rf_merge<T, COMB>(a, o);
  }
  if constexpr (TPR == 256) {
    __shared__ float part_v[4];
    __shared__ uint32_t part_m[4];
    if ((threadIdx.x & 63) == 0) {
      part_v[threadIdx.x >> 6] = a.v;
      part_m[threadIdx.x >> 6] = a.mag;
    }
    __syncthreads();
    a = rf_merge<T, COMB>(
        rf_merge<T, COMB>(Acc{part_v[0], part_m[0]}, Acc{part_v[1], part_m[1]}),
        rf_merge<T, COMB>(Acc{part_v[2], part_m[2]}, Acc{part_v[3], part_m[3]}));
  }
  float acc = rf_finish<T, MAP, COMB>(a);
  if (lane == 0 && live) {
    if (g.post == P_MEAN)
      acc *= g.inv_count;
    else if (g.post == P_SQRT)
      acc = sqrtf(acc);
    if (g.y_dt == FHIP_FLOAT)
      ((RF_AS1 float *)g.y)[row] = acc;
    else if (g.y_dt == FHIP_BFLOAT16)
      ((RF_AS1 __bf16 *)g.y)[row] = (__bf16)acc;
    else
      ((RF_AS1 _Float16 *)g.y)[row] = (_Float16)acc;
  }
}

struct ReducePlan {
  bool ok = false;
  int64_t rows = 0, cols = 0;
  int map = M_NONE, comb = C_ADD, post = P_NONE;
};

bool dense_row_major(const fhip_tensor_desc &t) {
  int64_t expect = 1;
  for (int i = t.rank - 1; i >= 0; --i) {
    if (t.dim[i] != 1 && t.stride[i] != expect)
      return false;
    expect *= t.dim[i];
  }
  return true;
}

ReducePlan make_plan(const fhip_reduce_desc *d) {
  ReducePlan p;
  const int xdt = d->x.dtype, ydt = d->y.dtype;
  auto f = [](int dt) {
    return dt == FHIP_FLOAT || dt == FHIP_BFLOAT16 || dt == FHIP_HALF;
  };
  if (!f(xdt) || !f(ydt))
    return p;
  if (!dense_row_major(d->x) || !dense_row_major(d->y))
    return p;
  // kept dims first, reduced dims last (unit dims may sit anywhere)
  p.rows = p.cols = 1;
  bool in_tail = false;
  for (int i = 0; i < d->x.rank; ++i) {
    if (d->x.dim[i] == 1)
      continue;
    const bool reduced = d->y.dim[i] == 1;
    if (reduced) {
      in_tail = true;
      p.cols *= d->x.dim[i];
    } else {
      if (in_tail)
        return p;
      p.rows *= d->x.dim[i];
    }
  }
  if (p.cols < 2 || (p.cols * fhip_dtype_size(xdt)) % 16 != 0)
    return p;
  if (p.rows >= (1ll << 31) * 16)
    return p;
  switch (d->mode) {
  case FHIP_RED_ADD:
  case FHIP_RED_SUM:
    break;
  case FHIP_RED_MUL:
    p.comb = C_MUL;
    break;
  case FHIP_RED_MUL_NO_ZEROS:
    p.comb = C_MUL;
    p.map = M_ZERO_TO_ONE;
    break;
  case FHIP_RED_MIN:
    p.comb = C_MIN;
    break;
  case FHIP_RED_MAX:
    p.comb = C_MAX;
    break;
  case FHIP_RED_AMAX:
    p.comb = C_MAX;
    p.map = M_ABS;
    break;
  case FHIP_RED_AVG:
    p.post = P_MEAN;
    break;
  case FHIP_RED_NORM1:
    p.map = M_ABS;
    break;
  case FHIP_RED_NORM2:
    p.map = M_SQUARE;
    p.post = P_SQRT;
    break;
  default:
    return p;
  }
  p.ok = true;
  return p;
}

template <typename T, int MAP, int COMB>
int launch_tpr(fhip_ctx *ctx, const ReduceRowsArgs &g) {
  const int64_t row_bytes = g.chunks * 16;
  if (row_bytes >= 4096) {
    hipLaunchKernelGGL((reduce_rows_kernel<T, MAP, COMB, 256>),
                       dim3((unsigned)g.rows), dim3(256), 0, ctx->stream, g);
  } else if (row_bytes >= 512) {
    hipLaunchKernelGGL((reduce_rows_kernel<T, MAP, COMB, 64>),
                       dim3((unsigned)((g.rows + 3) / 4)), dim3(256), 0,
                       ctx->stream, g);
  } else {
    hipLaunchKernelGGL((reduce_rows_kernel<T, MAP, COMB, 16>),
                       dim3((unsigned)((g.rows + 15) / 16)), dim3(256), 0,
                       ctx->stream, g);
  }
  FHIP_HIP_CHECK(ctx, hipGetLastError());
  return 0;
}

// The amax of |x| starts from 0, the others from their combine's identity;
// only these (map, combine) pairs occur.
template <typename T>
int launch_mode(fhip_ctx *ctx, const ReducePlan &p, const ReduceRowsArgs &g) {
  if (p.comb == C_ADD && p.map == M_NONE)
    return launch_tpr<T, M_NONE, C_ADD>(ctx, g);
  if (p.comb == C_ADD && p.map == M_ABS)
    return launch_tpr<T, M_ABS, C_ADD>(ctx, g);
  if (p.comb == C_ADD && p.map == M_SQUARE)
    return launch_tpr<T, M_SQUARE, C_ADD>(ctx, g);
  if (p.comb == C_MUL && p.map == M_NONE)
    return launch_tpr<T, M_NONE, C_MUL>(ctx, g);
  if (p.comb == C_MUL && p.map == M_ZERO_TO_ONE)
    return launch_tpr<T, M_ZERO_TO_ONE, C_MUL>(ctx, g);
  if (p.comb == C_MIN)
    return launch_tpr<T, M_NONE, C_MIN>(ctx, g);
  if (p.comb == C_MAX && p.map == M_ABS)
    return launch_tpr<T, M_ABS, C_MAX>(ctx, g);
  return launch_tpr<T, M_NONE, C_MAX>(ctx, g);
}

} // namespace

bool fhip_fast_reduce_applicable(const fhip_reduce_desc *d) {
  return make_plan(d).ok;
}

int fhip_fast_reduce(fhip_ctx *ctx, const fhip_reduce_desc *d, const void *x,
                     void *y) {
  const ReducePlan p = make_plan(d);
  FHIP_REQUIRE(ctx, p.ok, "reduce: descriptor not supported by the row kernel");
  FHIP_REQUIRE(ctx, ((uintptr_t)x & 15) == 0, "reduce: X must be 16-byte aligned");
  ReduceRowsArgs g{};
  g.x = (const char *)x;
  g.y = y;
  g.rows = p.rows;
  g.chunks = p.cols * fhip_dtype_size(d->x.dtype) / 16;
  g.y_dt = d->y.dtype;
  g.post = p.post;
  g.inv_count = 1.0f / (float)p.cols;
  fhip_note_kernel(ctx, "reduce_rows");
  switch (d->x.dtype) {
  case FHIP_FLOAT:
    return launch_mode<float>(ctx, p, g);
  case FHIP_BFLOAT16:
    return launch_mode<__bf16>(ctx, p, g);
  default:
    return launch_mode<_Float16>(ctx, p, g);
  }
}
