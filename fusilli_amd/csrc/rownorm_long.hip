// RMSNorm / LayerNorm forward for rows too long to hold in registers (more
// than 16384 16-byte chunks; e.g. a [16, 128, 64, 32] tensor normalised over
// everything but the batch dim is 16 rows of 262144 elements).
//
// A row is cut into segments, one workgroup each, so that a few rows still
// fill the machine:
//   pass 1  every workgroup reduces its segment to (sum (x - p), sum (x - p)^2)
//           around a pivot p = the row's first element (LayerNorm; RMSNorm
//           sums x^2) and leaves the pair in the context's scratch buffer;
//   pass 2  every workgroup adds up the pairs of its row in a fixed order,
//           derives mean and 1 / sqrt(var + eps), and normalises its segment
//           (the second read of X comes from the caches: a segment is a few KB).
// Rows are dense in memory and X, OUT, scale and bias walk a row alike, so the
// kernels go through a row's storage linearly whatever the order of its dims.
//
// Reference semantics: aten.rms_norm / aten.layer_norm over all dims except
// dim 0 (reference support/asm_emitter.h:1592-1626, 1427-1503;
// node/norm_utils.h:27-99).
#include "common.h"
#include "fast_paths.h"

namespace {

constexpr int kRlThreads = 256;

struct RowNormLongArgs {
  const void *x, *scale, *bias;
  void *out, *mean, *rstd;
  float *partial; // [rows][splits][2]
  int64_t rows, inner, x_row_stride, out_row_stride;
  int64_t seg; // elements per segment, a multiple of the vector width
  int32_t splits;
  int32_t scale_dt, bias_dt, y_dt, stats_dt;
  int32_t is_layernorm, emit_stats;
  float eps;
};

template <typename T> struct RlVec;
template <> struct RlVec<float> {
  static constexpr int kN = 4;
  static constexpr int kDt = FHIP_FLOAT;
  static __device__ __forceinline__ void load(const void *p, int64_t i, float (&v)[4]) {
    const float4 t = *(const float4 *)((const float *)p + i);
    v[0] = t.x, v[1] = t.y, v[2] = t.z, v[3] = t.w;
  }
  static __device__ __forceinline__ void store(void *p, int64_t i, const float (&v)[4]) {
    *(float4 *)((float *)p + i) = make_float4(v[0], v[1], v[2], v[3]);
  }
};
template <typename H> struct RlVec16 {
  static constexpr int kN = 8;
  typedef H hx8 __attribute__((ext_vector_type(8)));
  static __device__ __forceinline__ void load(const void *p, int64_t i, float (&v)[8]) {
    const hx8 t = *(const hx8 *)((const H *)p + i);
#pragma unroll
    for (int k = 0; k < 8; ++k)
      v[k] = (float)t[k];
  }
  static __device__ __forceinline__ void store(void *p, int64_t i, const float (&v)[8]) {
    hx8 t;
#pragma unroll
    for (int k = 0; k < 8; ++k)
      t[k] = (H)v[k];
    *(hx8 *)((H *)p + i) = t;
  }
};
template <> struct RlVec<__bf16> : RlVec16<__bf16> {
  static constexpr int kDt = FHIP_BFLOAT16;
};
template <> struct RlVec<_Float16> : RlVec16<_Float16> {
  static constexpr int kDt = FHIP_HALF;
};

__device__ __forceinline__ float rl_wave_sum(float v) {
  for (int o = 32; o > 0; o >>= 1)
    v += __shfl_xor(v, o, 64);
  return v;
}

// sums of a and b over the workgroup, the same value in every thread
__device__ __forceinline__ void rl_block_sum2(float &a, float &b, float (*lds)[2]) {
  a = rl_wave_sum(a);
  b = rl_wave_sum(b);
  const int wave = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) {
    lds[wave][0] = a;
    lds[wave][1] = b;
  }
  __syncthreads();
  a = b = 0.f;
  for (int i = 0; i < kRlThreads / 64; ++i) {
    a += lds[i][0];
    b += lds[i][1];
  }
}

template <typename T>
__global__ __launch_bounds__(kRlThreads) void rownorm_long_stats_kernel(RowNormLongArgs g) {
  using V = RlVec<T>;
  __shared__ float lds[kRlThreads / 64][2];
  const int64_t row = blockIdx.y, s = blockIdx.x;
  const T *xr = (const T *)g.x + row * g.x_row_stride;
  const float pivot = g.is_layernorm ? (float)xr[0] : 0.f;
  const int64_t lo = s * g.seg;
  const int64_t hi = lo + g.seg < g.inner ? lo + g.seg : g.inner;
  float s1 = 0.f, s2 = 0.f;
  for (int64_t i = lo + (int64_t)threadIdx.x * V::kN; i < hi; i += (int64_t)kRlThreads * V::kN) {
    float v[V::kN];
    V::load(xr, i, v);
#pragma unroll
    for (int k = 0; k < V::kN; ++k) {
      const float d = v[k] - pivot;
      s1 += d;
      s2 += d * d;
    }
  }
  rl_block_sum2(s1, s2, lds);
  if (threadIdx.x == 0) {
    float *p = g.partial + (row * g.splits + s) * 2;
    p[0] = s1;
    p[1] = s2;
    // the pivot travels with the sums: when OUT is X, the second kernel's
    // workgroups must not re-read it from a row that one of them is rewriting
    if (s == 0)
      g.partial[g.rows * g.splits * 2 + row] = pivot;
  }
}

template <typename T>
__global__ __launch_bounds__(kRlThreads) void rownorm_long_apply_kernel(RowNormLongArgs g) {
  using V = RlVec<T>;
  __shared__ float lds[kRlThreads / 64][2];
  const int64_t row = blockIdx.y, s = blockIdx.x;
  const T *xr = (const T *)g.x + row * g.x_row_stride;
  const float pivot = g.partial[g.rows * g.splits * 2 + row];
  // the row's statistics from its segments' sums (at most one per thread)
  float s1 = 0.f, s2 = 0.f;
  if ((int)threadIdx.x < g.splits) {
    const float *p = g.partial + (row * g.splits + threadIdx.x) * 2;
    s1 = p[0];
    s2 = p[1];
  }
  rl_block_sum2(s1, s2, lds);
  const float n = (float)g.inner;
  const float m1 = s1 / n;
  float mean = 0.f, var;
  if (g.is_layernorm) {
    mean = pivot + m1;
    var = s2 / n - m1 * m1;
    var = var > 0.f ? var : 0.f;
  } else {
    var = s2 / n;
  }
  const float rstd = 1.0f / sqrtf(var + g.eps);
  if (g.emit_stats && s == 0 && threadIdx.x == 0) {
    if (g.mean)
      fhip_store<float>(g.mean, g.stats_dt, row, mean);
    if (g.rstd)
      fhip_store<float>(g.rstd, g.stats_dt, row, rstd);
  }
  T *orow = (T *)g.out + row * g.out_row_stride;
  const int64_t lo = s * g.seg;
  const int64_t hi = lo + g.seg < g.inner ? lo + g.seg : g.inner;
  // scale and bias of the row's own type come as whole vectors, like the row
  const bool scale_vec = g.scale && g.scale_dt == V::kDt;
  const bool bias_vec = g.bias && g.bias_dt == V::kDt;
  for (int64_t i = lo + (int64_t)threadIdx.x * V::kN; i < hi; i += (int64_t)kRlThreads * V::kN) {
    float v[V::kN], sc[V::kN], bi[V::kN];
    V::load(xr, i, v);
    if (scale_vec) {
      V::load(g.scale, i, sc);
    } else {
#pragma unroll
      for (int k = 0; k < V::kN; ++k)
        sc[k] = g.scale ? fhip_load<float>(g.scale, g.scale_dt, i + k) : 1.f;
    }
    if (bias_vec) {
      V::load(g.bias, i, bi);
    } else {
#pragma unroll
      for (int k = 0; k < V::kN; ++k)
        bi[k] = g.bias ? fhip_load<float>(g.bias, g.bias_dt, i + k) : 0.f;
    }
#pragma unroll
    for (int k = 0; k < V::kN; ++k) {
      float y = (v[k] - mean) * rstd;
      if (g.scale)
        y *= sc[k];
      if (g.bias)
        y += bi[k];
      v[k] = fhip_round_through<float>(g.y_dt, y);
    }
    V::store(orow, i, v);
  }
}

template <typename T> void rl_launch(fhip_ctx *ctx, const RowNormLongArgs &g) {
  const dim3 grid((unsigned)g.splits, (unsigned)g.rows);
  hipLaunchKernelGGL(rownorm_long_stats_kernel<T>, grid, dim3(kRlThreads), 0, ctx->stream, g);
  hipLaunchKernelGGL(rownorm_long_apply_kernel<T>, grid, dim3(kRlThreads), 0, ctx->stream, g);
}

} // namespace

// The caller (rownorm.hip) has checked the layout conditions shared with the
// register-resident kernels: dense rows, X / OUT / scale / bias walking a row
// alike, inner % vector width == 0, aligned row strides.
bool fhip_norm_long_applicable(const fhip_norm_desc *d) {
  return d->epilogue.count == 0 && d->x.dim[0] <= 65535;
}

int fhip_norm_long(fhip_ctx *ctx, const fhip_norm_desc *d, int64_t inner,
                   const void *x, const void *scale, const void *bias, void *out,
                   void *mean, void *inv_variance) {
  FHIP_REQUIRE(ctx, fhip_norm_long_applicable(d),
               "rownorm: descriptor not supported by the long-row kernels");
  const int vec = 16 / (int)fhip_dtype_size(d->x.dtype);
  RowNormLongArgs g{};
  g.x = x, g.scale = scale, g.bias = bias, g.out = out;
  g.mean = mean, g.rstd = inv_variance;
  g.rows = d->x.dim[0];
  g.inner = inner;
  g.x_row_stride = d->x.dim[0] > 1 ? d->x.stride[0] : inner;
  g.out_row_stride = d->out.dim[0] > 1 ? d->out.stride[0] : inner;
  g.scale_dt = d->scale.dtype, g.bias_dt = d->bias.dtype;
  g.y_dt = d->y.dtype, g.stats_dt = d->stats_dtype;
  g.is_layernorm = d->is_layernorm, g.emit_stats = d->emit_stats;
  g.eps = d->epsilon;
  // segments: about eight workgroups per compute unit over all rows, at least
  // two vector loads per thread, at most one segment per thread of pass 2
  const int64_t cus = ctx->num_cus > 0 ? ctx->num_cus : 256;
  const int64_t min_seg = (int64_t)kRlThreads * vec * 2;
  int64_t splits = (8 * cus + g.rows - 1) / g.rows;
  const int64_t most = (inner + min_seg - 1) / min_seg;
  splits = splits < most ? splits : most;
  splits = splits < kRlThreads ? splits : kRlThreads;
  splits = splits < 1 ? 1 : splits;
  int64_t seg = (inner + splits - 1) / splits;
  seg = (seg + vec - 1) / vec * vec;
  splits = (inner + seg - 1) / seg;
  g.seg = seg;
  g.splits = (int32_t)splits;
  void *scratch = nullptr;
  // per row: a pair of sums per segment, and behind all pairs the rows' pivots
  if (fhip_ctx_scratch(ctx, (size_t)(g.rows * splits * 2 + g.rows) * sizeof(float), &scratch) != 0)
    return 1;
  g.partial = (float *)scratch;
  auto aligned = [](const void *p) { return ((uintptr_t)p & 15u) == 0; };
  FHIP_REQUIRE(ctx, aligned(x) && aligned(out),
               "rownorm: tensor base pointers must be 16-byte aligned");
  switch (d->x.dtype) {
  case FHIP_BFLOAT16:
    rl_launch<__bf16>(ctx, g);
    break;
  case FHIP_HALF:
    rl_launch<_Float16>(ctx, g);
    break;
  default:
    rl_launch<float>(ctx, g);
    break;
  }
  FHIP_HIP_CHECK(ctx, hipGetLastError());
  fhip_note_kernel(ctx, "rownorm_long segments=%d", g.splits);
  return 0;
}
