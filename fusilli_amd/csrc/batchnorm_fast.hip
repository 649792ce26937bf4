// Batch normalisation forward for dense channels-last tensors.
//
// X [N, C, spatial...] with the channel as the fastest dim is a matrix of
// rows = N * spatial pixels by C channels, and the statistics are column
// sums.  A thread owns one 16-byte chunk of channels (8 of a 16-bit type, 4
// floats) -- the same chunk in every row it visits -- so loads are whole
// pixel vectors, the per-channel parameters stay in registers, and nothing is
// indexed per element:
//
//   training   pass 1  a workgroup walks a block of rows; its threads add
//                      (x - p) and (x - p)^2 per channel around a pivot p =
//                      the channel's value in row 0 (the variance does not
//                      cancel for channels far from 0), the row lanes of a
//                      chunk meet in LDS, and the workgroup's 2 C sums go to
//                      the context's scratch;
//              pass 2  per channel, 64 lanes add the workgroups' sums (in a
//                      fixed order), store mean and 1 / sqrt(var + eps) and
//                      leave the multiplier, the mean and the bias as vectors;
//              pass 3  y = (x - mean) * a + b over all rows (X comes from the caches
//                      where it still is there);
//   inference  pass 2' a and b from the running statistics, then pass 3.
//
// Reference semantics: aten.native_batch_norm (reference
// support/asm_emitter.h:1066-1290, node/batchnorm_node.h:33-245): biased
// variance, saved statistics = (mean, 1 / sqrt(var + eps)).
#include "common.h"
#include "fast_paths.h"

namespace {

constexpr int kBnThreads = 256;

struct BnFastArgs {
  const void *x;
  void *y;
  const void *scale, *bias, *mean, *var; // per-channel vectors (may be null)
  void *saved_mean, *saved_inv;
  float *partial; // [workgroups][2][C], then multiplier[C], mean[C], bias[C]
  int64_t rows;
  int32_t C, chunks, row_lanes, rows_per_wg, nwg;
  int32_t scale_dt, bias_dt, running_dt, stats_dt;
  int32_t training;
  float eps;
};

template <typename T> struct BnVec;
template <> struct BnVec<float> {
  static constexpr int kN = 4;
  static __device__ __forceinline__ void load(const void *p, int64_t i, float (&v)[4]) {
    const float4 t = *(const float4 *)((const float *)p + i);
    v[0] = t.x, v[1] = t.y, v[2] = t.z, v[3] = t.w;
  }
  static __device__ __forceinline__ void store(void *p, int64_t i, const float (&v)[4]) {
    *(float4 *)((float *)p + i) = make_float4(v[0], v[1], v[2], v[3]);
  }
};
template <typename H> struct BnVec16 {
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
    __builtin_nontemporal_store(t, (hx8 *)((H *)p + i));
  }
};
template <> struct BnVec<__bf16> : BnVec16<__bf16> {};
template <> struct BnVec<_Float16> : BnVec16<_Float16> {};

// pass 1: partial[wg][0][c] = sum (x - p), partial[wg][1][c] = sum (x - p)^2
template <typename T>
__global__ __launch_bounds__(kBnThreads) void bn_stats_kernel(BnFastArgs g) {
  using V = BnVec<T>;
  extern __shared__ __attribute__((aligned(16))) float red[]; // [row_lanes][2][C]
  const int chunk = threadIdx.x % g.chunks, lane = threadIdx.x / g.chunks;
  const int c0 = chunk * V::kN;
  float s1[V::kN], s2[V::kN];
#pragma unroll
  for (int k = 0; k < V::kN; ++k)
    s1[k] = s2[k] = 0.f;
  if (lane < g.row_lanes) {
    float pv[V::kN];
    V::load(g.x, c0, pv); // row 0
    const int64_t r0 = (int64_t)blockIdx.x * g.rows_per_wg;
    const int64_t r1 = r0 + g.rows_per_wg < g.rows ? r0 + g.rows_per_wg : g.rows;
    // eight rows in flight per lane (a workgroup has a dozen or so in all:
    // the loop is as long as its loads' latency, not its arithmetic); rows
    // past the end re-read the last one and count as zero
    constexpr int kFly = 8;
    for (int64_t r = r0 + lane; r < r1; r += (int64_t)kFly * g.row_lanes) {
      float v[kFly][V::kN];
#pragma unroll
      for (int u = 0; u < kFly; ++u) {
        const int64_t rr = r + (int64_t)u * g.row_lanes;
        V::load(g.x, (rr < r1 ? rr : r1 - 1) * g.C + c0, v[u]);
      }
#pragma unroll
      for (int u = 0; u < kFly; ++u) {
        const bool live = r + (int64_t)u * g.row_lanes < r1;
#pragma unroll
        for (int k = 0; k < V::kN; ++k) {
          const float d = live ? v[u][k] - pv[k] : 0.f;
          s1[k] += d;
          s2[k] = __builtin_fmaf(d, d, s2[k]);
        }
      }
    }
    // (whole 16-byte stores: scalar ones would meet on the banks eight at a time)
#pragma unroll
    for (int k = 0; k < V::kN; k += 4) {
      *(float4 *)&red[(lane * 2 + 0) * g.C + c0 + k] =
          make_float4(s1[k], s1[k + 1], s1[k + 2], s1[k + 3]);
      *(float4 *)&red[(lane * 2 + 1) * g.C + c0 + k] =
          make_float4(s2[k], s2[k + 1], s2[k + 2], s2[k + 3]);
    }
  }
  __syncthreads();
  // the row lanes' sums, in lane order, by the first 2 C threads (in turns)
  for (int o = threadIdx.x; o < 2 * g.C; o += kBnThreads) {
    float acc = 0.f;
#pragma unroll 8
    for (int l = 0; l < g.row_lanes; ++l)
      acc += red[l * 2 * g.C + o];
    g.partial[(int64_t)blockIdx.x * 2 * g.C + o] = acc;
  }
}

// pass 2 / 2': per channel the multiplier inv * scale, the mean and the bias.
// A workgroup serves 4 channels: 64 lanes per channel add the workgroups'
// sums w, w + 64, ... and meet through a fixed tree (lanes of a wavefront by
// cross-lane moves, the four wavefronts in LDS), the same for every run.
constexpr int kBnFinCh = 4;
template <typename T>
__global__ __launch_bounds__(kBnThreads) void bn_finalize_kernel(BnFastArgs g) {
  __shared__ float red[kBnThreads / 64][kBnFinCh][2];
  const int ci = threadIdx.x % kBnFinCh, wl = threadIdx.x / kBnFinCh;
  const int c = blockIdx.x * kBnFinCh + ci;
  const bool live = c < g.C;
  float s1 = 0.f, s2 = 0.f;
  if (g.training) {
    if (live) {
#pragma unroll 8
      for (int w = wl; w < g.nwg; w += kBnThreads / kBnFinCh) {
        s1 += g.partial[(int64_t)w * 2 * g.C + c];
        s2 += g.partial[(int64_t)w * 2 * g.C + g.C + c];
      }
    }
    // lanes l, l ^ 4, l ^ 8, ... hold the same channel
#pragma unroll
    for (int m = kBnFinCh; m < 64; m <<= 1) {
      s1 += __shfl_xor(s1, m, 64);
      s2 += __shfl_xor(s2, m, 64);
    }
    if ((threadIdx.x & 63) < kBnFinCh) {
      red[threadIdx.x >> 6][ci][0] = s1;
      red[threadIdx.x >> 6][ci][1] = s2;
    }
  }
  __syncthreads();
  if (wl != 0 || !live)
    return;
  float mean, inv;
  if (g.training) {
    s1 = s2 = 0.f;
#pragma unroll
    for (int l = 0; l < kBnThreads / 64; ++l) {
      s1 += red[l][ci][0];
      s2 += red[l][ci][1];
    }
    const float n = (float)g.rows;
    const float m1 = s1 / n;
    const float pivot = (float)((const T *)g.x)[c];
    mean = pivot + m1;
    float var = s2 / n - m1 * m1;
    var = var > 0.f ? var : 0.f;
    inv = 1.0f / sqrtf(var + g.eps);
    fhip_store<float>(g.saved_mean, g.stats_dt, c, mean);
    fhip_store<float>(g.saved_inv, g.stats_dt, c, inv);
  } else {
    mean = fhip_load<float>(g.mean, g.running_dt, c);
    inv = 1.0f / sqrtf(fhip_load<float>(g.var, g.running_dt, c) + g.eps);
  }
  const float sc = g.scale ? fhip_load<float>(g.scale, g.scale_dt, c) : 1.f;
  const float bi = g.bias ? fhip_load<float>(g.bias, g.bias_dt, c) : 0.f;
  float *ab = g.partial + (int64_t)g.nwg * 2 * g.C;
  ab[c] = inv * sc;
  ab[g.C + c] = mean;
  ab[2 * g.C + c] = bi;
}

// pass 3: y = (x - mean) * (inv * scale) + bias
template <typename T>
__global__ __launch_bounds__(kBnThreads) void bn_apply_kernel(BnFastArgs g) {
  using V = BnVec<T>;
  const int chunk = threadIdx.x % g.chunks, lane = threadIdx.x / g.chunks;
  if (lane >= g.row_lanes)
    return;
  const int c0 = chunk * V::kN;
  const float *ab = g.partial + (int64_t)g.nwg * 2 * g.C;
  float a[V::kN], m[V::kN], b[V::kN];
#pragma unroll
  for (int k = 0; k < V::kN; ++k) {
    a[k] = ab[c0 + k];
    m[k] = ab[g.C + c0 + k];
    b[k] = ab[2 * g.C + c0 + k];
  }
  const int64_t step = (int64_t)gridDim.x * g.row_lanes;
  for (int64_t r = (int64_t)blockIdx.x * g.row_lanes + lane; r < g.rows; r += step) {
    float v[V::kN];
    V::load(g.x, r * g.C + c0, v);
#pragma unroll
    for (int k = 0; k < V::kN; ++k)
      v[k] = __builtin_fmaf(v[k] - m[k], a[k], b[k]);
    V::store(g.y, r * g.C + c0, v);
  }
}

// dense channels-last strides of dims [N, C, spatial...]
bool bn_channels_last(const fhip_tensor_desc &t) {
  if (t.dim[1] != 1 && t.stride[1] != 1)
    return false;
  int64_t expect = t.dim[1];
  for (int i = t.rank - 1; i >= 2; --i) {
    if (t.dim[i] != 1 && t.stride[i] != expect)
      return false;
    expect *= t.dim[i];
  }
  return t.dim[0] == 1 || t.stride[0] == expect;
}

bool bn_plan(const fhip_batchnorm_desc *d, BnFastArgs &g) {
  if (d->x.rank < 2 || d->x.dtype != d->y.dtype)
    return false;
  const int dt = d->x.dtype;
  if (dt != FHIP_FLOAT && dt != FHIP_BFLOAT16 && dt != FHIP_HALF)
    return false;
  const int vec = dt == FHIP_FLOAT ? 4 : 8;
  const int64_t C = d->x.dim[1];
  if (C < vec || C % vec != 0 || C / vec > kBnThreads)
    return false;
  if (!bn_channels_last(d->x) || !bn_channels_last(d->y))
    return false;
  const int64_t total = fhip_desc_volume(d->x);
  if (total <= 0 || total >= (1ll << 40))
    return false;
  g.C = (int32_t)C;
  g.rows = total / C;
  g.chunks = (int32_t)(C / vec);
  g.row_lanes = kBnThreads / g.chunks;
  g.training = d->training;
  g.scale_dt = d->scale_dtype, g.bias_dt = d->bias_dtype;
  g.running_dt = d->running_dtype, g.stats_dt = d->stats_dtype;
  g.eps = d->epsilon;
  // about two workgroups per compute unit, at least one round of the row lanes each
  int64_t nwg = 512;
  const int64_t most = (g.rows + g.row_lanes - 1) / g.row_lanes;
  nwg = nwg < most ? nwg : most;
  g.rows_per_wg = (int32_t)((g.rows + nwg - 1) / nwg);
  g.nwg = (int32_t)((g.rows + g.rows_per_wg - 1) / g.rows_per_wg);
  // LDS of pass 1: row_lanes x 2 x C floats
  return (int64_t)g.row_lanes * 2 * C * 4 <= 64 * 1024;
}

template <typename T> void bn_launch(fhip_ctx *ctx, const BnFastArgs &g) {
  if (g.training)
    hipLaunchKernelGGL(bn_stats_kernel<T>, dim3((unsigned)g.nwg), dim3(kBnThreads),
                       (size_t)g.row_lanes * 2 * g.C * 4, ctx->stream, g);
  hipLaunchKernelGGL(bn_finalize_kernel<T>, dim3((unsigned)((g.C + kBnFinCh - 1) / kBnFinCh)),
                     dim3(kBnThreads), 0, ctx->stream, g);
  // workgroups walk the rows with their channels' (a, mean, b) in registers
  int64_t blocks = (g.rows + g.row_lanes - 1) / g.row_lanes;
  const int64_t cap = 256 * 24;
  blocks = blocks < cap ? blocks : cap;
  hipLaunchKernelGGL(bn_apply_kernel<T>, dim3((unsigned)blocks), dim3(kBnThreads), 0, ctx->stream,
                     g);
}

} // namespace

bool fhip_fast_batchnorm_applicable(const fhip_batchnorm_desc *d) {
  BnFastArgs g{};
  return bn_plan(d, g);
}

int fhip_fast_batchnorm(fhip_ctx *ctx, const fhip_batchnorm_desc *d, const void *x,
                        const void *scale, const void *bias, const void *running_mean,
                        const void *running_var, void *y, void *saved_mean,
                        void *saved_inv_variance) {
  BnFastArgs g{};
  FHIP_REQUIRE(ctx, bn_plan(d, g), "batchnorm: descriptor not supported by the channels-last kernels");
  FHIP_REQUIRE(ctx, (((uintptr_t)x | (uintptr_t)y) & 15) == 0,
               "batchnorm: X and Y must be 16-byte aligned");
  void *scratch = nullptr;
  if (fhip_ctx_scratch(ctx, ((size_t)g.nwg * 2 + 3) * (size_t)g.C * sizeof(float), &scratch) != 0)
    return 1;
  g.x = x, g.y = y;
  g.scale = scale, g.bias = bias, g.mean = running_mean, g.var = running_var;
  g.saved_mean = saved_mean, g.saved_inv = saved_inv_variance;
  g.partial = (float *)scratch;
  if (d->x.dtype == FHIP_FLOAT)
    bn_launch<float>(ctx, g);
  else if (d->x.dtype == FHIP_BFLOAT16)
    bn_launch<__bf16>(ctx, g);
  else
    bn_launch<_Float16>(ctx, g);
  FHIP_HIP_CHECK(ctx, hipGetLastError());
  fhip_note_kernel(ctx, "batchnorm_channels_last training=%d workgroups=%d", (int)d->training,
                   g.nwg);
  return 0;
}
