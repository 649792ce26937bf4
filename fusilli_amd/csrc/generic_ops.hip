// Generic strided kernels: one straightforward gfx950 kernel per op that accepts
// every layout, broadcast and element type the descriptors can express.  They
// keep the API surface honest; the MFMA / bandwidth-tuned kernels in the other
// files take over for the shapes they support.  This file also holds the op
// entry points of the C ABI, which choose between the two.
#include "common.h"
#include "fast_paths.h"

namespace {

struct Dims {
  int32_t rank;
  int64_t dim[FHIP_MAX_RANK];
};

__device__ __forceinline__ void unravel(int64_t lin, const Dims &s,
                                        int64_t *coord) {
  for (int r = s.rank - 1; r >= 0; --r) {
    const int64_t d = s.dim[r];
    coord[r] = lin % d;
    lin /= d;
  }
}

struct Strides {
  int64_t s[FHIP_MAX_RANK];
};

__device__ __forceinline__ int64_t dot(const int64_t *coord, const Strides &st,
                                       int rank) {
  int64_t off = 0;
  for (int r = 0; r < rank; ++r)
    off += coord[r] * st.s[r];
  return off;
}

Dims make_dims(const fhip_tensor_desc &t) {
  Dims d{};
  d.rank = t.rank;
  for (int i = 0; i < t.rank; ++i)
    d.dim[i] = t.dim[i];
  return d;
}

Strides make_strides(const fhip_tensor_desc &t) {
  Strides s{};
  for (int i = 0; i < t.rank; ++i)
    s.s[i] = t.dim[i] == 1 ? 0 : t.stride[i];
  return s;
}

inline unsigned grid_for(int64_t n, int block) {
  int64_t g = (n + block - 1) / block;
  return (unsigned)g;
}

// --------------------------------------------------------------------------
// matmul
// --------------------------------------------------------------------------
struct MatmulArgs {
  Dims out;          // logical output dims [..., M, N]
  Strides a, b, o;   // strides on output coords (batch dims broadcast -> 0)
  int64_t a_k, b_k;  // K strides
  int64_t K;
  int32_t a_dt, b_dt, c_dt, o_dt;
  DevEpilogue epi;
};

template <typename Acc>
__global__ void generic_matmul_kernel(MatmulArgs g, const void *a,
                                      const void *b, void *out,
                                      int64_t total) {
  const int64_t lin = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (lin >= total)
    return;
  int64_t coord[FHIP_MAX_RANK];
  unravel(lin, g.out, coord);
  const int rank = g.out.rank;
  // a uses (batch..., m), b uses (batch..., n)
  int64_t ao = 0, bo = 0;
  for (int r = 0; r < rank; ++r) {
    ao += coord[r] * g.a.s[r];
    bo += coord[r] * g.b.s[r];
  }
  Acc acc = 0;
  for (int64_t k = 0; k < g.K; ++k) {
    const Acc av = fhip_load<Acc>(a, g.a_dt, ao + k * g.a_k);
    const Acc bv = fhip_load<Acc>(b, g.b_dt, bo + k * g.b_k);
    acc += av * bv;
  }
  double v = fhip_round_through<double>(g.c_dt, (double)acc);
  v = fhip_apply_epilogue<double>(g.epi, v, coord);
  fhip_store<double>(out, g.o_dt, dot(coord, g.o, rank), v);
}

// Floating-point matmul on the f32 matrix instruction (v_mfma_f32_32x32x2_f32):
// any strides, batch broadcasting and epilogue of the strided kernel above;
// f32, bf16 and f16 operands (also mixed) are widened to f32 as they are
// staged, which is exact.  A
// workgroup of 4 wavefronts owns a 64 x 64 output tile of one batch entry and
// walks K in steps of 16 through LDS (As[k][m], Bs[k][n]); the next step's
// global loads are in flight while the current one is multiplied.
constexpr int kF32Tile = 64, kF32K = 16, kF32Pitch = kF32Tile + 4;

// Operand element as f32.  DT is the element type fixed at compile time (both
// operands f32, bf16 or f16: a plain load and at most one conversion); -1
// takes the type from the descriptor per element (mixed operand types).
template <int DT>
__device__ __forceinline__ float matmul_operand(const void *p, int dt, int64_t idx) {
  if constexpr (DT == FHIP_FLOAT)
    return ((const float *)p)[idx];
  else if constexpr (DT == FHIP_BFLOAT16)
    return (float)((const __bf16 *)p)[idx];
  else if constexpr (DT == FHIP_HALF)
    return (float)((const _Float16 *)p)[idx];
  else
    return fhip_load<float>(p, dt, idx);
}

template <int DT>
__global__ __launch_bounds__(256) void tiled_matmul_f32_kernel(
    MatmulArgs g, const void *a, const void *b, void *out, int tiles_n) {
  typedef float f32x16 __attribute__((ext_vector_type(16)));
  __shared__ float As[kF32K][kF32Pitch], Bs[kF32K][kF32Pitch];
  const int rank = g.out.rank;
  const int64_t M = g.out.dim[rank - 2], N = g.out.dim[rank - 1];
  const int64_t m0 = (int64_t)(blockIdx.x / tiles_n) * kF32Tile;
  const int64_t n0 = (int64_t)(blockIdx.x % tiles_n) * kF32Tile;
  // batch coordinates of this workgroup
  int64_t coord[FHIP_MAX_RANK];
  {
    int64_t lin = blockIdx.y;
    for (int r = rank - 3; r >= 0; --r) {
      coord[r] = lin % g.out.dim[r];
      lin /= g.out.dim[r];
    }
  }
  int64_t ab = 0, bb = 0;
  for (int r = 0; r < rank - 2; ++r) {
    ab += coord[r] * g.a.s[r];
    bb += coord[r] * g.b.s[r];
  }
  const int64_t a_sm = g.a.s[rank - 2], b_sn = g.b.s[rank - 1];
  const int t = threadIdx.x, wave = t >> 6, l = t & 63;
  const int wm = wave >> 1, wn = wave & 1;
  // each thread stages 4 elements of A and 4 of B per step; the fastest thread
  // index runs along whichever dimension is contiguous in memory
  const bool a_kfast = g.a_k == 1, b_kfast = g.b_k == 1;
  int a_m[4], a_kk[4], b_n[4], b_kk[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int e = t + i * 256;
    a_kk[i] = a_kfast ? e % kF32K : e / kF32Tile;
    a_m[i] = a_kfast ? e / kF32K : e % kF32Tile;
    b_kk[i] = b_kfast ? e % kF32K : e / kF32Tile;
    b_n[i] = b_kfast ? e / kF32K : e % kF32Tile;
  }
  auto fetch = [&](int64_t k0, float (&ra)[4], float (&rb)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int64_t m = m0 + a_m[i], n = n0 + b_n[i];
      const int64_t ka = k0 + a_kk[i], kb = k0 + b_kk[i];
      ra[i] = m < M && ka < g.K
                  ? matmul_operand<DT>(a, g.a_dt, ab + m * a_sm + ka * g.a_k)
                  : 0.f;
      rb[i] = n < N && kb < g.K
                  ? matmul_operand<DT>(b, g.b_dt, bb + n * b_sn + kb * g.b_k)
                  : 0.f;
    }
  };
  f32x16 acc;
#pragma unroll
  for (int r = 0; r < 16; ++r)
    acc[r] = 0.f;
  float ra[4], rb[4];
  fetch(0, ra, rb);
  for (int64_t k0 = 0; k0 < g.K; k0 += kF32K) {
    __syncthreads(); // the previous step's reads are done
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      As[a_kk[i]][a_m[i]] = ra[i];
      Bs[b_kk[i]][b_n[i]] = rb[i];
    }
    __syncthreads();
    if (k0 + kF32K < g.K)
      fetch(k0 + kF32K, ra, rb);
#pragma unroll
    for (int kk = 0; kk < kF32K; kk += 2) {
      const float av = As[kk + (l >> 5)][wm * 32 + (l & 31)];
      const float bv = Bs[kk + (l >> 5)][wn * 32 + (l & 31)];
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc, 0, 0, 0);
    }
  }
  // lane holds column l % 32, rows (r / 4) * 8 + (l / 32) * 4 + r % 4
  const int64_t n = n0 + wn * 32 + (l & 31);
  if (n >= N)
    return;
  coord[rank - 1] = n;
  // (the 16 rows of a lane together: a fused operand's values are fetched as
  // one batch of loads, not one after the other)
  // (in f32, like the accumulators and the tuned kernels' fused chains)
  float v[16];
  int64_t rows[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int64_t m = m0 + wm * 32 + (r >> 2) * 8 + (l >> 5) * 4 + (r & 3);
    rows[r] = m < M ? m : M - 1;
    v[r] = acc[r];
  }
  if (g.c_dt == FHIP_BFLOAT16 || g.c_dt == FHIP_HALF) {
    fhip_round_fast_vec<16>(g.c_dt, v);
  } else if (g.c_dt != FHIP_FLOAT) {
#pragma clang loop unroll(disable)
    for (int r = 0; r < 16; ++r)
      v[r] = fhip_round_through<float>(g.c_dt, v[r]);
  }
  if (g.epi.count > 0)
    fhip_apply_epilogue_many<float, 16>(g.epi, v, coord, rank - 2, rows);
  coord[rank - 2] = 0;
  const int64_t ob = dot(coord, g.o, rank), o_sm = g.o.s[rank - 2];
  int64_t idx[16];
  uint32_t live = 0;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int64_t m = m0 + wm * 32 + (r >> 2) * 8 + (l >> 5) * 4 + (r & 3);
    idx[r] = ob + m * o_sm;
    live |= (uint32_t)(m < M) << r;
  }
  fhip_store_many<float, 16>(out, g.o_dt, idx, v, live);
}

// Small outputs (few 64 x 64 tiles): a workgroup owns a 32 x 32 tile and its 4
// wavefronts split K four ways (K-steps w, w + 4, ...), each staging its own
// A / B sub-tiles in a private LDS region (no workgroup barriers in the loop);
// the partial sums meet in LDS and every wavefront finishes a quarter of the
// accumulator registers.
template <int DT>
__global__ __launch_bounds__(256) void splitk_matmul_f32_kernel(
    MatmulArgs g, const void *a, const void *b, void *out, int tiles_n) {
  typedef float f32x16 __attribute__((ext_vector_type(16)));
  constexpr int T = 32, PITCH = T + 4;
  __shared__ float As[4][kF32K][PITCH], Bs[4][kF32K][PITCH];
  __shared__ float part[4][16][64];
  const int rank = g.out.rank;
  const int64_t M = g.out.dim[rank - 2], N = g.out.dim[rank - 1];
  const int64_t m0 = (int64_t)(blockIdx.x / tiles_n) * T;
  const int64_t n0 = (int64_t)(blockIdx.x % tiles_n) * T;
  int64_t coord[FHIP_MAX_RANK];
  {
    int64_t lin = blockIdx.y;
    for (int r = rank - 3; r >= 0; --r) {
      coord[r] = lin % g.out.dim[r];
      lin /= g.out.dim[r];
    }
  }
  int64_t ab = 0, bb = 0;
  for (int r = 0; r < rank - 2; ++r) {
    ab += coord[r] * g.a.s[r];
    bb += coord[r] * g.b.s[r];
  }
  const int64_t a_sm = g.a.s[rank - 2], b_sn = g.b.s[rank - 1];
  const int wave = threadIdx.x >> 6, l = threadIdx.x & 63;
  const bool a_kfast = g.a_k == 1, b_kfast = g.b_k == 1;
  // a lane stages 8 elements of A and 8 of B per step (16 x 32 each)
  int a_m[8], a_kk[8], b_n[8], b_kk[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int e = l + i * 64;
    a_kk[i] = a_kfast ? e % kF32K : e / T;
    a_m[i] = a_kfast ? e / kF32K : e % T;
    b_kk[i] = b_kfast ? e % kF32K : e / T;
    b_n[i] = b_kfast ? e / kF32K : e % T;
  }
  // element offsets at K-step 0 (a step adds k0 times the K stride) and the
  // rows / columns that exist
  int64_t a_off[8], b_off[8];
  uint32_t a_live = 0, b_live = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int64_t m = m0 + a_m[i], n = n0 + b_n[i];
    a_off[i] = ab + m * a_sm + a_kk[i] * g.a_k;
    b_off[i] = bb + n * b_sn + b_kk[i] * g.b_k;
    a_live |= (uint32_t)(m < M) << i;
    b_live |= (uint32_t)(n < N) << i;
  }
  auto fetch = [&](int64_t k0, float (&ra)[8], float (&rb)[8]) {
    const int64_t ka0 = k0 * g.a_k, kb0 = k0 * g.b_k;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      ra[i] = ((a_live >> i) & 1) && k0 + a_kk[i] < g.K
                  ? matmul_operand<DT>(a, g.a_dt, a_off[i] + ka0)
                  : 0.f;
      rb[i] = ((b_live >> i) & 1) && k0 + b_kk[i] < g.K
                  ? matmul_operand<DT>(b, g.b_dt, b_off[i] + kb0)
                  : 0.f;
    }
  };
  f32x16 acc;
#pragma unroll
  for (int r = 0; r < 16; ++r)
    acc[r] = 0.f;
  float ra[8], rb[8];
  const int64_t stride = 4 * kF32K;
  fetch((int64_t)wave * kF32K, ra, rb);
  for (int64_t k0 = (int64_t)wave * kF32K; k0 < g.K; k0 += stride) {
    // wavefront-private LDS: program order (with the waits the compiler puts
    // before dependent LDS accesses) is all the synchronisation needed
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      As[wave][a_kk[i]][a_m[i]] = ra[i];
      Bs[wave][b_kk[i]][b_n[i]] = rb[i];
    }
    if (k0 + stride < g.K)
      fetch(k0 + stride, ra, rb);
#pragma unroll
    for (int kk = 0; kk < kF32K; kk += 2) {
      const float av = As[wave][kk + (l >> 5)][l & 31];
      const float bv = Bs[wave][kk + (l >> 5)][l & 31];
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc, 0, 0, 0);
    }
  }
#pragma unroll
  for (int r = 0; r < 16; ++r)
    part[wave][r][l] = acc[r];
  __syncthreads();
  const int64_t n = n0 + (l & 31);
  if (n >= N)
    return;
  coord[rank - 1] = n;
  float v[4];
  int64_t rows[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int r = wave * 4 + q;
    const int64_t m = m0 + (r >> 2) * 8 + (l >> 5) * 4 + (r & 3);
    const float sum = (part[0][r][l] + part[1][r][l]) + (part[2][r][l] + part[3][r][l]);
    rows[q] = m < M ? m : M - 1;
    v[q] = sum;
  }
  if (g.c_dt == FHIP_BFLOAT16 || g.c_dt == FHIP_HALF) {
    fhip_round_fast_vec<4>(g.c_dt, v);
  } else if (g.c_dt != FHIP_FLOAT) {
#pragma clang loop unroll(disable)
    for (int q = 0; q < 4; ++q)
      v[q] = fhip_round_through<float>(g.c_dt, v[q]);
  }
  if (g.epi.count > 0)
    fhip_apply_epilogue_many<float, 4>(g.epi, v, coord, rank - 2, rows);
  coord[rank - 2] = 0;
  const int64_t ob = dot(coord, g.o, rank), o_sm = g.o.s[rank - 2];
  int64_t idx[4];
  uint32_t live = 0;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int r = wave * 4 + q;
    const int64_t m = m0 + (r >> 2) * 8 + (l >> 5) * 4 + (r & 3);
    idx[q] = ob + m * o_sm;
    live |= (uint32_t)(m < M) << q;
  }
  fhip_store_many<float, 4>(out, g.o_dt, idx, v, live);
}

// --------------------------------------------------------------------------
// convolution forward (cross-correlation, zero padding, groups = C / fC)
// --------------------------------------------------------------------------
struct ConvArgs {
  Dims y;            // [N, K, out spatial...]
  Strides x, w, o;   // strides of X [N,C,sp..], W [K,fC,fsp..], OUT [N,K,sp..]
  int64_t x_dim[FHIP_MAX_RANK];
  int64_t w_dim[FHIP_MAX_RANK];
  int32_t spatial;
  int64_t pad[3], str[3], dil[3];
  int64_t groups;
  int32_t x_dt, w_dt, y_dt, o_dt;
  DevEpilogue epi;
};

__global__ void generic_conv_kernel(ConvArgs g, const void *x, const void *w,
                                    void *out, int64_t total) {
  const int64_t lin = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (lin >= total)
    return;
  int64_t coord[FHIP_MAX_RANK];
  unravel(lin, g.y, coord);
  const int sp = g.spatial;
  const int64_t n = coord[0], k = coord[1];
  const int64_t fC = g.w_dim[1];
  const int64_t kPerGroup = g.y.dim[1] / g.groups;
  const int64_t grp = k / kPerGroup;
  int64_t fvol = 1;
  for (int i = 0; i < sp; ++i)
    fvol *= g.w_dim[2 + i];
  float acc = 0.f;
  for (int64_t fc = 0; fc < fC; ++fc) {
    const int64_t c = grp * fC + fc;
    for (int64_t f = 0; f < fvol; ++f) {
      int64_t rem = f;
      int64_t xo = n * g.x.s[0] + c * g.x.s[1];
      int64_t wo = k * g.w.s[0] + fc * g.w.s[1];
      bool inside = true;
      for (int i = sp - 1; i >= 0; --i) {
        const int64_t fd = g.w_dim[2 + i];
        const int64_t fi = rem % fd;
        rem /= fd;
        const int64_t xi = coord[2 + i] * g.str[i] - g.pad[i] + fi * g.dil[i];
        if (xi < 0 || xi >= g.x_dim[2 + i])
          inside = false;
        xo += xi * g.x.s[2 + i];
        wo += fi * g.w.s[2 + i];
      }
      if (inside)
        acc += fhip_load<float>(x, g.x_dt, xo) * fhip_load<float>(w, g.w_dt, wo);
    }
  }
  float v = fhip_round_through<float>(g.y_dt, acc);
  v = fhip_apply_epilogue<float>(g.epi, v, coord);
  fhip_store<float>(out, g.o_dt, dot(coord, g.o, g.y.rank), v);
}

// --------------------------------------------------------------------------
// SDPA forward: one wavefront per query row, online softmax over 64-key chunks
// --------------------------------------------------------------------------
struct SdpaArgs {
  int64_t B, Hq, Hkv, Sq, Skv, D, Dv;
  int64_t q[4], k[4], v[4], o[4], m[4]; // element strides (mask: broadcast->0)
  int32_t q_dt, k_dt, v_dt, o_dt, m_dt;
  int32_t has_mask, causal;
  float scale;
};

__device__ __forceinline__ float wave_max(float v) {
  for (int o = 32; o > 0; o >>= 1)
    v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
  for (int o = 32; o > 0; o >>= 1)
    v += __shfl_xor(v, o, 64);
  return v;
}

// --------------------------------------------------------------------------
// convolution backward: data gradient and weight gradient of the forward
// above (reference node/conv_node.h:255-598; aten.convolution_backward).
// Both are gathers with f32 accumulation, no atomics.
// --------------------------------------------------------------------------
struct ConvBwdArgs {
  Dims out;          // dgrad: DX [N, C, sp..]; wgrad: DW [K, fC, fsp..]
  Strides x, w, y;   // strides of X / DX, W / DW, DY
  int64_t x_dim[FHIP_MAX_RANK];
  int64_t w_dim[FHIP_MAX_RANK];
  int64_t y_dim[FHIP_MAX_RANK];
  int32_t spatial;
  int64_t pad[3], str[3], dil[3];
  int64_t groups;
  int32_t x_dt, w_dt, y_dt;
};

// DX[n, c, i..] = sum over k of c's group, filter taps f with
// i + pad - f * dil = o * stride:  DY[n, k, o..] * W[k, c % fC, f..]
__global__ void generic_conv_dgrad_kernel(ConvBwdArgs g, const void *dy,
                                          const void *w, void *dx,
                                          int64_t total) {
  const int64_t lin = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (lin >= total)
    return;
  int64_t coord[FHIP_MAX_RANK];
  unravel(lin, g.out, coord);
  const int sp = g.spatial;
  const int64_t n = coord[0], c = coord[1];
  const int64_t fC = g.w_dim[1];
  const int64_t kPerGroup = g.w_dim[0] / g.groups;
  const int64_t grp = c / fC, fc = c - grp * fC;
  int64_t fvol = 1;
  for (int i = 0; i < sp; ++i)
    fvol *= g.w_dim[2 + i];
  float acc = 0.f;
  for (int64_t f = 0; f < fvol; ++f) {
    int64_t rem = f;
    int64_t yo = n * g.y.s[0];
    int64_t wo = fc * g.w.s[1];
    bool hit = true;
    for (int i = sp - 1; i >= 0; --i) {
      const int64_t fd = g.w_dim[2 + i];
      const int64_t fi = rem % fd;
      rem /= fd;
      const int64_t t = coord[2 + i] + g.pad[i] - fi * g.dil[i];
      const int64_t o = t / g.str[i];
      if (t < 0 || o * g.str[i] != t || o >= g.y_dim[2 + i])
        hit = false;
      yo += o * g.y.s[2 + i];
      wo += fi * g.w.s[2 + i];
    }
    if (!hit)
      continue;
    for (int64_t kk = 0; kk < kPerGroup; ++kk) {
      const int64_t k = grp * kPerGroup + kk;
      acc += fhip_load<float>(dy, g.y_dt, yo + k * g.y.s[1]) *
             fhip_load<float>(w, g.w_dt, wo + k * g.w.s[0]);
    }
  }
  fhip_store<float>(dx, g.x_dt, dot(coord, g.x, g.out.rank), acc);
}

// DW[k, fc, f..] = sum over n, o..:  DY[n, k, o..] * X[n, c, o * stride - pad +
// f * dil] with c = group(k) * fC + fc.  A workgroup owns one (k, filter tap)
// and 64 filter channels: lane = channel (channels-last X is read in
// contiguous runs, the DY value is the same for the whole wavefront), the four
// wavefronts split the pixels and their sums meet in LDS.  The pixel
// decomposition is wavefront-uniform.  Filters are small and batches large:
// with gridDim.z > 1 the pixels are cut into that many runs, one workgroup
// each, whose sums go to `partial` [run][k][tap][fc] for
// generic_conv_wgrad_sum_kernel.
__global__ __launch_bounds__(256) void generic_conv_wgrad_kernel(
    ConvBwdArgs g, const void *dy, const void *x, void *dw, float *partial,
    int64_t per_run) {
  __shared__ float part[4][64];
  const int sp = g.spatial;
  int64_t fvol = 1;
  for (int i = 0; i < sp; ++i)
    fvol *= g.w_dim[2 + i];
  const int64_t k = blockIdx.x / fvol;
  int64_t tap = blockIdx.x - k * fvol;
  int64_t f[3] = {0, 0, 0};
  for (int i = sp - 1; i >= 0; --i) {
    f[i] = tap % g.w_dim[2 + i];
    tap /= g.w_dim[2 + i];
  }
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t fC = g.w_dim[1];
  const int64_t fc = (int64_t)blockIdx.y * 64 + lane;
  const int64_t kPerGroup = g.w_dim[0] / g.groups;
  const int64_t c = (k / kPerGroup) * fC + (fc < fC ? fc : 0);
  int64_t ovol = 1;
  for (int i = 0; i < sp; ++i)
    ovol *= g.y_dim[2 + i];
  const int64_t all = g.y_dim[0] * ovol;
  const int64_t first = (int64_t)blockIdx.z * per_run;
  const int64_t total = first + per_run < all ? first + per_run : all;
  const int64_t y_k = k * g.y.s[1], x_c = c * g.x.s[1];
  // This wavefront's pixels are wave, wave + 4, ...: coordinates advance by
  // carries (no division in the loop), and eight pixels' loads are in flight
  // together.
  int64_t o[3] = {0, 0, 0}, n = 0;
  {
    int64_t rem = first + wave;
    for (int i = sp - 1; i >= 0; --i) {
      o[i] = rem % g.y_dim[2 + i];
      rem /= g.y_dim[2 + i];
    }
    n = rem;
  }
  constexpr int U = 8;
  float acc = 0.f;
  for (int64_t it = first + wave; it < total; it += 4 * U) {
    int64_t yo[U], xo[U];
    bool ok[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      bool inside = it + 4 * u < total;
      int64_t yy = y_k + n * g.y.s[0], xx = x_c + n * g.x.s[0];
      for (int i = 0; i < sp; ++i) {
        const int64_t xi = o[i] * g.str[i] - g.pad[i] + f[i] * g.dil[i];
        if (xi < 0 || xi >= g.x_dim[2 + i])
          inside = false;
        yy += o[i] * g.y.s[2 + i];
        xx += xi * g.x.s[2 + i];
      }
      ok[u] = inside;
      yo[u] = inside ? yy : y_k; // a valid address either way
      xo[u] = inside ? xx : x_c;
      // next pixel of this wavefront
      o[sp - 1] += 4;
      for (int i = sp - 1; i > 0; --i)
        while (o[i] >= g.y_dim[2 + i]) {
          o[i] -= g.y_dim[2 + i];
          ++o[i - 1];
        }
      while (o[0] >= g.y_dim[2]) {
        o[0] -= g.y_dim[2];
        ++n;
      }
    }
    float gy[U], xv[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      gy[u] = fhip_load<float>(dy, g.y_dt, yo[u]);
      xv[u] = fhip_load<float>(x, g.x_dt, xo[u]);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
      acc += ok[u] ? gy[u] * xv[u] : 0.f;
  }
  part[wave][lane] = acc;
  __syncthreads();
  if (wave == 0 && fc < fC) {
    const float sum = (part[0][lane] + part[1][lane]) + (part[2][lane] + part[3][lane]);
    if (gridDim.z > 1) {
      partial[((int64_t)blockIdx.z * gridDim.x + blockIdx.x) * fC + fc] = sum;
      return;
    }
    int64_t off = k * g.w.s[0] + fc * g.w.s[1];
    for (int i = 0; i < sp; ++i)
      off += f[i] * g.w.s[2 + i];
    fhip_store<float>(dw, g.w_dt, off, sum);
  }
}

// The same sum for filters with few channels per group (lane = channel would
// leave most of a wavefront idle): one workgroup per filter element
// (k, fc, tap), its 256 threads stride over the output pixels -- consecutive
// threads read consecutive pixels of DY and X -- and their sums meet in LDS.
__global__ __launch_bounds__(256) void generic_conv_wgrad_pixel_kernel(
    ConvBwdArgs g, const void *dy, const void *x, void *dw) {
  __shared__ float part[4];
  const int sp = g.spatial;
  // blockIdx.x = ((k * fC + fc) * f0 + ..) in DW's logical order
  int64_t rem = blockIdx.x;
  int64_t f[3] = {0, 0, 0};
  int64_t w_off = 0;
  for (int i = sp - 1; i >= 0; --i) {
    f[i] = rem % g.w_dim[2 + i];
    rem /= g.w_dim[2 + i];
    w_off += f[i] * g.w.s[2 + i];
  }
  const int64_t fC = g.w_dim[1];
  const int64_t fc = rem % fC, k = rem / fC;
  w_off += k * g.w.s[0] + fc * g.w.s[1];
  const int64_t kPerGroup = g.w_dim[0] / g.groups;
  const int64_t c = (k / kPerGroup) * fC + fc;
  uint32_t od[3] = {1, 1, 1};
  uint32_t ovol = 1;
  for (int i = 0; i < sp; ++i) {
    od[i] = (uint32_t)g.y_dim[2 + i];
    ovol *= od[i];
  }
  const uint32_t total = (uint32_t)g.y_dim[0] * ovol; // the host checked the range
  const int64_t y_k = k * g.y.s[1], x_c = c * g.x.s[1];
  float acc = 0.f;
  for (uint32_t pix = threadIdx.x; pix < total; pix += 256) {
    uint32_t r = pix;
    int64_t yy = y_k, xx = x_c;
    bool inside = true;
    for (int i = sp - 1; i >= 0; --i) {
      const uint32_t o = r % od[i];
      r /= od[i];
      const int64_t xi = (int64_t)o * g.str[i] - g.pad[i] + f[i] * g.dil[i];
      inside = inside && xi >= 0 && xi < g.x_dim[2 + i];
      yy += (int64_t)o * g.y.s[2 + i];
      xx += xi * g.x.s[2 + i];
    }
    yy += (int64_t)r * g.y.s[0];
    xx += (int64_t)r * g.x.s[0];
    if (inside)
      acc += fhip_load<float>(dy, g.y_dt, yy) * fhip_load<float>(x, g.x_dt, xx);
  }
  acc = wave_sum(acc);
  if ((threadIdx.x & 63) == 0)
    part[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0)
    fhip_store<float>(dw, g.w_dt, w_off, (part[0] + part[1]) + (part[2] + part[3]));
}

// DW = sum of the runs' partial sums, in run order; one thread per element.
__global__ __launch_bounds__(256) void generic_conv_wgrad_sum_kernel(
    ConvBwdArgs g, const float *partial, void *dw, int64_t elems, int runs) {
  const int64_t lin = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (lin >= elems)
    return;
  float sum = 0.f;
#pragma unroll 8
  for (int r = 0; r < runs; ++r)
    sum += partial[(int64_t)r * elems + lin];
  const int sp = g.spatial;
  const int64_t fC = g.w_dim[1];
  const int64_t fc = lin % fC;
  int64_t tap = lin / fC;
  int64_t off = fc * g.w.s[1];
  for (int i = sp - 1; i >= 0; --i) {
    off += (tap % g.w_dim[2 + i]) * g.w.s[2 + i];
    tap /= g.w_dim[2 + i];
  }
  off += tap * g.w.s[0]; // what is left is k
  fhip_store<float>(dw, g.w_dt, off, sum);
}

constexpr int kSdpaMaxDvPerLane = 8; // Dv <= 512

__global__ __launch_bounds__(64) void generic_sdpa_kernel(SdpaArgs g,
                                                          const void *q,
                                                          const void *k,
                                                          const void *v,
                                                          const void *mask,
                                                          void *o) {
  __shared__ float p_lds[64];
  const int lane = threadIdx.x;
  int64_t row = blockIdx.x;
  const int64_t sq = row % g.Sq;
  row /= g.Sq;
  const int64_t h = row % g.Hq;
  const int64_t b = row / g.Hq;
  const int64_t hk = h / (g.Hq / g.Hkv);
  const int64_t qo = b * g.q[0] + h * g.q[1] + sq * g.q[2];
  const int64_t ko = b * g.k[0] + hk * g.k[1];
  const int64_t vo = b * g.v[0] + hk * g.v[1];
  const int64_t mo = b * g.m[0] + h * g.m[1] + sq * g.m[2];
  float acc[kSdpaMaxDvPerLane];
  for (int i = 0; i < kSdpaMaxDvPerLane; ++i)
    acc[i] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  int64_t kv_end = g.Skv;
  if (g.causal && sq + 1 < kv_end)
    kv_end = sq + 1;
  for (int64_t j0 = 0; j0 < kv_end; j0 += 64) {
    const int64_t j = j0 + lane;
    float s = -INFINITY;
    if (j < kv_end) {
      float d = 0.f;
      for (int64_t e = 0; e < g.D; ++e)
        d += fhip_load<float>(q, g.q_dt, qo + e * g.q[3]) *
             fhip_load<float>(k, g.k_dt, ko + j * g.k[2] + e * g.k[3]);
      s = d * g.scale;
      if (g.has_mask) {
        if (g.m_dt == FHIP_BOOLEAN) {
          if (((const uint8_t *)mask)[mo + j * g.m[3]] == 0)
            s = -INFINITY;
        } else {
          s += fhip_load<float>(mask, g.m_dt, mo + j * g.m[3]);
        }
      }
    }
    const float m_new = fmaxf(m_run, wave_max(s));
    const float p = (m_new == -INFINITY) ? 0.f : __expf(s - m_new);
    const float corr = (m_new == -INFINITY) ? 1.f : __expf(m_run - m_new);
    l_run = l_run * corr + wave_sum(p);
    m_run = m_new;
    __syncthreads();
    p_lds[lane] = p;
    __syncthreads();
    const int64_t cnt = (kv_end - j0 < 64) ? (kv_end - j0) : 64;
    for (int i = 0; i < kSdpaMaxDvPerLane; ++i) {
      const int64_t dv = lane + 64 * i;
      if (dv < g.Dv) {
        float a = acc[i] * corr;
        for (int64_t jj = 0; jj < cnt; ++jj)
          a += p_lds[jj] *
               fhip_load<float>(v, g.v_dt, vo + (j0 + jj) * g.v[2] + dv * g.v[3]);
        acc[i] = a;
      }
    }
  }
  const int64_t oo = b * g.o[0] + h * g.o[1] + sq * g.o[2];
  for (int i = 0; i < kSdpaMaxDvPerLane; ++i) {
    const int64_t dv = lane + 64 * i;
    if (dv < g.Dv)
      fhip_store<float>(o, g.o_dt, oo + dv * g.o[3], acc[i] / l_run);
  }
}

// --------------------------------------------------------------------------
// RMSNorm / LayerNorm forward over all dims but dim 0
// --------------------------------------------------------------------------
struct NormArgs {
  Dims x;           // logical dims of X
  Strides xs, ss, bs, os;
  int64_t inner;    // product of dims 1..
  int32_t x_dt, s_dt, b_dt, y_dt, o_dt, stats_dt;
  int32_t has_scale, has_bias, is_layernorm, emit_stats;
  float eps;
  DevEpilogue epi;
};

__device__ __forceinline__ float block_sum_256(float v, float *lds) {
  v = wave_sum(v);
  const int wave = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0)
    lds[wave] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < (int)(blockDim.x >> 6); ++i)
    t += lds[i];
  return t;
}

__global__ __launch_bounds__(256) void generic_norm_kernel(
    NormArgs g, const void *x, const void *scale, const void *bias, void *out,
    void *mean_out, void *rstd_out) {
  __shared__ float lds[4];
  const int64_t b = blockIdx.x;
  Dims inner{};
  inner.rank = g.x.rank;
  inner.dim[0] = 1;
  for (int r = 1; r < g.x.rank; ++r)
    inner.dim[r] = g.x.dim[r];
  int64_t coord[FHIP_MAX_RANK];
  float mean = 0.f;
  if (g.is_layernorm) {
    float s = 0.f;
    for (int64_t i = threadIdx.x; i < g.inner; i += blockDim.x) {
      unravel(i, inner, coord);
      coord[0] = b;
      s += fhip_load<float>(x, g.x_dt, dot(coord, g.xs, g.x.rank));
    }
    mean = block_sum_256(s, lds) / (float)g.inner;
  }
  float ss = 0.f;
  for (int64_t i = threadIdx.x; i < g.inner; i += blockDim.x) {
    unravel(i, inner, coord);
    coord[0] = b;
    const float d =
        fhip_load<float>(x, g.x_dt, dot(coord, g.xs, g.x.rank)) - mean;
    ss += d * d;
  }
  const float var = block_sum_256(ss, lds) / (float)g.inner;
  const float rstd = 1.0f / sqrtf(var + g.eps);
  if (g.emit_stats && threadIdx.x == 0) {
    fhip_store<float>(mean_out, g.stats_dt, b, mean);
    fhip_store<float>(rstd_out, g.stats_dt, b, rstd);
  }
  for (int64_t i = threadIdx.x; i < g.inner; i += blockDim.x) {
    unravel(i, inner, coord);
    coord[0] = b;
    float v =
        (fhip_load<float>(x, g.x_dt, dot(coord, g.xs, g.x.rank)) - mean) * rstd;
    if (g.has_scale)
      v *= fhip_load<float>(scale, g.s_dt, dot(coord, g.ss, g.x.rank));
    if (g.has_bias)
      v += fhip_load<float>(bias, g.b_dt, dot(coord, g.bs, g.x.rank));
    v = fhip_round_through<float>(g.y_dt, v);
    v = fhip_apply_epilogue<float>(g.epi, v, coord);
    fhip_store<float>(out, g.o_dt, dot(coord, g.os, g.x.rank), v);
  }
}

// --------------------------------------------------------------------------
// reduction (keep-dim)
// --------------------------------------------------------------------------
struct ReduceArgs {
  Dims y;        // output logical dims (1 where reduced)
  Dims red;      // reduced extents per dim (1 where kept)
  Strides xs, ys;
  int64_t red_count;
  int32_t x_dt, y_dt;
  int32_t map_kind, comb_kind, post_kind;
  double identity;
};

// The host splits a reduction mode into: a per-element map, a combine, an
// identity and a final step.
enum { RMAP_NONE = 0, RMAP_ABS, RMAP_SQUARE, RMAP_ZERO_TO_ONE };
enum { RCOMB_ADD = 0, RCOMB_MUL, RCOMB_MIN, RCOMB_MAX };
enum { RPOST_NONE = 0, RPOST_MEAN, RPOST_SQRT };

template <typename CT>
__device__ __forceinline__ CT red_map(int kind, CT v) {
  if (kind == RMAP_ABS)
    return v < (CT)0 ? -v : v;
  if (kind == RMAP_SQUARE)
    return v * v;
  if (kind == RMAP_ZERO_TO_ONE)
    return v == (CT)0 ? (CT)1 : v;
  return v;
}

template <typename CT>
__device__ __forceinline__ CT red_combine(int kind, CT a, CT b) {
  if (kind == RCOMB_MUL)
    return a * b;
  if (kind == RCOMB_MIN)
    return (a != a || b != b) ? (a != a ? a : b) : (a < b ? a : b);
  if (kind == RCOMB_MAX)
    return (a != a || b != b) ? (a != a ? a : b) : (a > b ? a : b);
  return a + b;
}

// One workgroup per output element and slice of the reduced index range
// (gridDim.y slices of `per_slice` indices; with several slices the
// workgroup's result goes to partial[slice][output] for
// generic_reduce_finish_kernel).  SMALL: the reduced index fits 32 bits, and
// the index arithmetic runs in them.
template <typename CT, bool SMALL>
__global__ __launch_bounds__(256) void generic_reduce_kernel(
    ReduceArgs g, const void *x, void *y, CT *partial, int64_t per_slice) {
  __shared__ CT lds[256];
  int64_t ocoord[FHIP_MAX_RANK], rcoord[FHIP_MAX_RANK];
  unravel((int64_t)blockIdx.x, g.y, ocoord);
  const int rank = g.y.rank;
  const int64_t base = dot(ocoord, g.xs, rank);
  CT acc = (CT)g.identity;
  const int64_t first = (int64_t)blockIdx.y * per_slice;
  const int64_t last =
      first + per_slice < g.red_count ? first + per_slice : g.red_count;
  for (int64_t i = first + threadIdx.x; i < last; i += blockDim.x) {
    int64_t off = base;
    if (SMALL) {
      uint32_t rem = (uint32_t)i;
      for (int r = rank - 1; r >= 0; --r) {
        const uint32_t dim = (uint32_t)g.red.dim[r];
        const uint32_t q = rem / dim;
        off += (int64_t)(rem - q * dim) * g.xs.s[r];
        rem = q;
      }
    } else {
      unravel(i, g.red, rcoord);
      off += dot(rcoord, g.xs, rank);
    }
    const CT v = fhip_load<CT>(x, g.x_dt, off);
    acc = red_combine<CT>(g.comb_kind, acc, red_map<CT>(g.map_kind, v));
  }
  lds[threadIdx.x] = acc;
  __syncthreads();
  for (int s = 128; s > 0; s >>= 1) {
    if ((int)threadIdx.x < s)
      lds[threadIdx.x] =
          red_combine<CT>(g.comb_kind, lds[threadIdx.x], lds[threadIdx.x + s]);
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    CT r = lds[0];
    if (gridDim.y > 1) {
      partial[(int64_t)blockIdx.y * gridDim.x + blockIdx.x] = r;
      return;
    }
    if (g.post_kind == RPOST_MEAN)
      r = r / (CT)g.red_count;
    else if (g.post_kind == RPOST_SQRT)
      r = sqrt(r);
    fhip_store<CT>(y, g.y_dt, dot(ocoord, g.ys, rank), r);
  }
}

// Combines the slices' results of one output element in slice order.
template <typename CT>
__global__ __launch_bounds__(256) void generic_reduce_finish_kernel(
    ReduceArgs g, const CT *partial, void *y, int64_t outs, int slices) {
  const int64_t o = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (o >= outs)
    return;
  CT r = partial[o];
  for (int s = 1; s < slices; ++s)
    r = red_combine<CT>(g.comb_kind, r, partial[(int64_t)s * outs + o]);
  if (g.post_kind == RPOST_MEAN)
    r = r / (CT)g.red_count;
  else if (g.post_kind == RPOST_SQRT)
    r = sqrt(r);
  int64_t ocoord[FHIP_MAX_RANK];
  unravel(o, g.y, ocoord);
  fhip_store<CT>(y, g.y_dt, dot(ocoord, g.ys, g.y.rank), r);
}

// --------------------------------------------------------------------------
// batch normalisation forward (reference node/batchnorm_node.h:33-245;
// aten.native_batch_norm, support/asm_emitter.h:1066-1290): per channel c
//   inference: y = (x - mean[c]) / sqrt(var[c] + eps) * scale[c] + bias[c]
//   training:  mean and biased variance of x over batch and space, y from
//              them, and the two saved statistics (mean, 1 / sqrt(var + eps))
// --------------------------------------------------------------------------
struct BatchNormArgs {
  Dims x;        // [N, C, spatial...]
  Strides xs, ys;
  int32_t x_dt, y_dt, scale_dt, bias_dt, mean_dt, stats_dt;
  float eps;
};

__global__ void generic_batchnorm_infer_kernel(BatchNormArgs g, const void *x,
                                               const void *scale,
                                               const void *bias,
                                               const void *mean, const void *var,
                                               void *y, int64_t total) {
  const int64_t lin = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (lin >= total)
    return;
  int64_t coord[FHIP_MAX_RANK];
  unravel(lin, g.x, coord);
  const int64_t c = coord[1];
  const float m = fhip_load<float>(mean, g.mean_dt, c);
  const float v = fhip_load<float>(var, g.mean_dt, c);
  const float sc = scale ? fhip_load<float>(scale, g.scale_dt, c) : 1.f;
  const float b = bias ? fhip_load<float>(bias, g.bias_dt, c) : 0.f;
  const float xv = fhip_load<float>(x, g.x_dt, dot(coord, g.xs, g.x.rank));
  const float r = (xv - m) * (1.0f / sqrtf(v + g.eps)) * sc + b;
  fhip_store<float>(y, g.y_dt, dot(coord, g.ys, g.x.rank), r);
}

// One workgroup per channel, three walks over the channel's N x spatial
// elements: mean, centred second moment, output.
__global__ __launch_bounds__(256) void generic_batchnorm_train_kernel(
    BatchNormArgs g, const void *x, const void *scale, const void *bias,
    void *y, void *saved_mean, void *saved_inv_var) {
  __shared__ float part[4];
  const int64_t c = blockIdx.x;
  const int rank = g.x.rank;
  int64_t inner = 1; // spatial volume
  for (int i = 2; i < rank; ++i)
    inner *= g.x.dim[i];
  const int64_t count = g.x.dim[0] * inner;
  auto offset = [&](int64_t it, const Strides &st) {
    int64_t rem = it, off = c * st.s[1];
    for (int i = rank - 1; i >= 2; --i) {
      off += (rem % g.x.dim[i]) * st.s[i];
      rem /= g.x.dim[i];
    }
    return off + rem * st.s[0];
  };
  float acc = 0.f;
  for (int64_t it = threadIdx.x; it < count; it += blockDim.x)
    acc += fhip_load<float>(x, g.x_dt, offset(it, g.xs));
  const float mean = block_sum_256(acc, part) / (float)count;
  acc = 0.f;
  for (int64_t it = threadIdx.x; it < count; it += blockDim.x) {
    const float dv = fhip_load<float>(x, g.x_dt, offset(it, g.xs)) - mean;
    acc += dv * dv;
  }
  const float var = block_sum_256(acc, part) / (float)count;
  const float inv = 1.0f / sqrtf(var + g.eps);
  const float sc = scale ? fhip_load<float>(scale, g.scale_dt, c) : 1.f;
  const float b = bias ? fhip_load<float>(bias, g.bias_dt, c) : 0.f;
  for (int64_t it = threadIdx.x; it < count; it += blockDim.x) {
    const float xv = fhip_load<float>(x, g.x_dt, offset(it, g.xs));
    fhip_store<float>(y, g.y_dt, offset(it, g.ys), (xv - mean) * inv * sc + b);
  }
  if (threadIdx.x == 0) {
    fhip_store<float>(saved_mean, g.stats_dt, c, mean);
    fhip_store<float>(saved_inv_var, g.stats_dt, c, inv);
  }
}

// --------------------------------------------------------------------------
// pointwise
// --------------------------------------------------------------------------
struct PointwiseArgs {
  Dims out;
  Strides in[3], os;
  int32_t in_dt[3], o_dt;
  int32_t is_scalar[3];
  double scalar[3];
  int32_t mode, num_inputs;
  fhip_pointwise_params params;
};

template <typename CT>
__global__ void generic_pointwise_kernel(PointwiseArgs g, const void *in0,
                                         const void *in1, const void *in2,
                                         void *out, int64_t total) {
  const int64_t lin = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (lin >= total)
    return;
  int64_t coord[FHIP_MAX_RANK];
  unravel(lin, g.out, coord);
  const int rank = g.out.rank;
  const void *ptr[3] = {in0, in1, in2};
  CT v[3] = {(CT)0, (CT)0, (CT)0};
  for (int i = 0; i < g.num_inputs; ++i)
    v[i] = g.is_scalar[i]
               ? (CT)g.scalar[i]
               : fhip_load<CT>(ptr[i], g.in_dt[i], dot(coord, g.in[i], rank));
  CT r;
  if (g.num_inputs == 1)
    r = fhip_pw_unary<CT>(g.mode, v[0], g.params);
  else if (g.num_inputs == 2)
    r = fhip_pw_binary<CT>(g.mode, v[0], v[1], g.params);
  else
    r = (v[0] != (CT)0) ? v[1] : v[2]; // BINARY_SELECT = where(in0, in1, in2)
  fhip_store<CT>(out, g.o_dt, dot(coord, g.os, rank), r);
}

bool needs_double(int dt) {
  return dt == FHIP_DOUBLE || dt == FHIP_INT32 || dt == FHIP_INT64;
}

// Whether dims of `t` equal the given list.
bool dims_equal(const fhip_tensor_desc &t, int rank, const int64_t *dims) {
  if (t.rank != rank)
    return false;
  for (int i = 0; i < rank; ++i)
    if (t.dim[i] != dims[i])
      return false;
  return true;
}

} // namespace

extern "C" {

// ---- matmul ---------------------------------------------------------------
static int matmul_validate(fhip_ctx *ctx, const fhip_matmul_desc *d) {
  FHIP_REQUIRE(ctx, d != nullptr, "fhip_matmul: null descriptor");
  if (!fhip_check_desc(ctx, d->a, "matmul A") ||
      !fhip_check_desc(ctx, d->b, "matmul B") ||
      !fhip_check_desc(ctx, d->c, "matmul C") ||
      !fhip_check_desc(ctx, d->out, "matmul OUT"))
    return 1;
  const int r = d->a.rank;
  FHIP_REQUIRE(ctx, r >= 2 && d->b.rank == r && d->c.rank == r &&
                        d->out.rank == r,
               "fhip_matmul: A, B, C and OUT must share a rank >= 2");
  FHIP_REQUIRE(ctx, d->a.dim[r - 1] == d->b.dim[r - 2],
               "fhip_matmul: K mismatch (%lld vs %lld)",
               (long long)d->a.dim[r - 1], (long long)d->b.dim[r - 2]);
  FHIP_REQUIRE(ctx,
               d->c.dim[r - 2] == d->a.dim[r - 2] &&
                   d->c.dim[r - 1] == d->b.dim[r - 1],
               "fhip_matmul: C dims do not match M x N");
  for (int i = 0; i < r - 2; ++i) {
    const int64_t ad = d->a.dim[i], bd = d->b.dim[i], cd = d->c.dim[i];
    const int64_t mx = ad > bd ? ad : bd;
    FHIP_REQUIRE(ctx, (ad == bd || ad == 1 || bd == 1) && cd == mx,
                 "fhip_matmul: batch dim %d (%lld x %lld -> %lld) is not a "
                 "1-to-N broadcast",
                 i, (long long)ad, (long long)bd, (long long)cd);
  }
  FHIP_REQUIRE(ctx, dims_equal(d->out, r, d->c.dim),
               "fhip_matmul: OUT dims differ from C dims");
  FHIP_REQUIRE(ctx, d->out.dtype == d->out_dtype,
               "fhip_matmul: out_dtype disagrees with OUT descriptor");
  return 0;
}

int fhip_matmul_workspace_size(const fhip_matmul_desc *d, size_t *bytes) {
  FHIP_REQUIRE(nullptr, d && bytes, "fhip_matmul_workspace_size: null");
  *bytes = 0;
  return 0;
}

int fhip_matmul_supported(const fhip_matmul_desc *d) {
  if (!d || matmul_validate(nullptr, d) != 0)
    return 0;
  return fhip_fast_matmul_applicable(d) ? 2 : 1;
}

int fhip_matmul(fhip_ctx *ctx, const fhip_matmul_desc *d, const void *a,
                const void *b, const void *const *epilogue_operands, void *out,
                void *workspace, size_t workspace_bytes) {
  FHIP_REQUIRE(ctx, ctx != nullptr, "fhip_matmul: null context");
  if (matmul_validate(ctx, d) != 0)
    return 1;
  FHIP_REQUIRE(ctx, a && b && out, "fhip_matmul: null tensor pointer");
  (void)workspace;
  (void)workspace_bytes;
  FHIP_HIP_CHECK(ctx, hipSetDevice(ctx->device));
  const int r = d->a.rank;
  DevEpilogue epi;
  if (fhip_build_epilogue(ctx, d->epilogue, r, d->c.dim, epilogue_operands,
                          &epi) != 0)
    return 1;
  if (fhip_fast_matmul_applicable(d))
    return fhip_fast_matmul(ctx, d, a, b, epi, out);
  fhip_note_kernel(ctx, "matmul_generic");

  MatmulArgs g{};
  g.out = make_dims(d->c);
  for (int i = 0; i < r; ++i) {
    g.a.s[i] = (i < r - 2) ? (d->a.dim[i] == 1 ? 0 : d->a.stride[i]) : 0;
    g.b.s[i] = (i < r - 2) ? (d->b.dim[i] == 1 ? 0 : d->b.stride[i]) : 0;
    g.o.s[i] = d->out.dim[i] == 1 ? 0 : d->out.stride[i];
  }
  g.a.s[r - 2] = d->a.stride[r - 2]; // m
  g.b.s[r - 1] = d->b.stride[r - 1]; // n
  g.a_k = d->a.stride[r - 1];
  g.b_k = d->b.stride[r - 2];
  g.K = d->a.dim[r - 1];
  g.a_dt = d->a.dtype;
  g.b_dt = d->b.dtype;
  g.c_dt = d->c.dtype;
  g.o_dt = d->out.dtype;
  g.epi = epi;
  const int64_t total = fhip_desc_volume(d->c);
  auto widens = [](int dt) {
    return dt == FHIP_FLOAT || dt == FHIP_BFLOAT16 || dt == FHIP_HALF;
  };
  if (widens(d->a.dtype) && widens(d->b.dtype)) {
    const int64_t M = d->c.dim[r - 2], N = d->c.dim[r - 1];
    const int64_t tm = (M + kF32Tile - 1) / kF32Tile, tn = (N + kF32Tile - 1) / kF32Tile;
    const int64_t batch = total / (M * N);
    const int64_t sm = (M + 31) / 32, sn = (N + 31) / 32;
    // the operands' common element type, compiled into the kernel (-1: mixed)
    const int same_dt = d->a.dtype == d->b.dtype ? (int)d->a.dtype : -1;
    if (tm * tn * batch < 128 && g.K >= 8 * kF32K && batch <= 65535 &&
        sm * sn < (1ll << 31)) {
      // few tiles: 32 x 32 tiles with K split over the wavefronts
      const dim3 grid((unsigned)(sm * sn), (unsigned)batch);
      auto go = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, grid, dim3(256), 0, ctx->stream, g, a, b, out, (int)sn);
      };
      if (same_dt == FHIP_FLOAT)
        go(splitk_matmul_f32_kernel<FHIP_FLOAT>);
      else if (same_dt == FHIP_BFLOAT16)
        go(splitk_matmul_f32_kernel<FHIP_BFLOAT16>);
      else if (same_dt == FHIP_HALF)
        go(splitk_matmul_f32_kernel<FHIP_HALF>);
      else
        go(splitk_matmul_f32_kernel<-1>);
      FHIP_HIP_CHECK(ctx, hipGetLastError());
      fhip_note_kernel(ctx, "matmul_f32_splitk");
      return 0;
    }
    if (tm * tn < (1ll << 31) && batch <= 65535 && tn < (1ll << 31)) {
      const dim3 grid((unsigned)(tm * tn), (unsigned)batch);
      auto go = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, grid, dim3(256), 0, ctx->stream, g, a, b, out, (int)tn);
      };
      if (same_dt == FHIP_FLOAT)
        go(tiled_matmul_f32_kernel<FHIP_FLOAT>);
      else if (same_dt == FHIP_BFLOAT16)
        go(tiled_matmul_f32_kernel<FHIP_BFLOAT16>);
      else if (same_dt == FHIP_HALF)
        go(tiled_matmul_f32_kernel<FHIP_HALF>);
      else
        go(tiled_matmul_f32_kernel<-1>);
      FHIP_HIP_CHECK(ctx, hipGetLastError());
      fhip_note_kernel(ctx, "matmul_f32_tiled");
      return 0;
    }
  }
  const bool int_path = fhip_dtype_is_int(d->a.dtype) &&
                        fhip_dtype_is_int(d->b.dtype);
  if (int_path)
    hipLaunchKernelGGL(generic_matmul_kernel<int32_t>, dim3(grid_for(total, 256)),
                       dim3(256), 0, ctx->stream, g, a, b, out, total);
  else
    hipLaunchKernelGGL(generic_matmul_kernel<float>, dim3(grid_for(total, 256)),
                       dim3(256), 0, ctx->stream, g, a, b, out, total);
  FHIP_HIP_CHECK(ctx, hipGetLastError());
  return 0;
}

// ---- conv fprop -----------------------------------------------------------
static int conv_validate(fhip_ctx *ctx, const fhip_conv_desc *d) {
  FHIP_REQUIRE(ctx, d != nullptr, "fhip_conv_fprop: null descriptor");
  if (!fhip_check_desc(ctx, d->x, "conv X") ||
      !fhip_check_desc(ctx, d->w, "conv W") ||
      !fhip_check_desc(ctx, d->y, "conv Y") ||
      !fhip_check_desc(ctx, d->out, "conv OUT"))
    return 1;
  const int sp = d->spatial_rank;
  FHIP_REQUIRE(ctx, sp >= 1 && sp <= 3, "fhip_conv_fprop: spatial rank %d", sp);
  FHIP_REQUIRE(ctx,
               d->x.rank == sp + 2 && d->w.rank == sp + 2 &&
                   d->y.rank == sp + 2 && d->out.rank == sp + 2,
               "fhip_conv_fprop: tensor ranks must equal spatial rank + 2");
  const int64_t C = d->x.dim[1], fC = d->w.dim[1], K = d->w.dim[0];
  FHIP_REQUIRE(ctx, fC > 0 && C % fC == 0,
               "fhip_conv_fprop: input channels %lld not divisible by filter "
               "channels %lld",
               (long long)C, (long long)fC);
  const int64_t groups = C / fC;
  FHIP_REQUIRE(ctx, K % groups == 0,
               "fhip_conv_fprop: output channels %lld not divisible by groups "
               "%lld",
               (long long)K, (long long)groups);
  FHIP_REQUIRE(ctx, d->y.dim[0] == d->x.dim[0] && d->y.dim[1] == K,
               "fhip_conv_fprop: Y batch/channel dims mismatch");
  for (int i = 0; i < sp; ++i) {
    FHIP_REQUIRE(ctx, d->stride[i] >= 1 && d->dilation[i] >= 1 &&
                          d->padding[i] >= 0,
                 "fhip_conv_fprop: invalid stride/dilation/padding");
    const int64_t expect =
        1 + (d->x.dim[2 + i] + 2 * d->padding[i] -
             d->dilation[i] * (d->w.dim[2 + i] - 1) - 1) /
                d->stride[i];
    FHIP_REQUIRE(ctx, d->y.dim[2 + i] == expect,
                 "fhip_conv_fprop: Y spatial dim %d is %lld, expected %lld", i,
                 (long long)d->y.dim[2 + i], (long long)expect);
  }
  FHIP_REQUIRE(ctx, dims_equal(d->out, d->y.rank, d->y.dim),
               "fhip_conv_fprop: OUT dims differ from Y dims");
  FHIP_REQUIRE(ctx, d->out.dtype == d->out_dtype,
               "fhip_conv_fprop: out_dtype disagrees with OUT descriptor");
  return 0;
}

int fhip_conv_fprop_workspace_size(const fhip_conv_desc *d, size_t *bytes) {
  FHIP_REQUIRE(nullptr, d && bytes, "fhip_conv_fprop_workspace_size: null");
  *bytes = 0;
  return 0;
}

int fhip_conv_fprop_supported(const fhip_conv_desc *d) {
  if (!d || conv_validate(nullptr, d) != 0)
    return 0;
  return fhip_fast_conv_applicable(d) || fhip_direct_conv_cl_applicable(d) ? 2 : 1;
}

int fhip_conv_fprop(fhip_ctx *ctx, const fhip_conv_desc *d, const void *x,
                    const void *w, const void *const *epilogue_operands,
                    void *out, void *workspace, size_t workspace_bytes) {
  FHIP_REQUIRE(ctx, ctx != nullptr, "fhip_conv_fprop: null context");
  if (conv_validate(ctx, d) != 0)
    return 1;
  FHIP_REQUIRE(ctx, x && w && out, "fhip_conv_fprop: null tensor pointer");
  (void)workspace;
  (void)workspace_bytes;
  FHIP_HIP_CHECK(ctx, hipSetDevice(ctx->device));
  DevEpilogue epi;
  if (fhip_build_epilogue(ctx, d->epilogue, d->y.rank, d->y.dim,
                          epilogue_operands, &epi) != 0)
    return 1;
  bool tuned = false;
  if (fhip_fast_conv(ctx, d, x, w, epi, out, &tuned) != 0)
    return 1;
  if (tuned)
    return 0;
  if (fhip_direct_conv_applicable(d))
    return fhip_direct_conv_fprop(ctx, d, x, w, epi, out);
  fhip_note_kernel(ctx, "conv_generic");

  ConvArgs g{};
  g.y = make_dims(d->y);
  g.x = make_strides(d->x);
  g.w = make_strides(d->w);
  g.o = make_strides(d->out);
  for (int i = 0; i < d->x.rank; ++i) {
    g.x_dim[i] = d->x.dim[i];
    g.w_dim[i] = d->w.dim[i];
  }
  g.spatial = d->spatial_rank;
  for (int i = 0; i < 3; ++i) {
    g.pad[i] = d->padding[i];
    g.str[i] = d->stride[i];
    g.dil[i] = d->dilation[i];
  }
  g.groups = d->x.dim[1] / d->w.dim[1];
  g.x_dt = d->x.dtype;
  g.w_dt = d->w.dtype;
  g.y_dt = d->y.dtype;
  g.o_dt = d->out.dtype;
  g.epi = epi;
  const int64_t total = fhip_desc_volume(d->y);
  hipLaunchKernelGGL(generic_conv_kernel, dim3(grid_for(total, 256)), dim3(256),
                     0, ctx->stream, g, x, w, out, total);
  FHIP_HIP_CHECK(ctx, hipGetLastError());
  return 0;
}

// ---- conv backward (data and weight gradients) -----------------------------
// The descriptor names the forward problem: x is X (wgrad input) or DX (dgrad
// output), w is W (dgrad input) or DW (wgrad output), y is DY.
static int conv_bwd_validate(fhip_ctx *ctx, const fhip_conv_desc *d,
                             const char *who) {
  FHIP_REQUIRE(ctx, d != nullptr, "%s: null descriptor", who);
  if (!fhip_check_desc(ctx, d->x, "conv X/DX") ||
      !fhip_check_desc(ctx, d->w, "conv W/DW") ||
      !fhip_check_desc(ctx, d->y, "conv DY"))
    return 1;
  const int sp = d->spatial_rank;
  FHIP_REQUIRE(ctx, sp >= 1 && sp <= 3, "%s: spatial rank %d", who, sp);
  FHIP_REQUIRE(ctx,
               d->x.rank == sp + 2 && d->w.rank == sp + 2 && d->y.rank == sp + 2,
               "%s: tensor ranks must equal spatial rank + 2", who);
  FHIP_REQUIRE(ctx, d->epilogue.count == 0,
               "%s: no pointwise chain can be fused into a gradient", who);
  const int64_t C = d->x.dim[1], fC = d->w.dim[1], K = d->w.dim[0];
  FHIP_REQUIRE(ctx, fC > 0 && C % fC == 0,
               "%s: input channels %lld not divisible by filter channels %lld",
               who, (long long)C, (long long)fC);
  const int64_t groups = C / fC;
  FHIP_REQUIRE(ctx, K % groups == 0,
               "%s: output channels %lld not divisible by groups %lld", who,
               (long long)K, (long long)groups);
  FHIP_REQUIRE(ctx, d->y.dim[0] == d->x.dim[0] && d->y.dim[1] == K,
               "%s: DY batch/channel dims mismatch", who);
  for (int i = 0; i < sp; ++i) {
    FHIP_REQUIRE(ctx, d->stride[i] >= 1 && d->dilation[i] >= 1 &&
                          d->padding[i] >= 0,
                 "%s: invalid stride/dilation/padding", who);
    const int64_t expect =
        1 + (d->x.dim[2 + i] + 2 * d->padding[i] -
             d->dilation[i] * (d->w.dim[2 + i] - 1) - 1) /
                d->stride[i];
    FHIP_REQUIRE(ctx, d->y.dim[2 + i] == expect,
                 "%s: DY spatial dim %d is %lld, expected %lld", who, i,
                 (long long)d->y.dim[2 + i], (long long)expect);
  }
  return 0;
}

static ConvBwdArgs conv_bwd_args(const fhip_conv_desc *d, bool dgrad) {
  ConvBwdArgs g{};
  g.out = make_dims(dgrad ? d->x : d->w);
  g.x = make_strides(d->x);
  g.w = make_strides(d->w);
  g.y = make_strides(d->y);
  for (int i = 0; i < d->x.rank; ++i) {
    g.x_dim[i] = d->x.dim[i];
    g.w_dim[i] = d->w.dim[i];
    g.y_dim[i] = d->y.dim[i];
  }
  g.spatial = d->spatial_rank;
  for (int i = 0; i < 3; ++i) {
    g.pad[i] = d->padding[i];
    g.str[i] = d->stride[i];
    g.dil[i] = d->dilation[i];
  }
  g.groups = d->x.dim[1] / d->w.dim[1];
  g.x_dt = d->x.dtype;
  g.w_dt = d->w.dtype;
  g.y_dt = d->y.dtype;
  return g;
}

int fhip_conv_dgrad_workspace_size(const fhip_conv_desc *d, size_t *bytes) {
  FHIP_REQUIRE(nullptr, d && bytes, "fhip_conv_dgrad_workspace_size: null");
  *bytes = 0;
  if (conv_bwd_validate(nullptr, d, "fhip_conv_dgrad") != 0)
    return 1;
  fhip_fast_conv_dgrad_applicable(d, bytes);
  return 0;
}

int fhip_conv_dgrad_supported(const fhip_conv_desc *d) {
  if (!d || conv_bwd_validate(nullptr, d, "fhip_conv_dgrad") != 0)
    return 0;
  return fhip_fast_conv_dgrad_applicable(d, nullptr) ? 2 : 1;
}

int fhip_conv_dgrad(fhip_ctx *ctx, const fhip_conv_desc *d, const void *dy,
                    const void *w, void *dx, void *workspace,
                    size_t workspace_bytes) {
  FHIP_REQUIRE(ctx, ctx != nullptr, "fhip_conv_dgrad: null context");
  if (conv_bwd_validate(ctx, d, "fhip_conv_dgrad") != 0)
    return 1;
  FHIP_REQUIRE(ctx, dy && w && dx, "fhip_conv_dgrad: null tensor pointer");
  FHIP_HIP_CHECK(ctx, hipSetDevice(ctx->device));
  size_t need = 0;
  if (fhip_fast_conv_dgrad_applicable(d, &need)) {
    FHIP_REQUIRE(ctx, workspace && workspace_bytes >= need,
                 "fhip_conv_dgrad: this descriptor needs %zu bytes of workspace "
                 "(fhip_conv_dgrad_workspace_size), got %zu",
                 need, workspace ? workspace_bytes : (size_t)0);
    return fhip_fast_conv_dgrad(ctx, d, dy, w, dx, workspace);
  }
  if (fhip_direct_conv_applicable(d))
    return fhip_direct_conv_dgrad(ctx, d, dy, w, dx);
  fhip_note_kernel(ctx, "conv_dgrad_generic");
  const ConvBwdArgs g = conv_bwd_args(d, true);
  const int64_t total = fhip_desc_volume(d->x);
  hipLaunchKernelGGL(generic_conv_dgrad_kernel, dim3(grid_for(total, 256)),
                     dim3(256), 0, ctx->stream, g, dy, w, dx, total);
  FHIP_HIP_CHECK(ctx, hipGetLastError());
  return 0;
}

int fhip_conv_dgrad_static(fhip_ctx *ctx, const fhip_conv_desc *d,
                           const void *dy, const void *w, void *dx) {
  FHIP_REQUIRE(ctx, ctx != nullptr, "fhip_conv_dgrad_static: null context");
  if (conv_bwd_validate(ctx, d, "fhip_conv_dgrad_static") != 0)
    return 1;
  FHIP_REQUIRE(ctx, dy && w && dx, "fhip_conv_dgrad_static: null tensor pointer");
  FHIP_HIP_CHECK(ctx, hipSetDevice(ctx->device));
  size_t need = 0;
  // (only plans that leave the context's growable scratch alone)
  if (fhip_fast_conv_dgrad_applicable(d, &need, false)) {
    FHIP_REQUIRE(ctx, need <= (size_t)FHIP_CONV_DGRAD_STATIC_MAX_BYTES,
                 "fhip_conv_dgrad_static: this descriptor needs %zu bytes of "
                 "scratch, the static array holds %zu; use fhip_conv_dgrad "
                 "with caller workspace",
                 need, (size_t)FHIP_CONV_DGRAD_STATIC_MAX_BYTES);
    FHIP_REQUIRE(ctx, ctx->dgrad_static_scratch != nullptr,
                 "fhip_conv_dgrad_static: scratch address not resolved");
    return fhip_fast_conv_dgrad(ctx, d, dy, w, dx, ctx->dgrad_static_scratch, false);
  }
  // the direct and the strided kernel use no scratch at all
  if (fhip_direct_conv_applicable(d))
    return fhip_direct_conv_dgrad(ctx, d, dy, w, dx);
  fhip_note_kernel(ctx, "conv_dgrad_generic");
  const ConvBwdArgs g = conv_bwd_args(d, true);
  const int64_t total = fhip_desc_volume(d->x);
  hipLaunchKernelGGL(generic_conv_dgrad_kernel, dim3(grid_for(total, 256)),
                     dim3(256), 0, ctx->stream, g, dy, w, dx, total);
  FHIP_HIP_CHECK(ctx, hipGetLastError());
  return 0;
}

int fhip_conv_wgrad_workspace_size(const fhip_conv_desc *d, size_t *bytes) {
  FHIP_REQUIRE(nullptr, d && bytes, "fhip_conv_wgrad_workspace_size: null");
  *bytes = 0;
  if (conv_bwd_validate(nullptr, d, "fhip_conv_wgrad") != 0)
    return 1;
  fhip_fast_conv_wgrad_applicable(d, bytes);
  return 0;
}

// grid of the weight-gradient kernel: x = K * filter taps, y = blocks of 64
// filter channels
static bool conv_wgrad_grid(const fhip_conv_desc *d, dim3 *grid) {
  int64_t fvol = 1;
  for (int i = 0; i < d->spatial_rank; ++i)
    fvol *= d->w.dim[2 + i];
  const int64_t gx = d->w.dim[0] * fvol, gy = (d->w.dim[1] + 63) / 64;
  if (gx >= (1ll << 31) || gy > 65535)
    return false;
  *grid = dim3((unsigned)gx, (unsigned)gy);
  return true;
}

// The weight gradient of a 1 x 1 convolution (unit stride, no padding, one
// group, dense channels-last 16-bit X and DY) is the matrix product DY^T X
// over the pixels: M = K, N = C, both operands with the reduction dim as the
// slow one.  The MFMA GEMM takes it as it lies and cuts the long reduction
// into parts (needs no caller workspace).
static bool conv_wgrad_as_matmul(const fhip_conv_desc *d, fhip_matmul_desc *m) {
  const int sp = d->spatial_rank;
  if (d->w.dim[1] != d->x.dim[1] || d->x.dtype != d->y.dtype ||
      (d->x.dtype != FHIP_BFLOAT16 && d->x.dtype != FHIP_HALF))
    return false;
  int64_t pixels = d->x.dim[0];
  for (int i = 0; i < sp; ++i) {
    if (d->w.dim[2 + i] != 1 || d->stride[i] != 1 || d->padding[i] != 0)
      return false;
    pixels *= d->x.dim[2 + i];
  }
  const int64_t C = d->x.dim[1], K = d->w.dim[0];
  auto dense_cl = [&](const fhip_tensor_desc &t, int64_t ch) {
    // [N, ch, spatial...] with the channel as the fastest dim and pixels dense
    if (ch != 1 && t.stride[1] != 1)
      return false;
    int64_t expect = ch;
    for (int i = t.rank - 1; i >= 2; --i) {
      if (t.dim[i] != 1 && t.stride[i] != expect)
        return false;
      expect *= t.dim[i];
    }
    return t.dim[0] == 1 || t.stride[0] == expect;
  };
  if (!dense_cl(d->x, C) || !dense_cl(d->y, K))
    return false;
  // DW [K, C, 1...]: rows of C contiguous elements
  if ((C != 1 && d->w.stride[1] != 1) || (K != 1 && d->w.stride[0] != C))
    return false;
  std::memset(m, 0, sizeof(*m));
  m->a.rank = m->b.rank = m->c.rank = m->out.rank = 2;
  m->a.dtype = m->b.dtype = d->x.dtype;
  m->a.dim[0] = K, m->a.dim[1] = pixels, m->a.stride[0] = 1, m->a.stride[1] = K;
  m->b.dim[0] = pixels, m->b.dim[1] = C, m->b.stride[0] = C, m->b.stride[1] = 1;
  m->c.dim[0] = K, m->c.dim[1] = C, m->c.stride[0] = C, m->c.stride[1] = 1;
  m->c.dtype = FHIP_FLOAT;
  m->out = m->c;
  m->out.dtype = d->w.dtype;
  m->out_dtype = d->w.dtype;
  return fhip_fast_matmul_applicable(m);
}

int fhip_conv_wgrad_supported(const fhip_conv_desc *d) {
  if (!d || conv_bwd_validate(nullptr, d, "fhip_conv_wgrad") != 0)
    return 0;
  fhip_matmul_desc md;
  if (conv_wgrad_as_matmul(d, &md))
    return 2;
  if (fhip_fast_conv_wgrad_applicable(d, nullptr))
    return 2;
  dim3 grid;
  return conv_wgrad_grid(d, &grid) ? 1 : 0;
}

int fhip_conv_wgrad(fhip_ctx *ctx, const fhip_conv_desc *d, const void *dy,
                    const void *x, void *dw, void *workspace,
                    size_t workspace_bytes) {
  FHIP_REQUIRE(ctx, ctx != nullptr, "fhip_conv_wgrad: null context");
  if (conv_bwd_validate(ctx, d, "fhip_conv_wgrad") != 0)
    return 1;
  FHIP_REQUIRE(ctx, dy && x && dw, "fhip_conv_wgrad: null tensor pointer");
  {
    fhip_matmul_desc md;
    if (conv_wgrad_as_matmul(d, &md) &&
        (((uintptr_t)dy | (uintptr_t)x | (uintptr_t)dw) & 15) == 0) {
      FHIP_HIP_CHECK(ctx, hipSetDevice(ctx->device));
      const int rc = fhip_fast_matmul(ctx, &md, dy, x, DevEpilogue{}, dw);
      char inner[sizeof(ctx->last_kernel)];
      std::snprintf(inner, sizeof(inner), "%s", ctx->last_kernel);
      fhip_note_kernel(ctx, "wgrad 1x1 as %s", inner);
      return rc;
    }
  }
  size_t need = 0;
  if (fhip_fast_conv_wgrad_applicable(d, &need)) {
    FHIP_REQUIRE(ctx, workspace && workspace_bytes >= need,
                 "fhip_conv_wgrad: this descriptor needs %zu bytes of workspace "
                 "(fhip_conv_wgrad_workspace_size), got %zu",
                 need, workspace ? workspace_bytes : (size_t)0);
    FHIP_HIP_CHECK(ctx, hipSetDevice(ctx->device));
    return fhip_fast_conv_wgrad(ctx, d, dy, x, dw, workspace);
  }
  dim3 grid;
  FHIP_REQUIRE(ctx, conv_wgrad_grid(d, &grid),
               "fhip_conv_wgrad: the filter exceeds the grid limits");
  (void)workspace;
  (void)workspace_bytes;
  FHIP_HIP_CHECK(ctx, hipSetDevice(ctx->device));
  if (fhip_direct_conv_applicable(d))
    return fhip_direct_conv_wgrad(ctx, d, dy, x, dw);
  fhip_note_kernel(ctx, "conv_wgrad_generic");
  const ConvBwdArgs g = conv_bwd_args(d, false);
  if (fhip_desc_volume(d->w) == 0)
    return 0;
  int64_t pixels = d->y.dim[0];
  for (int i = 0; i < d->spatial_rank; ++i)
    pixels *= d->y.dim[2 + i];
  // few channels per group: one workgroup per filter element, threads over pixels
  if (d->w.dim[1] < 32 && pixels < (1ll << 31) && fhip_desc_volume(d->w) < (1ll << 31)) {
    hipLaunchKernelGGL(generic_conv_wgrad_pixel_kernel,
                       dim3((unsigned)fhip_desc_volume(d->w)), dim3(256), 0,
                       ctx->stream, g, dy, x, dw);
    FHIP_HIP_CHECK(ctx, hipGetLastError());
    return 0;
  }
  // Few workgroups (one per filter tap and output channel) and many pixels:
  // cut the pixels into runs of at least 256 until the launch has about 16
  // workgroups per compute unit; the runs' sums meet in the context's scratch.
  const int64_t wgs = (int64_t)grid.x * grid.y;
  const int64_t cus = ctx->num_cus > 0 ? ctx->num_cus : 256;
  int64_t runs = (16 * cus + wgs - 1) / wgs;
  runs = runs < pixels / 256 ? runs : pixels / 256;
  runs = runs < 1024 ? runs : 1024;
  if (runs < 2 || grid.y != 1) {
    hipLaunchKernelGGL(generic_conv_wgrad_kernel, grid, dim3(256), 0, ctx->stream,
                       g, dy, x, dw, (float *)nullptr, pixels);
    FHIP_HIP_CHECK(ctx, hipGetLastError());
    return 0;
  }
  // whole groups of 32 pixels (4 wavefronts x 8 in flight) per run
  int64_t per_run = (pixels + runs - 1) / runs;
  per_run = (per_run + 31) / 32 * 32;
  runs = (pixels + per_run - 1) / per_run;
  const int64_t elems = (int64_t)grid.x * d->w.dim[1];
  void *scratch = nullptr;
  if (fhip_ctx_scratch(ctx, (size_t)(runs * elems) * sizeof(float), &scratch) != 0)
    return 1;
  grid.z = (unsigned)runs;
  hipLaunchKernelGGL(generic_conv_wgrad_kernel, grid, dim3(256), 0, ctx->stream,
                     g, dy, x, dw, (float *)scratch, per_run);
  hipLaunchKernelGGL(generic_conv_wgrad_sum_kernel,
                     dim3((unsigned)((elems + 255) / 256)), dim3(256), 0,
                     ctx->stream, g, (const float *)scratch, dw, elems, (int)runs);
  FHIP_HIP_CHECK(ctx, hipGetLastError());
  return 0;
}

// ---- sdpa -----------------------------------------------------------------
static int sdpa_validate(fhip_ctx *ctx, const fhip_sdpa_desc *d) {
  FHIP_REQUIRE(ctx, d != nullptr, "fhip_sdpa_fwd: null descriptor");
  if (!fhip_check_desc(ctx, d->q, "sdpa Q") ||
      !fhip_check_desc(ctx, d->k, "sdpa K") ||
      !fhip_check_desc(ctx, d->v, "sdpa V") ||
      !fhip_check_desc(ctx, d->o, "sdpa O"))
    return 1;
  FHIP_REQUIRE(ctx,
               d->q.rank == 4 && d->k.rank == 4 && d->v.rank == 4 &&
                   d->o.rank == 4,
               "fhip_sdpa_fwd: Q, K, V, O must be rank 4");
  const int64_t B = d->q.dim[0], Hq = d->q.dim[1], Sq = d->q.dim[2],
                D = d->q.dim[3];
  const int64_t Hkv = d->k.dim[1], Skv = d->k.dim[2];
  FHIP_REQUIRE(ctx, d->k.dim[0] == B && d->v.dim[0] == B,
               "fhip_sdpa_fwd: batch mismatch");
  FHIP_REQUIRE(ctx, d->k.dim[3] == D, "fhip_sdpa_fwd: Q/K head dim mismatch");
  FHIP_REQUIRE(ctx, d->v.dim[1] == Hkv && d->v.dim[2] == Skv,
               "fhip_sdpa_fwd: K/V head count or sequence mismatch");
  FHIP_REQUIRE(ctx, Hkv > 0 && Hq % Hkv == 0,
               "fhip_sdpa_fwd: Hq %lld not divisible by Hkv %lld",
               (long long)Hq, (long long)Hkv);
  const int64_t Dv = d->v.dim[3];
  FHIP_REQUIRE(ctx,
               d->o.dim[0] == B && d->o.dim[1] == Hq && d->o.dim[2] == Sq &&
                   d->o.dim[3] == Dv,
               "fhip_sdpa_fwd: O dims must be [B, Hq, Sq, Dv]");
  FHIP_REQUIRE(ctx, Dv <= 64 * kSdpaMaxDvPerLane,
               "fhip_sdpa_fwd: value head dim %lld above %d", (long long)Dv,
               64 * kSdpaMaxDvPerLane);
  if (d->mask.rank != 0) {
    if (!fhip_check_desc(ctx, d->mask, "sdpa MASK"))
      return 1;
    FHIP_REQUIRE(ctx, !d->is_causal,
                 "fhip_sdpa_fwd: mask and is_causal are mutually exclusive");
    int64_t dims[4] = {B, Hq, Sq, Skv};
    int64_t st[4];
    FHIP_REQUIRE(ctx, fhip_broadcast_strides(d->mask, 4, dims, st),
                 "fhip_sdpa_fwd: mask is not broadcastable to [B,Hq,Sq,Skv]");
  }
  return 0;
}

int fhip_sdpa_fwd_workspace_size(const fhip_sdpa_desc *d, size_t *bytes) {
  FHIP_REQUIRE(nullptr, d && bytes, "fhip_sdpa_fwd_workspace_size: null");
  *bytes = 0;
  return 0;
}

int fhip_sdpa_fwd_supported(const fhip_sdpa_desc *d) {
  if (!d || sdpa_validate(nullptr, d) != 0)
    return 0;
  return fhip_fast_sdpa_applicable(d) ? 2 : 1;
}

int fhip_sdpa_fwd(fhip_ctx *ctx, const fhip_sdpa_desc *d, const void *q,
                  const void *k, const void *v, const void *mask, void *o,
                  void *workspace, size_t workspace_bytes) {
  FHIP_REQUIRE(ctx, ctx != nullptr, "fhip_sdpa_fwd: null context");
  if (sdpa_validate(ctx, d) != 0)
    return 1;
  FHIP_REQUIRE(ctx, q && k && v && o, "fhip_sdpa_fwd: null tensor pointer");
  FHIP_REQUIRE(ctx, (d->mask.rank != 0) == (mask != nullptr),
               "fhip_sdpa_fwd: mask pointer and mask descriptor disagree");
  (void)workspace;
  (void)workspace_bytes;
  FHIP_HIP_CHECK(ctx, hipSetDevice(ctx->device));
  if (fhip_fast_sdpa_applicable(d))
    return fhip_fast_sdpa(ctx, d, q, k, v, mask, o);
  fhip_note_kernel(ctx, "sdpa_generic");

  SdpaArgs g{};
  g.B = d->q.dim[0];
  g.Hq = d->q.dim[1];
  g.Sq = d->q.dim[2];
  g.D = d->q.dim[3];
  g.Hkv = d->k.dim[1];
  g.Skv = d->k.dim[2];
  g.Dv = d->v.dim[3];
  for (int i = 0; i < 4; ++i) {
    g.q[i] = d->q.stride[i];
    g.k[i] = d->k.stride[i];
    g.v[i] = d->v.stride[i];
    g.o[i] = d->o.stride[i];
    g.m[i] = 0;
  }
  g.q_dt = d->q.dtype;
  g.k_dt = d->k.dtype;
  g.v_dt = d->v.dtype;
  g.o_dt = d->o.dtype;
  g.has_mask = d->mask.rank != 0;
  g.causal = d->is_causal;
  if (g.has_mask) {
    int64_t dims[4] = {g.B, g.Hq, g.Sq, g.Skv};
    fhip_broadcast_strides(d->mask, 4, dims, g.m);
    g.m_dt = d->mask.dtype;
  }
  g.scale = d->has_scale ? d->scale : 1.0f / sqrtf((float)g.D);
  const int64_t rows = g.B * g.Hq * g.Sq;
  hipLaunchKernelGGL(generic_sdpa_kernel, dim3((unsigned)rows), dim3(64), 0,
                     ctx->stream, g, q, k, v, mask, o);
  FHIP_HIP_CHECK(ctx, hipGetLastError());
  return 0;
}

// ---- norms ----------------------------------------------------------------
static int norm_validate(fhip_ctx *ctx, const fhip_norm_desc *d) {
  FHIP_REQUIRE(ctx, d != nullptr, "fhip_norm_fwd: null descriptor");
  if (!fhip_check_desc(ctx, d->x, "norm X") ||
      !fhip_check_desc(ctx, d->y, "norm Y") ||
      !fhip_check_desc(ctx, d->out, "norm OUT"))
    return 1;
  FHIP_REQUIRE(ctx, d->x.rank >= 2, "fhip_norm_fwd: X rank must be >= 2");
  FHIP_REQUIRE(ctx, dims_equal(d->y, d->x.rank, d->x.dim) &&
                        dims_equal(d->out, d->x.rank, d->x.dim),
               "fhip_norm_fwd: Y / OUT dims differ from X dims");
  int64_t sdim[FHIP_MAX_RANK];
  for (int i = 0; i < d->x.rank; ++i)
    sdim[i] = i == 0 ? 1 : d->x.dim[i];
  if (d->scale.rank != 0) {
    if (!fhip_check_desc(ctx, d->scale, "norm SCALE"))
      return 1;
    FHIP_REQUIRE(ctx, dims_equal(d->scale, d->x.rank, sdim),
                 "fhip_norm_fwd: SCALE dims must equal X dims with dim 0 = 1");
  }
  if (d->bias.rank != 0) {
    FHIP_REQUIRE(ctx, d->is_layernorm, "fhip_norm_fwd: RMSNorm takes no bias");
    if (!fhip_check_desc(ctx, d->bias, "norm BIAS"))
      return 1;
    FHIP_REQUIRE(ctx, dims_equal(d->bias, d->x.rank, sdim),
                 "fhip_norm_fwd: BIAS dims must equal X dims with dim 0 = 1");
  }
  if (d->emit_stats)
    FHIP_REQUIRE(ctx, d->is_layernorm && fhip_dtype_is_float(d->stats_dtype),
                 "fhip_norm_fwd: statistics are a LayerNorm training output "
                 "of floating type");
  FHIP_REQUIRE(ctx, d->out.dtype == d->out_dtype,
               "fhip_norm_fwd: out_dtype disagrees with OUT descriptor");
  return 0;
}

int fhip_norm_fwd_workspace_size(const fhip_norm_desc *d, size_t *bytes) {
  FHIP_REQUIRE(nullptr, d && bytes, "fhip_norm_fwd_workspace_size: null");
  *bytes = 0;
  return 0;
}

int fhip_norm_fwd_supported(const fhip_norm_desc *d) {
  if (!d || norm_validate(nullptr, d) != 0)
    return 0;
  return fhip_fast_norm_applicable(d) ? 2 : 1;
}

int fhip_norm_fwd(fhip_ctx *ctx, const fhip_norm_desc *d, const void *x,
                  const void *scale, const void *bias,
                  const void *const *epilogue_operands, void *out, void *mean,
                  void *inv_variance, void *workspace, size_t workspace_bytes) {
  FHIP_REQUIRE(ctx, ctx != nullptr, "fhip_norm_fwd: null context");
  if (norm_validate(ctx, d) != 0)
    return 1;
  FHIP_REQUIRE(ctx, x && out, "fhip_norm_fwd: null tensor pointer");
  FHIP_REQUIRE(ctx, (d->scale.rank != 0) == (scale != nullptr),
               "fhip_norm_fwd: scale pointer and descriptor disagree");
  FHIP_REQUIRE(ctx, (d->bias.rank != 0) == (bias != nullptr),
               "fhip_norm_fwd: bias pointer and descriptor disagree");
  FHIP_REQUIRE(ctx, !d->emit_stats || (mean && inv_variance),
               "fhip_norm_fwd: statistics requested but pointers are null");
  (void)workspace;
  (void)workspace_bytes;
  FHIP_HIP_CHECK(ctx, hipSetDevice(ctx->device));
  DevEpilogue epi;
  if (fhip_build_epilogue(ctx, d->epilogue, d->x.rank, d->x.dim,
                          epilogue_operands, &epi) != 0)
    return 1;
  if (fhip_fast_norm_applicable(d))
    return fhip_fast_norm(ctx, d, x, scale, bias, epi, out, mean, inv_variance);
  fhip_note_kernel(ctx, "norm_generic");

  NormArgs g{};
  g.x = make_dims(d->x);
  g.xs = make_strides(d->x);
  g.os = make_strides(d->out);
  if (d->scale.rank)
    g.ss = make_strides(d->scale);
  if (d->bias.rank)
    g.bs = make_strides(d->bias);
  g.inner = fhip_desc_volume(d->x) / d->x.dim[0];
  g.x_dt = d->x.dtype;
  g.s_dt = d->scale.dtype;
  g.b_dt = d->bias.dtype;
  g.y_dt = d->y.dtype;
  g.o_dt = d->out.dtype;
  g.stats_dt = d->stats_dtype;
  g.has_scale = d->scale.rank != 0;
  g.has_bias = d->bias.rank != 0;
  g.is_layernorm = d->is_layernorm;
  g.emit_stats = d->emit_stats;
  g.eps = d->epsilon;
  g.epi = epi;
  hipLaunchKernelGGL(generic_norm_kernel, dim3((unsigned)d->x.dim[0]),
                     dim3(256), 0, ctx->stream, g, x, scale, bias, out, mean,
                     inv_variance);
  FHIP_HIP_CHECK(ctx, hipGetLastError());
  return 0;
}

// ---- batch norm -----------------------------------------------------------
static int batchnorm_validate(fhip_ctx *ctx, const fhip_batchnorm_desc *d) {
  FHIP_REQUIRE(ctx, d != nullptr, "fhip_batchnorm_fwd: null descriptor");
  if (!fhip_check_desc(ctx, d->x, "batchnorm X") ||
      !fhip_check_desc(ctx, d->y, "batchnorm Y"))
    return 1;
  FHIP_REQUIRE(ctx, d->x.rank >= 2, "fhip_batchnorm_fwd: X rank %d < 2",
               d->x.rank);
  FHIP_REQUIRE(ctx, dims_equal(d->y, d->x.rank, d->x.dim),
               "fhip_batchnorm_fwd: Y dims differ from X dims");
  auto fl = [](int dt) {
    return dt == FHIP_FLOAT || dt == FHIP_HALF || dt == FHIP_BFLOAT16 ||
           dt == FHIP_DOUBLE;
  };
  FHIP_REQUIRE(ctx, fl(d->x.dtype) && fl(d->y.dtype),
               "fhip_batchnorm_fwd: X and Y must be floating point");
  FHIP_REQUIRE(ctx, !d->has_scale || fl(d->scale_dtype),
               "fhip_batchnorm_fwd: SCALE must be floating point");
  FHIP_REQUIRE(ctx, !d->has_bias || fl(d->bias_dtype),
               "fhip_batchnorm_fwd: BIAS must be floating point");
  if (d->training)
    FHIP_REQUIRE(ctx, fl(d->stats_dtype),
                 "fhip_batchnorm_fwd: saved statistics must be floating point");
  else
    FHIP_REQUIRE(ctx, fl(d->running_dtype),
                 "fhip_batchnorm_fwd: running statistics must be floating "
                 "point");
  FHIP_REQUIRE(ctx, d->epsilon >= 0.f, "fhip_batchnorm_fwd: negative epsilon");
  FHIP_REQUIRE(ctx, !d->training || d->x.dim[1] < (1ll << 31),
               "fhip_batchnorm_fwd: channel count exceeds the grid limit");
  return 0;
}

int fhip_batchnorm_fwd_workspace_size(const fhip_batchnorm_desc *d,
                                      size_t *bytes) {
  FHIP_REQUIRE(nullptr, d && bytes, "fhip_batchnorm_fwd_workspace_size: null");
  *bytes = 0;
  return 0;
}

int fhip_batchnorm_fwd_supported(const fhip_batchnorm_desc *d) {
  if (!d || batchnorm_validate(nullptr, d) != 0)
    return 0;
  return fhip_fast_batchnorm_applicable(d) ? 2 : 1;
}

int fhip_batchnorm_fwd(fhip_ctx *ctx, const fhip_batchnorm_desc *d,
                       const void *x, const void *scale, const void *bias,
                       const void *running_mean, const void *running_var,
                       void *y, void *saved_mean, void *saved_inv_variance,
                       void *workspace, size_t workspace_bytes) {
  FHIP_REQUIRE(ctx, ctx != nullptr, "fhip_batchnorm_fwd: null context");
  if (batchnorm_validate(ctx, d) != 0)
    return 1;
  FHIP_REQUIRE(ctx, x && y, "fhip_batchnorm_fwd: null tensor pointer");
  FHIP_REQUIRE(ctx, !d->has_scale == !scale && !d->has_bias == !bias,
               "fhip_batchnorm_fwd: SCALE / BIAS pointers disagree with the "
               "descriptor");
  if (d->training)
    FHIP_REQUIRE(ctx, saved_mean && saved_inv_variance,
                 "fhip_batchnorm_fwd: training needs the saved statistics' "
                 "buffers");
  else
    FHIP_REQUIRE(ctx, running_mean && running_var,
                 "fhip_batchnorm_fwd: inference needs running mean and "
                 "variance");
  (void)workspace;
  (void)workspace_bytes;
  FHIP_HIP_CHECK(ctx, hipSetDevice(ctx->device));
  if (fhip_desc_volume(d->x) > 0 && fhip_fast_batchnorm_applicable(d) &&
      (((uintptr_t)x | (uintptr_t)y) & 15) == 0)
    return fhip_fast_batchnorm(ctx, d, x, scale, bias, running_mean, running_var, y,
                               saved_mean, saved_inv_variance);
  fhip_note_kernel(ctx, "batchnorm_generic training=%d", (int)d->training);
  BatchNormArgs g{};
  g.x = make_dims(d->x);
  g.xs = make_strides(d->x);
  g.ys = make_strides(d->y);
  g.x_dt = d->x.dtype;
  g.y_dt = d->y.dtype;
  g.scale_dt = d->scale_dtype;
  g.bias_dt = d->bias_dtype;
  g.mean_dt = d->running_dtype;
  g.stats_dt = d->stats_dtype;
  g.eps = d->epsilon;
  const int64_t total = fhip_desc_volume(d->x);
  if (total == 0)
    return 0;
  if (d->training)
    hipLaunchKernelGGL(generic_batchnorm_train_kernel,
                       dim3((unsigned)d->x.dim[1]), dim3(256), 0, ctx->stream, g,
                       x, scale, bias, y, saved_mean, saved_inv_variance);
  else
    hipLaunchKernelGGL(generic_batchnorm_infer_kernel,
                       dim3(grid_for(total, 256)), dim3(256), 0, ctx->stream, g,
                       x, scale, bias, running_mean, running_var, y, total);
  FHIP_HIP_CHECK(ctx, hipGetLastError());
  return 0;
}

// ---- reduction ------------------------------------------------------------
static int reduce_validate(fhip_ctx *ctx, const fhip_reduce_desc *d) {
  FHIP_REQUIRE(ctx, d != nullptr, "fhip_reduce: null descriptor");
  if (!fhip_check_desc(ctx, d->x, "reduce X") ||
      !fhip_check_desc(ctx, d->y, "reduce Y"))
    return 1;
  FHIP_REQUIRE(ctx, d->x.rank == d->y.rank,
               "fhip_reduce: X and Y must share a rank (keep-dim)");
  for (int i = 0; i < d->x.rank; ++i)
    FHIP_REQUIRE(ctx, d->y.dim[i] == d->x.dim[i] || d->y.dim[i] == 1,
                 "fhip_reduce: Y dim %d must be 1 or equal X's", i);
  FHIP_REQUIRE(ctx, d->mode > FHIP_RED_NOT_SET && d->mode <= FHIP_RED_MUL_NO_ZEROS,
               "fhip_reduce: invalid mode %d", d->mode);
  FHIP_REQUIRE(ctx, d->mode != FHIP_RED_AVG || fhip_dtype_is_float(d->x.dtype),
               "fhip_reduce: AVG needs a floating-point input");
  return 0;
}

int fhip_reduce_workspace_size(const fhip_reduce_desc *d, size_t *bytes) {
  FHIP_REQUIRE(nullptr, d && bytes, "fhip_reduce_workspace_size: null");
  *bytes = 0;
  return 0;
}

int fhip_reduce_supported(const fhip_reduce_desc *d) {
  if (!d || reduce_validate(nullptr, d) != 0)
    return 0;
  return fhip_fast_reduce_applicable(d) ? 2 : 1;
}

int fhip_reduce(fhip_ctx *ctx, const fhip_reduce_desc *d, const void *x,
                void *y, void *workspace, size_t workspace_bytes) {
  FHIP_REQUIRE(ctx, ctx != nullptr, "fhip_reduce: null context");
  if (reduce_validate(ctx, d) != 0)
    return 1;
  FHIP_REQUIRE(ctx, x && y, "fhip_reduce: null tensor pointer");
  (void)workspace;
  (void)workspace_bytes;
  FHIP_HIP_CHECK(ctx, hipSetDevice(ctx->device));
  // the row kernel moves 16-byte chunks: an unaligned base takes the generic one
  if (fhip_fast_reduce_applicable(d) && ((uintptr_t)x & 15) == 0)
    return fhip_fast_reduce(ctx, d, x, y);
  fhip_note_kernel(ctx, "reduce_generic");
  ReduceArgs g{};
  g.y = make_dims(d->y);
  g.red.rank = d->x.rank;
  g.red_count = 1;
  for (int i = 0; i < d->x.rank; ++i) {
    const bool reduced = d->y.dim[i] == 1 && d->x.dim[i] > 1;
    g.red.dim[i] = reduced ? d->x.dim[i] : 1;
    g.red_count *= g.red.dim[i];
  }
  g.xs = make_strides(d->x);
  g.ys = make_strides(d->y);
  g.x_dt = d->x.dtype;
  g.y_dt = d->y.dtype;
  g.map_kind = RMAP_NONE;
  g.comb_kind = RCOMB_ADD;
  g.post_kind = RPOST_NONE;
  g.identity = 0.0;
  switch (d->mode) {
  case FHIP_RED_MUL:
    g.comb_kind = RCOMB_MUL;
    g.identity = 1.0;
    break;
  case FHIP_RED_MUL_NO_ZEROS:
    g.comb_kind = RCOMB_MUL;
    g.map_kind = RMAP_ZERO_TO_ONE;
    g.identity = 1.0;
    break;
  case FHIP_RED_MIN:
    g.comb_kind = RCOMB_MIN;
    g.identity = (double)INFINITY;
    break;
  case FHIP_RED_MAX:
    g.comb_kind = RCOMB_MAX;
    g.identity = -(double)INFINITY;
    break;
  case FHIP_RED_AMAX:
    g.comb_kind = RCOMB_MAX;
    g.map_kind = RMAP_ABS;
    break;
  case FHIP_RED_AVG:
    g.post_kind = RPOST_MEAN;
    break;
  case FHIP_RED_NORM1:
    g.map_kind = RMAP_ABS;
    break;
  case FHIP_RED_NORM2:
    g.map_kind = RMAP_SQUARE;
    g.post_kind = RPOST_SQRT;
    break;
  default:
    break;
  }
  const int64_t outs = fhip_desc_volume(d->y);
  if (outs == 0)
    return 0;
  // few outputs over long ranges: slices of the range on workgroups of their
  // own (about two workgroups per compute unit, at least 2048 indices each),
  // combined in slice order by a second kernel
  const int64_t cus = ctx->num_cus > 0 ? ctx->num_cus : 256;
  int64_t slices = 2 * cus / outs;
  const int64_t most = g.red_count / 2048;
  slices = slices < most ? slices : most;
  slices = slices < 1024 ? slices : 1024;
  slices = slices < 1 ? 1 : slices;
  int64_t per_slice = (g.red_count + slices - 1) / slices;
  per_slice = per_slice < 1 ? 1 : per_slice;
  slices = g.red_count > 0 ? (g.red_count + per_slice - 1) / per_slice : 1;
  const bool small = g.red_count < (1ll << 31);
  const dim3 grid((unsigned)outs, (unsigned)slices);
  auto run = [&](auto zero) {
    using CT = decltype(zero);
    void *scratch = nullptr;
    if (slices > 1 &&
        fhip_ctx_scratch(ctx, (size_t)(slices * outs) * sizeof(CT), &scratch) != 0)
      return 1;
    if (small)
      hipLaunchKernelGGL((generic_reduce_kernel<CT, true>), grid, dim3(256), 0,
                         ctx->stream, g, x, y, (CT *)scratch, per_slice);
    else
      hipLaunchKernelGGL((generic_reduce_kernel<CT, false>), grid, dim3(256), 0,
                         ctx->stream, g, x, y, (CT *)scratch, per_slice);
    if (slices > 1)
      hipLaunchKernelGGL(generic_reduce_finish_kernel<CT>,
                         dim3((unsigned)((outs + 255) / 256)), dim3(256), 0,
                         ctx->stream, g, (const CT *)scratch, y, outs,
                         (int)slices);
    return 0;
  };
  if ((needs_double(d->x.dtype) ? run(0.0) : run(0.f)) != 0)
    return 1;
  FHIP_HIP_CHECK(ctx, hipGetLastError());
  return 0;
}

// ---- pointwise ------------------------------------------------------------
static int pointwise_validate(fhip_ctx *ctx, const fhip_pointwise_desc *d) {
  FHIP_REQUIRE(ctx, d != nullptr, "fhip_pointwise: null descriptor");
  FHIP_REQUIRE(ctx, d->mode > FHIP_PW_NOT_SET && d->mode < FHIP_PW_MODE_COUNT,
               "fhip_pointwise: invalid mode %d", d->mode);
  FHIP_REQUIRE(ctx, d->num_inputs == fhip_pw_arity(d->mode),
               "fhip_pointwise: mode %d takes %d inputs, got %d", d->mode,
               fhip_pw_arity(d->mode), d->num_inputs);
  if (!fhip_check_desc(ctx, d->out, "pointwise OUT"))
    return 1;
  for (int i = 0; i < d->num_inputs; ++i) {
    if (d->in_is_scalar[i])
      continue;
    if (!fhip_check_desc(ctx, d->in[i], "pointwise IN"))
      return 1;
    int64_t st[FHIP_MAX_RANK];
    FHIP_REQUIRE(ctx,
                 fhip_broadcast_strides(d->in[i], d->out.rank, d->out.dim, st),
                 "fhip_pointwise: input %d does not broadcast to the output", i);
  }
  return 0;
}

int fhip_pointwise_supported(const fhip_pointwise_desc *d) {
  if (!d || pointwise_validate(nullptr, d) != 0)
    return 0;
  return fhip_fast_pointwise_applicable(d) ? 2 : 1;
}

int fhip_pointwise(fhip_ctx *ctx, const fhip_pointwise_desc *d, const void *in0,
                   const void *in1, const void *in2, void *out) {
  FHIP_REQUIRE(ctx, ctx != nullptr, "fhip_pointwise: null context");
  if (pointwise_validate(ctx, d) != 0)
    return 1;
  const void *ptr[3] = {in0, in1, in2};
  for (int i = 0; i < d->num_inputs; ++i)
    FHIP_REQUIRE(ctx, d->in_is_scalar[i] || ptr[i] != nullptr,
                 "fhip_pointwise: input %d pointer is null", i);
  FHIP_REQUIRE(ctx, out != nullptr, "fhip_pointwise: null output pointer");
  FHIP_HIP_CHECK(ctx, hipSetDevice(ctx->device));
  {
    // the vector kernel needs 16-byte aligned tensors
    bool aligned = ((uintptr_t)out & 15) == 0;
    for (int i = 0; i < d->num_inputs; ++i)
      aligned = aligned && (d->in_is_scalar[i] || ((uintptr_t)ptr[i] & 15) == 0);
    if (aligned && fhip_fast_pointwise_applicable(d))
      return fhip_fast_pointwise(ctx, d, in0, in1, in2, out);
  }
  fhip_note_kernel(ctx, "pointwise_generic");
  PointwiseArgs g{};
  g.out = make_dims(d->out);
  g.os = make_strides(d->out);
  g.o_dt = d->out.dtype;
  g.mode = d->mode;
  g.num_inputs = d->num_inputs;
  g.params = d->params;
  bool dbl = needs_double(d->out.dtype);
  for (int i = 0; i < d->num_inputs; ++i) {
    g.is_scalar[i] = d->in_is_scalar[i];
    g.scalar[i] = d->in_scalar[i];
    if (!d->in_is_scalar[i]) {
      fhip_broadcast_strides(d->in[i], d->out.rank, d->out.dim, g.in[i].s);
      g.in_dt[i] = d->in[i].dtype;
      dbl = dbl || needs_double(d->in[i].dtype);
    }
  }
  const int64_t total = fhip_desc_volume(d->out);
  if (dbl)
    hipLaunchKernelGGL(generic_pointwise_kernel<double>,
                       dim3(grid_for(total, 256)), dim3(256), 0, ctx->stream, g,
                       in0, in1, in2, out, total);
  else
    hipLaunchKernelGGL(generic_pointwise_kernel<float>,
                       dim3(grid_for(total, 256)), dim3(256), 0, ctx->stream, g,
                       in0, in1, in2, out, total);
  FHIP_HIP_CHECK(ctx, hipGetLastError());
  return 0;
}

} // extern "C"
