// Convolution weight gradient for 3 x 3 filters, straight from X and DY.
//
//   DW[k, r, s, c] = sum over n, p, q of DY[n, p, q, k] * X[n, p + r - 1, q + s - 1, c]
//
// (channels-last 16-bit tensors, one group, unit strides and dilations,
// padding 1, images of up to 56 columns, C and K multiples of 32).  As a GEMM
// this is skinny: 9 * C * K outputs, reduced over every pixel of the batch, and
// the reduction runs along the tensors' slow dimension.  The kernel therefore
//
//  * gives a workgroup one 32 x 32 block of (k, c) for all nine taps -- 144
//    accumulator registers per lane -- and lets its eight wavefronts reduce
//    different image rows; their results are summed through LDS at the end, so
//    a workgroup leaves 36 KB of partial sums, not 288 KB;
//  * streams image rows through small per-wavefront LDS rings by LDS-DMA (a
//    pixel's 32 channels of this block are 64 contiguous bytes) and takes the
//    MFMA operands out of them with transposing reads: 16 consecutive pixels of
//    a row are the K extent of one 32 x 32 x 16 MFMA;
//  * walks the rows of X: row rho pairs with the DY rows rho + 1, rho, rho - 1
//    (filter rows 0, 1, 2), whose fragments stay in registers for the three
//    visits, and the three column taps are the same LDS row read one pixel
//    apart -- six fragment reads feed nine MFMAs;
//  * needs no barrier in the main loop: a wavefront only waits for its own DMA.
//
// A second, small kernel sums the workgroups' partial results in a fixed
// order (the result does not depend on scheduling) and writes DW in its dtype
// and strides.
//
// Reference semantics: node/conv_node.h:255-426 (ConvWGradNode),
// aten.convolution_backward, weight gradient.
#include "common.h"
#include "fast_paths.h"
#include "gemm_kernel.h"

namespace {

constexpr int kWdWaves = 8;
constexpr int kWdThreads = kWdWaves * 64;
constexpr int kWdRow = 4096;   // LDS bytes of a row slice: 64 pixel slots x 64 bytes
constexpr int kWdXSlots = 3;   // X rows in flight per wavefront
constexpr int kWdYSlots = 2;   // DY rows in flight per wavefront
constexpr int kWdWaveLds = (kWdXSlots + kWdYSlots) * kWdRow;
constexpr int kWdLds = kWdWaves * kWdWaveLds; // 160 KB
constexpr int kWdMaxW = 56;
constexpr int kWdBlock = 9 * 16 * 64; // partial sums of one workgroup (floats)

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

struct WgDirectArgs {
  const char *x, *dy;
  float *part;
  int32_t N, H, W, C, K;
  int32_t rpw;    // image rows per wavefront
  int32_t chunks; // row chunks (8 * rpw rows) per image
  int32_t ipw;    // images per workgroup
  int32_t nparts; // workgroups per (k, c) block
  int32_t ctypes; // C / 32
  uint32_t x_bytes, dy_bytes;
};

template <int KIND>
__device__ __forceinline__ f32x16 wd_mfma(const u32x2 &a0, const u32x2 &a1,
                                          const u32x2 &b0, const u32x2 &b1,
                                          const f32x16 &c) {
  const u32x4 a = {a0.x, a0.y, a1.x, a1.y};
  const u32x4 b = {b0.x, b0.y, b1.x, b1.y};
  if constexpr (KIND == GK_BF16)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(
        __builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(
        __builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

// Transposing LDS read: the 16 lanes of a group address a 4-pixel x 16-channel
// block (lane i: pixel i / 4, channels 4 * (i % 4) ..+3) and lane i receives
// channel i of the four pixels.  Written as asm so that the compiler does not
// tie it to the LDS-DMA loads in flight; wd_wait_lgkm says when the registers
// may be used.
template <int OFFSET>
__device__ __forceinline__ void wd_read_tr(u32x2 &dst, uint32_t addr) {
  static_assert(OFFSET >= 0 && OFFSET < 65536, "16-bit offset field");
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2"
               : "=v"(dst)
               : "v"(addr), "n"(OFFSET));
}

template <int N> __device__ __forceinline__ void wd_wait_lgkm() {
  static_assert(N >= 0 && N <= 15, "lgkmcnt is a 4-bit field");
  asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(N) : "memory");
}

__device__ __forceinline__ void wd_pin(u32x2 &a) { asm volatile("" : "+v"(a)); }

__device__ __forceinline__ __amdgpu_buffer_rsrc_t wd_rsrc(const void *base,
                                                          uint32_t bytes) {
  const uint64_t b64 = (uint64_t)base;
  const uint32_t blo = __builtin_amdgcn_readfirstlane((uint32_t)b64);
  const uint32_t bhi = __builtin_amdgcn_readfirstlane((uint32_t)(b64 >> 32));
  return __builtin_amdgcn_make_buffer_rsrc(
      (void *)(((uint64_t)bhi << 32) | blo), 0,
      (int)__builtin_amdgcn_readfirstlane(bytes), 0x00020000);
}

template <int KIND>
__global__ __launch_bounds__(kWdThreads)
__attribute__((amdgpu_waves_per_eu(2, 2))) void
conv_wgrad_direct_kernel(WgDirectArgs g) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int l = threadIdx.x & 63;
  const int a_H = g.H, a_W = g.W, a_C = g.C, a_K = g.K, a_N = g.N;
  const int a_rpw = g.rpw, a_chunks = g.chunks, a_ipw = g.ipw;

  // workgroup -> (k block, c block), images, row chunk
  const int type = (int)(blockIdx.x / (unsigned)g.nparts);
  const int part = (int)(blockIdx.x - (unsigned)type * (unsigned)g.nparts);
  const int kb = type / g.ctypes, cb = type - kb * g.ctypes;
  const int igroup = part / a_chunks, chunk = part - igroup * a_chunks;
  const int n0 = igroup * a_ipw;
  const int n1 = n0 + a_ipw < a_N ? n0 + a_ipw : a_N;
  const int p0 = (chunk * kWdWaves + wave) * a_rpw;
  int nrows = a_H - p0;
  nrows = nrows < a_rpw ? nrows : a_rpw;
  nrows = nrows > 0 ? nrows : 0;
  const int n_it = nrows > 0 ? nrows + 2 : 0;

  // ---- LDS-DMA lane offsets (relative to a row's first byte) --------------------
  // instruction j fills pixel slots 16 j .. 16 j + 15 of a row slice: lane d
  // carries 16 bytes (8 channels) d % 4 of slot 16 j + d / 4.  X slot t holds
  // image column t - 1 (slot 0 and the slots past the image are the zero
  // padding), DY slot t holds column t (zeros past the image).
  uint32_t xrel[4], yrel[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int slot = 16 * j + (l >> 2);
    const int q = slot - 1;
    xrel[j] = (unsigned)q < (unsigned)a_W
                  ? (uint32_t)(q * a_C * 2 + cb * 64 + (l & 3) * 16)
                  : 0x80000000u;
    yrel[j] = slot < a_W ? (uint32_t)(slot * a_K * 2 + kb * 64 + (l & 3) * 16)
                         : 0x80000000u;
  }
  const __amdgpu_buffer_rsrc_t rx = wd_rsrc(g.x, g.x_bytes);
  const __amdgpu_buffer_rsrc_t ry = wd_rsrc(g.dy, g.dy_bytes);
  const __amdgpu_buffer_rsrc_t rnone = wd_rsrc(g.x, 0); // every lane reads zero

  const uint32_t wbase = lds0 + (uint32_t)wave * kWdWaveLds;
  // fragment read address inside a row slice: lane l is MFMA row / column
  // l % 32 and K half l / 32 (pixels 8 h .. 8 h + 7 of the K-step)
  const uint32_t tbase = (uint32_t)(((l >> 5) * 8 + ((l & 15) >> 2)) * 64 +
                                    ((l >> 4) & 1) * 32 + (l & 3) * 8);
  const uint32_t xbase = wbase + tbase;
  const uint32_t ybase = wbase + kWdXSlots * kWdRow + tbase;
  const bool upper = l >= 32;

  f32x16 acc[9];
#pragma unroll
  for (int t = 0; t < 9; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i)
      acc[t][i] = 0.f;

  for (int n = n0; n < n1; ++n) {
    // group gi of loads: X row p0 - 1 + gi into X slot xs, DY row p0 + gi into
    // DY slot gi % 2; rows outside the image (or this wavefront's share of DY)
    // arrive as zeros.  Always eight instructions, so the waits can count.
    auto issue = [&](int gi, int xs) __attribute__((always_inline)) {
      const int rho = p0 - 1 + gi;
      const bool xok = (unsigned)rho < (unsigned)a_H && gi < n_it;
      const __amdgpu_buffer_rsrc_t rsx = xok ? rx : rnone;
      const int xoff = xok ? ((n * a_H + rho) * a_W) * a_C * 2 : 0;
      const uint32_t xdst = wbase + (uint32_t)xs * kWdRow;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rsx, (GEMM_AS3 char *)__builtin_amdgcn_readfirstlane(xdst + j * 1024u),
            16, (int)xrel[j], xoff, 0, 0);
      const bool yok = gi < nrows;
      const __amdgpu_buffer_rsrc_t rsy = yok ? ry : rnone;
      const int yoff = yok ? ((n * a_H + p0 + gi) * a_W) * a_K * 2 : 0;
      const uint32_t ydst = wbase + (uint32_t)(kWdXSlots + (gi & 1)) * kWdRow;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rsy, (GEMM_AS3 char *)__builtin_amdgcn_readfirstlane(ydst + j * 1024u),
            16, (int)yrel[j], yoff, 0, 0);
    };

    // DY fragments of three rows: dyf[j] holds row it with it % 3 == j
    u32x2 dyf[3][4][2];
#pragma unroll
    for (int j = 0; j < 3; ++j)
#pragma unroll
      for (int ks = 0; ks < 4; ++ks)
        dyf[j][ks][0] = dyf[j][ks][1] = u32x2{0u, 0u};

    if (n_it > 0) {
      issue(0, 0);
      issue(1, 1);
    }

    // iteration it (it % 3 == J): X row p0 - 1 + it against DY rows it, it - 1,
    // it - 2 of this wavefront's share
    auto body = [&](auto jc, int it) __attribute__((always_inline)) {
      constexpr int J = decltype(jc)::value;
      constexpr int J1 = (J + 2) % 3, J2 = (J + 1) % 3;
      // group `it` has landed when only the eight loads of group it + 1 are out
      __builtin_amdgcn_s_waitcnt(gemm_wait_imm(8));
      const uint32_t ya = ybase + (uint32_t)(it & 1) * kWdRow;
      gemm_static_for<4>([&](auto kc) {
        constexpr int ks = decltype(kc)::value;
        wd_read_tr<ks * 1024>(dyf[J][ks][0], ya);
        wd_read_tr<ks * 1024 + 256>(dyf[J][ks][1], ya);
      });
      const uint32_t xa = xbase + (uint32_t)J * kWdRow;
      u32x2 xf[2][3][2];
      auto read_x = [&](auto kc) __attribute__((always_inline)) {
        constexpr int ks = decltype(kc)::value;
        gemm_static_for<3>([&](auto sc) {
          constexpr int s = decltype(sc)::value;
          wd_read_tr<ks * 1024 + s * 64>(xf[ks & 1][s][0], xa);
          wd_read_tr<ks * 1024 + s * 64 + 256>(xf[ks & 1][s][1], xa);
        });
      };
      read_x(std::integral_constant<int, 0>{});
      // the DY row is in registers: its slot (and the X slot read last
      // iteration) can be refilled
      wd_wait_lgkm<6>();
      issue(it + 2, (J + 2) % 3);
      // Every MFMA runs: rows that do not exist (outside the image, or DY
      // rows of another wavefront's share) were loaded as zeros, so the
      // accumulators are updated in place by straight-line code.
      gemm_static_for<4>([&](auto kc) {
        constexpr int ks = decltype(kc)::value;
        if constexpr (ks + 1 < 4) {
          read_x(std::integral_constant<int, ks + 1>{});
          wd_wait_lgkm<6>();
        } else {
          wd_wait_lgkm<0>();
        }
        u32x2(&xk)[3][2] = xf[ks & 1];
#pragma unroll
        for (int s = 0; s < 3; ++s) {
          wd_pin(xk[s][0]);
          wd_pin(xk[s][1]);
        }
        wd_pin(dyf[J][ks][0]);
        wd_pin(dyf[J][ks][1]);
        if constexpr (ks == 3) {
          // pixels 56 .. 63 of the row do not exist: X reads past the slice
#pragma unroll
          for (int s = 0; s < 3; ++s)
#pragma unroll
            for (int hh = 0; hh < 2; ++hh) {
              xk[s][hh].x = upper ? 0u : xk[s][hh].x;
              xk[s][hh].y = upper ? 0u : xk[s][hh].y;
            }
        }
#pragma unroll
        for (int s = 0; s < 3; ++s)
          acc[0 + s] = wd_mfma<KIND>(dyf[J][ks][0], dyf[J][ks][1], xk[s][0],
                                     xk[s][1], acc[0 + s]);
#pragma unroll
        for (int s = 0; s < 3; ++s)
          acc[3 + s] = wd_mfma<KIND>(dyf[J1][ks][0], dyf[J1][ks][1], xk[s][0],
                                     xk[s][1], acc[3 + s]);
#pragma unroll
        for (int s = 0; s < 3; ++s)
          acc[6 + s] = wd_mfma<KIND>(dyf[J2][ks][0], dyf[J2][ks][1], xk[s][0],
                                     xk[s][1], acc[6 + s]);
      });
    };

    int it = 0;
    while (true) {
      if (it >= n_it)
        break;
      body(std::integral_constant<int, 0>{}, it);
      ++it;
      if (it >= n_it)
        break;
      body(std::integral_constant<int, 1>{}, it);
      ++it;
      if (it >= n_it)
        break;
      body(std::integral_constant<int, 2>{}, it);
      ++it;
    }
    // the two groups still in flight land before the next image reuses the slots
    __builtin_amdgcn_s_waitcnt(gemm_wait_imm(0));
  }

  // ---- sum of the eight wavefronts through LDS, one filter row at a time ------
  __builtin_amdgcn_s_waitcnt(gemm_wait_imm(0));
  __syncthreads();
  float *scr = (float *)smem; // [wavefront][48 = 3 taps x 16 registers][64 lanes]
  float *dst = g.part + (size_t)blockIdx.x * kWdBlock;
  gemm_static_for<3>([&](auto rc) {
    constexpr int r = decltype(rc)::value;
#pragma unroll
    for (int s = 0; s < 3; ++s)
#pragma unroll
      for (int i = 0; i < 16; ++i)
        scr[(wave * 48 + s * 16 + i) * 64 + l] = acc[r * 3 + s][i];
    __syncthreads();
#pragma unroll
    for (int e6 = 0; e6 < 6; ++e6) {
      const int e = wave * 6 + e6;
      float sum = 0.f;
#pragma unroll
      for (int v = 0; v < kWdWaves; ++v)
        sum += scr[(v * 48 + e) * 64 + l];
      dst[(r * 48 + e) * 64 + l] = sum;
    }
    __syncthreads();
  });
}

struct WgDirectSumArgs {
  int32_t nparts, ctypes;
  int64_t sk, sc, sr, ss; // element strides of DW [K, C, R, S]
  int32_t dt;
};

// DW[k][c][r][s] = sum over the workgroups of a (k, c) block of their partial
// sums, in workgroup order; one thread per output element.
__global__ void conv_wgrad_direct_sum_kernel(WgDirectSumArgs a, const float *part,
                                             void *dw, int64_t total) {
  const int64_t lin = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (lin >= total)
    return;
  const int lane = (int)(lin & 63), i = (int)((lin >> 6) & 15);
  const int tap = (int)((lin >> 10) % 9);
  const int type = (int)(lin / kWdBlock);
  const float *src = part + (int64_t)type * a.nparts * kWdBlock + lin % kWdBlock;
  float acc = 0.f;
#pragma unroll 8 // independent loads: several in flight
  for (int p = 0; p < a.nparts; ++p)
    acc += src[(int64_t)p * kWdBlock];
  const int kb = type / a.ctypes, cb = type - kb * a.ctypes;
  const int64_t k = kb * 32 + 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3);
  const int64_t c = cb * 32 + (lane & 31);
  const int r = tap / 3, s = tap - r * 3;
  fhip_store<float>(dw, a.dt, k * a.sk + c * a.sc + r * a.sr + s * a.ss, acc);
}

struct WgDirectPlan {
  bool ok = false;
  int kind = GK_BF16;
  WgDirectArgs a{};
  int grid = 0;
  size_t part_bytes = 0;
};

bool wd_channels_last(const fhip_tensor_desc &t) {
  int64_t expect = 1;
  int order[FHIP_MAX_RANK], n = 0;
  order[n++] = 1;
  for (int i = t.rank - 1; i >= 2; --i)
    order[n++] = i;
  order[n++] = 0;
  for (int i = 0; i < n; ++i) {
    const int d = order[i];
    if (t.dim[d] != 1 && t.stride[d] != expect)
      return false;
    expect *= t.dim[d];
  }
  return true;
}

WgDirectPlan make_wd_plan(const fhip_conv_desc *d, int num_cus) {
  WgDirectPlan p;
  if (fhip_knobs().wgrad_direct == 0)
    return p;
  if (d->spatial_rank != 2)
    return p;
  const int dt = d->x.dtype;
  if (dt == FHIP_BFLOAT16)
    p.kind = GK_BF16;
  else if (dt == FHIP_HALF)
    p.kind = GK_F16;
  else
    return p;
  if (d->y.dtype != dt)
    return p;
  const int wdt = d->w.dtype;
  if (wdt != FHIP_BFLOAT16 && wdt != FHIP_HALF && wdt != FHIP_FLOAT)
    return p;
  const int64_t N = d->x.dim[0], C = d->x.dim[1], H = d->x.dim[2], W = d->x.dim[3];
  const int64_t K = d->w.dim[0];
  if (d->w.dim[1] != C || d->w.dim[2] != 3 || d->w.dim[3] != 3)
    return p;
  for (int i = 0; i < 2; ++i)
    if (d->stride[i] != 1 || d->dilation[i] != 1 || d->padding[i] != 1)
      return p;
  if (d->y.dim[2] != H || d->y.dim[3] != W || d->y.dim[0] != N || d->y.dim[1] != K)
    return p;
  if (C % 32 != 0 || K % 32 != 0 || W > kWdMaxW || W < 1 || H < 1 || N < 1)
    return p;
  if (!wd_channels_last(d->x) || !wd_channels_last(d->y))
    return p;
  const int64_t x_bytes = N * H * W * C * 2, dy_bytes = N * H * W * K * 2;
  if (x_bytes >= (1ll << 31) || dy_bytes >= (1ll << 31))
    return p;
  const int cus = num_cus > 0 ? num_cus : 256;
  const int64_t types = (C / 32) * (K / 32);
  if (types > 4096)
    return p;
  // One workgroup per (block, image group, row chunk): as few partial results
  // as fill the machine once.  Small batches cut the image into row chunks,
  // large ones give a workgroup several images.
  int64_t chunks = 1, ipw = 1;
  if (types * N < cus) {
    chunks = (cus + types * N - 1) / (types * N);
    const int64_t most = (H + kWdWaves - 1) / kWdWaves;
    chunks = chunks < most ? chunks : most;
  } else {
    ipw = types * N / cus;
    ipw = ipw < 1 ? 1 : ipw;
  }
  const int64_t rpw = (H + kWdWaves * chunks - 1) / (kWdWaves * chunks);
  chunks = (H + kWdWaves * rpw - 1) / (kWdWaves * rpw);
  const int64_t igroups = (N + ipw - 1) / ipw;
  const int64_t nparts = igroups * chunks;
  if (types * nparts >= (1ll << 31) / kWdBlock)
    return p;
  WgDirectArgs &a = p.a;
  a.N = (int32_t)N, a.H = (int32_t)H, a.W = (int32_t)W, a.C = (int32_t)C, a.K = (int32_t)K;
  a.rpw = (int32_t)rpw, a.chunks = (int32_t)chunks, a.ipw = (int32_t)ipw;
  a.nparts = (int32_t)nparts, a.ctypes = (int32_t)(C / 32);
  a.x_bytes = (uint32_t)x_bytes, a.dy_bytes = (uint32_t)dy_bytes;
  p.grid = (int)(types * nparts);
  p.part_bytes = (size_t)p.grid * kWdBlock * sizeof(float);
  p.ok = true;
  return p;
}

template <int KIND> int wd_launch(fhip_ctx *ctx, const WgDirectPlan &p) {
  auto kernel = conv_wgrad_direct_kernel<KIND>;
  static FhipOncePerDevice configured;
  if (!configured.done(ctx->device)) {
    FHIP_HIP_CHECK(ctx, hipFuncSetAttribute(
                            reinterpret_cast<const void *>(kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, kWdLds));
    configured.mark(ctx->device);
  }
  hipLaunchKernelGGL(kernel, dim3((unsigned)p.grid), dim3(kWdThreads), kWdLds,
                     ctx->stream, p.a);
  FHIP_HIP_CHECK(ctx, hipGetLastError());
  return 0;
}

} // namespace

bool fhip_fast_conv_wgrad_direct_applicable(const fhip_conv_desc *d,
                                            size_t *workspace_bytes) {
  const WgDirectPlan p = make_wd_plan(d, 256);
  if (workspace_bytes)
    *workspace_bytes = p.ok ? p.part_bytes : 0;
  return p.ok;
}

int fhip_fast_conv_wgrad_direct(fhip_ctx *ctx, const fhip_conv_desc *d,
                                const void *dy, const void *x, void *dw,
                                void *workspace) {
  // planned for 256 compute units whatever the device: the workspace size was
  // answered without one
  WgDirectPlan p = make_wd_plan(d, 256);
  FHIP_REQUIRE(ctx, p.ok, "conv wgrad: descriptor not supported by the direct kernel");
  FHIP_REQUIRE(ctx, ((uintptr_t)workspace & 255) == 0 && ((uintptr_t)x & 15) == 0 &&
                        ((uintptr_t)dy & 15) == 0,
               "conv wgrad: workspace must be 256-byte and tensors 16-byte aligned");
  p.a.x = (const char *)x;
  p.a.dy = (const char *)dy;
  p.a.part = (float *)workspace;
  if ((p.kind == GK_BF16 ? wd_launch<GK_BF16>(ctx, p) : wd_launch<GK_F16>(ctx, p)) != 0)
    return 1;
  WgDirectSumArgs s;
  s.nparts = p.a.nparts, s.ctypes = p.a.ctypes;
  s.sk = d->w.dim[0] == 1 ? 0 : d->w.stride[0];
  s.sc = d->w.dim[1] == 1 ? 0 : d->w.stride[1];
  s.sr = d->w.dim[2] == 1 ? 0 : d->w.stride[2];
  s.ss = d->w.dim[3] == 1 ? 0 : d->w.stride[3];
  s.dt = d->w.dtype;
  const int64_t total = (int64_t)(p.a.C / 32) * (p.a.K / 32) * kWdBlock;
  hipLaunchKernelGGL(conv_wgrad_direct_sum_kernel,
                     dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                     ctx->stream, s, (const float *)p.a.part, dw, total);
  FHIP_HIP_CHECK(ctx, hipGetLastError());
  return 0;
}
