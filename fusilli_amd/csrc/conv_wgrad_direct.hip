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

#ifndef WD_EXP
#define WD_EXP 0 // timing experiments: 1 no MFMA, 2 no loads in the loop, 4 no LDS sum, 8 no fragment reads
#endif

#ifdef WD_PROFILE // experiment builds: cycle stamps of workgroup 0 replace its results
#define WD_STAMP(i) st[i] = __builtin_amdgcn_s_memtime()
#else
#define WD_STAMP(i)                                                            \
  do {                                                                         \
  } while (0)
#endif

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
typedef float f32x4 __attribute__((ext_vector_type(4)));

struct WgDirectArgs {
  const char *x, *dy;
  float *part;
  int32_t N, H, W, C, K;
  int32_t rpw;    // image rows per pair of wavefronts (w, w + 4) that share a SIMD
  int32_t rfirst; // of which wavefront w takes the first rfirst, w + 4 the rest
  int32_t chunks; // row chunks (4 * rpw rows) per image
  int32_t ipw;    // images per workgroup
  int32_t nparts; // workgroups per (k, c) block
  int32_t ctypes; // C / 32
  uint32_t magic_ctypes;
  uint32_t x_bytes, dy_bytes;
};

template <int KIND>
__device__ __forceinline__ f32x16 wd_mfma(const u32x2 &a0, const u32x2 &a1,
                                          const u32x2 &b0, const u32x2 &b1,
                                          const f32x16 &c) {
  const u32x4 a = {a0.x, a0.y, a1.x, a1.y};
  const u32x4 b = {b0.x, b0.y, b1.x, b1.y};
  if (WD_EXP & 1) {
    f32x16 r = c;
    asm volatile("" : "+v"(r) : "v"(a), "v"(b));
    return r;
  }
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
  if (WD_EXP & 8) {
    asm volatile("" : "=v"(dst) : "v"(addr));
    return;
  }
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
#ifdef WD_PROFILE
  uint64_t st[8] = {};
#endif
  WD_STAMP(0);
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int l = threadIdx.x & 63;
  const int a_H = g.H, a_W = g.W, a_C = g.C, a_K = g.K, a_N = g.N;
  const int a_rpw = g.rpw, a_ipw = g.ipw;

  // workgroup (x, y, z) -> row chunk, image group, (k block, c block)
  const int chunk = (int)blockIdx.x, igroup = (int)blockIdx.y, type = (int)blockIdx.z;
  const int kb = conv_div(type, g.ctypes, g.magic_ctypes), cb = type - kb * g.ctypes;
  const int n0 = igroup * a_ipw;
  const int n1 = n0 + a_ipw < a_N ? n0 + a_ipw : a_N;
  // rows: the pair (w, w + 4) of a SIMD shares a_rpw rows; the first of the
  // pair, which the SIMD serves first, takes the larger part
  const int second = wave >> 2;
  const int p0 = (chunk * 4 + (wave & 3)) * a_rpw + (second ? g.rfirst : 0);
  const int share = second ? a_rpw - g.rfirst : g.rfirst;
  int nrows = a_H - p0;
  nrows = nrows < share ? nrows : share;
  nrows = nrows > 0 ? nrows : 0;
  // Step t of a wavefront's walk brings DY row p0 - 1 + t into registers and,
  // from t = 2 on, multiplies X row p0 + t - 2 with the three DY rows held:
  // the newest is filter row 0, the oldest filter row 2.
  const int n_st = nrows > 0 ? nrows + 2 : 0;

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

  for (int n = n0; n < n1 && n_st > 0; ++n) {
    // Loads of step t: four instructions each, so that the waits can count.
    // Rows outside the image arrive as zeros (DY rows of the neighbouring
    // wavefronts' shares are real: they are this share's halo).
    auto issue_y = [&](int t) __attribute__((always_inline)) {
      const int row = p0 - 1 + t;
      const bool ok = t < n_st && (unsigned)row < (unsigned)a_H;
      const __amdgpu_buffer_rsrc_t rs = ok ? ry : rnone;
      const int off = ok ? ((n * a_H + row) * a_W) * a_K * 2 : 0;
      const uint32_t dst = wbase + (uint32_t)(kWdXSlots + (t & 1)) * kWdRow;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rs, (GEMM_AS3 char *)__builtin_amdgcn_readfirstlane(dst + j * 1024u),
            16, (int)yrel[j], off, 0, 0);
    };
    auto issue_x = [&](int t, int xs) __attribute__((always_inline)) {
      const int row = p0 + t - 2;
      const bool ok = t < n_st;
      const __amdgpu_buffer_rsrc_t rs = ok ? rx : rnone;
      const int off = ok ? ((n * a_H + row) * a_W) * a_C * 2 : 0;
      const uint32_t dst = wbase + (uint32_t)xs * kWdRow;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rs, (GEMM_AS3 char *)__builtin_amdgcn_readfirstlane(dst + j * 1024u),
            16, (int)xrel[j], off, 0, 0);
    };

    // DY fragments of three rows: dyf[j] holds the row of step t, t % 3 == j
    u32x2 dyf[3][4][2];

    WD_STAMP(1);
    issue_y(0);
    issue_y(1);
    issue_x(2, 0);
    WD_STAMP(2);

    auto read_y = [&](auto jc, int t) __attribute__((always_inline)) {
      constexpr int J = decltype(jc)::value;
      const uint32_t ya = ybase + (uint32_t)(t & 1) * kWdRow;
      gemm_static_for<4>([&](auto kc) {
        constexpr int ks = decltype(kc)::value;
        wd_read_tr<ks * 1024>(dyf[J][ks][0], ya);
        wd_read_tr<ks * 1024 + 256>(dyf[J][ks][1], ya);
      });
    };
    // steps 0 and 1: a DY row into registers, its slot refilled.  The order of
    // all loads is Y0 Y1 X2 | Y2 X3 | Y3 | X4 Y4 | X5 Y5 ...: from step 2 on a
    // step finds exactly eight loads issued after the ones it needs.
    auto light = [&](auto jc, auto vmc, int t) __attribute__((always_inline)) {
      if (!(WD_EXP & 2))
        __builtin_amdgcn_s_waitcnt(gemm_wait_imm(decltype(vmc)::value));
      read_y(jc, t);
      wd_wait_lgkm<0>();
      if (!(WD_EXP & 2)) {
        issue_y(t + 2);
        if (t == 0)
          issue_x(3, 1);
      }
    };
    // step t >= 2 (t % 3 == J): X row p0 + t - 2 against the three DY rows
    auto full = [&](auto jc, auto vmc, int t) __attribute__((always_inline)) {
      constexpr int J = decltype(jc)::value;
      constexpr int J1 = (J + 2) % 3, J2 = (J + 1) % 3;
      constexpr int XS = (J + 1) % 3; // (t - 2) % 3
      // the loads of this step have landed when only the eight issued after
      // them are out
      if (!(WD_EXP & 2))
        __builtin_amdgcn_s_waitcnt(gemm_wait_imm(decltype(vmc)::value));
      read_y(jc, t);
      const uint32_t xa = xbase + (uint32_t)XS * kWdRow;
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
      // the DY row is in registers: its slot, and the X slot read in the
      // step before, can be refilled
      wd_wait_lgkm<6>();
      if (!(WD_EXP & 2)) {
        issue_x(t + 2, J);
        issue_y(t + 2);
      }
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

    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    using V8 = std::integral_constant<int, 8>;
    using V12 = std::integral_constant<int, 12>;
    light(I0{}, V8{}, 0);
    light(I1{}, V12{}, 1);
    int t = 2;
    while (true) {
      if (t >= n_st)
        break;
      full(I2{}, V8{}, t);
      ++t;
      if (t >= n_st)
        break;
      full(I0{}, V8{}, t);
      ++t;
      if (t >= n_st)
        break;
      full(I1{}, V8{}, t);
      ++t;
    }
    // the loads still in flight land before the next image reuses the slots
    __builtin_amdgcn_s_waitcnt(gemm_wait_imm(0));
  }

  // ---- sum of the eight wavefronts through LDS, half of the block at a time ---
  WD_STAMP(4);
  __builtin_amdgcn_s_waitcnt(gemm_wait_imm(0));
  __syncthreads();
  WD_STAMP(5);
  const unsigned wg = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
  f32x4 *dst4 = (f32x4 *)(g.part + (size_t)wg * kWdBlock);
  if (WD_EXP & 4) {
    float v = 0.f;
#pragma unroll
    for (int t = 0; t < 9; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i)
        v += acc[t][i];
    ((float *)dst4)[wave * 64 + l] = v;
    return;
  }
  // entry e = 4 * tap + j is registers 4 j .. 4 j + 3 of a tap's accumulator:
  // one 16-byte LDS access per lane
  f32x4 *scr4 = (f32x4 *)smem; // [wavefront][18 entries][64 lanes]
  constexpr int kHalf = 18 * 64;
  gemm_static_for<2>([&](auto hc) {
    constexpr int h = decltype(hc)::value;
    gemm_static_for<18>([&](auto kc) {
      constexpr int k = decltype(kc)::value;
      constexpr int e = 18 * h + k, tap = e / 4, j = e % 4;
      const f32x4 v = {acc[tap][4 * j], acc[tap][4 * j + 1], acc[tap][4 * j + 2],
                       acc[tap][4 * j + 3]};
      scr4[(wave * 18 + k) * 64 + l] = v;
    });
    __syncthreads();
    for (int f = (int)threadIdx.x; f < kHalf; f += kWdThreads) {
      f32x4 sum = scr4[f];
#pragma unroll
      for (int v = 1; v < kWdWaves; ++v) {
        const f32x4 o = scr4[v * kHalf + f];
        sum[0] += o[0], sum[1] += o[1], sum[2] += o[2], sum[3] += o[3];
      }
      dst4[h * kHalf + f] = sum;
    }
    __syncthreads();
  });
#ifdef WD_PROFILE
  __builtin_amdgcn_s_waitcnt(gemm_wait_imm(0));
  WD_STAMP(6);
  if (wg == 0 && l == 0)
    for (int i = 0; i < 8; ++i)
      ((uint64_t *)dst4)[wave * 8 + i] = st[i];
#endif
}

struct WgDirectSumArgs {
  int32_t nparts, ctypes;
  int64_t sk, sc, sr, ss; // element strides of DW [K, C, R, S]
  int32_t dt;
};

// DW[k][c][r][s] = sum of the partial results of a (k, c) block's workgroups.
// 64 outputs per workgroup of 256 threads: thread (o, j) adds the partials
// j, j + 4, ... (all loads independent), the four sums are added in order.
// A partial block is [entry e = 4 * tap + i / 4][lane][i % 4].
__global__ __launch_bounds__(256) void
conv_wgrad_direct_sum_kernel(WgDirectSumArgs a, const float *part, void *dw) {
  // A workgroup adds 256 results: thread (o, j) the parts j, j + 4, ... of
  // four consecutive ones (16-byte loads; a wavefront reads 1 KB runs), then
  // the four j of a group meet in LDS, always in the same order.
  __shared__ f32x4 red[4][64];
  const int o = threadIdx.x & 63, j = threadIdx.x >> 6;
  const int64_t lin = ((int64_t)blockIdx.x * 64 + o) * 4;
  const int type = (int)(lin / kWdBlock);
  const int within = (int)(lin - (int64_t)type * kWdBlock);
  const float *src = part + (int64_t)type * a.nparts * kWdBlock + within;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 8
  for (int p = j; p < a.nparts; p += 4)
    acc += *(const f32x4 *)(src + (int64_t)p * kWdBlock);
  red[j][o] = acc;
  __syncthreads();
  if (j != 0)
    return;
  acc = ((red[0][o] + red[1][o]) + red[2][o]) + red[3][o];
  // within = [entry e = 4 * tap + i / 4][lane][i % 4]: the four values are i % 4 = 0 .. 3
  const int lane = (within >> 2) & 63, e = within >> 8;
  const int tap = e >> 2;
  const int kb = type / a.ctypes, cb = type - kb * a.ctypes;
  const int64_t c = cb * 32 + (lane & 31);
  const int r = tap / 3, sx = tap - r * 3;
#pragma unroll
  for (int comp = 0; comp < 4; ++comp) {
    const int i = 4 * (e & 3) + comp;
    const int64_t k = kb * 32 + 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3);
    fhip_store<float>(dw, a.dt, k * a.sk + c * a.sc + r * a.sr + sx * a.ss, acc[comp]);
  }
}

struct WgDirectPlan {
  bool ok = false;
  int kind = GK_BF16;
  WgDirectArgs a{};
  dim3 grid;
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
  const FhipKnobs &knobs = fhip_knobs();
  if (knobs.wgrad_direct == 0)
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
  // rows per pair of wavefronts
  const int64_t rpw = (H + 4 * chunks - 1) / (4 * chunks);
  chunks = (H + 4 * rpw - 1) / (4 * rpw);
  const int64_t rfirst = (rpw + 1) / 2;
  const int64_t igroups = (N + ipw - 1) / ipw;
  const int64_t nparts = igroups * chunks;
  if (types * nparts >= (1ll << 31) / kWdBlock)
    return p;
  WgDirectArgs &a = p.a;
  a.N = (int32_t)N, a.H = (int32_t)H, a.W = (int32_t)W, a.C = (int32_t)C, a.K = (int32_t)K;
  a.rpw = (int32_t)rpw, a.rfirst = (int32_t)rfirst;
  a.chunks = (int32_t)chunks, a.ipw = (int32_t)ipw;
  a.nparts = (int32_t)nparts, a.ctypes = (int32_t)(C / 32);
  a.magic_ctypes = conv_magic(a.ctypes);
  a.x_bytes = (uint32_t)x_bytes, a.dy_bytes = (uint32_t)dy_bytes;
  if (chunks > 65535 || igroups > 65535 || types > 65535)
    return p;
  p.grid = dim3((unsigned)chunks, (unsigned)igroups, (unsigned)types);
  p.part_bytes = (size_t)(types * nparts) * kWdBlock * sizeof(float);
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
  hipLaunchKernelGGL(kernel, p.grid, dim3(kWdThreads), kWdLds, ctx->stream, p.a);
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
  hipLaunchKernelGGL(conv_wgrad_direct_sum_kernel, dim3((unsigned)(total / 256)),
                     dim3(256), 0, ctx->stream, s, (const float *)p.a.part, dw);
  FHIP_HIP_CHECK(ctx, hipGetLastError());
  fhip_note_kernel(ctx, "conv_wgrad_direct");
  return 0;
}
