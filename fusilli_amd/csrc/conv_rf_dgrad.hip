// Convolution data gradient with the filter held in registers.
//
//   DX[n, i, j, c] = sum over r, s, k of DY[n, i + pad - r, j + pad - s, k] * W[k, r, s, c]
//
// (channels-last 16-bit tensors, one group, unit strides and dilations; the
// 3 x 3 x 128-channel family).  It is the forward problem of conv_rf.hip with
// DY as the image, the mirrored and transposed filter and padding R - 1 - pad,
// with two differences that shape the kernel:
//
//   * the reduction is twice as long (9 taps x 128 channels of DY): the filter
//     of 32 output channels is 36 K-steps x 2 tiles x 4 = 288 registers, more
//     than a wavefront has at two per SIMD (and 16 channels per wavefront
//     would read one LDS fragment per MFMA: the LDS, not the matrix pipe, then
//     sets the pace -- measured: 24.6 us).  So a workgroup is 4 wavefronts, one
//     per SIMD with the whole register file (2 channel slices of 32 x 2 that
//     alternate pixel blocks = 64 output channels), every fragment read feeds
//     two v_mfma_f32_16x16x32, and a lane ends up with 8 consecutive channels
//     of one pixel (16-byte stores);
//   * no mirrored copy of the filter is made: W's rows [k][r][s][c] are staged
//     as they lie, 32 k x 64 c per K-step by LDS-DMA (tap R - 1 - r', S - 1 -
//     s' for the kernel's tap r', s'), and the transposing LDS read hands a
//     lane the 8 consecutive k of its channel, the MFMA's A operand.  The whole
//     filter (144 KB) is staged at once, before the first slab.
//
// The slab (tile rows plus halo, zero-padded, pixel pitch 128 * 2 + 16 bytes)
// and the fragment ring are those of conv_rf.hip; tiles may also split the
// image's width, so that they come out as whole rounds of the machine.  DY is
// twice the size of the output, so the slab loads are what the kernel has to
// hide: two slab buffers alternate (under the filter stage until the filter is
// in registers), the next tile's rows arrive by LDS-DMA while the current tile
// is multiplied.  Fragment reads are written as asm with their own wait
// counts, so that they do not wait for the loads in flight.
//
// Reference semantics: node/conv_node.h:427-598 (ConvDGradNode),
// aten.convolution_backward, input gradient.
#include "common.h"
#include "fast_paths.h"
#include "gemm_kernel.h"

#ifdef RD_PROFILE // experiment builds: cycle stamps of workgroup 0 replace the start of DX
#define RD_STAMP(i) st[i] = __builtin_amdgcn_s_memtime()
#else
#define RD_STAMP(i)                                                            \
  do {                                                                         \
  } while (0)
#endif

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kRdWaves = 4; // one per SIMD: the whole register file each
constexpr int kRdThreads = kRdWaves * 64;
constexpr int kRdChannels = 64; // output channels per workgroup
constexpr int kRdMaxNI = 16;    // KB of LDS per slab row, at most

struct RfDgradArgs {
  const char *dy, *w;
  char *dx;
  int32_t N, H, W;  // DY's batch and extent
  int32_t P, Q;     // DX's extent
  int32_t CO;       // DX's channels, a multiple of 64
  int32_t pad_h, pad_w; // of the forward-shaped problem: R - 1 - padding
  int32_t TR, tiles_per_image, ntiles, kgroups, NI;
  int32_t TQ, ctiles; // output columns per tile (Q = TQ * ctiles), column tiles per row tile
  uint32_t magic_q;   // of TQ
  uint32_t dy_bytes, w_bytes;
};

template <int KIND>
__device__ __forceinline__ f32x4 rd_mfma(const u32x4 &a, const u32x4 &b,
                                         const f32x4 &c) {
  if constexpr (KIND == GK_BF16)
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(
        __builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(
        __builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t rd_rsrc(const void *base,
                                                          uint32_t bytes) {
  const uint64_t b64 = (uint64_t)base;
  const uint32_t blo = __builtin_amdgcn_readfirstlane((uint32_t)b64);
  const uint32_t bhi = __builtin_amdgcn_readfirstlane((uint32_t)(b64 >> 32));
  return __builtin_amdgcn_make_buffer_rsrc(
      (void *)(((uint64_t)bhi << 32) | blo), 0,
      (int)__builtin_amdgcn_readfirstlane(bytes), 0x00020000);
}

// 16-byte LDS read that the compiler does not tie to the LDS-DMA loads in
// flight, and the wait that goes with it: at most N LDS operations still
// outstanding, after which `reg` may be used.
template <int OFFSET>
__device__ __forceinline__ void rd_read_b128(u32x4 &dst, uint32_t addr) {
  static_assert(OFFSET >= 0 && OFFSET < 65536, "16-bit offset field");
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFFSET));
}
template <int N> __device__ __forceinline__ void rd_wait_lgkm(u32x4 &reg) {
  static_assert(N >= 0 && N <= 15, "lgkmcnt is a 4-bit field");
  asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(reg) : "n"(N));
}

// CK: channels of DY (the reduction)
template <int CK, int R, int S> struct RdGeom {
  static constexpr int kCPP = CK * 2 / 16 + 1;  // chunks per slab pixel (one is padding)
  static constexpr int kKPT = CK / 32;          // K-steps per tap
  static constexpr int kNK = R * S * kKPT;      // K-steps of 32 channels
  static constexpr int kStageBytes = kNK * 4096; // 32 k x 64 c x 2 bytes per K-step
};

template <int KIND, int CK, int R, int S>
__global__ __launch_bounds__(kRdThreads)
__attribute__((amdgpu_waves_per_eu(1, 1))) void
conv_rf_dgrad_kernel(RfDgradArgs g) {
  using G = RdGeom<CK, R, S>;
  constexpr int CPP = G::kCPP, PITCH = CPP * 16, KPT = G::kKPT, NK = G::kNK;
#ifndef RD_RING
#define RD_RING 9
#endif
  constexpr int RING = RD_RING; // fragment buffers (K-steps in flight)
  constexpr int NFE = RING - 1; // fragments of the next block fetched early
  constexpr int NF0 = NK - 2 * NFE - RING - 1; // step of the first early fetch, then every other step
  static_assert(RING <= 9 && CK % 32 == 0 && NK % RING == 0 && NF0 >= 0,
                "filter shape not covered");
  static_assert((S - 1) * PITCH + (KPT - 1) * 64 + 48 < 65536, "ds offset range");
  const int a_Q = g.Q, a_P = g.P, a_TR = g.TR, a_NI = g.NI, a_CO = g.CO;
  const int a_W = g.W, a_H = g.H, a_pad_w = g.pad_w, a_pad_h = g.pad_h;
  const int a_tiles_per_image = g.tiles_per_image, a_ntiles = g.ntiles;
  const int a_kgroups = g.kgroups;
  const uint32_t a_magic_q = g.magic_q;
  const int a_TQ = g.TQ, a_ctiles = g.ctiles;

  extern __shared__ __attribute__((aligned(16))) char smem[];
#ifdef RD_PROFILE
  uint64_t st[8] = {};
  int iter = 0;
#endif
  RD_STAMP(0);
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int slice = wave & 1; // 32 output channels
  const int half = wave >> 1; // which of the two that alternate pixel blocks
  const int l = threadIdx.x & 63;
  const int px = l & 15, q = l >> 4;
  const uint32_t rowpitch = (uint32_t)a_NI * 1024u;
  // two slab buffers; the filter stage lies over them until the filter is in
  // registers
  const uint32_t slab_bytes = (uint32_t)(a_TR + R - 1) * rowpitch;
  const uint32_t buf0 = lds0, buf1 = lds0 + slab_bytes;

  const int kg = (int)(blockIdx.x % (unsigned)a_kgroups);
  const int ch_wave = kg * kRdChannels + slice * 32;
  // Tiles of a workgroup.  Workgroups go to the 8 XCDs round-robin; with one
  // channel group and a multiple of 8 workgroups, XCD x takes a contiguous
  // eighth of the tiles, so that the halo rows neighbouring tiles share are
  // found in its L2.
  const int slot = (int)(blockIdx.x / (unsigned)a_kgroups);
  const int nslots = (int)(gridDim.x / (unsigned)a_kgroups);
  int tile0 = slot, tile_end = a_ntiles, tile_step = nslots;
  if (a_kgroups == 1 && (nslots & 7) == 0) {
    const int chunk = (a_ntiles + 7) >> 3, x = slot & 7;
    tile0 = x * chunk + (slot >> 3);
    tile_end = (x + 1) * chunk < a_ntiles ? (x + 1) * chunk : a_ntiles;
    tile_step = nslots >> 3;
  }

  // ---- filter: W[k][r][s][c] -> registers, through LDS ------------------------
  // K-step j = (tap', part) covers k = 32 part .. 32 part + 31 of kernel tap
  // tap' = (r', s'), which is filter tap (R - 1 - r', S - 1 - s').  Its stage
  // slot holds 32 rows (k) of this workgroup's 64 channels (128 bytes), written
  // by four LDS-DMA instructions (8 rows each: lane d carries chunk d % 8 of
  // row d / 8); wavefront w issues the K-steps j = w, w + 4, ...
  const int64_t wrow = (int64_t)R * S * a_CO * 2; // bytes between W's k rows
  const __amdgpu_buffer_rsrc_t rw = rd_rsrc(g.w, g.w_bytes);
  {
    uint32_t fvoff[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      // chunk c of stage row r sits at position c ^ 4 * (r / 2 % 2): the 64 lanes
      // of a fragment read then meet 4 to a bank pair instead of 8
      const int row = i * 8 + (l >> 3);
      const int c = (l & 7) ^ (((row >> 1) & 1) << 2);
      fvoff[i] = (uint32_t)(row * wrow + kg * 128 + c * 16);
    }
    gemm_static_for<NK / 4>([&](auto jc) {
      const int j = decltype(jc)::value * 4 + wave;
      const int tap = j / KPT, part = j - tap * KPT;
      const int src = (R - 1 - tap / S) * S + (S - 1 - tap % S);
      const int soff = (int)(part * 32 * wrow + src * a_CO * 2);
#pragma unroll
      for (int i = 0; i < 4; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rw,
            (GEMM_AS3 char *)__builtin_amdgcn_readfirstlane(
                lds0 + (uint32_t)(j * 4096 + i * 1024)),
            16, (int)fvoff[i], soff, 0, 0);
    });
  }
  // MFMA row rho of tile t is output channel ch_wave + 8 * (rho / 4) + 4 * t +
  // rho % 4, so that a lane's 8 results (rows 4 q .. 4 q + 3 of both tiles) are
  // 8 consecutive channels.  MFMA lane (rho = l % 16, kq = l / 16) takes k = 8
  // kq .. 8 kq + 7 of its channel: two transposing reads of 4 k each, for which
  // the 16 lanes of a group address rows 8 kq + rho / 4 (+ 4) and the four
  // channels 8 (rho % 4) + 4 t ..+3 of the slice.
  // (with one wavefront per SIMD the compiler has the accumulation registers
  // as well: it keeps most of these 288 registers there, where the MFMA takes
  // its A operand from directly)
  u32x4 filt[NK][2];
  __builtin_amdgcn_s_waitcnt(gemm_wait_imm(0));
  gemm_barrier();
  RD_STAMP(1);
  {
    const int frow = 8 * q + (px >> 2);
    const uint32_t fread =
        lds0 + (uint32_t)(frow * 128 + (((slice * 4 + (px & 3)) ^ (((frow >> 1) & 1) << 2)) << 4));
    gemm_static_for<NK>([&](auto jc) {
      constexpr int j = decltype(jc)::value;
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const u32x2 lo = __builtin_bit_cast(
            u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                       (GEMM_AS3 s16x4 *)(uintptr_t)(fread + j * 4096 + t * 8)));
        const u32x2 hi = __builtin_bit_cast(
            u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                       (GEMM_AS3 s16x4 *)(uintptr_t)(fread + j * 4096 + t * 8 + 512)));
        const u32x4 f = {lo.x, lo.y, hi.x, hi.y};
        filt[j][t] = f;
      }
    });
  }
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt(gemm_wait_imm(63)); // the reads returned
  gemm_barrier(); // the stage is dead: slabs may cover it

  const __amdgpu_buffer_rsrc_t rx = rd_rsrc(g.dy, g.dy_bytes);
  const __amdgpu_buffer_rsrc_t rnone = rd_rsrc(g.dy, 0); // every lane out of range

  // ---- slab of a tile: its rows plus halo by LDS-DMA; wavefront w loads rows
  // w, w + 4, ...  LDS chunk x = i * 64 + lane of a slab row is chunk x % CPP
  // of slab pixel x / CPP, i.e. input column q0 - pad_w + x / CPP; the padding
  // chunk, columns outside the image or the tile's reach and the tail of the
  // row's last KB read as zeros.
  // tile -> (image, first output row, first output column)
  auto tile_origin = [&](int tile, int &n, int &p0, int &q0) __attribute__((always_inline)) {
    const int rt = tile / a_ctiles; // row tile of the batch
    q0 = (tile - rt * a_ctiles) * a_TQ;
    n = rt / a_tiles_per_image;
    p0 = (rt - n * a_tiles_per_image) * a_TR;
  };
  // s_sp / s_off: slab pixel and byte offset (pixel and chunk) of this lane's
  // chunk of instruction i, the same for every tile; a chunk that no tile
  // fetches has a pixel far below zero, which fails the column test.
  int s_sp[kRdMaxNI];
  uint32_t s_off[kRdMaxNI];
#pragma unroll
  for (int i = 0; i < kRdMaxNI; ++i)
    if (i < a_NI) {
      const int xk = i * 64 + l;
      const int sp = (xk * (65536 / CPP + 1)) >> 16; // xk / CPP for xk < 2^12
      const int c = xk - sp * CPP;
      const bool ok = c < CPP - 1 && sp < a_TQ + S - 1;
      s_sp[i] = ok ? sp : -0x40000000;
      s_off[i] = (uint32_t)(sp * (CK * 2) + c * 16);
    }
  auto issue_slab = [&](int tile, uint32_t dst0) __attribute__((always_inline)) {
    int n, p0, q0;
    tile_origin(tile, n, p0, q0);
    // slab pixel sp is input column q0 - pad_w + sp; only the TQ + S - 1
    // columns the tile needs are fetched
    const int iw0 = q0 - a_pad_w;
    uint32_t rel[kRdMaxNI];
#pragma unroll
    for (int i = 0; i < kRdMaxNI; ++i)
      if (i < a_NI)
        rel[i] = (unsigned)(iw0 + s_sp[i]) < (unsigned)a_W
                     ? s_off[i] + (uint32_t)(iw0 * (CK * 2))
                     : 0x80000000u;
    const int tr = a_P - p0 < a_TR ? a_P - p0 : a_TR;
    const int rows_in = tr + R - 1;
    const int ih0 = p0 - a_pad_h;
    for (int sr = wave; sr < rows_in; sr += kRdWaves) {
      const int ih = ih0 + sr;
      const bool row_ok = (unsigned)ih < (unsigned)a_H;
      const __amdgpu_buffer_rsrc_t rs = row_ok ? rx : rnone;
      const int soff = row_ok ? ((n * a_H + ih) * a_W) * (CK * 2) : 0;
      const uint32_t dst = dst0 + (uint32_t)sr * rowpitch;
#pragma unroll
      for (int i = 0; i < kRdMaxNI; ++i)
        if (i < a_NI)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(
              rs, (GEMM_AS3 char *)__builtin_amdgcn_readfirstlane(dst + i * 1024u),
              16, (int)rel[i], soff, 0, 0);
    }
  };
  if (tile0 < tile_end)
    issue_slab(tile0, buf0);
  RD_STAMP(2);

  int cur = 0; // buffer of the current tile
  for (int tile = tile0; tile < tile_end; tile += tile_step) {
    int n, p0, q0;
    tile_origin(tile, n, p0, q0);
    const int tr = a_P - p0 < a_TR ? a_P - p0 : a_TR;
    const int npix = tr * a_TQ;
    const uint32_t lds_s = cur ? buf1 : buf0;
    const int next = tile + tile_step;
    // this tile's slab has landed, and every wavefront has left the previous
    // tile: its buffer is free for the next tile's rows
    __builtin_amdgcn_s_waitcnt(gemm_wait_imm(0));
    gemm_barrier();
#ifdef RD_PROFILE
    if (iter == 0)
      RD_STAMP(3);
    if (iter == 1)
      RD_STAMP(5);
#endif
    if (next < tile_end)
      issue_slab(next, cur ? buf0 : buf1);

    // outputs of this tile: TQ pixels of CO channels out of every image row
    const __amdgpu_buffer_rsrc_t ro =
        rd_rsrc(g.dx + ((int64_t)(n * a_P + p0) * a_Q + q0) * a_CO * 2,
                (uint32_t)((tr - 1) * a_Q + a_TQ) * (uint32_t)a_CO * 2u);
    const uint32_t lane_out = (uint32_t)(ch_wave + 8 * q) * 2u;
    const int nblocks = (npix + 15) >> 4;

    // Slab addresses (one per filter row, this lane's K quarter) and output
    // offset of this lane's pixel of block b.
    auto block_setup = [&](int b, uint32_t (&base)[R], uint32_t &ooff) __attribute__((always_inline)) {
      const int pl = b * 16 + px;
      const int plc = pl < npix ? pl : npix - 1;
      const int prow = (int)conv_div(plc, a_TQ, a_magic_q);
      const int pcol = plc - prow * a_TQ;
      base[0] = lds_s + (uint32_t)prow * rowpitch + (uint32_t)pcol * PITCH + (uint32_t)q * 16u;
#pragma unroll
      for (int r = 1; r < R; ++r)
        base[r] = base[r - 1] + rowpitch;
      ooff = pl < npix ? (uint32_t)(prow * a_Q + pcol) * (uint32_t)a_CO * 2u + lane_out
                       : 0x80000000u;
    };
    u32x4 frag[RING];
    auto fetch = [&](auto jc, const uint32_t (&base)[R], u32x4 &dst) __attribute__((always_inline)) {
      constexpr int j = decltype(jc)::value;
      constexpr int tap = j / KPT, part = j % KPT;
      constexpr int r = tap / S, s = tap % S;
      rd_read_b128<s * PITCH + part * 64>(dst, base[r]);
    };
    f32x4 acc[2];
    uint32_t base[R], nbase[R], ooff, nooff;
    // The K-steps of the block at `base`.  Step j fetches the fragment of step
    // j + RING - 1; the first RING - 1 fragments of the NEXT block (at `nbase`)
    // are fetched into registers of their own a dozen steps before the end, so
    // that they have landed when the block ends: values that cross the loop's
    // back edge may be copied there, which must not happen to a register a
    // load is still to write.  LDS returns in order, so a step waits until at
    // most `younger` reads issued after its own fragment's are outstanding.
    u32x4 nfrag[NFE];
    auto ksteps = [&]() __attribute__((always_inline)) {
      gemm_static_for<NK>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        constexpr int ahead = j + RING - 1;
        if constexpr (ahead < NK)
          fetch(std::integral_constant<int, ahead>{}, base, frag[ahead % RING]);
        if constexpr (j >= NF0 && j < NF0 + 2 * NFE && (j - NF0) % 2 == 0)
          fetch(std::integral_constant<int, (j - NF0) / 2>{}, nbase, nfrag[(j - NF0) / 2]);
        // reads issued after this step's fragment's: the regular ones of the
        // steps since, and the early ones issued at steps j - (RING - 1) .. j
        constexpr int regular = NK - 1 - j < RING - 1 ? NK - 1 - j : RING - 1;
        constexpr int early = [] {
          int n = 0;
          for (int k = 0; k < NFE; ++k) {
            const int st = NF0 + 2 * k;
            n += (st >= j - (RING - 1) && st <= j) ? 1 : 0;
          }
          return n;
        }();
        static_assert(regular + early <= 15, "lgkmcnt is a 4-bit field");
        rd_wait_lgkm<regular + early>(frag[j % RING]);
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          acc[t] = rd_mfma<KIND>(filt[j][t], frag[j % RING],
                                 j == 0 ? f32x4{0.f, 0.f, 0.f, 0.f} : acc[t]);
        }
        // (keeps the step's MFMAs at its reads: with registers to spare the
        // compiler would otherwise gather all reads of a block in front of all
        // its MFMAs, or put off the second tile's MFMAs to the block's end, and
        // nothing would overlap.  The empty statement orders both accumulators
        // among the reads, which are volatile as well.)
        asm volatile("" : "+a"(acc[0]), "+a"(acc[1]));
        __builtin_amdgcn_sched_barrier(0);
      });
      // every read has returned (the early ones long ago)
      gemm_static_for<NFE>([&](auto kc) {
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(nfrag[decltype(kc)::value]));
        frag[decltype(kc)::value] = nfrag[decltype(kc)::value];
      });
    };
    // rounding and the 16-byte store of a finished block
    auto finish = [&](uint32_t off) __attribute__((always_inline)) {
      typedef float f2 __attribute__((ext_vector_type(2)));
      uint32_t w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const f2 pair = {acc[i >> 1][2 * (i & 1)], acc[i >> 1][2 * (i & 1) + 1]};
        if constexpr (KIND == GK_BF16) {
          typedef __bf16 b2 __attribute__((ext_vector_type(2)));
          w[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, b2));
        } else {
          typedef _Float16 h2 __attribute__((ext_vector_type(2)));
          w[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, h2));
        }
      }
      __builtin_amdgcn_raw_buffer_store_b128(u32x4{w[0], w[1], w[2], w[3]}, ro, (int)off, 0, 19);
    };

    // This wavefront's blocks: b0, b0 + 2, ... with b0 = half on even tiles of
    // the workgroup and 1 - half on odd ones, so that the odd block of a tile
    // falls to either pair of wavefronts in turn.  (A block index past the last
    // one addresses the last pixel and stores nothing.)
    int b = half ^ cur;
    block_setup(b, base, ooff);
    gemm_static_for<RING - 1>(
        [&](auto jc) { fetch(jc, base, frag[decltype(jc)::value]); });
    for (; b < nblocks; b += 2) {
      block_setup(b + 2, nbase, nooff);
      ksteps();
      const uint32_t done_off = ooff;
#pragma unroll
      for (int r = 0; r < R; ++r)
        base[r] = nbase[r];
      ooff = nooff;
      finish(done_off);
    }
    // the fragments fetched ahead for a block that does not exist
    __builtin_amdgcn_s_waitcnt(gemm_wait_imm(63));
    cur ^= 1;
#ifdef RD_PROFILE
    if (iter == 0)
      RD_STAMP(4);
    ++iter;
#endif
  }
#ifdef RD_PROFILE
  RD_STAMP(6);
  __builtin_amdgcn_s_waitcnt(gemm_wait_imm(0));
  if (blockIdx.x == 0 && l < 8)
    ((uint64_t *)g.dx)[wave * 8 + l] = st[l < 7 ? l : 7];
#endif
}

struct RdPlan {
  bool ok = false;
  int kind = 0;
  RfDgradArgs a{};
  int lds = 0;
  int grid = 0;
};

bool rd_channels_last(const fhip_tensor_desc &t) {
  int64_t expect = 1;
  int order[FHIP_MAX_RANK];
  int n = 0;
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

constexpr int kRdCK = 128, kRdR = 3, kRdS = 3;

RdPlan make_rd_plan(const fhip_conv_desc *d, int num_cus) {
  RdPlan p;
  const FhipKnobs &knobs = fhip_knobs();
  if (knobs.dgrad_rf == 0)
    return p;
  if (d->spatial_rank != 2 || d->x.rank != 4 || d->epilogue.count != 0)
    return p;
  const int dt = d->y.dtype;
  if (dt == FHIP_BFLOAT16)
    p.kind = GK_BF16;
  else if (dt == FHIP_HALF)
    p.kind = GK_F16;
  else
    return p;
  if (d->x.dtype != dt || d->w.dtype != dt)
    return p;
  const int64_t CO = d->x.dim[1], K = d->w.dim[0];
  if (d->w.dim[1] != CO || CO % kRdChannels != 0 || K != kRdCK ||
      d->w.dim[2] != kRdR || d->w.dim[3] != kRdS)
    return p;
  for (int i = 0; i < 2; ++i)
    if (d->stride[i] != 1 || d->dilation[i] != 1 || d->padding[i] > kRdR - 1)
      return p;
  if (!rd_channels_last(d->x) || !rd_channels_last(d->w) || !rd_channels_last(d->y))
    return p;
  RfDgradArgs &a = p.a;
  a.N = (int32_t)d->y.dim[0], a.H = (int32_t)d->y.dim[2], a.W = (int32_t)d->y.dim[3];
  a.P = (int32_t)d->x.dim[2], a.Q = (int32_t)d->x.dim[3];
  a.CO = (int32_t)CO;
  a.pad_h = kRdR - 1 - (int32_t)d->padding[0];
  a.pad_w = kRdS - 1 - (int32_t)d->padding[1];
  if (a.P != a.H + 2 * a.pad_h - kRdR + 1 || a.Q != a.W + 2 * a.pad_w - kRdS + 1)
    return p;
  const int64_t dy_bytes = (int64_t)a.N * a.H * a.W * kRdCK * 2;
  const int64_t w_bytes = K * kRdR * kRdS * CO * 2;
  if (dy_bytes >= (1ll << 31) || w_bytes >= (1ll << 31) ||
      (int64_t)a.P * a.Q * CO * 2 >= (1ll << 31) || d->x.dim[0] != d->y.dim[0])
    return p;
  a.dy_bytes = (uint32_t)dy_bytes;
  a.w_bytes = (uint32_t)w_bytes;
  using G = RdGeom<kRdCK, kRdR, kRdS>;
  // two slab buffers, under the filter stage until the filter is in registers
  const int64_t lds_total = 160 * 1024;
  auto lds_of = [&](int tr, int ni) {
    const int64_t slab = (int64_t)(tr + kRdR - 1) * ni * 1024;
    return 2 * slab > G::kStageBytes ? 2 * slab : (int64_t)G::kStageBytes;
  };
  // Tile = TR output rows x TQ output columns (Q = TQ * ctiles): the split
  // that fills whole rounds of the machine best.  Time of a round ~ the blocks
  // of the busier wavefront of a pair plus a share that grows with the slab
  // bytes a tile loads (measured on N32 56 x 56 with full-width tiles: 2 rows
  // per tile 24.8 us, 3 rows 25.9 us, 1 row 28.7 us).
  const int cus = num_cus > 0 ? num_cus : 256;
  const int kgroups = (int)(CO / kRdChannels);
  double best = 0;
  int best_tr = 0, best_ct = 1;
  for (int ct = 1; ct <= 4; ct *= 2) {
    if (a.Q % ct != 0)
      continue;
    const int tq = a.Q / ct;
    const int ni = ((tq + kRdS - 1) * G::kCPP + 63) / 64;
    if (ni > kRdMaxNI || (ct > 1 && tq < 16))
      continue;
    for (int tr = 1; tr <= a.P; ++tr) {
      if (lds_of(tr, ni) > lds_total)
        break;
      const int64_t tiles = (int64_t)a.N * ((a.P + tr - 1) / tr) * ct * kgroups;
      const int64_t rounds = (tiles + cus - 1) / cus;
      const int64_t blocks = ((int64_t)tr * tq + 15) / 16;
      const double cost =
          (double)rounds * ((blocks + 1) / 2 * 2 * 16 + 2 * (tr + kRdR - 1) * ni);
      const double eff = (double)a.N * a.P * a.Q * kgroups / (cost * cus);
      if (eff > best + 1e-9) {
        best = eff;
        best_tr = tr;
        best_ct = ct;
      }
    }
  }
  if (knobs.dgrad_rf > 0) {
    // rows per tile, and column tiles in the hundreds: 207 = 7 rows, 2 column tiles
    const int tr = knobs.dgrad_rf % 100, ct = knobs.dgrad_rf >= 100 ? knobs.dgrad_rf / 100 : 1;
    if (tr >= 1 && tr <= a.P && ct >= 1 && a.Q % ct == 0) {
      const int ni = ((a.Q / ct + kRdS - 1) * G::kCPP + 63) / 64;
      if (ni <= kRdMaxNI && lds_of(tr, ni) <= lds_total)
        best_tr = tr, best_ct = ct;
    }
  }
  if (best_tr == 0)
    return p;
  // small problems that leave most of the machine idle stay with the tiled kernels
  if (best < 0.3 && knobs.dgrad_rf < 0)
    return p;
  a.TR = best_tr;
  a.ctiles = best_ct;
  a.TQ = a.Q / best_ct;
  a.NI = ((a.TQ + kRdS - 1) * G::kCPP + 63) / 64;
  a.tiles_per_image = (a.P + a.TR - 1) / a.TR;
  a.ntiles = a.N * a.tiles_per_image * a.ctiles;
  a.kgroups = kgroups;
  a.magic_q = conv_magic(a.TQ);
  p.lds = (int)lds_of(a.TR, a.NI);
  const int64_t items = (int64_t)a.ntiles * kgroups;
  const int64_t slots =
      (int64_t)cus / kgroups * kgroups > 0 ? (int64_t)cus / kgroups * kgroups : kgroups;
  p.grid = (int)(items < slots ? items : slots);
  p.ok = true;
  return p;
}

template <int KIND> int rd_launch(fhip_ctx *ctx, const RdPlan &p) {
  auto kernel = conv_rf_dgrad_kernel<KIND, kRdCK, kRdR, kRdS>;
  static FhipOncePerDevice configured;
  if (!configured.done(ctx->device)) {
    FHIP_HIP_CHECK(ctx, hipFuncSetAttribute(
                            reinterpret_cast<const void *>(kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize,
                            160 * 1024));
    configured.mark(ctx->device);
  }
  hipLaunchKernelGGL(kernel, dim3((unsigned)p.grid), dim3(kRdThreads), p.lds,
                     ctx->stream, p.a);
  FHIP_HIP_CHECK(ctx, hipGetLastError());
  fhip_note_kernel(ctx, "conv_rf_dgrad rows=%d cols=%d", p.a.TR, p.a.TQ);
  return 0;
}

} // namespace

bool fhip_fast_conv_dgrad_rf_applicable(const fhip_conv_desc *d) {
  return make_rd_plan(d, 256).ok;
}

int fhip_fast_conv_dgrad_rf(fhip_ctx *ctx, const fhip_conv_desc *d,
                            const void *dy, const void *w, void *dx) {
  // planned for 256 compute units, like the applicability query that the
  // caller went by: on a device or partition of another size the tile choice
  // must not flip between the two (the grid runs anywhere)
  RdPlan p = make_rd_plan(d, 256);
  FHIP_REQUIRE(ctx, p.ok,
               "conv: descriptor not supported by the register-filter data gradient");
  FHIP_REQUIRE(ctx, ((uintptr_t)dy & 15) == 0 && ((uintptr_t)w & 15) == 0 &&
                        ((uintptr_t)dx & 15) == 0,
               "conv: DY, W and DX must be 16-byte aligned");
  p.a.dy = (const char *)dy;
  p.a.w = (const char *)w;
  p.a.dx = (char *)dx;
  return p.kind == GK_BF16 ? rd_launch<GK_BF16>(ctx, p) : rd_launch<GK_F16>(ctx, p);
}
