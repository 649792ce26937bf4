// Convolution forward with the filter held in registers.
//
// For channels-last tensors with unit stride and unit dilation and a filter
// small enough that a 32-channel slice of it fits a wavefront's registers
// (R * S * C <= 640: the 3 x 3 x 64 family), the whole problem is one pass:
//
//   * a workgroup (8 wavefronts, two per SIMD) owns TR output rows of one
//     image and 128 output channels; the wavefronts w and w + 4 share 32 of
//     those channels, both keep that 32 x (R*S*C) filter slice in registers as
//     ready-made MFMA A operands for the kernel's whole life (staged once
//     through LDS, all of it at once -- one part in a stage of its own, the
//     other where the slab will be -- by LDS-DMA instructions that each cover
//     eight whole 128-byte lines of filter rows), and they draw blocks of 16
//     pixels from a counter they share;
//   * the tile's input rows plus halo go into LDS once, by LDS-DMA, into a
//     zero-padded image (W + S - 1 pixels per row, rows above / below the image
//     as zeros) with a pixel pitch of C * 2 + 16 bytes: every filter tap is then
//     a constant byte offset from an output pixel's slab address, no border
//     masks exist, and the pitch keeps the 16-byte fragment reads of 16
//     consecutive pixels on distinct banks;
//   * the product is computed transposed, OUT^T[channel, pixel] = W . X^T, with
//     v_mfma_f32_16x16x32: the pixels' B fragments are one ds_read_b128 per 16
//     pixels and K-step, feeding two MFMAs (the wavefront's two 16-channel
//     tiles).  A lane then holds 8 consecutive output channels of one pixel:
//     bias / scale / ReLU run on the accumulators and the result leaves with
//     one 16-byte store per lane, no trip through LDS;
//   * the fragments run through a ring of registers a few K-steps ahead of the
//     MFMAs, across block boundaries, and a block's epilogue and store are
//     issued while the SIMD's other wavefront keeps the matrix pipe busy.
//
// Grouped convolutions of 64 -> 64 channels per group run on the same kernel
// with two groups per workgroup: the slab holds both groups' input channels
// of a pixel and a wavefront reads the half of its channel slice's group.
//
// Reference semantics: aten.convolution (reference
// support/asm_emitter.h:690-701, node/conv_node.h:38-56) followed by the fused
// pointwise chain (support/asm_emitter.h:1806-2122).
#include "common.h"
#include "fast_paths.h"
#include "gemm_kernel.h"

#ifdef RF_PROFILE // experiment builds (-DRF_PROFILE=<workgroup>): cycle stamps per wavefront
__device__ uint64_t rf_prof[8 * 48];
#define RF_STAMP(i)                                                            \
  do {                                                                         \
    if (blockIdx.x == RF_PROFILE && (threadIdx.x & 63) == 0 && (i) < 48)       \
      rf_prof[(threadIdx.x >> 6) * 48 + (i)] = __builtin_amdgcn_s_memtime();   \
  } while (0)
extern "C" int fhip_debug_rf_prof(unsigned long long *out) {
  return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(rf_prof), sizeof(rf_prof));
}
#else
#define RF_STAMP(i)                                                            \
  do {                                                                         \
  } while (0)
#endif

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kRfWaves = 8;      // two per SIMD
constexpr int kRfThreads = kRfWaves * 64;
constexpr int kRfMaxNI = 16;     // KB of LDS per slab row, at most

// s_waitcnt immediate: lgkmcnt <= n, the other counters untouched
constexpr int rf_wait_lgkm_imm(int n) { return 0xF | (0x7 << 4) | (n << 8) | (0x3 << 14); }

// Compile-time geometry shared by the kernel and the host's LDS budget.
// GW: groups of the convolution that a workgroup's 128 output channels span
// (1, or 2 groups of 64 -> 64 channels: the slab then holds both groups' C
// input channels of a pixel, and a channel slice reads its group's half).
// SL: channel slices of 32 output channels per workgroup.  4: two wavefronts
// per slice, the filter staged in two parts (one in front of the slab, one in
// its place).  2: four wavefronts per slice and 64 output channels per
// workgroup -- half the filter to bring in per workgroup, all of it staged at
// once where the slab will be, and twice the tiles, which run in pairs that
// share their halo rows in LDS.
template <int C, int R, int S, int GW = 1, int SL = 4> struct RfGeom {
  static constexpr int kCS = C * GW;            // input channels of a slab pixel
  static constexpr int kCPP = kCS * 2 / 16 + 1; // chunks per slab pixel (one is padding)
  static constexpr int kNK = R * S * (C / 32);  // K-steps of 32 channels
  static constexpr int kNKA = SL == 2 ? kNK : kNK / 4 * 2; // K-steps of the first stage
  // filter stages: per channel slice two KB per K-step (one per 16-channel tile)
  static constexpr int kStageBytes = SL * kNKA * 2 * 1024;
  static constexpr int kStage2Bytes = SL * (kNK - kNKA) * 2 * 1024; // in the slab's place
};

struct ConvRfArgs {
  const char *x, *w;
  char *out;
  int32_t N, H, W, P, Q;
  int32_t K;               // output channels (of all groups), a multiple of 128
  int32_t x_pitch;         // bytes between pixels of X (all groups' channels)
  int32_t pad_h, pad_w;
  int32_t TR;              // output rows per tile
  int32_t tiles_per_image; // ceil(P / TR)
  int32_t ntiles;          // N * tiles_per_image
  int32_t kgroups;         // K / 128
  int32_t NI;              // 1 KB LDS-DMA instructions per slab row
  int32_t slab_org;        // LDS byte offset of slab row 0
  int32_t slab_rows;       // slab rows that fit LDS from there
  int32_t first_row;       // slab row of a workgroup's first tile (clear of the filter stage)
  uint32_t magic_q, magic_ni;
  uint32_t x_bytes, w_bytes;
  int32_t o_dt;
  int32_t unit_scale; // every op of the chain is additive with factor 1
  // linear epilogue before the optional ReLU: per op y = mul ? y * o : a * y + b * o
  int32_t nops;
  float lin_a[FHIP_MAX_EPILOGUE], lin_b[FHIP_MAX_EPILOGUE];
  int32_t lin_mul[FHIP_MAX_EPILOGUE];
  DevEpilogue epi; // operand pointers; stride[2] = per-channel step
};

template <int KIND>
__device__ __forceinline__ f32x4 rf_mfma(const u32x4 &a, const u32x4 &b,
                                         const f32x4 &c) {
  if constexpr (KIND == GK_BF16)
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(
        __builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(
        __builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t rf_rsrc(const void *base,
                                                          uint32_t bytes) {
  const uint64_t b64 = (uint64_t)base;
  const uint32_t blo = __builtin_amdgcn_readfirstlane((uint32_t)b64);
  const uint32_t bhi = __builtin_amdgcn_readfirstlane((uint32_t)(b64 >> 32));
  return __builtin_amdgcn_make_buffer_rsrc(
      (void *)(((uint64_t)bhi << 32) | blo), 0,
      (int)__builtin_amdgcn_readfirstlane(bytes), 0x00020000);
}

template <int KIND, int C, int R, int S, bool RELU, bool UNIT, int GW, int SL>
__global__ __launch_bounds__(kRfThreads)
__attribute__((amdgpu_waves_per_eu(2, 2))) void
conv_rf_kernel(ConvRfArgs g) {
  static_assert(SL == 4 || (SL == 2 && GW == 1), "slices per workgroup");
  using Geom = RfGeom<C, R, S, GW, SL>;
  constexpr int MEMBERS = kRfWaves / SL; // wavefronts that share a channel slice
  // scalar arguments as locals (only the loop over the epilogue table indexes
  // the argument block at run time)
  const int a_Q = g.Q;
  const int a_kgroups = g.kgroups;
  const int a_TR = g.TR;
  const int a_P = g.P;
  const int a_NI = g.NI;
  const int a_K = g.K;
  const int a_tiles_per_image = g.tiles_per_image;
  const int a_ntiles = g.ntiles;
  const int a_W = g.W;
  const int a_H = g.H;
  const int a_pad_w = g.pad_w;
  const int a_pad_h = g.pad_h;
  const uint32_t a_magic_q = g.magic_q;
  const uint32_t a_x_bytes = g.x_bytes;
  const uint32_t a_w_bytes = g.w_bytes;
  const int a_nops = g.nops;
  constexpr int CPP = Geom::kCPP; // 16-byte chunks per slab pixel
  constexpr int CS = Geom::kCS;   // input channels of a slab pixel
  constexpr int PITCH = CPP * 16;
  constexpr int KPT = C / 32;                // K-steps per filter tap
  constexpr int NK = Geom::kNK;   // K-steps
  constexpr int NKA = Geom::kNKA; // K-steps of the filter's first part
  // fragment buffers (K-steps in flight); a divisor of NK, so that a block's
  // K-step j always sits in buffer j % RING
  constexpr int RING = NK % 6 == 0 ? 6 : (NK % 4 == 0 ? 4 : 3);
  constexpr int FROW = R * S * C * 2;        // bytes of a filter row
  static_assert(C % 64 == 0 && NK % RING == 0 && NKA % 2 == 0, "filter shape outside this kernel");
  static_assert((S - 1) * PITCH + (GW - 1) * C * 2 + (KPT - 1) * 64 + 48 < 65536, "ds offset range");

  extern __shared__ __attribute__((aligned(16))) char smem[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  // 32 output channels per slice; the wavefronts of a slice sit on one SIMD
  // (w and w + 4) or two
  const int slice = wave & (SL - 1);
  const int half = wave / SL; // which of the slice's wavefronts: its first block, its share of the filter
  const int l = threadIdx.x & 63;
  const int px = l & 15, q = l >> 4;
  const uint32_t rowpitch = (uint32_t)a_NI * 1024u;
  // LDS: [block counters, 1 KB | filter stage | rest of the filter]; the slab
  // is a grid of rows over all of it above the counters, a workgroup's first
  // tile in the rows behind the filter stage (in the place of the filter's
  // second part, which has left LDS by then)
  const uint32_t lds_f = lds0 + 1024u + (uint32_t)slice * (NKA * 2 * 1024);
  const uint32_t lds_b = lds0 + 1024u + Geom::kStageBytes;
  const uint32_t slab_org = lds0 + (uint32_t)g.slab_org;
  const int a_slab_rows = g.slab_rows;

  // this workgroup's channel group stays fixed; it takes a run of consecutive
  // tiles (consecutive row bands of an image share their halo rows in LDS)
  const int kg = (int)(blockIdx.x % (unsigned)a_kgroups);
  const int wg = (int)(blockIdx.x / (unsigned)a_kgroups);
  const int nwg = (int)(gridDim.x / (unsigned)a_kgroups);
  const int tile_end = (int)(((int64_t)(wg + 1) * a_ntiles) / nwg);
  int tile = (int)(((int64_t)wg * a_ntiles) / nwg);
  const int ch_wave = kg * (SL * 32) + slice * 32;
  RF_STAMP(0);

  // ---- filter slice -> registers, through LDS --------------------------------
  // MFMA row rho of tile t is output channel ch_wave + 8 * (rho / 4) + 4 * t +
  // rho % 4, so that a lane's 8 results (rows 4 q .. 4 q + 3 of both tiles) are
  // 8 consecutive channels.  K-step j covers the 64 bytes at j * 64 of a
  // channel's R * S * C run; MFMA lane (rho, kq) takes the 16 bytes of K
  // quarter kq.  Loading those straight into registers would touch four cache
  // lines per lane quad (adjacent lanes are adjacent rho: rows FROW bytes
  // apart), so the fragments go through LDS: per (pair of K-steps, tile) two
  // LDS-DMA instructions, one per eight MFMA rows, each fetching the 128
  // contiguous bytes that the pair covers of its eight filter rows.  The two
  // wavefronts of a slice stage one tile each and both read all fragments.
  // The pair is the instructions' scalar offset (the immediate offset would
  // also move the LDS destination), so there is no address arithmetic per
  // instruction.
  u32x4 filt[NK][2];
  const __amdgpu_buffer_rsrc_t rw = rf_rsrc(g.w, a_w_bytes);
  // DMA lane d of the instruction for (K-step pair jp, row half h) carries
  // MFMA row 8 h + d / 8 and the 16-byte chunk (d % 8) ^ (d / 16 | 4 h) of the
  // 128 bytes at jp * 128 of that row: eight whole lines per instruction.  The
  // MFMA lane (rho, kq) of K-step 2 jp + jo finds its chunk jo * 4 + kq at
  // position ((jo ^ h) * 4 + (kq ^ (rho % 8 / 2))) of its row's eight: the 16
  // lanes of a quarter wavefront then read 16 different bank groups.
  // The wavefronts of a slice share the staging: of two, each takes one tile
  // (both row halves); of four, each takes one row half of one tile.
  constexpr int NH = MEMBERS == 2 ? 2 : 1; // row halves this wavefront stages
  const int ftile = MEMBERS == 2 ? half : (half & 1);
  uint32_t fvoff[NH];
  int fh[NH];
#pragma unroll
  for (int i = 0; i < NH; ++i) {
    const int h = MEMBERS == 2 ? i : (half >> 1);
    const int r8 = l >> 3, cpos = l & 7;
    const int rho = 8 * h + r8;
    const int chunk = cpos ^ ((r8 >> 1) | (h << 2));
    const int ch = ch_wave + 8 * (rho >> 2) + 4 * ftile + (rho & 3);
    fvoff[i] = (uint32_t)ch * (uint32_t)FROW + (uint32_t)chunk * 16u;
    fh[i] = h;
  }
  const uint32_t lds_f2 = lds_b + (uint32_t)slice * ((NK - NKA) * 2 * 1024);
  uint32_t fread[2]; // per K-step parity, relative to the stage of the slice
#pragma unroll
  for (int jo = 0; jo < 2; ++jo) {
    const int h = px >> 3, r8 = px & 7;
    fread[jo] = (uint32_t)(h * 1024 + (r8 * 8 + ((jo ^ h) * 4 + (q ^ (r8 >> 1)))) * 16);
  }
  auto filter_dma = [&](auto j0c, auto j1c, uint32_t stage) __attribute__((always_inline)) {
    constexpr int J0 = decltype(j0c)::value, J1 = decltype(j1c)::value;
    gemm_static_for<(J1 - J0) / 2>([&](auto dc) {
      constexpr int jp = decltype(dc)::value;
#pragma unroll
      for (int i = 0; i < NH; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rw,
            (GEMM_AS3 char *)__builtin_amdgcn_readfirstlane(
                stage + (uint32_t)((jp * 2 + ftile) * 2048 + fh[i] * 1024)),
            16, (int)fvoff[i], (J0 / 2 + jp) * 128, 0, 0);
    });
  };
  auto filter_read = [&](auto j0c, auto j1c, uint32_t from) __attribute__((always_inline)) {
    constexpr int J0 = decltype(j0c)::value, J1 = decltype(j1c)::value;
    gemm_static_for<J1 - J0>([&](auto dc) {
      constexpr int j = J0 + decltype(dc)::value;
      constexpr int jp = (j - J0) / 2, jo = j % 2;
#pragma unroll
      for (int t = 0; t < 2; ++t)
        filt[j][t] = *(const GEMM_AS3 u32x4 *)(uintptr_t)(
            from + fread[jo] + (uint32_t)((jp * 2 + t) * 2048));
    });
  };
  using JA0 = std::integral_constant<int, 0>;
  using JA1 = std::integral_constant<int, NKA>;
  using JB1 = std::integral_constant<int, NK>;
  // Both parts are requested at once: the first into the stage, the second
  // into the slab's place (the slab is loaded after the filter has left LDS).
  filter_dma(JA0{}, JA1{}, lds_f);
  filter_dma(JA1{}, JB1{}, lds_f2);
  RF_STAMP(14);

  const __amdgpu_buffer_rsrc_t rx = rf_rsrc(g.x, a_x_bytes);
  const __amdgpu_buffer_rsrc_t rnone = rf_rsrc(g.x, 0); // every lane out of range
  float sc[8], sh[8];
  f32x4 acc0[2];

  // ---- slab: rows of NI KB by LDS-DMA; wavefront w carries the KBs w and w + 8
  // of every row.  LDS chunk x = i * 64 + lane of a slab row is chunk x % CPP of
  // slab pixel x / CPP, i.e. input column x / CPP - pad_w; the padding chunk,
  // columns outside the image and the tail of the row's last KB read as
  // zeros.  The lane offsets are the same for every row, the row is the
  // instructions' scalar offset.
  uint32_t rel[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int xk = (wave + 8 * i) * 64 + l;
    const int sp = (xk * (65536 / CPP + 1)) >> 16; // xk / CPP for xk < 2^12
    const int c = xk - sp * CPP;
    const int iw = sp - a_pad_w;
    const bool ok = c < CPP - 1 && (unsigned)iw < (unsigned)a_W;
    rel[i] = ok ? (uint32_t)(iw * g.x_pitch + (GW > 1 ? kg * (CS * 2) : 0) + c * 16)
                : 0x80000000u;
  }
  const int npr = wave + 8 < a_NI ? 2 : (wave < a_NI ? 1 : 0); // instructions per row
  // `count` input rows from row ih0 of image n into the slab rows from `row`
  auto slab_rows = [&](int count, int n, int ih0, int row) __attribute__((always_inline)) {
    for (int sr = 0; sr < count; ++sr) {
      const int ih = ih0 + sr;
      const bool row_ok = (unsigned)ih < (unsigned)a_H;
      const __amdgpu_buffer_rsrc_t rs = row_ok ? rx : rnone;
      const int soff = row_ok ? ((n * a_H + ih) * a_W) * g.x_pitch : 0;
      const uint32_t dst = slab_org + (uint32_t)(row + sr) * rowpitch + (uint32_t)wave * 1024u;
      if (npr > 0)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rs, (GEMM_AS3 char *)__builtin_amdgcn_readfirstlane(dst), 16, (int)rel[0], soff, 0, 0);
      if (npr > 1)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rs, (GEMM_AS3 char *)__builtin_amdgcn_readfirstlane(dst + 8192u), 16, (int)rel[1],
            soff, 0, 0);
    }
  };

  // block counters of the slice (one per tile parity), in the KB at the bottom of LDS
  const uint32_t draw0 = lds0 + (uint32_t)slice * 8u;
  uint32_t draw = draw0;
  auto draw_block = [&]() __attribute__((always_inline)) {
    // one LDS atomic of lane 0; the result is in flight when this returns (the
    // compiler does not know: the reader waits by count, LDS answers in order)
    uint32_t v;
    uint64_t saved;
    asm volatile("s_mov_b64 %1, exec\n\t"
                 "s_mov_b64 exec, 1\n\t"
                 "ds_add_rtn_u32 %0, %2, %3\n\t"
                 "s_mov_b64 exec, %1"
                 : "=&v"(v), "=&s"(saved)
                 : "v"(draw), "v"(1u)
                 : "memory");
    return v;
  };
  // image, first output row, output rows and first input row of a tile
  auto tile_geom = [&](int t, int &n, int &p0, int &tr, int &ih0) __attribute__((always_inline)) {
    n = t / a_tiles_per_image;
    p0 = (t - n * a_tiles_per_image) * a_TR;
    tr = a_P - p0 < a_TR ? a_P - p0 : a_TR;
    ih0 = p0 - a_pad_h;
  };
  int n, p0, tr, ih0;
  tile_geom(tile, n, p0, tr, ih0);
  int srow = g.first_row; // the tile's first slab row

  {
    RF_STAMP(15);
    // ---- epilogue constants: y = acc * sc[c] + sh[c] for the lane's 8 channels
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      sc[c] = 1.f;
      sh[c] = 0.f;
    }
    for (int e = 0; e < a_nops; ++e) {
      const DevEpiOp &o = g.epi.op[e];
      // the 8 operand values of an op are fetched by loads issued back to back
      float ovs[8];
#pragma unroll
      for (int c = 0; c < 8; ++c)
        ovs[c] = o.kind == FHIP_OPERAND_SCALAR ? o.scalar : 0.f;
      if (o.kind == FHIP_OPERAND_TENSOR) {
        int64_t off[8];
#pragma unroll
        for (int c = 0; c < 8; ++c)
          off[c] = (int64_t)(ch_wave + 8 * q + c) * o.stride[2];
        load_operand_vec<8>(o.ptr, o.operand_dtype, off, ovs);
      }
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        const float ov = ovs[c];
        if (g.lin_mul[e]) {
          sc[c] *= ov;
          sh[c] *= ov;
        } else {
          sc[c] *= g.lin_a[e];
          sh[c] = sh[c] * g.lin_a[e] + g.lin_b[e] * ov;
        }
      }
    }
    // with unit scales (UNIT: the host found every op additive with factor
    // 1) the shift is the accumulators' start value and the multiply-add
    // drops out of the epilogue
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        acc0[t][i] = UNIT ? sh[4 * t + i] : 0.f;
    RF_STAMP(1);
    __builtin_amdgcn_s_waitcnt(gemm_wait_imm(0));
    RF_STAMP(2);
    gemm_barrier();
    RF_STAMP(3);
    if constexpr (SL == 2) {
      // the whole filter leaves LDS, then the slab takes its place
      filter_read(JA0{}, JA1{}, lds_f);
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_waitcnt(gemm_wait_imm(63));
      RF_STAMP(6);
      gemm_barrier();
      slab_rows(tr + R - 1, n, ih0, srow);
      RF_STAMP(7);
    } else {
      // the second part leaves the slab's place first; the first part is read
      // while the slab's loads are in flight
      filter_read(JA1{}, JB1{}, lds_f2);
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_waitcnt(gemm_wait_imm(63));
      RF_STAMP(6);
      gemm_barrier();
      slab_rows(tr + R - 1, n, ih0, srow);
      RF_STAMP(7);
      filter_read(JA0{}, JA1{}, lds_f);
    }
    // the wavefronts of a slice draw their blocks from a counter (the first
    // ones are dealt out): the SIMD serves its older wavefront first, so
    // equal shares would leave the younger one to finish alone
    if (half == 0 && l == 0)
      *(GEMM_AS3 uint32_t *)(uintptr_t)draw = (uint32_t)MEMBERS;
    __builtin_amdgcn_s_waitcnt(gemm_wait_imm(0));
    RF_STAMP(9);
    gemm_barrier();
    RF_STAMP(10);
  }

  for (;;) {
    const int npix = tr * a_Q;
    const uint32_t lds_s = slab_org + (uint32_t)srow * rowpitch;
    RF_STAMP(16 + 4 * (tile - tile_end + 8)); // (profile builds: per tile, the run's last eight)

    // ---- the next tile's rows are requested now and land during this tile's
    // blocks.  Below this tile in the same image it starts on this tile's last
    // R - 1 rows and only the new rows are loaded; otherwise it goes to the
    // slab rows in front of this tile's or behind them, wherever it fits; when
    // it fits nowhere its rows are loaded once this tile is done.
    const bool more = tile + 1 < tile_end;
    int n2 = n, p02 = p0, tr2 = tr, ih02 = ih0, srow2 = 0;
    bool deferred = false;
    if (more) {
      tile_geom(tile + 1, n2, p02, tr2, ih02);
      const int rows_in = tr + R - 1, rows_in2 = tr2 + R - 1;
      int skip = 0;
      if (n2 == n && srow + tr + rows_in2 <= a_slab_rows) {
        srow2 = srow + tr;
        skip = R - 1;
      } else if (srow >= rows_in2) {
        srow2 = 0;
      } else if (srow + rows_in + rows_in2 <= a_slab_rows) {
        srow2 = srow + rows_in;
      } else {
        deferred = true;
      }
      if (!deferred)
        slab_rows(rows_in2 - skip, n2, ih02 + skip, srow2 + skip);
      // the other counter: its last draws were the tile's before this one
      if (half == 0 && l == 0)
        *(GEMM_AS3 uint32_t *)(uintptr_t)(draw ^ 4u) = (uint32_t)MEMBERS;
    }

    // outputs of this tile: dense rows of K channels, pixel index tile-relative
    const __amdgpu_buffer_rsrc_t ro =
        rf_rsrc(g.out + ((int64_t)(n * a_P + p0) * a_Q) * a_K * 2,
                (uint32_t)npix * (uint32_t)a_K * 2u);
    const uint32_t lane_out = (uint32_t)(ch_wave + 8 * q) * 2u;
    const int nblocks = (npix + 15) >> 4;

    // Slab address (filter row 0, this lane's K quarter) and output offset of
    // this lane's pixel of block b.
    auto block_setup = [&](int b, uint32_t &base, uint32_t &ooff) __attribute__((always_inline)) {
      const int pl = b * 16 + px;
      const int plc = pl < npix ? pl : npix - 1;
      const int prow = (int)conv_div(plc, a_Q, a_magic_q);
      const int pcol = plc - prow * a_Q;
      base = lds_s + (uint32_t)prow * rowpitch + (uint32_t)pcol * PITCH + (uint32_t)q * 16u +
             (GW > 1 ? (uint32_t)(slice >> 1) * (C * 2) : 0u);
      ooff = pl < npix ? (uint32_t)pl * (uint32_t)a_K * 2u + lane_out : 0x80000000u;
    };
    u32x4 frag[RING];
    auto fetch = [&](auto jc, uint32_t base) __attribute__((always_inline)) {
      constexpr int j = decltype(jc)::value;
      constexpr int tap = j / KPT, part = j % KPT;
      constexpr int r = tap / S, s = tap % S;
      frag[j % RING] = *(const GEMM_AS3 u32x4 *)(uintptr_t)(
          base + (uint32_t)r * rowpitch + (uint32_t)(s * PITCH + part * 64));
    };
    f32x4 acc[2];
    uint32_t base, ooff, nbase, nooff;
    uint32_t drawn;
    int nb;
    // The K-steps of the block at `base`; the first fragments of the next
    // block (at `nbase`) are fetched during the last steps.
    auto ksteps = [&]() __attribute__((always_inline)) {
      gemm_static_for<NK>([&](auto dc) {
        constexpr int j = decltype(dc)::value;
        constexpr int ahead = j + RING - 1;
        if constexpr (ahead == NK) {
          // the block drawn at the top of this one: j fragment reads have been
          // issued since, so "at most j outstanding" says the draw is back
          // (one statement: nothing may move between the wait and the read)
          asm volatile("s_waitcnt lgkmcnt(%2)\n\t"
                       "v_readfirstlane_b32 %0, %1\n\t"
                       "s_nop 4"
                       : "=s"(nb)
                       : "v"(drawn), "n"(j < 15 ? j : 15));
          block_setup(nb, nbase, nooff);
        }
        if constexpr (ahead < NK)
          fetch(std::integral_constant<int, ahead>{}, base);
        else
          fetch(std::integral_constant<int, ahead - NK>{}, nbase);
#pragma unroll
        for (int t = 0; t < 2; ++t)
          acc[t] = rf_mfma<KIND>(filt[j][t], frag[j % RING], j == 0 ? acc0[t] : acc[t]);
        // (keeps the fragment reads where they are written: RING - 1 K-steps
        // ahead of their MFMAs)
        __builtin_amdgcn_sched_barrier(0);
      });
    };
    // scale / ReLU, rounding and the 16-byte store of a finished block
    auto finish = [&](const float (&yin)[8], uint32_t off) __attribute__((always_inline)) {
      float y[8];
#pragma unroll
      for (int c = 0; c < 8; ++c)
        y[c] = UNIT ? yin[c] : __builtin_fmaf(yin[c], sc[c], sh[c]);
      // (scalar words: bit-casting an element of a vector in place reads
      // element 0)
      uint32_t w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        // one packed round-to-nearest-even conversion per pair (a vector
        // conversion: inline asm here would hide the MFMA -> VALU hazard of
        // its operands from the compiler's hazard handling)
        typedef float f2 __attribute__((ext_vector_type(2)));
        const f2 pair = {y[2 * i], y[2 * i + 1]};
        if constexpr (KIND == GK_BF16) {
          typedef __bf16 b2 __attribute__((ext_vector_type(2)));
          const b2 r = __builtin_convertvector(pair, b2);
          w[i] = __builtin_bit_cast(uint32_t, r);
        } else {
          typedef _Float16 h2 __attribute__((ext_vector_type(2)));
          const h2 r = __builtin_convertvector(pair, h2);
          w[i] = __builtin_bit_cast(uint32_t, r);
        }
        if constexpr (RELU) {
          // max(x, 0) on the rounded pair: as 16-bit integers the negative
          // values (and -0) are exactly the patterns below zero
          typedef short s2 __attribute__((ext_vector_type(2)));
          const s2 v = __builtin_bit_cast(s2, w[i]);
          w[i] = __builtin_bit_cast(uint32_t,
                                    __builtin_elementwise_max(v, s2{0, 0}));
        }
      }
      const u32x4 pk = {w[0], w[1], w[2], w[3]};
      // (sc0 sc1 nt: the output is written once and not read back here;
      // measured 8 % faster end to end than the default write-back policy)
      __builtin_amdgcn_raw_buffer_store_b128(pk, ro, (int)off, 0, 19);
    };

    // This wavefront's blocks: `half`, then whatever it draws (block indices
    // past the last one address the last pixel and store nothing).
    int b = half;
    block_setup(b, base, ooff);
    gemm_static_for<RING - 1>([&](auto jc) {
      fetch(jc, base);
      __builtin_amdgcn_sched_barrier(0); // (in this order: the loop waits for the oldest)
    });
    RF_STAMP(4);
    RF_STAMP(17 + 4 * (tile - tile_end + 8));
    while (b < nblocks) {
      drawn = draw_block();
      ksteps();
      float y[8];
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          y[4 * t + i] = acc[t][i];
      const uint32_t done_off = ooff;
      base = nbase;
      ooff = nooff;
      finish(y, done_off);
      if (b == half)
        RF_STAMP(5);
      b = nb;
    }
    RF_STAMP(12);
    RF_STAMP(18 + 4 * (tile - tile_end + 8));
    if (!more)
      break;
    if (deferred) {
      // every wavefront is done with the slab before the next tile overwrites it
      __builtin_amdgcn_s_waitcnt(gemm_wait_imm(0));
      gemm_barrier();
      slab_rows(tr2 + R - 1, n2, ih02, 0);
    }
    // the next tile's rows are in LDS, and every wavefront has left this tile
    __builtin_amdgcn_s_waitcnt(gemm_wait_imm(0));
    gemm_barrier();
    RF_STAMP(19 + 4 * (tile - tile_end + 8));
    ++tile;
    n = n2, p0 = p02, tr = tr2, ih0 = ih02, srow = srow2;
    draw ^= 4u;
  }
  RF_STAMP(13);
}

struct RfPlan {
  bool ok = false;
  int kind = 0;
  int C = 0, R = 0, S = 0; // C: input channels of a group
  int gw = 1;              // groups per workgroup
  int sl = 4;              // channel slices (of 32 output channels) per workgroup
  bool relu = false;
  ConvRfArgs a{};
  int lds = 0;
  int grid = 0;
};

bool rf_channels_last(const fhip_tensor_desc &t) {
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

// The (C, R, S) instances that are compiled.
bool rf_instance(int C, int R, int S) {
  return C == 64 && R == 3 && S == 3;
}

RfPlan make_rf_plan(const fhip_conv_desc *d, int num_cus) {
  RfPlan p;
  const FhipKnobs &knobs = fhip_knobs();
  if (knobs.conv_rows == 0)
    return p;
  if (d->spatial_rank != 2 || d->x.dtype != d->w.dtype)
    return p;
  if (d->x.dtype == FHIP_BFLOAT16)
    p.kind = GK_BF16;
  else if (d->x.dtype == FHIP_HALF)
    p.kind = GK_F16;
  else
    return p;
  if (d->out.dtype != d->x.dtype) // the element kind also fixes the rounding
    return p;
  if (d->y.dtype != FHIP_FLOAT && !(d->epilogue.count == 0 && d->y.dtype == d->out.dtype))
    return p;
  // C: input channels of a group.  One group, or an even number of groups of
  // 64 -> 64 channels (a workgroup's 128 output channels are then two groups)
  const int64_t Call = d->x.dim[1], C = d->w.dim[1], K = d->w.dim[0];
  if (C <= 0 || Call % C != 0 || K % 64 != 0)
    return p;
  const int64_t groups = Call / C;
  if (groups != 1 && !(groups % 2 == 0 && C == 64 && K == groups * 64))
    return p;
  p.gw = groups == 1 ? 1 : 2;
  const int64_t R = d->w.dim[2], S = d->w.dim[3];
  if (!rf_instance((int)C, (int)R, (int)S))
    return p;
  for (int i = 0; i < 2; ++i)
    if (d->stride[i] != 1 || d->dilation[i] != 1)
      return p;
  if (!rf_channels_last(d->x) || !rf_channels_last(d->w) || !rf_channels_last(d->out))
    return p;
  ConvRfArgs &a = p.a;
  a.N = (int32_t)d->x.dim[0], a.H = (int32_t)d->x.dim[2], a.W = (int32_t)d->x.dim[3];
  a.P = (int32_t)d->y.dim[2], a.Q = (int32_t)d->y.dim[3];
  a.K = (int32_t)K;
  a.pad_h = (int32_t)d->padding[0], a.pad_w = (int32_t)d->padding[1];
  if (a.P != a.H + 2 * a.pad_h - (int)R + 1 || a.Q != a.W + 2 * a.pad_w - (int)S + 1)
    return p;
  const int64_t x_bytes = (int64_t)a.N * a.H * a.W * Call * 2;
  a.x_pitch = (int32_t)(Call * 2);
  const int64_t o_tile_max = (int64_t)a.P * a.Q * K * 2;
  if (x_bytes >= (1ll << 31) || o_tile_max >= (1ll << 31) || K * R * S * C * 2 >= (1ll << 31))
    return p;
  a.x_bytes = (uint32_t)x_bytes;
  a.w_bytes = (uint32_t)(K * R * S * C * 2);
  // epilogue: linear ops with scalar / per-channel operands and f32
  // intermediates, optionally closed by one ReLU
  int nops = d->epilogue.count;
  if (nops > 0 && d->epilogue.op[nops - 1].mode == FHIP_PW_RELU_FWD) {
    p.relu = true;
    --nops;
  }
  {
    GemmArgs tmp{};
    tmp.c_dt = d->y.dtype;
    tmp.o_dt = d->out.dtype;
    for (int i = 0; i < d->epilogue.count; ++i) {
      const fhip_epilogue_op &o = d->epilogue.op[i];
      if (o.operand_kind == FHIP_OPERAND_TENSOR) {
        int64_t st[FHIP_MAX_RANK];
        if (!fhip_broadcast_strides(o.operand, d->y.rank, d->y.dim, st))
          return p;
        // per-channel vectors only
        if ((d->y.dim[0] != 1 && st[0] != 0) || (d->y.dim[2] != 1 && st[2] != 0) ||
            (d->y.dim[3] != 1 && st[3] != 0))
          return p;
        const int dt = o.operand.dtype;
        if (dt != FHIP_FLOAT && dt != FHIP_BFLOAT16 && dt != FHIP_HALF)
          return p;
        tmp.epi.op[i].stride[2] = st[1];
      }
    }
    gemm_fill_linear(d->epilogue, tmp);
    if (!tmp.epi_reg)
      return p;
    a.unit_scale = 1;
    for (int i = 0; i < nops; ++i) {
      if (tmp.lin_relu[i])
        return p; // a ReLU in the middle of the chain
      a.lin_a[i] = tmp.lin_a[i];
      a.lin_b[i] = tmp.lin_b[i];
      a.lin_mul[i] = tmp.lin_mul[i];
      if (tmp.lin_mul[i] || tmp.lin_a[i] != 1.f)
        a.unit_scale = 0;
    }
  }
  a.nops = nops;
  a.o_dt = d->out.dtype;
  // slab geometry
  const int cpp = (int)C * p.gw * 2 / 16 + 1;
  const int wp = a.W + (int)S - 1 + 0; // = W + 2 * pad_w
  if (a.W + 2 * a.pad_w != a.Q + (int)S - 1)
    return p;
  a.NI = ((a.W + 2 * a.pad_w) * cpp + 63) / 64;
  (void)wp;
  if (a.NI > kRfMaxNI)
    return p;
  // LDS: a KB of block counters, the filter stage(s) and the slab.  Four
  // slices: the slab's place first stages the filter's second part, and the
  // slab's rows form a grid anchored so that a row starts right behind the
  // first stage: that row takes a workgroup's first tile, the rows in front of
  // it (over the stage, free once the filter is in registers) serve later
  // tiles.  Two slices: the whole filter is staged where the slab will be.
  const int nk = (int)(R * S * (C / 32));
  const int lds_max = 160 * 1024;
  const int rowpitch = a.NI * 1024;
  const int cus = num_cus > 0 ? num_cus : 256;
  struct Choice {
    int sl = 0, tr = 0;
    double eff = 0;
  } best;
  struct Layout {
    int stage, stage2, first_row, slab_org, rows_max, kgroups;
    int64_t slots;
  };
  auto layout_of = [&](int sl) {
    Layout y;
    const int nka = sl == 2 ? nk : nk / 4 * 2;
    y.stage = sl * nka * 2 * 1024;
    y.stage2 = sl * (nk - nka) * 2 * 1024;
    y.first_row = sl == 2 ? 0 : y.stage / rowpitch;
    y.slab_org = sl == 2 ? 1024 : 1024 + y.stage - y.first_row * rowpitch;
    y.rows_max = (lds_max - y.slab_org) / rowpitch; // slab rows with all of LDS
    y.kgroups = (int)(K / (sl * 32));
    y.slots = (int64_t)cus / y.kgroups * y.kgroups > 0 ? (int64_t)cus / y.kgroups * y.kgroups
                                                      : y.kgroups;
    return y;
  };
  // the work in units of 1/8 of a block of a channel slice on one SIMD, spread
  // over the machine's SIMDs
  const double ideal = (double)a.N * a.P * a.Q / 16.0 * (double)(K / 32) * 8.0 / (cus * 4.0);
  for (int sl = 4; sl >= 2; sl -= 2) {
    if (K % (sl * 32) != 0 || (sl == 2 && p.gw != 1))
      continue;
    if (knobs.conv_slices && knobs.conv_slices != sl)
      continue;
    const Layout y = layout_of(sl);
    const int members = kRfWaves / sl;
    // rows a first tile may have: behind the first stage, or (two slices) all of LDS
    const int first_cap = sl == 2 ? lds_max - 1024 : lds_max - 1024 - y.stage;
    // Cost of a workgroup's run of tiles [t0, t1), same units: the placement
    // rules of the kernel, a tile's blocks on the busiest wavefront of a
    // slice, and the rows loaded for the next tile, which hide behind the
    // blocks unless they had to wait for them.
    auto run_cost = [&](int tr_full, int t0, int t1) {
      const int tpi = (a.P + tr_full - 1) / tr_full;
      // until the first block: the filter's KB, then the first tile's rows
      // (fitted to cycle stamps: 144 KB + 81 KB = 10 k cycles)
      const int rows0 = ((a.P - (t0 % tpi) * tr_full < tr_full ? a.P - (t0 % tpi) * tr_full : tr_full) +
                         (int)R - 1);
      double cost = 0.45 * (sl * nk * 2) + 0.55 * rows0 * a.NI;
      int srow = y.first_row;
      for (int t = t0; t < t1; ++t) {
        const int n = t / tpi, p0 = (t - n * tpi) * tr_full;
        const int tr = a.P - p0 < tr_full ? a.P - p0 : tr_full;
        const int64_t blocks = ((int64_t)tr * a.Q + 15) / 16;
        // (+ 40: requesting the next rows and the barrier, 2.6 k cycles per tile)
        const double compute = (double)((blocks + members - 1) / members * 16 + 40);
        if (t + 1 == t1) {
          cost += compute;
          break;
        }
        const int n2 = (t + 1) / tpi, p02 = (t + 1 - n2 * tpi) * tr_full;
        const int tr2 = a.P - p02 < tr_full ? a.P - p02 : tr_full;
        const int rows_in = tr + (int)R - 1, rows_in2 = tr2 + (int)R - 1;
        int loaded = rows_in2;
        bool deferred = false;
        if (n2 == n && srow + tr + rows_in2 <= y.rows_max) {
          srow += tr;
          loaded = tr2;
        } else if (srow >= rows_in2) {
          srow = 0;
        } else if (srow + rows_in + rows_in2 <= y.rows_max) {
          srow += rows_in;
        } else {
          srow = 0;
          deferred = true;
        }
        // (KB of rows: 1.5 units each behind the blocks, 2.5 when nothing hides them)
        const double kb = (double)loaded * a.NI;
        cost += deferred ? compute + 2.5 * kb : (compute > 1.5 * kb ? compute : 1.5 * kb);
      }
      return cost;
    };
    for (int tr = 1; tr <= a.P; ++tr) {
      if ((tr + (int)R - 1) * rowpitch > first_cap)
        break;
      const int64_t ntiles = (int64_t)a.N * ((a.P + tr - 1) / tr);
      if (ntiles >= (1 << 24))
        continue;
      const int64_t items = ntiles * y.kgroups;
      const int64_t nwg = (items < y.slots ? items : y.slots) / y.kgroups;
      // the longest runs: the first workgroup with a run of the larger size,
      // from its first tile (the runs differ in where they meet image borders)
      double cost = 0;
      const int64_t probes[3] = {0, nwg / 2, nwg - 1};
      for (int64_t wi : probes) {
        const double c = run_cost(tr, (int)(wi * ntiles / nwg), (int)((wi + 1) * ntiles / nwg));
        cost = c > cost ? c : cost;
      }
      if (ntiles % nwg != 0) {
        int64_t wi = 0;
        const int64_t big = ntiles / nwg + 1;
        while (wi < nwg && (wi + 1) * ntiles / nwg - wi * ntiles / nwg != big)
          ++wi;
        if (wi < nwg) {
          const double c = run_cost(tr, (int)(wi * ntiles / nwg), (int)((wi + 1) * ntiles / nwg));
          cost = c > cost ? c : cost;
        }
      }
      // (measured: where both apply and the model sees them within a few
      // percent, four slices are the faster by 2-4 %)
      const double eff = ideal / cost * (sl == 2 ? 0.93 : 1.0);
      const bool forced = knobs.conv_rows > 0 && knobs.conv_rows == tr;
      if (knobs.conv_rows > 0 ? (forced && best.sl == 0) : eff > best.eff + 1e-9) {
        best.eff = eff;
        best.tr = tr;
        best.sl = sl;
      }
    }
  }
  if (best.tr == 0)
    return p;
  // (also for problems that leave most of the machine idle: a workgroup's 5 us
  // of filter and slab set-up is half of what the tiled kernels' K loop of
  // dependent slices takes on the same problem)
  const Layout y = layout_of(best.sl);
  p.sl = best.sl;
  a.TR = best.tr;
  a.tiles_per_image = (a.P + a.TR - 1) / a.TR;
  a.ntiles = a.N * a.tiles_per_image;
  a.kgroups = y.kgroups;
  a.magic_q = conv_magic(a.Q);
  a.magic_ni = conv_magic(a.NI);
  p.C = (int)C, p.R = (int)R, p.S = (int)S;
  const int64_t items = (int64_t)a.ntiles * y.kgroups;
  p.grid = (int)(items < y.slots ? items : y.slots);
  // one tile per workgroup: the first tile's rows and what the filter's
  // staging needs; more: all of LDS
  const int slab_bytes = (a.TR + (int)R - 1) * rowpitch;
  const int stage_end = 1024 + y.stage + y.stage2;
  const int slab_end = y.slab_org + y.first_row * rowpitch + slab_bytes;
  p.lds = items > p.grid ? lds_max : (slab_end > stage_end ? slab_end : stage_end);
  a.slab_org = y.slab_org;
  a.first_row = y.first_row;
  a.slab_rows = (p.lds - y.slab_org) / rowpitch;
  p.ok = true;
  return p;
}

template <int KIND, int C, int R, int S, bool RELU, bool UNIT, int GW, int SL>
int rf_launch(fhip_ctx *ctx, const RfPlan &p) {
  auto kernel = conv_rf_kernel<KIND, C, R, S, RELU, UNIT, GW, SL>;
  static FhipOncePerDevice configured;
  if (!configured.done(ctx->device)) {
    FHIP_HIP_CHECK(ctx, hipFuncSetAttribute(
                            reinterpret_cast<const void *>(kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize,
                            160 * 1024));
    configured.mark(ctx->device);
  }
  hipLaunchKernelGGL(kernel, dim3((unsigned)p.grid), dim3(kRfThreads), p.lds,
                     ctx->stream, p.a);
  FHIP_HIP_CHECK(ctx, hipGetLastError());
  if (GW > 1)
    fhip_note_kernel(ctx, "conv_rf c=%d r=%d s=%d rows=%d relu=%d unit=%d groups_per_wg=%d", C, R,
                     S, p.a.TR, (int)RELU, (int)UNIT, GW);
  else if (SL == 2)
    fhip_note_kernel(ctx, "conv_rf c=%d r=%d s=%d rows=%d relu=%d unit=%d slices=2", C, R, S,
                     p.a.TR, (int)RELU, (int)UNIT);
  else
    fhip_note_kernel(ctx, "conv_rf c=%d r=%d s=%d rows=%d relu=%d unit=%d", C, R, S, p.a.TR,
                     (int)RELU, (int)UNIT);
  return 0;
}

template <int KIND, int C, int R, int S, int GW, int SL>
int rf_launch_relu(fhip_ctx *ctx, const RfPlan &p) {
  if (p.a.unit_scale)
    return p.relu ? rf_launch<KIND, C, R, S, true, true, GW, SL>(ctx, p)
                  : rf_launch<KIND, C, R, S, false, true, GW, SL>(ctx, p);
  return p.relu ? rf_launch<KIND, C, R, S, true, false, GW, SL>(ctx, p)
                : rf_launch<KIND, C, R, S, false, false, GW, SL>(ctx, p);
}

template <int KIND> int rf_launch_shape(fhip_ctx *ctx, const RfPlan &p) {
  if (p.C == 64 && p.R == 3 && p.S == 3)
    return p.gw == 2   ? rf_launch_relu<KIND, 64, 3, 3, 2, 4>(ctx, p)
           : p.sl == 2 ? rf_launch_relu<KIND, 64, 3, 3, 1, 2>(ctx, p)
                       : rf_launch_relu<KIND, 64, 3, 3, 1, 4>(ctx, p);
  return fhip_fail(ctx, "conv: no register-filter kernel for this filter");
}

} // namespace

bool fhip_fast_conv_rf_applicable(const fhip_conv_desc *d) {
  return make_rf_plan(d, 256).ok;
}


int fhip_fast_conv_rf(fhip_ctx *ctx, const fhip_conv_desc *d, const void *x,
                      const void *w, const DevEpilogue &epi, void *out,
                      bool *handled) {
  RfPlan p = make_rf_plan(d, ctx->num_cus);
  if (handled) {
    // one planning pass: tells the caller whether this kernel took the call
    *handled = p.ok && ((uintptr_t)out & 15) == 0;
    if (!*handled)
      return 0;
  }
  FHIP_REQUIRE(ctx, p.ok, "conv: descriptor not supported by the register-filter kernel");
  FHIP_REQUIRE(ctx, ((uintptr_t)x & 15) == 0 && ((uintptr_t)w & 15) == 0 &&
                        ((uintptr_t)out & 15) == 0,
               "conv: X, W and OUT must be 16-byte aligned");
  p.a.x = (const char *)x;
  p.a.w = (const char *)w;
  p.a.out = (char *)out;
  p.a.epi = epi;
  for (int i = 0; i < epi.count; ++i)
    p.a.epi.op[i].stride[2] = epi.op[i].stride[1]; // per-channel step
  return p.kind == GK_BF16 ? rf_launch_shape<GK_BF16>(ctx, p)
                           : rf_launch_shape<GK_F16>(ctx, p);
}
