// MFMA GEMM kernel template and launch helpers; instantiated once per element
// kind in gemm_<kind>.hip.
//
// Data path of one workgroup (4 wavefronts as 2 x 2, or 8 as 2 x 4 / 4 x 2, each
// owning a block of 32x32 MFMA tiles; the eight-wavefront kernels compute them
// as 16x16 MFMA tiles of twice the K):
//   * 128-byte K slices of A and B go from global memory straight into LDS
//     with the LDS-DMA form of the buffer load (no staging registers), into a
//     ring of NSTAGE stages ahead of the MFMAs; the convolution modes gather A
//     from the NHWC input per filter tap, or keep the tile's input pixels and
//     halo resident in LDS for all taps;
//   * LDS rows are unpadded; 16-byte chunks are XOR-permuted inside a row so
//     both the 16-byte fragment reads (K-contiguous operand) and the
//     transposing 8-byte reads (M/N-contiguous operand) are bank-conflict free;
//   * 4-wave tiles double-buffer MFMA fragments in registers (the reads for
//     K-step s + 1 are in flight during the MFMAs of step s, one barrier per K
//     slice); 8-wave tiles alternate a memory phase and an MFMA phase per K
//     slice between the two wavefronts of each SIMD;
//   * the fused epilogue runs on the accumulators when it is linear with
//     per-column operands (16-bit results then leave through LDS as packed
//     row pairs), otherwise after a trip through LDS in 32-row bands; either
//     way a lane stores 8 consecutive columns with 16-byte writes.
#ifndef FUSILLI_AMD_CSRC_GEMM_KERNEL_H
#define FUSILLI_AMD_CSRC_GEMM_KERNEL_H

#include "common.h"

#include <cstdlib>
#include <type_traits>


typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef float gemm_f32x4 __attribute__((ext_vector_type(4)));

// Pointer into LDS (address space 3) at a byte offset from a generic pointer
// that is known to point into shared memory.
#define LDS_PTR(T, base, byte_off)                                             \
  ((T __attribute__((address_space(3))) *)((                                   \
      char __attribute__((address_space(3))) *)(uint32_t)(uintptr_t)(base) +   \
      (byte_off)))

enum GemmKind { GK_BF16 = 0, GK_F16 = 1, GK_I8 = 2, GK_FP8E4M3 = 3, GK_FP8E5M2 = 4 };

template <int KIND> struct KindTraits;
template <> struct KindTraits<GK_BF16> {
  static constexpr int kElemBytes = 2;
  static constexpr int kStepBytes = 32; // K bytes per row per MFMA
  using Acc = float;
  using AccVec = f32x16;
  using AccVec4 = gemm_f32x4; // accumulators of a 16 x 16 MFMA
};
template <> struct KindTraits<GK_F16> {
  static constexpr int kElemBytes = 2;
  static constexpr int kStepBytes = 32;
  using Acc = float;
  using AccVec = f32x16;
  using AccVec4 = gemm_f32x4;
};
template <> struct KindTraits<GK_I8> {
  static constexpr int kElemBytes = 1;
  static constexpr int kStepBytes = 32;
  using Acc = int;
  using AccVec = i32x16;
  using AccVec4 = i32x4;
};
template <> struct KindTraits<GK_FP8E4M3> {
  static constexpr int kElemBytes = 1;
  static constexpr int kStepBytes = 64;
  using Acc = float;
  using AccVec = f32x16;
  using AccVec4 = gemm_f32x4;
};
template <> struct KindTraits<GK_FP8E5M2> {
  static constexpr int kElemBytes = 1;
  static constexpr int kStepBytes = 64;
  using Acc = float;
  using AccVec = f32x16;
  using AccVec4 = gemm_f32x4;
};

template <int N, typename F>
__device__ __forceinline__ void gemm_static_for(F &&f) {
  if constexpr (N > 0) {
    gemm_static_for<N - 1>(f);
    f(std::integral_constant<int, N - 1>{});
  }
}

constexpr int kTileKBytes = 128; // bytes of K per LDS slice
constexpr int kThreads = 256;

// Geometry of an implicit-GEMM convolution: A is never materialised; row m of
// the GEMM is output pixel (n, p, q) and K-slice kt is filter tap (r, s) with a
// 128-byte run of channels, gathered from the NHWC input (zero outside it).
struct ConvGeom {
  int32_t H, W, C;        // input spatial extents and channels (of one group)
  int32_t x_pitch;        // bytes between input pixels (all groups' channels)
  int32_t P, Q;           // output spatial extents
  int32_t S;              // filter width (taps per filter row)
  int32_t pad_h, pad_w, str_h, str_w, dil_h, dil_w;
  int32_t slices_per_tap; // C * elem / 128
  uint32_t x_bytes;       // bytes of the input tensor (< 2^31)
  int32_t R;              // filter height
  // floor(2^32 / d) for d = Q, P, S, slices_per_tap (see conv_div)
  uint32_t magic_q, magic_p, magic_s, magic_spt;
  // halo mode: rows (input pixels) of the LDS slab, a multiple of 8, and the
  // slab's bytes including its trailing 128-byte row of zeros
  int32_t halo_rows;
  uint32_t slab_bytes;
};

// n / d for 0 <= n < 2^31 with magic = floor(2^32 / d): the estimate is at
// most one too small.
__host__ __device__ inline uint32_t conv_magic(int32_t d) {
  return d <= 1 ? 0u : (uint32_t)((1ull << 32) / (uint32_t)d);
}
__device__ __forceinline__ int32_t conv_div(int32_t n, int32_t d, uint32_t magic) {
  if (d == 1)
    return n;
  int32_t q = (int32_t)__umulhi((uint32_t)n, magic);
  if (n - q * d >= d)
    ++q;
  return q;
}

// A_CONV gathers one filter tap per K slice from global memory.  A_HALO (unit
// stride, output extent == input extent) loads the tile's input pixels and
// their halo into LDS once; every tap then reads its fragments from that slab
// at a shifted row, and only the filter streams through the stage ring.
enum GemmAMode { A_KCONTIG = 0, A_MCONTIG = 1, A_CONV = 2, A_HALO = 3 };

struct GemmArgs {
  ConvGeom conv;
  const char *a;
  const char *b;
  char *out;
  int64_t M, N, K;            // K in elements
  int64_t a_ld, b_ld;         // leading dimension in elements (stride of the
                              // non-contiguous one of the two matrix dims)
  int64_t a_batch, b_batch;   // batch strides in elements (0 = broadcast)
  int64_t o_sm, o_sn, o_batch; // output strides in elements
  // optional outer batch dim (grid z) with strides of its own; fused operands
  // do not see it
  int64_t a_outer, b_outer, o_outer;
  // column offset per outer index that fused operands DO see (grouped
  // convolution: the group's first output channel); 0 otherwise
  int64_t epi_n_outer;
  int32_t outer; // extent (0 or 1: none)
  // The reduction cut into `outer` parts of kt_split K slices each (0: not
  // cut; not in halo mode): part z accumulates slices z * kt_split .. and
  // writes its own f32 result, which the caller adds up
  int32_t kt_split;
  int32_t c_dt, o_dt;
  int32_t tiles_m, tiles_n;
  // rows of an M tile that are computed and stored (0: all BM); a smaller
  // value lets the host match the tile count to the machine
  int32_t tile_rows;
  int32_t o_vec;              // output rows allow aligned 16-byte stores
  // columns that are stored (0: N).  The parts of a split reduction store
  // whole column tiles into rows padded to the tile width, so that no cache
  // line of the partial sums is written by two workgroups
  int64_t n_store;
  // Epilogue applied to the accumulators in registers: every op is one of
  // ADD / SUB / MUL / RELU / NEG / IDENTITY with a scalar or per-column
  // operand: v = mul ? v * o : a * v + b * o, then max(v, 0) if relu.
  int32_t epi_reg;
  float lin_a[FHIP_MAX_EPILOGUE], lin_b[FHIP_MAX_EPILOGUE];
  int32_t lin_mul[FHIP_MAX_EPILOGUE], lin_relu[FHIP_MAX_EPILOGUE];
  DevEpilogue epi;            // strides refer to (batch, m, n)
};

// Fragment (per-lane MFMA operand) holder: FRAG_REGS 32-bit registers.
template <int KIND> struct Frag {
  static constexpr int kRegs = KindTraits<KIND>::kStepBytes / 2 / 4;
  uint32_t r[kRegs];
};

template <int KIND>
__device__ __forceinline__ void mfma32(typename KindTraits<KIND>::AccVec &c,
                                       const Frag<KIND> &a,
                                       const Frag<KIND> &b) {
  if constexpr (KIND == GK_BF16) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
        __builtin_bit_cast(bf16x8, a.r), __builtin_bit_cast(bf16x8, b.r), c, 0,
        0, 0);
  } else if constexpr (KIND == GK_F16) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_f16(
        __builtin_bit_cast(f16x8, a.r), __builtin_bit_cast(f16x8, b.r), c, 0, 0,
        0);
  } else if constexpr (KIND == GK_I8) {
    c = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, a.r),
                                              __builtin_bit_cast(i32x4, b.r), c,
                                              0, 0, 0);
  } else {
    constexpr int fmt = KIND == GK_FP8E4M3 ? 0 : 1; // 0 = e4m3, 1 = e5m2
    c = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
        __builtin_bit_cast(i32x8, a.r), __builtin_bit_cast(i32x8, b.r), c, fmt,
        fmt, 0, 0, 0, 0);
  }
}

// The 16 x 16 shapes with twice the K of the 32 x 32 ones (16x16x32 16-bit,
// 16x16x64 int8, 16x16x128 fp8): the same operand bytes per lane, a quarter
// of the accumulator registers per instruction.  Measured on register-resident
// loops with random operand bits they sustain 13-21 % more than the 32 x 32
// shapes (bf16 2.34 against 2.03 PFLOP/s, int8 4.33 / 3.58, fp8 4.74 / 4.20):
// the matrix pipe is power-limited, and these shapes move less accumulator
// data per operation.  Lane (row or column l % 16, K block l / 16) holds the
// K block's STEPB / 2 consecutive bytes.
template <int KIND>
__device__ __forceinline__ void mfma16(typename KindTraits<KIND>::AccVec4 &c,
                                       const Frag<KIND> &a, const Frag<KIND> &b) {
  if constexpr (KIND == GK_BF16) {
    c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
        __builtin_bit_cast(bf16x8, a.r), __builtin_bit_cast(bf16x8, b.r), c, 0, 0, 0);
  } else if constexpr (KIND == GK_F16) {
    c = __builtin_amdgcn_mfma_f32_16x16x32_f16(
        __builtin_bit_cast(f16x8, a.r), __builtin_bit_cast(f16x8, b.r), c, 0, 0, 0);
  } else if constexpr (KIND == GK_I8) {
    c = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(i32x4, a.r),
                                              __builtin_bit_cast(i32x4, b.r), c, 0, 0, 0);
  } else {
    constexpr int fmt = KIND == GK_FP8E4M3 ? 0 : 1; // 0 = e4m3, 1 = e5m2
    c = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
        __builtin_bit_cast(i32x8, a.r), __builtin_bit_cast(i32x8, b.r), c, fmt, fmt, 0, 0, 0, 0);
  }
}

#ifndef GEMM_M16
#define GEMM_M16 1
#endif
#define GEMM_AS1 __attribute__((address_space(1)))
#define GEMM_AS3 __attribute__((address_space(3)))

// s_waitcnt immediate: vmcnt <= n, lgkmcnt = 0, expcnt untouched.
constexpr int gemm_wait_imm(int vm) {
  return (vm & 0xF) | ((vm >> 4) << 14) | (0x7 << 4) | (0x0 << 8);
}

// LDS geometry of one operand slice (128 K-bytes of ROWS rows).
//   K-contiguous operand: ROWS rows of 128 bytes; the 16-byte chunk c of row r
//   sits at chunk position c ^ (r & 7) ^ ((r >> 3) & 1).
//   Other operand: 128/elem K-rows of ROWS*elem bytes; chunk c of K-row k sits
//   at position nkc_pos(k, c).
template <int ROWS, int ELEM, bool KCONTIG, int NW = 4> struct SliceGeom {
  static constexpr int kBytes = ROWS * kTileKBytes;
  static constexpr int kLoads = kBytes / 1024 / NW; // DMA instructions per thread
  static constexpr int kKRows = kTileKBytes / ELEM;
  static constexpr int kRowBytes = KCONTIG ? kTileKBytes : ROWS * ELEM;
  static constexpr int kCPR = kRowBytes / 16;        // chunks per LDS row
  static constexpr int kRowsPerLoad = 1024 / kRowBytes; // LDS rows per wave DMA
};

__device__ __forceinline__ int kc_swz(int r) { return (r & 7) ^ ((r >> 3) & 1); }

// Chunk permutation of the M/N-contiguous layout.  A 32-lane half-wavefront
// of a transposing read covers 4 K-rows x 64 bytes (16-bit) or 8 K-rows x
// 32 bytes (8-bit); the permutation spreads those over all 64 banks.
// With the 16 x 16 MFMA shapes the two 16-lane groups of a half-wavefront read
// the same columns of K-rows that differ in bit XB of k (16 for 16-bit
// elements, 32 for 8-bit ones): that bit sends them to different banks as
// well.  XB = 0 for the 32 x 32 shapes.  (A bit of k above the lowest three
// may only enter where it depends on the lane alone: fragment reads reach the
// K-rows of later reads and K-steps through immediate offsets from one address.)
template <int ELEM, int RB, int XB> __device__ __forceinline__ int nkc_pos(int k, int c) {
  if constexpr (ELEM == 2)
    return c ^ ((k & 3) << 1) ^ ((c & 2) << 2) ^ ((k & XB) ? 8 : 0);
  else if constexpr (RB == 256)
    return c ^ ((k & 7) << 1) ^ ((k & XB) ? 1 : 0);
  else
    return c ^ (((k >> 1) & 3) << 1) ^ ((k & XB) ? 1 : 0);
}
template <int ELEM, int RB, int XB> __device__ __forceinline__ int nkc_chunk(int k, int p) {
  if constexpr (ELEM == 2) {
    const int t = p ^ ((k & 3) << 1) ^ ((k & XB) ? 8 : 0);
    return t ^ ((t & 2) << 2);
  } else {
    return nkc_pos<ELEM, RB, XB>(k, p);
  }
}

// Per-thread byte offsets (from the tile's first row / column at K = 0) of the
// chunks this thread's DMA instructions fetch; the same for every K slice.
template <int ROWS, int ELEM, bool KCONTIG, int NW, int XB>
__device__ __forceinline__ void
dma_setup(int64_t ld_bytes, int64_t row0, int64_t rows_total,
          uint32_t (&off)[SliceGeom<ROWS, ELEM, KCONTIG, NW>::kLoads]) {
  using G = SliceGeom<ROWS, ELEM, KCONTIG, NW>;
  const int w = threadIdx.x >> 6, l = threadIdx.x & 63;
#pragma unroll
  for (int j = 0; j < G::kLoads; ++j) {
    const int group = j * NW + w;
    if constexpr (KCONTIG) {
      const int row = group * 8 + (l >> 3);
      const int c = (l & 7) ^ kc_swz(row);
      int64_t r = row0 + row;
      r = r < rows_total ? r : rows_total - 1; // ragged edge tiles
      off[j] = (uint32_t)((r - row0) * ld_bytes + c * 16);
    } else {
      const int k = group * G::kRowsPerLoad + l / G::kCPR;
      const int c = nkc_chunk<ELEM, G::kRowBytes, XB>(k, l % G::kCPR);
      int64_t e = row0 + (int64_t)c * (16 / ELEM);
      const int64_t last = rows_total - 16 / ELEM;
      e = e < last ? e : last;
      off[j] = (uint32_t)(k * ld_bytes + (e - row0) * ELEM);
    }
  }
}

// One K slice of one operand, global -> LDS: each wavefront instruction moves
// 64 x 16 bytes to 1024 consecutive LDS bytes.  Buffer addressing (uniform
// 64-bit base + 32-bit lane offset) keeps these loads on the vector-memory
// counter only, so waits on LDS reads stay exact while they are in flight;
// offsets at or past `bytes` read as zero.
template <int NW, int LOADS, int J0 = 0, int J1 = LOADS>
__device__ __forceinline__ void dma_issue(const char *base, uint32_t bytes,
                                          const uint32_t (&off)[LOADS],
                                          uint32_t lds_stage) {
  const int w = threadIdx.x >> 6;
  // the descriptor must sit in scalar registers: say so, or 64-bit pointer
  // arithmetic done on the vector ALU forces a per-lane loop around each load
  const uint64_t b64 = (uint64_t)base;
  const uint32_t blo = __builtin_amdgcn_readfirstlane((uint32_t)b64);
  const uint32_t bhi = __builtin_amdgcn_readfirstlane((uint32_t)(b64 >> 32));
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
      (void *)(((uint64_t)bhi << 32) | blo), 0,
      (int)__builtin_amdgcn_readfirstlane(bytes), 0x00020000);
#pragma unroll
  for (int j = J0; j < J1; ++j) {
    const uint32_t dst = lds_stage + (uint32_t)(j * NW + w) * 1024u;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(
        rsrc, (GEMM_AS3 char *)__builtin_amdgcn_readfirstlane(dst), 16,
        (int)off[j], 0, 0, 0);
  }
}

// Fragment addressing: per-lane LDS byte offsets (within a stage) that stay
// fixed for the whole kernel; everything that varies is an immediate.
template <int KIND, int ROWS, bool KCONTIG, int NT> struct FragAddr {
  static constexpr int ELEM = KindTraits<KIND>::kElemBytes;
  static constexpr int STEPB = KindTraits<KIND>::kStepBytes;
  static constexpr int KSTEPS = kTileKBytes / STEPB;
  static constexpr int CH = STEPB / 16;  // chunks per row per K-step
  static constexpr int CHH = CH / 2;     // 16-byte reads per fragment
  static constexpr int RB = ROWS * ELEM; // M/N-contiguous: bytes per K-row
  static constexpr int N = KCONTIG ? KSTEPS * CHH : NT;
  uint32_t a[N];

  __device__ __forceinline__ void setup(int tile0) {
    const int l = threadIdx.x & 63;
    if constexpr (KCONTIG) {
      const int r = tile0 * 32 + (l & 31);
      const int sw = kc_swz(l & 31);
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s)
#pragma unroll
        for (int i = 0; i < CHH; ++i) {
          const int c = s * CH + (l >> 5) * CHH + i;
          a[s * CHH + i] = (uint32_t)(r * kTileKBytes + ((c ^ sw) << 4));
        }
    } else {
      const int L = l & 15, h = (l >> 4) & 1;
      constexpr int KPL = STEPB / 2 / ELEM; // K values per lane per step
      const int kq = ELEM == 2 ? (L >> 2) : (L >> 1);
      const int k = (l >> 5) * KPL + kq;
#pragma unroll
      for (int i = 0; i < NT; ++i) {
        const int rb = tile0 + i;
        int c, sub;
        if constexpr (ELEM == 2) {
          c = rb * 4 + h * 2 + ((L & 3) >> 1);
          sub = (L & 1) * 8;
        } else {
          c = rb * 2 + h;
          sub = (L & 1) * 8;
        }
        a[i] = (uint32_t)(k * RB + nkc_pos<ELEM, RB, 0>(k, c) * 16 + sub);
      }
    }
  }

  // Fragments of the NT tiles for K-step S from the stage at LDS address `st`.
  template <int S>
  __device__ __forceinline__ void load(uint32_t st, Frag<KIND> (&f)[NT]) const {
    if constexpr (KCONTIG) {
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int i = 0; i < CHH; ++i) {
          const u32x4 v = *(const GEMM_AS3 u32x4 *)(uintptr_t)(
              st + a[S * CHH + i] + t * 32 * kTileKBytes);
          f[t].r[4 * i + 0] = v.x;
          f[t].r[4 * i + 1] = v.y;
          f[t].r[4 * i + 2] = v.z;
          f[t].r[4 * i + 3] = v.w;
        }
    } else {
      // Written as asm: the compiler makes the transposing-read builtins wait
      // for every global -> LDS load in flight (vmcnt(0)), the prefetched
      // slices included, and spends an address addition on each.  The caller
      // waits for these reads itself (lgkmcnt) before it uses the fragments.
      constexpr int KPL = STEPB / 2 / ELEM;
      constexpr int RPK = ELEM == 2 ? 4 : 8; // K values per transposing read
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const uint32_t ad = st + a[t];
        gemm_static_for<KPL / RPK>([&](auto rc) {
          constexpr int r = decltype(rc)::value;
          constexpr int OFF = (S * (STEPB / ELEM) + RPK * r) * RB;
          static_assert(OFF >= 0 && OFF < 65536, "16-bit offset field");
          u32x2 w;
          if constexpr (ELEM == 2)
            asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(w) : "v"(ad), "n"(OFF));
          else
            asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(w) : "v"(ad), "n"(OFF));
          f[t].r[2 * r + 0] = w.x;
          f[t].r[2 * r + 1] = w.y;
        });
      }
    }
  }
};

// Fragment addressing for the 16 x 16 MFMA shapes: NT tiles of 16 rows, K-steps
// of 2 * STEPB bytes.  Same LDS layouts as above (with the bit XB in the
// M/N-contiguous one).  The 16-lane group g of a wavefront supplies K block
// g of a step.  A 16-byte LDS read serves 16 lanes per clock: lanes
// 32 h + 4 q + (0..3) for the four q in 0..7 of one parity of bit count, i.e.
// lanes 0-3 and 12-15 of one group with lanes 4-11 of the next.  Under the
// K-contiguous layout's swizzle such a set stays on distinct banks when lane i
// of a group reads tile row row16(i) = i with the blocks 8-11 and 12-15
// exchanged; the MFMA's output rows (A) or columns (B) are then permuted the
// same way, which the epilogue's LDS writes undo.  (The K blocks stay in their
// natural order: every tile shape adds a slice's products in the same order.)
template <int KIND> struct Frag16Geom {
  static constexpr int ELEM = KindTraits<KIND>::kElemBytes;
  static constexpr int STEPB = 2 * KindTraits<KIND>::kStepBytes;
  static constexpr int XB = STEPB / 4 / ELEM; // K values per lane: 8, 16 (int8), 32 (fp8)
  __device__ static __forceinline__ int row16(int i) { return i ^ ((i >> 1) & 4); }
};
template <int KIND, int ROWS, bool KCONTIG, int NT> struct FragAddr16 {
  static constexpr int XB = Frag16Geom<KIND>::XB;
  static constexpr int ELEM = KindTraits<KIND>::kElemBytes;
  static constexpr int STEPB = 2 * KindTraits<KIND>::kStepBytes; // K bytes per row per MFMA
  static constexpr int KSTEPS = kTileKBytes / STEPB;
  static constexpr int CH = STEPB / 16;  // chunks per row per K-step
  static constexpr int CHQ = CH / 4;     // 16-byte reads per fragment
  static constexpr int RB = ROWS * ELEM; // M/N-contiguous: bytes per K-row
  static constexpr int KPL = STEPB / 4 / ELEM; // K values per lane per step
  static constexpr int N = KCONTIG ? KSTEPS * CHQ : NT;
  uint32_t a[N];

  __device__ __forceinline__ void setup(int tile0) {
    const int l = threadIdx.x & 63;
    if constexpr (KCONTIG) {
      const int r16 = Frag16Geom<KIND>::row16(l & 15);
      const int r = tile0 * 16 + r16;
      const int sw = kc_swz(r16);
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s)
#pragma unroll
        for (int i = 0; i < CHQ; ++i) {
          const int c = s * CH + (l >> 4) * CHQ + i;
          a[s * CHQ + i] = (uint32_t)(r * kTileKBytes + ((c ^ sw) << 4));
        }
    } else {
      // a 16-lane group reads the K block l / 16: its lanes address 4 (16-bit)
      // or 8 (8-bit) K-rows x 16 matrix rows and each receives one matrix
      // row's run of K values
      const int L = l & 15;
      const int k = (l >> 4) * KPL + (ELEM == 2 ? (L >> 2) : (L >> 1));
#pragma unroll
      for (int i = 0; i < NT; ++i) {
        const int rb = tile0 + i; // 16 matrix rows: 32 bytes (16-bit) or 16 (8-bit)
        int c, sub;
        if constexpr (ELEM == 2) {
          c = rb * 2 + ((L & 3) >> 1);
          sub = (L & 1) * 8;
        } else {
          c = rb;
          sub = (L & 1) * 8;
        }
        a[i] = (uint32_t)(k * RB + nkc_pos<ELEM, RB, XB>(k, c) * 16 + sub);
      }
    }
  }

  template <int S>
  __device__ __forceinline__ void load(uint32_t st, Frag<KIND> (&f)[NT]) const {
    if constexpr (KCONTIG) {
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int i = 0; i < CHQ; ++i) {
          const u32x4 v = *(const GEMM_AS3 u32x4 *)(uintptr_t)(
              st + a[S * CHQ + i] + t * 16 * kTileKBytes);
          f[t].r[4 * i + 0] = v.x;
          f[t].r[4 * i + 1] = v.y;
          f[t].r[4 * i + 2] = v.z;
          f[t].r[4 * i + 3] = v.w;
        }
    } else {
      // Written as asm: the compiler makes the transposing-read builtins wait
      // for every global -> LDS load in flight (vmcnt(0)), the prefetched
      // slices included, and spends an address addition on each.  The caller
      // waits for these reads itself (lgkmcnt) before it uses the fragments.
      constexpr int RPK = ELEM == 2 ? 4 : 8; // K values per transposing read
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const uint32_t ad = st + a[t];
        gemm_static_for<KPL / RPK>([&](auto rc) {
          constexpr int r = decltype(rc)::value;
          constexpr int OFF = (S * (STEPB / ELEM) + RPK * r) * RB;
          static_assert(OFF >= 0 && OFF < 65536, "16-bit offset field");
          u32x2 w;
          if constexpr (ELEM == 2)
            asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(w) : "v"(ad), "n"(OFF));
          else
            asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(w) : "v"(ad), "n"(OFF));
          f[t].r[2 * r + 0] = w.x;
          f[t].r[2 * r + 1] = w.y;
        });
      }
    }
  }
};

// Scheduling recipe for one K-step: NM MFMAs with NR LDS reads spread over
// the leading MFMAs and NV global->LDS loads over the trailing quarter (the
// loads write LDS, so they stay behind the reads that precede them in program
// order).  Neither memory queue then fills up and stalls the wavefront while
// the matrix pipe has work.
template <int NM, int NR, int NV> __device__ __forceinline__ void gemm_interleave() {
  constexpr int MV0 = NV == 0 ? 0 : (NM / 4 < NV ? NM / 4 : NV);
  constexpr int MV = (NV + 1) / 2 > MV0 && (NV + 1) / 2 <= NM / 2 ? (NV + 1) / 2 : MV0;
  constexpr int MR = NM - MV;
  gemm_static_for<NM>([&](auto mc) {
    constexpr int m = decltype(mc)::value;
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); // MFMA
    if constexpr (m < MR) {
      constexpr int nr = ((m + 1) * NR) / MR - (m * NR) / MR;
      if constexpr (nr > 0)
        __builtin_amdgcn_sched_group_barrier(0x100, nr, 0); // DS read
    } else {
      constexpr int v = m - MR;
      constexpr int nv = ((v + 1) * NV) / MV - (v * NV) / MV;
      if constexpr (nv > 0)
        __builtin_amdgcn_sched_group_barrier(0x020, nv, 0); // VMEM read
    }
  });
}

// Workgroup barrier with nothing attached: the callers wait for exactly the
// loads and LDS reads that the hand-over needs; the empty asm statements keep
// the compiler from moving memory operations across.
__device__ __forceinline__ void gemm_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// Makes the compiler treat `x` as produced here (a value that a pending load
// delivers must have arrived).
__device__ __forceinline__ void gemm_pin(float &x) { asm volatile("" : "+v"(x)); }

template <int N>
__device__ __forceinline__ void load_operand_vec(const void *p, int dt,
                                                 const int64_t (&off)[N],
                                                 float (&o)[N]) {
  if (dt == FHIP_FLOAT) {
#pragma unroll
    for (int i = 0; i < N; ++i)
      o[i] = ((const GEMM_AS1 float *)p)[off[i]];
  } else if (dt == FHIP_BFLOAT16) {
#pragma unroll
    for (int i = 0; i < N; ++i)
      o[i] = (float)((const GEMM_AS1 __bf16 *)p)[off[i]];
  } else {
#pragma unroll
    for (int i = 0; i < N; ++i)
      o[i] = (float)((const GEMM_AS1 _Float16 *)p)[off[i]];
  }
}

// LDS bytes of the kernel: NSTAGE stages of (A slice + B slice); the epilogue
// reuses it for four 32-row accumulator bands (one per wavefront).
// Wavefront grid of a tile.  8 wavefronts (two per SIMD, scheduled in
// alternating memory / MFMA phases): 256 x 256 as 2 x 4 and 512 x 128 as 4 x 2,
// each wavefront owning 128 x 64 outputs, 256 x 128 as 4 x 2 of 64 x 64 and
// 128 x 128 (GEMM, gather convolution) as 2 x 4 of 64 x 32; 4 wavefronts (the
// halo convolution) as 2 x 2.
template <int BM, int BN, int NW = 0> struct GemmLayout {
  static constexpr bool kWide = BM == 256 && BN == 256;
  static constexpr bool kTall = (BM == 512 || (BM == 256 && NW == 8)) && BN == 128;
  static constexpr bool kSmall8 = BM == 128 && BN == 128 && NW == 8; // 64 x 32 per wavefront
  static constexpr int kWavesM = kTall ? 4 : 2;
  static constexpr int kWavesN = kWide || kSmall8 ? 4 : 2;
  static constexpr int kWaves = kWavesM * kWavesN;
};

template <int BM, int BN, int NSTAGE, int NW, bool HALO = false> struct GemmLds {
  static constexpr int kStage = (BM + BN) * kTileKBytes;
  static constexpr int kWN = BN / GemmLayout<BM, BN, NW>::kWavesN; // wave columns
  static constexpr int kEpiPitch = kWN * 4 + 32;
  static constexpr int kBand = 32 * kEpiPitch; // one wavefront, one tile row
  static constexpr int kTM = BM / GemmLayout<BM, BN, NW>::kWavesM / 32;
  // tile rows that leave together: as many as fit 160 KB, or 80 KB where the
  // stages leave room for two workgroups per compute unit
  static constexpr int kCap =
      HALO || NSTAGE * kStage <= 80 * 1024 ? 80 * 1024 : 160 * 1024;
  static constexpr int kBands =
      NW * kTM * kBand <= kCap ? kTM : (NW * 2 * kBand <= kCap ? 2 : 1);
  static constexpr int kEpiBytes = NW * kBands * kBand;
  static constexpr int kBytes =
      NSTAGE * kStage > kEpiBytes ? NSTAGE * kStage : kEpiBytes;
};

// Halo kernels are laid out for two workgroups per compute unit (two
// wavefronts per SIMD): at most 256 registers per lane.
template <int KIND, int BM, int BN, int A_MODE, bool B_KC, int NSTAGE, int NW>
__global__ __launch_bounds__(NW * 64)
__attribute__((amdgpu_waves_per_eu(A_MODE == A_HALO ? 2 : 1, 8))) void
gemm_kernel(GemmArgs g) {
  using Acc = typename KindTraits<KIND>::Acc;
  constexpr bool A_KC = A_MODE != A_MCONTIG;
  constexpr int ELEM = KindTraits<KIND>::kElemBytes;
  constexpr int STEPB = KindTraits<KIND>::kStepBytes;
  constexpr int KSTEPS = kTileKBytes / STEPB;
  static_assert(KSTEPS % 2 == 0, "fragment double buffering needs even KSTEPS");
  using GA = SliceGeom<BM, ELEM, A_KC, NW>;
  using GB = SliceGeom<BN, ELEM, B_KC, NW>;
  using L = GemmLds<BM, BN, NSTAGE, NW, A_MODE == A_HALO>;
  constexpr int WAVES_M = GemmLayout<BM, BN, NW>::kWavesM;
  constexpr int WAVES_N = GemmLayout<BM, BN, NW>::kWavesN;
  static_assert(WAVES_M * WAVES_N == NW, "wavefront grid");
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N; // wavefront tile
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr bool HALO = A_MODE == A_HALO;
  static_assert(!HALO || (ELEM == 2 && B_KC && NW == 4), "halo mode: 16-bit, 4 waves");
  // The ping-pong GEMM tiles use the 16 x 16 MFMA shapes (twice the K per
  // instruction): on operands with random bits the matrix pipe sustains 13 to
  // 21 % more with them than with the 32 x 32 shapes.
  constexpr bool M16 = GEMM_M16 && NW == 8;
  constexpr int XB = M16 ? Frag16Geom<KIND>::XB : 0; // (M/N-contiguous LDS layout)
  constexpr int KSTEPS16 = KSTEPS / 2;
  constexpr int TM16 = WM / 16, TN16 = WN / 16;
  // DMA instructions per slice
  constexpr int LPS = (HALO ? 0 : GA::kLoads) + GB::kLoads;

  extern __shared__ __attribute__((aligned(16))) char smem[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem;

  // XCD-aware tile order: hardware deals consecutive workgroup ids to the 8
  // XCDs in turn; give each XCD a contiguous run of logical ids, then walk the
  // tile grid in column-major groups of 8 row-tiles so a run is a compact
  // block sharing A row-panels and B column-panels in that XCD's L2.
  const int tiles = g.tiles_m * g.tiles_n;
  int pid = blockIdx.x;
  if (tiles % 8 == 0)
    pid = (pid % 8) * (tiles / 8) + pid / 8;
  constexpr int GROUP = 8;
  int tile_m = pid, tile_n = 0;
  if (g.tiles_n > 1) {
    const int per_group = GROUP * g.tiles_n;
    const int group = pid / per_group;
    const int first_m = group * GROUP;
    const int group_rows =
        g.tiles_m - first_m < GROUP ? g.tiles_m - first_m : GROUP;
    tile_m = first_m + (pid % per_group) % group_rows;
    tile_n = (pid % per_group) / group_rows;
  }
  const int64_t batch = blockIdx.y;
  const int64_t outer = blockIdx.z;

  const int tile_rows = g.tile_rows ? g.tile_rows : BM;
  const int64_t m0 = (int64_t)tile_m * tile_rows, n0 = (int64_t)tile_n * BN;
  // first row past this tile's share of the output
  const int64_t m_end = m0 + tile_rows < g.M ? m0 + tile_rows : g.M;
  const int64_t a_ldb = g.a_ld * ELEM, b_ldb = g.b_ld * ELEM;
  const int kt_count =
      !HALO && g.kt_split > 0 ? g.kt_split : (int)(g.K * ELEM / kTileKBytes);
  const int kt_base = !HALO && g.kt_split > 0 ? (int)outer * g.kt_split : 0;

  const int wave = threadIdx.x >> 6;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int l = threadIdx.x & 63;

  // ---- global -> LDS plumbing ---------------------------------------------
  // A and B tile base pointers at K = 0 and their per-slice advance.
  const char *a_base;
  int64_t a_step;
  uint32_t off_a[GA::kLoads], off_b[GB::kLoads];
  // implicit-GEMM gather: pixel index of tap (0, 0) and in-image row / column
  // masks of the filter
  int32_t cv_pix[A_MODE == A_CONV ? GA::kLoads : 1];
  uint32_t cv_mask[A_MODE == A_CONV ? GA::kLoads : 1];
  int cv_chunk = 0;
  // halo mode: slab row of tap (0, 0) and the validity masks of this lane's
  // fragment rows
  int32_t h_row[HALO ? TM : 1];
  uint32_t h_mask[HALO ? TM : 1];
  if constexpr (HALO) {
    a_base = g.a + outer * g.a_outer * ELEM; // a group's first channel
    a_step = 0;
  } else if constexpr (A_MODE == A_CONV) {
    a_base = g.a + outer * g.a_outer * ELEM;
    a_step = 0;
#pragma unroll
    for (int j = 0; j < GA::kLoads; ++j) {
      const int row = (j * NW + wave) * 8 + (l >> 3);
      const int64_t m = m0 + row;
      const bool live = m < m_end;
      const int32_t mm = (int32_t)(live ? m : 0);
      const int32_t pq = conv_div(mm, g.conv.Q, g.conv.magic_q);
      const int32_t q = mm - pq * g.conv.Q;
      const int32_t nn = conv_div(pq, g.conv.P, g.conv.magic_p);
      const int32_t pp = pq - nn * g.conv.P;
      const int32_t ih0 = pp * g.conv.str_h - g.conv.pad_h;
      const int32_t iw0 = q * g.conv.str_w - g.conv.pad_w;
      cv_pix[j] = (nn * g.conv.H + ih0) * g.conv.W + iw0;
      // bits 0..15: filter rows inside the image, 16..31: filter columns
      uint32_t mask = 0;
      for (int fr = 0; fr < g.conv.R; ++fr)
        mask |= (uint32_t)(live && (uint32_t)(ih0 + fr * g.conv.dil_h) <
                                       (uint32_t)g.conv.H)
                << fr;
      for (int fs = 0; fs < g.conv.S; ++fs)
        mask |= (uint32_t)((uint32_t)(iw0 + fs * g.conv.dil_w) <
                           (uint32_t)g.conv.W)
                << (16 + fs);
      cv_mask[j] = mask;
      cv_chunk = ((l & 7) ^ kc_swz(row)) * 16; // same for every j
    }
  } else if constexpr (A_KC) {
    a_step = kTileKBytes;
    a_base = g.a + (batch * g.a_batch + outer * g.a_outer) * ELEM + m0 * a_ldb +
             kt_base * a_step;
    dma_setup<BM, ELEM, true, NW, XB>(a_ldb, m0, m_end, off_a);
  } else {
    a_step = (int64_t)GA::kKRows * a_ldb;
    a_base = g.a + (batch * g.a_batch + outer * g.a_outer) * ELEM + m0 * ELEM +
             kt_base * a_step;
    dma_setup<BM, ELEM, false, NW, XB>(a_ldb, m0, m_end, off_a);
  }
  const char *b_base;
  int64_t b_step;
  if constexpr (B_KC) {
    b_base = g.b + (batch * g.b_batch + outer * g.b_outer) * ELEM + n0 * b_ldb +
             (int64_t)kt_base * kTileKBytes;
    b_step = kTileKBytes;
  } else {
    b_step = (int64_t)GB::kKRows * b_ldb;
    b_base = g.b + (batch * g.b_batch + outer * g.b_outer) * ELEM + n0 * ELEM +
             kt_base * b_step;
  }
  dma_setup<BN, ELEM, B_KC, NW, XB>(b_ldb, n0, g.N, off_b);

  // halo mode: [slab | ring of B slices]; otherwise a ring of (A, B) slices
  constexpr uint32_t STAGE = HALO ? GB::kBytes : L::kStage;
  const uint32_t ring0 = HALO ? lds0 + g.conv.slab_bytes : lds0;
  auto stage_a = [&](int st) { return ring0 + (uint32_t)st * STAGE; };
  auto stage_b = [&](int st) {
    return ring0 + (uint32_t)st * STAGE + (HALO ? 0 : GA::kBytes);
  };
  // Part PART of PARTS of slice kt's loads (A and B split alike).
  // Slices past the end of K are not loaded at all; the loops' waits by count
  // become waits for everything where a batch is missing.  (They used to be
  // "loaded" through zero-sized buffers, which kept every iteration identical;
  // but such a load counts as complete before its zeros are written to LDS:
  // on tiles whose real loads return quickly the zeros of the last batch
  // could land in the epilogue's bands, after the final wait and barrier.)
  auto issue = [&](int kt, int st, auto part_c, auto parts_c) {
    if (kt >= kt_count)
      return;
    const uint32_t lim = 0xffffffffu;
    constexpr int PART = decltype(part_c)::value;
    constexpr int PARTS = decltype(parts_c)::value;
    constexpr int A0 = PART * GA::kLoads / PARTS, A1 = (PART + 1) * GA::kLoads / PARTS;
    constexpr int B0 = PART * GB::kLoads / PARTS, B1 = (PART + 1) * GB::kLoads / PARTS;
    if constexpr (HALO) {
      // only the filter streams
    } else if constexpr (A_MODE == A_CONV) {
      const int32_t ktg = kt + kt_base;
      const int32_t tap = conv_div(ktg, g.conv.slices_per_tap, g.conv.magic_spt);
      const int32_t cb =
          (ktg - tap * g.conv.slices_per_tap) * kTileKBytes + cv_chunk;
      const int32_t fr = conv_div(tap, g.conv.S, g.conv.magic_s);
      const int32_t fs = tap - fr * g.conv.S;
      const int32_t dpix = fr * g.conv.dil_h * g.conv.W + fs * g.conv.dil_w;
      const int32_t cbytes = g.conv.x_pitch;
      uint32_t off[GA::kLoads];
#pragma unroll
      for (int j = A0; j < A1; ++j) {
        const bool in = (cv_mask[j] >> fr) & (cv_mask[j] >> (16 + fs)) & 1;
        // taps outside the image (and rows past M) read past the end: zeros
        off[j] = in ? (uint32_t)((cv_pix[j] + dpix) * cbytes + cb) : 0x80000000u;
      }
      dma_issue<NW, GA::kLoads, A0, A1>(a_base, g.conv.x_bytes & lim, off,
                                    stage_a(st));
    } else {
      dma_issue<NW, GA::kLoads, A0, A1>(a_base + kt * a_step, lim, off_a,
                                    stage_a(st));
    }
    dma_issue<NW, GB::kLoads, B0, B1>(b_base + kt * b_step, lim, off_b,
                                  stage_b(st));
  };
  using One = std::integral_constant<int, 1>;
  using Zero = std::integral_constant<int, 0>;

  // ---- prologue: fill all NSTAGE stages -------------------------------------
  if constexpr (HALO) {
    // Slab row r holds input pixel pix0 + r in the K-contiguous slice layout
    // (one 128-byte channel run per slice); pixels before the tensor or past
    // its end read as zeros, rows of other image lines are masked at use.
    const int32_t pix0 =
        (int32_t)m0 - g.conv.pad_h * g.conv.W - g.conv.pad_w;
    const int32_t cbytes = g.conv.x_pitch;
    const int groups = g.conv.halo_rows / 8;
    const uint64_t b64 = (uint64_t)a_base;
    const uint32_t blo = __builtin_amdgcn_readfirstlane((uint32_t)b64);
    const uint32_t bhi = __builtin_amdgcn_readfirstlane((uint32_t)(b64 >> 32));
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(((uint64_t)bhi << 32) | blo), 0,
        (int)__builtin_amdgcn_readfirstlane(g.conv.x_bytes), 0x00020000);
    for (int sl = 0; sl < g.conv.slices_per_tap; ++sl)
      for (int grp = __builtin_amdgcn_readfirstlane(wave); grp < groups;
           grp += NW) {
        const int row = grp * 8 + (l >> 3);
        const int c = (l & 7) ^ kc_swz(row);
        // modulo 2^32: pixels before the tensor wrap to offsets past its end
        const uint32_t off = (uint32_t)(pix0 + row) * (uint32_t)cbytes +
                             (uint32_t)(sl * kTileKBytes + c * 16);
        const uint32_t dst =
            lds0 + (uint32_t)(sl * g.conv.halo_rows + row - (l >> 3)) * kTileKBytes;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rsrc, (GEMM_AS3 char *)__builtin_amdgcn_readfirstlane(dst), 16,
            (int)off, 0, 0, 0);
      }
    // the row of zeros that masked taps read
    if (threadIdx.x < 8)
      *(GEMM_AS3 u32x4 *)(uintptr_t)(ring0 - kTileKBytes + threadIdx.x * 16) =
          u32x4{0, 0, 0, 0};
  }
  constexpr bool PINGPONG = NW == 8;
  if constexpr (PINGPONG) {
    // slice 0, and the share of slice 1 that wavefronts 4..7 own (see the loop)
    static_assert(NSTAGE == 2, "ping-pong tiles alternate two stages");
    issue(0, 0, Zero{}, One{});
    if (wave >= 4)
      issue(1, 1, Zero{}, One{}); // (nothing when there is one slice)
  } else {
#pragma unroll
    for (int p = 0; p < NSTAGE; ++p)
      issue(p, p, Zero{}, One{});
  }
  __builtin_amdgcn_sched_barrier(0);
  // ---- fragments and accumulators (set up while the first loads fly) --------
  FragAddr<KIND, BM, A_KC, TM> fa_addr;
  FragAddr<KIND, BN, B_KC, TN> fb_addr;
  fa_addr.setup(wm * TM);
  fb_addr.setup(wn * TN);
  Frag<KIND> fa[2][TM], fb[2][TN];

  // Accumulators: value r of 32 x 32 tile (i, j).  With the 16 x 16 shapes
  // that is value r & 3 of the 16 x 16 tile (2 i + (r >> 3), 2 j + ((r >> 2) & 1)).
  typename KindTraits<KIND>::AccVec acc[M16 ? 1 : TM][M16 ? 1 : TN];
  typename KindTraits<KIND>::AccVec4 acc16[M16 ? TM16 : 1][M16 ? TN16 : 1];
  auto acc_get = [&](int i, int j, int r) __attribute__((always_inline)) -> Acc {
    if constexpr (M16)
      return acc16[i * 2 + (r >> 3)][j * 2 + ((r >> 2) & 1)][r & 3];
    else
      return acc[i][j][r];
  };
  auto acc_set = [&](int i, int j, int r, Acc v) __attribute__((always_inline)) {
    if constexpr (M16)
      acc16[i * 2 + (r >> 3)][j * 2 + ((r >> 2) & 1)][r & 3] = v;
    else
      acc[i][j][r] = v;
  };
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        acc_set(i, j, r, 0);
  if constexpr (HALO) {
    // (computed while the prologue's loads are in flight)
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int rt = wm * WM + i * 32 + (l & 31);
      const int64_t m = m0 + rt;
      const bool live = m < m_end;
      const int32_t mm = (int32_t)(live ? m : 0);
      const int32_t pq = conv_div(mm, g.conv.Q, g.conv.magic_q);
      const int32_t q = mm - pq * g.conv.Q;
      const int32_t nn = conv_div(pq, g.conv.P, g.conv.magic_p);
      const int32_t ih0 = pq - nn * g.conv.P - g.conv.pad_h;
      const int32_t iw0 = q - g.conv.pad_w;
      uint32_t mask = 0;
      for (int fr = 0; fr < g.conv.R; ++fr)
        mask |= (uint32_t)(live && (uint32_t)(ih0 + fr * g.conv.dil_h) <
                                       (uint32_t)g.conv.H)
                << fr;
      for (int fs = 0; fs < g.conv.S; ++fs)
        mask |= (uint32_t)((uint32_t)(iw0 + fs * g.conv.dil_w) <
                           (uint32_t)g.conv.W)
                << (16 + fs);
      h_row[i] = rt;
      h_mask[i] = mask;
    }
  }
  if constexpr (PINGPONG) {
    // slice 0 has landed (wavefronts 4..7 keep their share of slice 1 in flight)
    if (wave >= 4 && kt_count > 1)
      __builtin_amdgcn_s_waitcnt(gemm_wait_imm(LPS));
    else
      __builtin_amdgcn_s_waitcnt(gemm_wait_imm(0));
    gemm_barrier();
  } else {
    __builtin_amdgcn_s_waitcnt(gemm_wait_imm(0));
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  }
  // halo mode: per-tap fragment addresses (row base, swizzled chunk bits)
  uint32_t h_base[HALO ? TM : 1], h_x[HALO ? TM : 1];
  auto halo_tap = [&](int kt) {
    const int32_t tap = conv_div(kt, g.conv.slices_per_tap, g.conv.magic_spt);
    const int32_t sl = kt - tap * g.conv.slices_per_tap;
    const int32_t fr = conv_div(tap, g.conv.S, g.conv.magic_s);
    const int32_t fs = tap - fr * g.conv.S;
    const int32_t dpix = fr * g.conv.dil_h * g.conv.W + fs * g.conv.dil_w;
    const uint32_t slab = lds0 + (uint32_t)(sl * g.conv.halo_rows) * kTileKBytes;
#pragma unroll
    for (int i = 0; i < (HALO ? TM : 1); ++i) {
      const bool in = (h_mask[i] >> fr) & (h_mask[i] >> (16 + fs)) & 1;
      const int row = h_row[i] + dpix;
      h_base[i] = in ? slab + (uint32_t)row * kTileKBytes : ring0 - kTileKBytes;
      h_x[i] = (uint32_t)(((l >> 5) ^ kc_swz(row)) << 4);
    }
  };
  auto halo_load = [&](auto ks_c, Frag<KIND> (&f)[TM]) {
    constexpr int ks = decltype(ks_c)::value;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const u32x4 v = *(const GEMM_AS3 u32x4 *)(uintptr_t)(
          h_base[i] + (h_x[i] ^ (uint32_t)(ks << 5)));
      f[i].r[0] = v.x;
      f[i].r[1] = v.y;
      f[i].r[2] = v.z;
      f[i].r[3] = v.w;
    }
  };
  // The in-order loop starts with K-step 0's fragments in hand.  (Not the
  // two-phase loop, which reads whole slices itself: a transposing read is asm
  // whose result nobody would use there, so its registers would be given to
  // other values at once -- and be overwritten when the read returns.)
  if constexpr (!PINGPONG) {
    if constexpr (HALO) {
      halo_tap(0);
      halo_load(Zero{}, fa[0]);
    } else {
      fa_addr.template load<0>(stage_a(0), fa[0]);
    }
    fb_addr.template load<0>(stage_b(0), fb[0]);
    if constexpr (!A_KC || !B_KC) {
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_waitcnt(gemm_wait_imm(63)); // (transposing reads are asm)
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  // Reads per fragment set and the loads of a slice spread over the K-steps
  // that precede the barrier.
  constexpr int NRA = TM * FragAddr<KIND, BM, A_KC, TM>::CHH *
                      (A_KC ? 1 : 2);
  constexpr int NRB = TN * FragAddr<KIND, BN, B_KC, TN>::CHH *
                      (B_KC ? 1 : 2);
  using Two = std::integral_constant<int, 2>;

  int cur = 0; // stage holding slice kt
  if constexpr (PINGPONG) {
    // Two wavefronts share each SIMD.  A K slice is a memory phase (all of the
    // slice's fragment reads and this wavefront's share of a later slice's
    // global -> LDS loads) and an MFMA phase (KSTEPS x TM x TN MFMAs), with a
    // barrier after each; wavefronts 4..7 (team 1) run one phase behind
    // wavefronts 0..3 (team 0), so on every SIMD one wavefront feeds the
    // matrix pipe while the other issues memory instructions.  With g = global
    // phase number:
    //   g = 2 kt     : team 0 reads slice kt, loads its share of slice kt + 1
    //                  into the other stage (team 1 finished reading that
    //                  stage in phase 2 kt - 1)            | team 1: MFMA(kt-1)
    //   g = 2 kt + 1 : team 0: MFMA(kt), then waits for its share of slice
    //                  kt + 1 | team 1 reads slice kt and, once those reads
    //                  have returned, loads its share of slice kt + 2 into the
    //                  same stage (team 0 read it in phase 2 kt); it then
    //                  waits for its share of slice kt + 1
    // so slice kt + 1 is complete when phase 2 kt + 2 starts, and every load
    // has two phases to land.
    // (A wavefront of team 1 requests its share of slice kt + 2 once ITS reads
    // of the stage have returned; its three team mates, released by the same
    // barrier and served by LDS in turns, finish theirs within a few hundred
    // clocks of it, and the requested data is at least a cache round trip and
    // the rest of the phase away.  Requesting after the next barrier instead,
    // in front of the MFMAs, measured 4-5 % slower; dealt out between the
    // MFMAs it needs a loop per team, and then the compiler no longer keeps
    // the asm transposing reads' results where they land.)
    const int team = __builtin_amdgcn_readfirstlane(wave >> 2);
    Frag<KIND> pa[KSTEPS][TM], pb[KSTEPS][TN];
    FragAddr16<KIND, BM, A_KC, TM16> fa16;
    FragAddr16<KIND, BN, B_KC, TN16> fb16;
    Frag<KIND> qa[M16 ? KSTEPS16 : 1][TM16], qb[M16 ? KSTEPS16 : 1][TN16];
    if constexpr (M16) {
      fa16.setup(wm * TM16);
      fb16.setup(wn * TN16);
    }
    if (team)
      gemm_barrier();
    for (int kt = 0; kt < kt_count; ++kt) {
      const int nxt = cur ^ 1;
      // ---- memory phase
      const uint32_t sa = stage_a(cur), sb = stage_b(cur);
      if constexpr (M16) {
        gemm_static_for<KSTEPS16>([&](auto uc) {
          constexpr int u = decltype(uc)::value;
          fa16.template load<u>(sa, qa[u]);
          fb16.template load<u>(sb, qb[u]);
        });
      } else {
        gemm_static_for<KSTEPS>([&](auto uc) {
          constexpr int u = decltype(uc)::value;
          fa_addr.template load<u>(sa, pa[u]);
          fb_addr.template load<u>(sb, pb[u]);
        });
      }
      if (team) {
        __builtin_amdgcn_s_waitcnt(gemm_wait_imm(63)); // the reads returned
        issue(kt + 2, cur, Zero{}, One{});
        // its share of slice kt + 1 (one batch older) has landed
        if (kt + 2 < kt_count)
          __builtin_amdgcn_s_waitcnt(gemm_wait_imm(LPS));
        else
          __builtin_amdgcn_s_waitcnt(gemm_wait_imm(0));
      } else {
        issue(kt + 1, nxt, Zero{}, One{});
        // the reads returned: the other team may overwrite the stage next
        __builtin_amdgcn_s_waitcnt(gemm_wait_imm(63));
      }
      __builtin_amdgcn_sched_barrier(0);
      gemm_barrier();
      __builtin_amdgcn_sched_barrier(0);
      // ---- MFMA phase
      __builtin_amdgcn_s_setprio(1);
      if constexpr (M16) {
        gemm_static_for<KSTEPS16>([&](auto uc) {
          constexpr int u = decltype(uc)::value;
#pragma unroll
          for (int i = 0; i < TM16; ++i)
#pragma unroll
            for (int j = 0; j < TN16; ++j)
              mfma16<KIND>(acc16[i][j], qa[u][i], qb[u][j]);
        });
      } else {
        gemm_static_for<KSTEPS>([&](auto uc) {
          constexpr int u = decltype(uc)::value;
#pragma unroll
          for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
              mfma32<KIND>(acc[i][j], pa[u][i], pb[u][j]);
        });
      }
      __builtin_amdgcn_s_setprio(0);
      __builtin_amdgcn_sched_barrier(0);
      if (!team)
        __builtin_amdgcn_s_waitcnt(gemm_wait_imm(0)); // its share of slice kt + 1
      gemm_barrier();
      __builtin_amdgcn_sched_barrier(0);
      cur = nxt;
    }
    if (!team)
      gemm_barrier();
  } else {
  // One K slice.  A stage is free again once the barrier of the iteration
  // that consumes it has passed, and is refilled at once with the slice
  // NSTAGE ahead: first half of its loads behind the MFMAs of the last
  // K-step, second half behind K-step 0 of the next iteration.  Every K-step
  // is one basic block, so the recipe can interleave.
  for (int kt = 0; kt < kt_count; ++kt) {
    const int nxt = cur + 1 == NSTAGE ? 0 : cur + 1;
    const int prv = cur == 0 ? NSTAGE - 1 : cur - 1;
    const uint32_t sa = stage_a(cur), sb = stage_b(cur);
    gemm_static_for<KSTEPS>([&](auto sc) {
      constexpr int s = decltype(sc)::value;
      constexpr int fc = s & 1, fn = fc ^ 1;
      constexpr bool LAST = s + 1 == KSTEPS;
      if constexpr (!LAST) {
        if constexpr (HALO)
          halo_load(std::integral_constant<int, s + 1>{}, fa[fn]);
        else
          fa_addr.template load<s + 1>(sa, fa[fn]);
        fb_addr.template load<s + 1>(sb, fb[fn]);
        if constexpr (s == 0)
          issue(kt + NSTAGE - 1, prv, One{}, Two{});
      } else {
        // Slice kt + 1 must be in LDS (this thread's DMA, then everyone's),
        // and every fragment read of this stage must have returned before
        // it is refilled.
        // (all but the NSTAGE - 2 slices behind it; everything where slices
        // past the end were not loaded)
        if (kt + NSTAGE - 1 < kt_count)
          __builtin_amdgcn_s_waitcnt(gemm_wait_imm((NSTAGE - 2) * LPS));
        else
          __builtin_amdgcn_s_waitcnt(gemm_wait_imm(0));
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (HALO) {
          halo_tap(kt + 1 < kt_count ? kt + 1 : kt);
          halo_load(Zero{}, fa[fn]);
        } else {
          fa_addr.template load<0>(stage_a(nxt), fa[fn]);
        }
        fb_addr.template load<0>(stage_b(nxt), fb[fn]);
        issue(kt + NSTAGE, cur, Zero{}, Two{});
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          mfma32<KIND>(acc[i][j], fa[fc][i], fb[fc][j]);
      constexpr int NV = LAST ? LPS / 2 : (s == 0 ? LPS - LPS / 2 : 0);
      gemm_interleave<TM * TN, NRA + NRB, NV>();
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (!A_KC || !B_KC) {
        // the next step's transposing reads (asm: the compiler does not wait
        // for them), issued a K-step of MFMAs ago
        __builtin_amdgcn_s_waitcnt(gemm_wait_imm(63));
        __builtin_amdgcn_sched_barrier(0);
      }
    });
    cur = nxt;
  }
  }
  // (nothing is in flight any more; the stages become the epilogue's bands)
  __builtin_amdgcn_s_waitcnt(gemm_wait_imm(0));
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");

  // ---- epilogue -------------------------------------------------------------
  // Each wavefront moves its accumulators through private LDS bands of 32
  // rows x WN columns (row pitch padded by 32 bytes), BANDS tile rows at a
  // time, and reads them back with 8 consecutive columns per lane.
  constexpr int PITCH = L::kEpiPitch;
  constexpr int BANDS = L::kBands;
  constexpr int LPR = WN / 8;   // lanes per row
  constexpr int RPP = 64 / LPR; // rows per pass
  constexpr int PPB = 32 / RPP; // passes per band
  const uint32_t band = lds0 + (uint32_t)wave * (BANDS * L::kBand);
  // a lane's value r of tile (., j) lands at wr + row_of(r) * PITCH + col_of(j, r)
  // (16 x 16 shapes: a K-contiguous operand's fragments hold the tile rows in
  // the order row16, so the output's row blocks 2 and 3 (A) or its columns (B)
  // come out exchanged the same way)
  const int g16 = A_KC ? (l >> 4) ^ (l >> 5) : l >> 4;
  const int c16 = B_KC ? Frag16Geom<KIND>::row16(l & 15) : l & 15;
  const uint32_t wr =
      band + (uint32_t)(M16 ? g16 * 4 * PITCH + c16 * 4
                            : (l >> 5) * 4 * PITCH + (l & 31) * 4);
  auto row_of = [](int r) { return M16 ? (r >> 3) * 16 + (r & 3) : (r >> 2) * 8 + (r & 3); };
  auto col_of = [](int j, int r) { return M16 ? j * 128 + ((r >> 2) & 1) * 64 : j * 128; };
  const uint32_t rd = band + (uint32_t)((l / LPR) * PITCH + (l % LPR) * 32);
  const int64_t ob = batch * g.o_batch + outer * g.o_outer;
  const int64_t ncol = n0 + wn * WN + (l % LPR) * 8;

  // Lean path: the epilogue is linear with scalar / per-column operands (bias,
  // scale, ReLU ...), the output rows allow aligned 16-byte stores and this
  // wavefront has no ragged columns.  A lane's 8 columns are the same in
  // every pass, so each operand is loaded once, before the passes.
  const int64_t n_store = g.n_store ? g.n_store : g.N;
  const bool lane_full = ncol + 8 <= n_store || ncol >= n_store;
  const bool lean = g.epi_reg && g.o_vec != 0 &&
                    __builtin_amdgcn_ballot_w64(!lane_full) == 0;
  const int64_t esz = fhip_dtype_size(g.o_dt);
  GEMM_AS1 char *lean_ptr =
      (GEMM_AS1 char *)g.out +
      (ob + (m0 + wm * WM + l / LPR) * g.o_sm + ncol) * esz;
  const int64_t lean_m = m0 + wm * WM + l / LPR;
  const int64_t row_bytes = g.o_sm * esz;
  const int nops = g.epi.count;
  const int64_t gM = m_end, gN = n_store; // rows and columns that are stored
  const int o_dt = g.o_dt;

  // Lean path, step 1: the chain runs on the accumulators where they are.  A
  // lane's accumulators of column tile j all belong to one output column, so
  // an op is y <- y * S + T with one (S, T) pair of registers per (op, j):
  // (operand, -0) for MUL, (a, b * operand) for the additive modes.
  if constexpr (!std::is_same<Acc, int>::value) {
    if (lean && nops > 0) {
      // (column tiles of 16 with the 16 x 16 shapes)
      constexpr int CT = M16 ? TN16 : TN, CW = M16 ? 16 : 32;
      float S[FHIP_MAX_EPILOGUE][CT], T[FHIP_MAX_EPILOGUE][CT];
      int lin_relu[FHIP_MAX_EPILOGUE];
      gemm_static_for<FHIP_MAX_EPILOGUE>([&](auto ec) {
        constexpr int e = decltype(ec)::value;
        lin_relu[e] = g.lin_relu[e];
        if (e >= nops)
          return;
        const DevEpiOp &o = g.epi.op[e];
        const bool mul = g.lin_mul[e] != 0;
        const float a = g.lin_a[e], b = g.lin_b[e];
#pragma unroll
        for (int j = 0; j < CT; ++j) {
          float ov;
          if (o.kind == FHIP_OPERAND_TENSOR) {
            int64_t n = n0 + wn * WN + j * CW + (M16 ? c16 : l & 31);
            n = n < g.N ? n : g.N - 1;
            const int64_t off[1] = {(n + outer * g.epi_n_outer) * o.stride[2]};
            float one[1];
            load_operand_vec<1>(o.ptr, o.operand_dtype, off, one);
            ov = one[0];
          } else {
            ov = o.kind == FHIP_OPERAND_SCALAR ? o.scalar : 0.f;
          }
          S[e][j] = mul ? ov : a;
          T[e][j] = mul ? -0.f : b * ov;
        }
      });
      gemm_static_for<FHIP_MAX_EPILOGUE>([&](auto ec) {
        constexpr int e = decltype(ec)::value;
        if (e >= nops)
          return;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const int c = M16 ? j * 2 + ((r >> 2) & 1) : j;
              acc_set(i, j, r, __builtin_fmaf(acc_get(i, j, r), S[e][c], T[e][c]));
            }
        if (lin_relu[e]) {
          // one instruction per value (fmaxf would first quiet its input);
          // NaN -> 0 like fmaxf
#pragma unroll
          for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
              for (int r = 0; r < 16; ++r) {
                float y = acc_get(i, j, r);
                asm("v_max_f32 %0, 0, %0" : "+v"(y));
                acc_set(i, j, r, y);
              }
        }
      });
    }
  }
  // Step 2, 16-bit outputs: the values are rounded here and leave through LDS
  // as packed pairs of consecutive rows (half the LDS traffic and passes).
  const bool packed = !std::is_same<Acc, int>::value && lean &&
                      (o_dt == FHIP_BFLOAT16 || o_dt == FHIP_HALF);
  const uint32_t wr2 =
      band + (uint32_t)(M16 ? g16 * 2 * PITCH + c16 * 4
                            : (l >> 5) * 2 * PITCH + (l & 31) * 4);
  auto pair_row_of = [](int r) {
    return M16 ? (r >> 3) * 8 + ((r & 3) >> 1) : (r >> 2) * 4 + ((r & 3) >> 1);
  };

  gemm_static_for<TM / BANDS>([&](auto rc) {
    constexpr int round = decltype(rc)::value;
    if constexpr (!std::is_same<Acc, int>::value) {
      if (packed) {
        // pair-row k of a band holds rows 2k and 2k + 1 as (low, high) halves
        auto run = [&](auto ot_c) {
          constexpr int OT = decltype(ot_c)::value; // 1 bf16, 2 f16
#pragma unroll
          for (int bi = 0; bi < BANDS; ++bi)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
              for (int r = 0; r < 16; r += 2) {
                const float lo = acc_get(round * BANDS + bi, j, r);
                const float hi = acc_get(round * BANDS + bi, j, r + 1);
                uint32_t pk;
                if constexpr (OT == 1) {
                  typedef __bf16 b2 __attribute__((ext_vector_type(2)));
                  pk = __builtin_bit_cast(uint32_t, b2{(__bf16)lo, (__bf16)hi});
                } else {
                  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
                  pk = __builtin_bit_cast(uint32_t,
                                          h2{(_Float16)lo, (_Float16)hi});
                }
                *(GEMM_AS3 uint32_t *)(uintptr_t)(
                    wr2 + bi * L::kBand + pair_row_of(r) * PITCH + col_of(j, r)) = pk;
              }
          // a pass covers RPP pair-rows = 2 * RPP rows
          constexpr int PPB2 = 16 / RPP;
#pragma unroll
          for (int p = 0; p < BANDS * PPB2; ++p) {
            const int bi = p / PPB2, pp = p % PPB2;
            const int rel = (round * BANDS + bi) * 32 + pp * 2 * RPP;
            const uint32_t src = rd + bi * L::kBand + pp * RPP * PITCH;
            const u32x4 v0 = *(const GEMM_AS3 u32x4 *)(uintptr_t)(src);
            const u32x4 v1 = *(const GEMM_AS3 u32x4 *)(uintptr_t)(src + 16);
            // lane's rows: lean_m' = tile row of pair-row (l / LPR)
            const int64_t mrow = m0 + wm * WM + rel + 2 * (l / LPR);
            if (ncol >= gN || mrow >= gM)
              continue;
            GEMM_AS1 char *dst =
                (GEMM_AS1 char *)g.out + (ob + mrow * g.o_sm + ncol) * 2;
            const u32x4 even = {
                __builtin_amdgcn_perm(v0.y, v0.x, 0x05040100u),
                __builtin_amdgcn_perm(v0.w, v0.z, 0x05040100u),
                __builtin_amdgcn_perm(v1.y, v1.x, 0x05040100u),
                __builtin_amdgcn_perm(v1.w, v1.z, 0x05040100u)};
            const u32x4 odd = {
                __builtin_amdgcn_perm(v0.y, v0.x, 0x07060302u),
                __builtin_amdgcn_perm(v0.w, v0.z, 0x07060302u),
                __builtin_amdgcn_perm(v1.y, v1.x, 0x07060302u),
                __builtin_amdgcn_perm(v1.w, v1.z, 0x07060302u)};
            __builtin_nontemporal_store(even, (GEMM_AS1 u32x4 *)dst);
            if (mrow + 1 < gM)
              __builtin_nontemporal_store(odd,
                                          (GEMM_AS1 u32x4 *)(dst + row_bytes));
          }
        };
        if (o_dt == FHIP_BFLOAT16)
          run(std::integral_constant<int, 1>{});
        else
          run(std::integral_constant<int, 2>{});
        return;
      }
    }
#pragma unroll
    for (int bi = 0; bi < BANDS; ++bi)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          *(GEMM_AS3 Acc *)(uintptr_t)(wr + bi * L::kBand + row_of(r) * PITCH +
                                       col_of(j, r)) =
              acc_get(round * BANDS + bi, j, r);
    if (lean) {
      // 4-byte outputs (the chain has already run on the accumulators)
#pragma unroll
      for (int p = 0; p < BANDS * PPB; ++p) {
        const int bi = p / PPB, pp = p % PPB;
        const int rel = (round * BANDS + bi) * 32 + pp * RPP;
        const uint32_t src = rd + bi * L::kBand + pp * RPP * PITCH;
        const u32x4 v0 = *(const GEMM_AS3 u32x4 *)(uintptr_t)(src);
        const u32x4 v1 = *(const GEMM_AS3 u32x4 *)(uintptr_t)(src + 16);
        if (lean_m + rel >= gM || ncol >= gN)
          continue;
        GEMM_AS1 char *dst = lean_ptr + rel * row_bytes;
        *(GEMM_AS1 u32x4 *)dst = v0;
        *(GEMM_AS1 u32x4 *)(dst + 16) = v1;
      }
      return;
    }
#pragma clang loop unroll(disable)
    for (int p = 0; p < BANDS * PPB; ++p) {
      const int bi = p / PPB, pp = p % PPB;
      const int64_t m =
          m0 + wm * WM + (round * BANDS + bi) * 32 + pp * RPP + l / LPR;
      const uint32_t src = rd + bi * L::kBand + pp * RPP * PITCH;
      const u32x4 v0 = *(const GEMM_AS3 u32x4 *)(uintptr_t)(src);
      const u32x4 v1 = *(const GEMM_AS3 u32x4 *)(uintptr_t)(src + 16);
      if (m >= m_end || ncol >= n_store)
        continue;
      const bool full = ncol + 8 <= n_store;
      const int64_t o0 = ob + m * g.o_sm + ncol * g.o_sn;
      if constexpr (std::is_same<Acc, int>::value) {
        GEMM_AS1 int32_t *out = (GEMM_AS1 int32_t *)g.out;
        if (full && g.o_vec) {
          *(GEMM_AS1 u32x4 *)(out + o0) = v0;
          *(GEMM_AS1 u32x4 *)(out + o0 + 4) = v1;
        } else {
          const uint32_t y[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (ncol + e < n_store)
              out[o0 + e * g.o_sn] = (int32_t)y[e];
        }
      } else {
        // (element-wise copies first: bit-casting a vector element directly
        // reads element 0)
        const uint32_t w[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
        float y[8];
#pragma unroll
        for (int c = 0; c < 8; ++c)
          y[c] = __builtin_bit_cast(float, w[c]);
        fhip_round_fast_vec<8>(g.c_dt, y);
        for (int e = 0; e < nops; ++e) {
          const DevEpiOp &o = g.epi.op[e];
          if (o.kind == FHIP_OPERAND_NONE) {
            fhip_pw_fast_unary_vec<true, 8>(o.mode, y, o.params.swish_beta);
          } else {
            float other[8];
            if (o.kind == FHIP_OPERAND_SCALAR) {
#pragma unroll
              for (int c = 0; c < 8; ++c)
                other[c] = o.scalar;
            } else {
              const int64_t base = batch * o.stride[0] + m * o.stride[1];
              int64_t off[8];
#pragma unroll
              for (int c = 0; c < 8; ++c) {
                int64_t n = ncol + c;
                n = n < g.N ? n : g.N - 1; // edge tiles stay in bounds
                off[c] = base + (n + outer * g.epi_n_outer) * o.stride[2];
              }
              load_operand_vec<8>(o.ptr, o.operand_dtype, off, other);
            }
            fhip_pw_fast_binary_vec<8>(o.mode, o.acc_is_in1 != 0, y, other);
          }
          fhip_round_fast_vec<8>(o.result_dtype, y);
        }
        if (g.o_dt == FHIP_FLOAT) {
          GEMM_AS1 float *out = (GEMM_AS1 float *)g.out;
          if (full && g.o_vec) {
            typedef float f32x4 __attribute__((ext_vector_type(4)));
            *(GEMM_AS1 f32x4 *)(out + o0) = f32x4{y[0], y[1], y[2], y[3]};
            *(GEMM_AS1 f32x4 *)(out + o0 + 4) = f32x4{y[4], y[5], y[6], y[7]};
          } else {
#pragma unroll
            for (int c = 0; c < 8; ++c)
              if (ncol + c < n_store)
                out[o0 + c * g.o_sn] = y[c];
          }
        } else if (g.o_dt == FHIP_BFLOAT16) {
          GEMM_AS1 __bf16 *out = (GEMM_AS1 __bf16 *)g.out;
          if (full && g.o_vec) {
            bf16x8 v;
#pragma unroll
            for (int c = 0; c < 8; ++c)
              v[c] = (__bf16)y[c];
            *(GEMM_AS1 bf16x8 *)(out + o0) = v;
          } else {
#pragma unroll
            for (int c = 0; c < 8; ++c)
              if (ncol + c < n_store)
                out[o0 + c * g.o_sn] = (__bf16)y[c];
          }
        } else {
          GEMM_AS1 _Float16 *out = (GEMM_AS1 _Float16 *)g.out;
          if (full && g.o_vec) {
            f16x8 v;
#pragma unroll
            for (int c = 0; c < 8; ++c)
              v[c] = (_Float16)y[c];
            *(GEMM_AS1 f16x8 *)(out + o0) = v;
          } else {
#pragma unroll
            for (int c = 0; c < 8; ++c)
              if (ncol + c < n_store)
                out[o0 + c * g.o_sn] = (_Float16)y[c];
          }
        }
      }
    }
  });
}

// Decides whether the epilogue can run on the accumulators in registers and
// fills its linear form.  `g.epi` must hold the (batch, m, n) strides already.
inline void gemm_fill_linear(const fhip_epilogue &e, GemmArgs &g) {
  g.epi_reg = 0;
  if (e.count == 0) {
    // the store's conversion is the only rounding
    g.epi_reg = g.c_dt == FHIP_FLOAT || g.c_dt == g.o_dt;
    return;
  }
  // no rounding between the steps: every intermediate is f32 (the last
  // result may already have the stored type, which the store's conversion
  // reproduces)
  if (g.c_dt != FHIP_FLOAT)
    return;
  for (int i = 0; i < e.count; ++i) {
    const int dt = e.op[i].result_dtype;
    if (dt != FHIP_FLOAT && !(i + 1 == e.count && dt == g.o_dt))
      return;
  }
  for (int i = 0; i < e.count; ++i) {
    const fhip_epilogue_op &o = e.op[i];
    float a = 1.f, b = 0.f;
    int mul = 0, relu = 0;
    switch (o.mode) {
    case FHIP_PW_ADD:
      b = 1.f;
      break;
    case FHIP_PW_SUB: // IN_0 - IN_1
      a = o.acc_is_in1 ? -1.f : 1.f;
      b = o.acc_is_in1 ? 1.f : -1.f;
      break;
    case FHIP_PW_MUL:
      mul = 1;
      break;
    case FHIP_PW_RELU_FWD:
      relu = 1;
      break;
    case FHIP_PW_NEG:
      a = -1.f;
      break;
    case FHIP_PW_IDENTITY:
      break;
    default:
      return;
    }
    // tensor operands must depend on the column only
    if (o.operand_kind == FHIP_OPERAND_TENSOR &&
        (g.epi.op[i].stride[0] != 0 || g.epi.op[i].stride[1] != 0))
      return;
    g.lin_a[i] = a;
    g.lin_b[i] = b;
    g.lin_mul[i] = mul;
    g.lin_relu[i] = relu;
  }
  g.epi_reg = 1;
}

// What the host decided about one matmul call.
struct GemmPlan {
  bool ok = false;
  int kind = 0;
  bool a_kc = true, b_kc = true;
  int64_t M = 0, N = 0, K = 0, batch = 1;
  int64_t a_ld = 0, b_ld = 0, a_batch = 0, b_batch = 0;
  int64_t o_sm = 0, o_sn = 0, o_batch = 0;
  int bm = 256, bn = 256;
  // parts the reduction is cut into (f32 partial results in the context's
  // scratch, added by a second kernel); 1: none
  int ksplit = 1;
};

// Stage count per tile: as many as fit the 160 KB LDS, at most 4.
template <int BM, int BN> struct GemmStages {
  static constexpr int kStage = (BM + BN) * kTileKBytes;
  static constexpr int value = 160 * 1024 / kStage >= 4 ? 4 : 160 * 1024 / kStage;
};

template <> struct GemmStages<256, 128> {
  static constexpr int value = 2; // the ping-pong loop alternates two stages
};

template <int BM, int BN> struct GemmWaves {
  static constexpr int value = BM == 256 && BN == 128 ? 8 : GemmLayout<BM, BN>::kWaves;
};

template <int KIND, int BM, int BN, int A_MODE, bool B_KC, int STAGES = 0, int WAVES = 0>
int launch(fhip_ctx *ctx, const GemmArgs &g, int64_t batch) {
  constexpr int NSTAGE = STAGES ? STAGES : GemmStages<BM, BN>::value;
  constexpr int NW = WAVES ? WAVES : GemmWaves<BM, BN>::value;
  constexpr int lds = GemmLds<BM, BN, NSTAGE, NW>::kBytes;
  auto kernel = gemm_kernel<KIND, BM, BN, A_MODE, B_KC, NSTAGE, NW>;
  static FhipOncePerDevice configured;
  if (!configured.done(ctx->device)) {
    FHIP_HIP_CHECK(ctx, hipFuncSetAttribute(
                            reinterpret_cast<const void *>(kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    configured.mark(ctx->device);
  }
  const dim3 grid((unsigned)(g.tiles_m * g.tiles_n), (unsigned)batch,
                  (unsigned)(g.outer > 1 ? g.outer : 1));
  hipLaunchKernelGGL(kernel, grid, dim3(NW * 64), lds, ctx->stream, g);
  FHIP_HIP_CHECK(ctx, hipGetLastError());
  return 0;
}

template <int KIND, int BM, int BN, int STAGES = 0, int WAVES = 0>
int launch_orient(fhip_ctx *ctx, const GemmPlan &p, const GemmArgs &g) {
  if (p.a_kc && p.b_kc)
    return launch<KIND, BM, BN, A_KCONTIG, true, STAGES, WAVES>(ctx, g, p.batch);
  if (p.a_kc && !p.b_kc)
    return launch<KIND, BM, BN, A_KCONTIG, false, STAGES, WAVES>(ctx, g, p.batch);
  if (!p.a_kc && p.b_kc)
    return launch<KIND, BM, BN, A_MCONTIG, true, STAGES, WAVES>(ctx, g, p.batch);
  return launch<KIND, BM, BN, A_MCONTIG, false, STAGES, WAVES>(ctx, g, p.batch);
}

template <int KIND>
int gemm_launch_kind(fhip_ctx *ctx, const GemmPlan &p, const GemmArgs &g) {
  if (p.bm == 256 && p.bn == 256)
    return launch_orient<KIND, 256, 256>(ctx, p, g);
  if (p.bm == 256 && p.bn == 128)
    return launch_orient<KIND, 256, 128>(ctx, p, g);
  // (eight wavefronts of 64 x 32 in two phases, two stages: two workgroups per
  // compute unit at 116-118 registers a lane)
  return launch_orient<KIND, 128, 128, 2, 8>(ctx, p, g);
}

// Implicit-GEMM convolution launchers (A gathered, B = filter, K-contiguous).
template <int KIND>
int conv_launch_kind(fhip_ctx *ctx, int bm, int bn, const GemmArgs &g) {
  if (bm == 512 && bn == 128)
    return launch<KIND, 512, 128, A_CONV, true>(ctx, g, 1);
  if (bm == 256 && bn == 256)
    return launch<KIND, 256, 256, A_CONV, true>(ctx, g, 1);
  if (bm == 256 && bn == 128)
    return launch<KIND, 256, 128, A_CONV, true>(ctx, g, 1);
  // eight wavefronts in two phases on two stages: two workgroups share a
  // compute unit, and one's prologue and epilogue hide behind the other's K
  // loop (convolutions have short K)
  return launch<KIND, 128, 128, A_CONV, true, 2, 8>(ctx, g, 1);
}

// Halo mode: 128 x 128 tiles with three filter stages behind the slab, or
// 256 x 128 tiles with two.
// Outputs of at most 64 channels take 64-wide column tiles (no padded MFMA
// columns).
template <int BM, int BN = 128> struct HaloShape {
  static constexpr int kStages = BM == 256 || BN == 64 ? 2 : 3;
  static constexpr int kRingBytes = kStages * BN * kTileKBytes;
};
template <int KIND, int BM, int BN = 128>
int conv_launch_halo(fhip_ctx *ctx, const GemmArgs &g) {
  constexpr int STAGES = HaloShape<BM, BN>::kStages;
  using L = GemmLds<BM, BN, STAGES, 4, true>;
  const int main_bytes = (int)g.conv.slab_bytes + HaloShape<BM, BN>::kRingBytes;
  // (the epilogue's bands stay within 80 KB so that two workgroups keep
  // sharing a compute unit)
  const int lds = main_bytes > L::kEpiBytes ? main_bytes : L::kEpiBytes;
  auto kernel = gemm_kernel<KIND, BM, BN, A_HALO, true, STAGES, 4>;
  static FhipOncePerDevice configured;
  if (!configured.done(ctx->device)) {
    FHIP_HIP_CHECK(ctx, hipFuncSetAttribute(
                            reinterpret_cast<const void *>(kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize,
                            160 * 1024));
    configured.mark(ctx->device);
  }
  const dim3 grid((unsigned)(g.tiles_m * g.tiles_n), 1,
                  (unsigned)(g.outer > 1 ? g.outer : 1));
  hipLaunchKernelGGL(kernel, grid, dim3(256), lds, ctx->stream, g);
  FHIP_HIP_CHECK(ctx, hipGetLastError());
  return 0;
}

int gemm_launch_bf16(fhip_ctx *ctx, const GemmPlan &p, const GemmArgs &g);
int gemm_launch_f16(fhip_ctx *ctx, const GemmPlan &p, const GemmArgs &g);
int gemm_launch_i8(fhip_ctx *ctx, const GemmPlan &p, const GemmArgs &g);
int gemm_launch_fp8e4m3(fhip_ctx *ctx, const GemmPlan &p, const GemmArgs &g);
int gemm_launch_fp8e5m2(fhip_ctx *ctx, const GemmPlan &p, const GemmArgs &g);

#endif // FUSILLI_AMD_CSRC_GEMM_KERNEL_H
