// MFMA GEMM kernel template and launch helpers; instantiated once per element
// kind in gemm_<kind>.hip.
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
};
template <> struct KindTraits<GK_F16> {
  static constexpr int kElemBytes = 2;
  static constexpr int kStepBytes = 32;
  using Acc = float;
  using AccVec = f32x16;
};
template <> struct KindTraits<GK_I8> {
  static constexpr int kElemBytes = 1;
  static constexpr int kStepBytes = 32;
  using Acc = int;
  using AccVec = i32x16;
};
template <> struct KindTraits<GK_FP8E4M3> {
  static constexpr int kElemBytes = 1;
  static constexpr int kStepBytes = 64;
  using Acc = float;
  using AccVec = f32x16;
};
template <> struct KindTraits<GK_FP8E5M2> {
  static constexpr int kElemBytes = 1;
  static constexpr int kStepBytes = 64;
  using Acc = float;
  using AccVec = f32x16;
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
  int32_t H, W, C;        // input spatial extents and channels
  int32_t P, Q;           // output spatial extents
  int32_t S;              // filter width (taps per filter row)
  int32_t pad_h, pad_w, str_h, str_w, dil_h, dil_w;
  int32_t slices_per_tap; // C * elem / 128
};

enum GemmAMode { A_KCONTIG = 0, A_MCONTIG = 1, A_CONV = 2 };

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
  int32_t c_dt, o_dt;
  int32_t tiles_m, tiles_n;
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

// LDS geometry of one operand slice.
//   K-contiguous operand: ROWS rows (m or n) of 128 K-bytes, row pitch 144 B
//   (16-byte reads by 16 lanes of consecutive rows then touch 64 distinct banks).
//   Other operand: 128/elem K-rows of ROWS*elem bytes; the row pitch is chosen
//   so the transposing 8-byte reads of a 32-lane half-wavefront are conflict
//   free (K-rows 16 words apart for 16-bit, 8 words apart for 8-bit elements).
template <int ROWS, int ELEM, bool KCONTIG> struct SliceGeom {
  static constexpr int kKRows = kTileKBytes / ELEM;
  static constexpr int kPitch =
      KCONTIG ? (kTileKBytes + 16)
              : (ROWS * ELEM + (ELEM == 2 ? 64 : 32));
  static constexpr int kBytes = KCONTIG ? ROWS * kPitch : kKRows * kPitch;
  // 16-byte chunks a thread moves per slice
  static constexpr int kChunks = ROWS * kTileKBytes / 16 / kThreads;
};

// Global -> registers for one slice of one operand.
template <int ROWS, int ELEM, bool KCONTIG>
__device__ __forceinline__ void
load_slice(const char *base, int64_t ld_bytes, int64_t row0, int64_t rows_total,
           int64_t k0_bytes, u32x4 (&regs)[SliceGeom<ROWS, ELEM, KCONTIG>::kChunks]) {
  using G = SliceGeom<ROWS, ELEM, KCONTIG>;
  const int t = threadIdx.x;
#pragma unroll
  for (int i = 0; i < G::kChunks; ++i) {
    const int c = t + i * kThreads;
    if constexpr (KCONTIG) {
      const int row = c >> 3, col = c & 7; // 8 chunks of 16 B per 128-B row
      int64_t r = row0 + row;
      r = r < rows_total ? r : rows_total - 1; // clamp: ragged edge tiles
      regs[i] = *reinterpret_cast<const u32x4 *>(base + r * ld_bytes + k0_bytes +
                                                 col * 16);
    } else {
      constexpr int cpr = ROWS * ELEM / 16; // chunks per K-row
      const int krow = c / cpr, col = c % cpr;
      // element index along the row dimension, clamped at the edge
      int64_t e = row0 + (int64_t)col * (16 / ELEM);
      const int64_t last = rows_total - 16 / ELEM;
      e = e < last ? e : last;
      regs[i] = *reinterpret_cast<const u32x4 *>(
          base + (k0_bytes / ELEM + krow) * ld_bytes + e * ELEM);
    }
  }
}

template <int ROWS, int ELEM, bool KCONTIG>
__device__ __forceinline__ void
store_slice(char *lds, const u32x4 (&regs)[SliceGeom<ROWS, ELEM, KCONTIG>::kChunks]) {
  using G = SliceGeom<ROWS, ELEM, KCONTIG>;
  const int t = threadIdx.x;
#pragma unroll
  for (int i = 0; i < G::kChunks; ++i) {
    const int c = t + i * kThreads;
    if constexpr (KCONTIG) {
      const int row = c >> 3, col = c & 7;
      *reinterpret_cast<u32x4 *>(lds + row * G::kPitch + col * 16) = regs[i];
    } else {
      constexpr int cpr = ROWS * ELEM / 16;
      const int krow = c / cpr, col = c % cpr;
      *reinterpret_cast<u32x4 *>(lds + krow * G::kPitch + col * 16) = regs[i];
    }
  }
}

// LDS -> MFMA fragment for rows [rb*32, rb*32+32) at K-step `s` of the slice.
template <int KIND, int ROWS, bool KCONTIG>
__device__ __forceinline__ void load_frag(const char *lds, int rb, int s,
                                          Frag<KIND> &f) {
  constexpr int ELEM = KindTraits<KIND>::kElemBytes;
  constexpr int STEPB = KindTraits<KIND>::kStepBytes;
  using G = SliceGeom<ROWS, ELEM, KCONTIG>;
  const int l = threadIdx.x & 63;
  if constexpr (KCONTIG) {
    const char *p = lds + (rb * 32 + (l & 31)) * G::kPitch + s * STEPB +
                    (l >> 5) * (STEPB / 2);
#pragma unroll
    for (int i = 0; i < STEPB / 32; ++i) {
      const u32x4 v = *reinterpret_cast<const u32x4 *>(p + 16 * i);
      f.r[4 * i + 0] = v.x;
      f.r[4 * i + 1] = v.y;
      f.r[4 * i + 2] = v.z;
      f.r[4 * i + 3] = v.w;
    }
  } else {
    // Elements of K this lane needs: (STEPB / 2) / ELEM consecutive K-rows.
    constexpr int KPL = STEPB / 2 / ELEM;
    const int kbase = s * (STEPB / ELEM) + (l >> 5) * KPL;
    const int L = l & 15;
    const int nsub = rb * 32 + ((l >> 4) & 1) * 16;
    if constexpr (ELEM == 2) {
      // 16 lanes cover 4 K-rows x 16 columns; a read returns 4 K values.
#pragma unroll
      for (int r = 0; r < KPL / 4; ++r) {
        const int k = kbase + 4 * r + (L >> 2);
        const int n = nsub + 4 * (L & 3);
        const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            LDS_PTR(s16x4, lds, k * G::kPitch + n * 2));
        const u32x2 w = __builtin_bit_cast(u32x2, v);
        f.r[2 * r + 0] = w.x;
        f.r[2 * r + 1] = w.y;
      }
    } else {
      // 16 lanes cover 8 K-rows x 16 columns; a read returns 8 K values.
#pragma unroll
      for (int r = 0; r < KPL / 8; ++r) {
        const int k = kbase + 8 * r + (L >> 1);
        const int n = nsub + 8 * (L & 1);
        const i32x2 v = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
            LDS_PTR(i32x2, lds, k * G::kPitch + n));
        f.r[2 * r + 0] = (uint32_t)v.x;
        f.r[2 * r + 1] = (uint32_t)v.y;
      }
    }
  }
}

template <int N>
__device__ __forceinline__ void load_operand_vec(const void *p, int dt,
                                                 const int64_t (&off)[N],
                                                 float (&o)[N]) {
  if (dt == FHIP_FLOAT) {
#pragma unroll
    for (int i = 0; i < N; ++i)
      o[i] = ((const float *)p)[off[i]];
  } else if (dt == FHIP_BFLOAT16) {
#pragma unroll
    for (int i = 0; i < N; ++i)
      o[i] = (float)((const __bf16 *)p)[off[i]];
  } else {
#pragma unroll
    for (int i = 0; i < N; ++i)
      o[i] = (float)((const _Float16 *)p)[off[i]];
  }
}

template <int KIND, int BM, int BN, int A_MODE, bool B_KC>
__global__ __launch_bounds__(kThreads) void gemm_kernel(GemmArgs g) {
  using Acc = typename KindTraits<KIND>::Acc;
  constexpr bool A_KC = A_MODE != A_MCONTIG;
  constexpr int ELEM = KindTraits<KIND>::kElemBytes;
  constexpr int STEPB = KindTraits<KIND>::kStepBytes;
  constexpr int KSTEPS = kTileKBytes / STEPB;
  using GA = SliceGeom<BM, ELEM, A_KC>;
  using GB = SliceGeom<BN, ELEM, B_KC>;
  constexpr int WM = BM / 2, WN = BN / 2; // wavefront tile
  constexpr int TM = WM / 32, TN = WN / 32;

  extern __shared__ __attribute__((aligned(16))) char smem[];
  // LDS map: A slice 0, A slice 1, B slice 0, B slice 1.
  auto lds_a = [&](int buf) { return smem + buf * GA::kBytes; };
  auto lds_b = [&](int buf) {
    return smem + 2 * GA::kBytes + buf * GB::kBytes;
  };

  // XCD-aware tile order: hardware deals consecutive workgroup ids to the 8
  // XCDs in turn; give each XCD a contiguous run of logical ids, then walk the
  // tile grid in column-major groups of 8 row-tiles so a run is a compact
  // block sharing A row-panels and B column-panels in that XCD's L2.
  const int tiles = g.tiles_m * g.tiles_n;
  int pid = blockIdx.x;
  if (tiles % 8 == 0)
    pid = (pid % 8) * (tiles / 8) + pid / 8;
  constexpr int GROUP = 8;
  const int per_group = GROUP * g.tiles_n;
  const int group = pid / per_group;
  const int first_m = group * GROUP;
  const int group_rows =
      g.tiles_m - first_m < GROUP ? g.tiles_m - first_m : GROUP;
  const int tile_m = first_m + (pid % per_group) % group_rows;
  const int tile_n = (pid % per_group) / group_rows;
  const int64_t batch = blockIdx.y;

  const int64_t m0 = (int64_t)tile_m * BM, n0 = (int64_t)tile_n * BN;
  const char *a = g.a + batch * g.a_batch * ELEM;
  const char *b = g.b + batch * g.b_batch * ELEM;

  const int wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int l = threadIdx.x & 63;

  typename KindTraits<KIND>::AccVec acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        acc[i][j][r] = 0;

  u32x4 ra[GA::kChunks], rb[GB::kChunks];
  const int64_t a_ldb = g.a_ld * ELEM, b_ldb = g.b_ld * ELEM;
  const int64_t kt_count = g.K * ELEM / kTileKBytes;

  // Implicit-GEMM gather state: the rows a thread copies are the same for
  // every K-slice, so their pixel coordinates are decoded once.
  constexpr int CONV_ROWS = A_MODE == A_CONV ? GA::kChunks : 1;
  int32_t cv_pix[CONV_ROWS], cv_ih[CONV_ROWS], cv_iw[CONV_ROWS];
  if constexpr (A_MODE == A_CONV) {
#pragma unroll
    for (int i = 0; i < GA::kChunks; ++i) {
      const int64_t m = m0 + (threadIdx.x >> 3) + 32 * i;
      const bool live = m < g.M;
      const int32_t mm = (int32_t)(live ? m : g.M - 1);
      const int32_t q = mm % g.conv.Q, pq = mm / g.conv.Q;
      const int32_t pp = pq % g.conv.P, nn = pq / g.conv.P;
      cv_pix[i] = nn * g.conv.H * g.conv.W;
      // rows past M read nothing: park them far outside the image
      cv_ih[i] = live ? pp * g.conv.str_h - g.conv.pad_h : -(1 << 28);
      cv_iw[i] = q * g.conv.str_w - g.conv.pad_w;
    }
  }
  auto load_a = [&](int64_t kt) {
    if constexpr (A_MODE == A_CONV) {
      const int32_t tap = (int32_t)(kt / g.conv.slices_per_tap);
      const int32_t cb = (int32_t)(kt % g.conv.slices_per_tap) * kTileKBytes;
      const int32_t fr = tap / g.conv.S, fs = tap % g.conv.S;
      const int32_t dh = fr * g.conv.dil_h, dw = fs * g.conv.dil_w;
      const int col = threadIdx.x & 7;
#pragma unroll
      for (int i = 0; i < GA::kChunks; ++i) {
        const int32_t ih = cv_ih[i] + dh, iw = cv_iw[i] + dw;
        const bool inside = (uint32_t)ih < (uint32_t)g.conv.H &&
                            (uint32_t)iw < (uint32_t)g.conv.W;
        const int64_t pix = (int64_t)cv_pix[i] + ih * g.conv.W + iw;
        ra[i] = inside ? *reinterpret_cast<const u32x4 *>(
                             a + pix * ((int64_t)g.conv.C * ELEM) + cb + col * 16)
                       : u32x4{0, 0, 0, 0};
      }
    } else {
      load_slice<BM, ELEM, A_KC>(a, a_ldb, m0, g.M, kt * kTileKBytes, ra);
    }
  };

  load_a(0);
  load_slice<BN, ELEM, B_KC>(b, b_ldb, n0, g.N, 0, rb);
  store_slice<BM, ELEM, A_KC>(lds_a(0), ra);
  store_slice<BN, ELEM, B_KC>(lds_b(0), rb);
  __syncthreads();

  for (int64_t kt = 0; kt < kt_count; ++kt) {
    const int cur = kt & 1;
    const bool more = kt + 1 < kt_count;
    if (more) {
      load_a(kt + 1);
      load_slice<BN, ELEM, B_KC>(b, b_ldb, n0, g.N, (kt + 1) * kTileKBytes, rb);
    }
    const char *sa = lds_a(cur);
    const char *sb = lds_b(cur);
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      Frag<KIND> fa[TM], fb[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        load_frag<KIND, BM, A_KC>(sa, wm * TM + i, s, fa[i]);
#pragma unroll
      for (int j = 0; j < TN; ++j)
        load_frag<KIND, BN, B_KC>(sb, wn * TN + j, s, fb[j]);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          mfma32<KIND>(acc[i][j], fa[i], fb[j]);
    }
    if (more) {
      store_slice<BM, ELEM, A_KC>(lds_a(cur ^ 1), ra);
      store_slice<BN, ELEM, B_KC>(lds_b(cur ^ 1), rb);
    }
    __syncthreads();
  }

  // Epilogue.  Lane l of a 32x32 tile holds column (l & 31) and rows
  // (r / 4) * 8 + (l >> 5) * 4 + r % 4 for r = 0..15.
  const int64_t ob = batch * g.o_batch;
  gemm_static_for<TM * TN>([&](auto idx) {
    constexpr int i = decltype(idx)::value / TN;
    constexpr int j = decltype(idx)::value % TN;
    const int64_t n = n0 + wn * WN + j * 32 + (l & 31);
    const int64_t mbase = m0 + wm * WM + i * 32 + (l >> 5) * 4;
    if (n >= g.N)
      return;
    if constexpr (std::is_same<Acc, int>::value) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int64_t m = mbase + (r >> 2) * 8 + (r & 3);
        if (m < g.M)
          ((int32_t *)g.out)[ob + m * g.o_sm + n * g.o_sn] = acc[i][j][r];
      }
    } else {
      float y[16];
#pragma unroll
      for (int r = 0; r < 16; ++r)
        y[r] = acc[i][j][r];
      fhip_round_fast_vec<16>(g.c_dt, y);
      for (int e = 0; e < g.epi.count; ++e) {
        const DevEpiOp &o = g.epi.op[e];
        if (o.kind == FHIP_OPERAND_NONE) {
          fhip_pw_fast_unary_vec<true, 16>(o.mode, y, o.params.swish_beta);
        } else {
          float other[16];
          if (o.kind == FHIP_OPERAND_SCALAR) {
#pragma unroll
            for (int r = 0; r < 16; ++r)
              other[r] = o.scalar;
          } else {
            const int64_t base = batch * o.stride[0] + n * o.stride[2];
            int64_t off[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              int64_t m = mbase + (r >> 2) * 8 + (r & 3);
              m = m < g.M ? m : g.M - 1; // edge tiles stay in bounds
              off[r] = base + m * o.stride[1];
            }
            load_operand_vec<16>(o.ptr, o.operand_dtype, off, other);
          }
          fhip_pw_fast_binary_vec<16>(o.mode, o.acc_is_in1 != 0, y, other);
        }
        fhip_round_fast_vec<16>(o.result_dtype, y);
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int64_t m = mbase + (r >> 2) * 8 + (r & 3);
        if (m >= g.M)
          continue;
        const int64_t off = ob + m * g.o_sm + n * g.o_sn;
        if (g.o_dt == FHIP_BFLOAT16)
          ((__bf16 *)g.out)[off] = (__bf16)y[r];
        else if (g.o_dt == FHIP_HALF)
          ((_Float16 *)g.out)[off] = (_Float16)y[r];
        else
          ((float *)g.out)[off] = y[r];
      }
    }
  });
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
};

template <int KIND, int BM, int BN, int A_MODE, bool B_KC>
int launch(fhip_ctx *ctx, const GemmArgs &g, int64_t batch) {
  constexpr int ELEM = KindTraits<KIND>::kElemBytes;
  constexpr bool A_KC = A_MODE != A_MCONTIG;
  constexpr int lds = 2 * SliceGeom<BM, ELEM, A_KC>::kBytes +
                      2 * SliceGeom<BN, ELEM, B_KC>::kBytes;
  auto kernel = gemm_kernel<KIND, BM, BN, A_MODE, B_KC>;
  static bool configured = false;
  if (!configured) {
    FHIP_HIP_CHECK(ctx, hipFuncSetAttribute(
                            reinterpret_cast<const void *>(kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    configured = true;
  }
  const dim3 grid((unsigned)(g.tiles_m * g.tiles_n), (unsigned)batch);
  hipLaunchKernelGGL(kernel, grid, dim3(kThreads), lds, ctx->stream, g);
  FHIP_HIP_CHECK(ctx, hipGetLastError());
  return 0;
}

template <int KIND, int BM, int BN>
int launch_orient(fhip_ctx *ctx, const GemmPlan &p, const GemmArgs &g) {
  if (p.a_kc && p.b_kc)
    return launch<KIND, BM, BN, A_KCONTIG, true>(ctx, g, p.batch);
  if (p.a_kc && !p.b_kc)
    return launch<KIND, BM, BN, A_KCONTIG, false>(ctx, g, p.batch);
  if (!p.a_kc && p.b_kc)
    return launch<KIND, BM, BN, A_MCONTIG, true>(ctx, g, p.batch);
  return launch<KIND, BM, BN, A_MCONTIG, false>(ctx, g, p.batch);
}

template <int KIND>
int gemm_launch_kind(fhip_ctx *ctx, const GemmPlan &p, const GemmArgs &g) {
  if (p.bm == 256 && p.bn == 256)
    return launch_orient<KIND, 256, 256>(ctx, p, g);
  if (p.bm == 256 && p.bn == 128)
    return launch_orient<KIND, 256, 128>(ctx, p, g);
  return launch_orient<KIND, 128, 128>(ctx, p, g);
}


// Implicit-GEMM convolution launchers (A gathered, B = filter, K-contiguous).
template <int KIND>
int conv_launch_kind(fhip_ctx *ctx, int bm, int bn, const GemmArgs &g) {
  if (bm == 256 && bn == 256)
    return launch<KIND, 256, 256, A_CONV, true>(ctx, g, 1);
  if (bm == 256 && bn == 128)
    return launch<KIND, 256, 128, A_CONV, true>(ctx, g, 1);
  return launch<KIND, 128, 128, A_CONV, true>(ctx, g, 1);
}

int gemm_launch_bf16(fhip_ctx *ctx, const GemmPlan &p, const GemmArgs &g);
int gemm_launch_f16(fhip_ctx *ctx, const GemmPlan &p, const GemmArgs &g);
int gemm_launch_i8(fhip_ctx *ctx, const GemmPlan &p, const GemmArgs &g);
int gemm_launch_fp8e4m3(fhip_ctx *ctx, const GemmPlan &p, const GemmArgs &g);
int gemm_launch_fp8e5m2(fhip_ctx *ctx, const GemmPlan &p, const GemmArgs &g);

#endif // FUSILLI_AMD_CSRC_GEMM_KERNEL_H
