// MFMA GEMM for gfx950: C[b] = A[b] x B[b] with fused pointwise epilogue.
//
//   * element types: bf16 / f16 (v_mfma_f32_32x32x16), int8
//     (v_mfma_i32_32x32x32_i8, exact int32 accumulate) and OCP fp8 e4m3 / e5m2
//     (v_mfma_f32_32x32x64_f8f6f4);
//   * either operand may be K-contiguous or M/N-contiguous (the reference
//     expresses transposes purely by strides, node/matmul_node.h:240-252):
//     K-contiguous tiles are read from LDS with 16-byte loads, the other kind
//     with the gfx950 transposing LDS reads (ds_read_b64_tr_b16 / _tr_b8), so
//     no operand is ever transposed in registers or in HBM;
//   * 256 threads = 2 x 2 wavefronts per workgroup, each wavefront owning a
//     (BM/2) x (BN/2) block of 32x32 MFMA tiles; K advances in 128-byte slices
//     through double-buffered, bank-conflict-padded LDS with the next slice's
//     global loads in flight during the MFMAs of the current one;
//   * workgroup ids are remapped so that the workgroups resident on one XCD
//     (one L2) cover a compact block of output tiles.
//
// Reference semantics: aten.matmul (reference support/asm_emitter.h:1669-1696).
#include "common.h"
#include "fast_paths.h"
#include "gemm_kernel.h"

#include <cstdlib>
#include <type_traits>

namespace {

// ---- host side --------------------------------------------------------------
bool kind_for(int a_dt, int b_dt, int *kind) {
  if (a_dt != b_dt)
    return false;
  switch (a_dt) {
  case FHIP_BFLOAT16:
    *kind = GK_BF16;
    return true;
  case FHIP_HALF:
    *kind = GK_F16;
    return true;
  case FHIP_INT8:
    *kind = GK_I8;
    return true;
  case FHIP_FP8E4M3:
    *kind = GK_FP8E4M3;
    return true;
  case FHIP_FP8E5M2:
    *kind = GK_FP8E5M2;
    return true;
  default:
    return false;
  }
}

GemmPlan make_plan(const fhip_matmul_desc *d, bool allow_split = true) {
  GemmPlan p;
  const int r = d->a.rank;
  if (r != 2 && r != 3)
    return p;
  if (!kind_for(d->a.dtype, d->b.dtype, &p.kind))
    return p;
  const int elem = fhip_dtype_size(d->a.dtype);
  p.M = d->a.dim[r - 2];
  p.K = d->a.dim[r - 1];
  p.N = d->b.dim[r - 1];
  p.batch = r == 3 ? d->c.dim[0] : 1;
  // operand orientation from strides
  const int64_t a_sm = d->a.stride[r - 2], a_sk = d->a.stride[r - 1];
  const int64_t b_sk = d->b.stride[r - 2], b_sn = d->b.stride[r - 1];
  if (a_sk == 1 || p.K == 1) {
    p.a_kc = true;
    p.a_ld = p.M == 1 ? p.K : a_sm;
  } else if (a_sm == 1 || p.M == 1) {
    p.a_kc = false;
    p.a_ld = a_sk;
  } else {
    return p;
  }
  if (b_sk == 1 || p.K == 1) {
    p.b_kc = true;
    p.b_ld = p.N == 1 ? p.K : b_sn;
  } else if (b_sn == 1 || p.N == 1) {
    p.b_kc = false;
    p.b_ld = b_sk;
  } else {
    return p;
  }
  // whole 128-byte K slices; 16-byte aligned rows; tiles no larger than the
  // matrix so edge clamping stays in bounds
  if ((p.K * elem) % kTileKBytes != 0)
    return p;
  if ((p.a_ld * elem) % 16 != 0 || (p.b_ld * elem) % 16 != 0)
    return p;
  if (p.a_kc ? p.a_ld < p.K : p.a_ld < p.M)
    return p;
  // (rows of an N-contiguous B may overlap, b_ld < N: the weight gradient
  // reads the filter taps of one row as one run of S * C elements per pixel)
  if (p.b_kc && p.b_ld < p.K)
    return p;
  if (p.M < 128 || p.N < 128)
    return p;
  // lane offsets inside a tile's rows are 32-bit
  if (p.a_ld * elem >= (1ll << 23) || p.b_ld * elem >= (1ll << 23))
    return p;
  // M/N-contiguous operands are moved in 16-byte column chunks
  if (!p.a_kc && (p.M * elem) % 16 != 0)
    return p;
  if (!p.b_kc && (p.N * elem) % 16 != 0)
    return p;
  if (p.batch > 65535) // grid y
    return p;
  if (r == 3) {
    p.a_batch = d->a.dim[0] == 1 ? 0 : d->a.stride[0];
    p.b_batch = d->b.dim[0] == 1 ? 0 : d->b.stride[0];
    p.o_batch = d->out.dim[0] == 1 ? 0 : d->out.stride[0];
    if ((p.a_batch * elem) % 16 != 0 || (p.b_batch * elem) % 16 != 0)
      return p;
  }
  p.o_sm = d->out.stride[r - 2];
  p.o_sn = d->out.stride[r - 1];
  // result / epilogue constraints
  if (p.kind == GK_I8) {
    if (d->c.dtype != FHIP_INT32 || d->out.dtype != FHIP_INT32 ||
        d->epilogue.count != 0)
      return p;
  } else {
    auto f = [](int dt) {
      return dt == FHIP_FLOAT || dt == FHIP_BFLOAT16 || dt == FHIP_HALF;
    };
    if (!f(d->c.dtype) || !f(d->out.dtype) ||
        !fhip_epilogue_is_fast(d->epilogue))
      return p;
    for (int i = 0; i < d->epilogue.count; ++i) {
      const fhip_epilogue_op &o = d->epilogue.op[i];
      if (o.operand_kind == FHIP_OPERAND_TENSOR && !f(o.operand.dtype))
        return p;
    }
  }
  // Tile shape and reduction split: the pair with the shortest estimated run.
  // A workgroup's time is a fixed part (prologue, epilogue: not overlapped
  // between the rounds of the large tiles, hidden behind the second resident
  // workgroup of the 128 x 128 tile) plus its K slices at the
  // tile's measured pace; the tiles run in rounds of 256 (one per compute
  // unit), and a round that leaves compute units idle runs at a higher clock
  // (fitted: 0.65 + 0.35 x the busy share).  Microseconds on this chip, from
  // 2048^3 ... 8192 x 8192 x 1024 problems of each type.
  const bool k16 = p.kind == GK_BF16 || p.kind == GK_F16;
  const int64_t slices = p.K * elem / kTileKBytes;
  auto tiles = [&](int bm, int bn) {
    return (double)(((p.M + bm - 1) / bm) * ((p.N + bn - 1) / bn) * p.batch);
  };
  auto estimate = [&](int bm, int bn, int sk) {
    const int shape = bm == 256 && bn == 256 ? 0 : (bm == 256 ? 1 : 2);
    static const double pace16[3] = {1.36, 0.90, 0.625}, pace8f[3] = {1.275, 0.876, 0.7125},
                        pace8i[3] = {1.38, 0.95, 0.66};
    static const double fixed16[3] = {11.0, 6.7, 6.4}, fixed8f[3] = {11.0, 5.7, 3.3},
                        fixed8i[3] = {18.0, 9.0, 7.7};
    const double pace = (k16 ? pace16 : p.kind == GK_I8 ? pace8i : pace8f)[shape];
    const double fixed = (k16 ? fixed16 : p.kind == GK_I8 ? fixed8i : fixed8f)[shape];
    const double t = tiles(bm, bn) * sk;
    const double full = floor(t / 256.0), rest = t - 256.0 * full;
    const double rounds = full + (rest > 0 ? 1 : 0);
    const double work = full + (rest > 0 ? 0.65 + 0.35 * rest / 256.0 : 0.0);
    double us = (double)(slices / sk) * pace * work +
                (shape != 2 ? fixed * rounds
                 : p.kind == GK_I8 ? fixed * (1.0 + 0.5 * (rounds - 1)) // (int32 stores)
                                   // (a partner with under 4.25 us of K slices does not cover it:
                                   // fp8 4096 x 4096 x 512 18.9 us against 16.1 on 256 x 256)
                                   : fixed + (rounds - 1) * fmax(0.0, 4.25 - (double)(slices / sk) * pace));
    if (sk > 1) // the parts' f32 stores and the kernel that adds them (~5 TB/s each way)
      us += 2.0 * sk * (double)p.M * (double)p.N * 4.0 / 5.0e6 + 2.5;
    return us;
  };
  const int forced = fhip_knobs().gemm_split; // (1: never split)
  const bool may_split = p.batch == 1 && p.N % 4 == 0 && p.o_sn == 1 &&
                         allow_split && forced != 1;
  double best = 0;
  p.bm = p.bn = 0;
  static const int shapes[3][2] = {{128, 128}, {256, 128}, {256, 256}};
  for (int i = 0; i < 3; ++i) {
    const int bm = shapes[i][0], bn = shapes[i][1];
    if (i > 0 && (p.M < bm || p.N < bn))
      continue;
    for (int sk = 1; sk <= 128; ++sk) {
      if (sk > 1 && (!may_split || slices % sk != 0 || slices / sk < 8))
        continue;
      // (a forced count must still divide the slices into runs of at least 8)
      if (forced > 1 && may_split && slices % forced == 0 && slices / forced >= 8 && sk != forced)
        continue;
      // a split must pay clearly; ties go to the larger tile (compute units
      // run faster while others idle)
      const double us = estimate(bm, bn, sk) * (sk > 1 ? 1.1 : 1.0);
      if (p.bm == 0 || us <= best) {
        best = us;
        p.bm = bm, p.bn = bn, p.ksplit = sk;
      }
    }
  }
  if (fhip_knobs().gemm_tile_bm) {
    const int bm = fhip_knobs().gemm_tile_bm, bn = fhip_knobs().gemm_tile_bn;
    if ((bm == 128 || bm == 256) &&
        (bn == 128 || bn == 256) && bm >= bn && bm <= p.M && bn <= p.N) {
      // the best split for the forced shape
      p.bm = bm, p.bn = bn, p.ksplit = 1;
      best = estimate(bm, bn, 1);
      for (int sk = 2; sk <= 128 && may_split; ++sk) {
        if (slices % sk != 0 || slices / sk < 8)
          continue;
        if (forced > 1 && slices % forced == 0 && slices / forced >= 8 && sk != forced)
          continue;
        const double us = estimate(bm, bn, sk) * 1.1;
        if (us < best || sk == forced)
          best = us, p.ksplit = sk;
      }
    }
  }
  p.ok = true;
  return p;
}

struct GemmSumArgs {
  const float *part; // [parts][M][pitch]: rows padded to whole column tiles
  void *out;
  int64_t part_stride; // M * pitch
  int64_t mn4, o_sm;   // mn4: M * N / 4
  int32_t N, pitch, parts, rank;
  int32_t c_dt, o_dt;
  int32_t ints;    // the parts are int32 sums (int8 operands): added exactly, no epilogue
  DevEpilogue epi; // strides over the matmul's result dims
};

// OUT[m][n] = epilogue(round(sum over the parts)), four columns per thread
// (N is a multiple of 4)
__global__ void gemm_splitk_sum_kernel(GemmSumArgs a) {
  const int64_t lin = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (lin >= a.mn4)
    return;
  const int64_t e = lin * 4;
  const int64_t m = e / a.N;
  const int64_t n0 = e - m * a.N;
  const float *src = a.part + m * a.pitch + n0;
  if (a.ints) {
    uint4 sum = *(const uint4 *)src; // (unsigned: wraps like the kernel's int32 accumulators)
    for (int z = 1; z < a.parts; ++z) {
      const uint4 v = *(const uint4 *)(src + (int64_t)z * a.part_stride);
      sum.x += v.x, sum.y += v.y, sum.z += v.z, sum.w += v.w;
    }
    uint32_t *o = (uint32_t *)a.out + m * a.o_sm + n0;
    o[0] = sum.x, o[1] = sum.y, o[2] = sum.z, o[3] = sum.w;
    return;
  }
  float4 acc = *(const float4 *)src;
  for (int z = 1; z < a.parts; ++z) {
    const float4 v = *(const float4 *)(src + (int64_t)z * a.part_stride);
    acc.x += v.x, acc.y += v.y, acc.z += v.z, acc.w += v.w;
  }
  int64_t coord[FHIP_MAX_RANK];
  coord[0] = 0;
  coord[a.rank - 2] = m;
  float v[4] = {acc.x, acc.y, acc.z, acc.w};
  int64_t cols[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    cols[i] = n0 + i;
    v[i] = fhip_round_through<float>(a.c_dt, v[i]);
  }
  fhip_apply_epilogue_many<float, 4>(a.epi, v, coord, a.rank - 1, cols);
#pragma unroll
  for (int i = 0; i < 4; ++i)
    fhip_store<float>(a.out, a.o_dt, m * a.o_sm + n0 + i, v[i]);
}

} // namespace

bool fhip_fast_matmul_applicable(const fhip_matmul_desc *d) {
  return make_plan(d).ok;
}

int fhip_fast_matmul(fhip_ctx *ctx, const fhip_matmul_desc *d, const void *a,
                     const void *b, const DevEpilogue &epi, void *out) {
  return fhip_fast_matmul_outer(ctx, d, a, b, epi, out, 1, 0, 0, 0);
}

int fhip_fast_matmul_outer(fhip_ctx *ctx, const fhip_matmul_desc *d,
                           const void *a, const void *b, const DevEpilogue &epi,
                           void *out, int outer, int64_t a_outer,
                           int64_t b_outer, int64_t o_outer) {
  const GemmPlan p = make_plan(d, outer == 1);
  FHIP_REQUIRE(ctx, outer >= 1 && outer <= 65535 && (outer == 1 || epi.count == 0),
               "gemm: outer batch extent %d (no fused operands with it)", outer);
  FHIP_REQUIRE(ctx, p.ok, "gemm: descriptor not supported by the MFMA kernel");
  FHIP_REQUIRE(ctx, ((uintptr_t)a & 15) == 0 && ((uintptr_t)b & 15) == 0,
               "gemm: A and B must be 16-byte aligned");
  GemmArgs g{};
  g.a = (const char *)a;
  g.b = (const char *)b;
  g.out = (char *)out;
  g.M = p.M;
  g.N = p.N;
  g.K = p.K;
  g.a_ld = p.a_ld;
  g.b_ld = p.b_ld;
  g.a_batch = p.a_batch;
  g.b_batch = p.b_batch;
  g.o_sm = p.o_sm;
  g.o_sn = p.o_sn;
  g.o_batch = p.o_batch;
  g.outer = outer;
  g.a_outer = a_outer;
  g.b_outer = b_outer;
  g.o_outer = o_outer;
  g.c_dt = d->c.dtype;
  g.o_dt = d->out.dtype;
  g.tiles_m = (int)((p.M + p.bm - 1) / p.bm);
  g.tiles_n = (int)((p.N + p.bn - 1) / p.bn);
  {
    const int64_t oe = fhip_dtype_size(d->out.dtype);
    g.o_vec = p.o_sn == 1 && (p.o_sm * oe) % 16 == 0 &&
              (p.o_batch * oe) % 16 == 0 && (o_outer * oe) % 16 == 0 &&
              ((uintptr_t)out & 15) == 0;
  }
  // epilogue strides on (batch, m, n)
  g.epi = epi;
  g.epi.rank = 3;
  const int r = d->a.rank;
  for (int i = 0; i < epi.count; ++i) {
    const DevEpiOp &s = epi.op[i];
    DevEpiOp &o = g.epi.op[i];
    o.stride[0] = r == 3 ? s.stride[0] : 0;
    o.stride[1] = s.stride[r - 2];
    o.stride[2] = s.stride[r - 1];
  }
  static const char *const kKindName[] = {"bf16", "f16", "i8", "fp8e4m3", "fp8e5m2"};
  fhip_note_kernel(ctx, "gemm_mfma %s %dx%d waves=8 split=%d", kKindName[p.kind], p.bm, p.bn,
                   p.ksplit);
  auto launch = [&]() {
    switch (p.kind) {
    case GK_BF16:
      return gemm_launch_bf16(ctx, p, g);
    case GK_F16:
      return gemm_launch_f16(ctx, p, g);
    case GK_I8:
      return gemm_launch_i8(ctx, p, g);
    case GK_FP8E4M3:
      return gemm_launch_fp8e4m3(ctx, p, g);
    default:
      return gemm_launch_fp8e5m2(ctx, p, g);
    }
  };
  if (p.ksplit > 1) {
    // every part writes plain f32 (int8 operands: int32) sums; rounding and
    // the fused operations follow in the kernel that adds them
    // (rows of the parts are padded to whole column tiles and the tiles are
    // stored whole: every cache line of the parts is written by one workgroup,
    // with full 16-byte stores)
    void *sp = nullptr;
    const int64_t pitch = (int64_t)g.tiles_n * p.bn;
    if (fhip_ctx_scratch(ctx, (size_t)p.ksplit * (size_t)(p.M * pitch) * sizeof(float), &sp) != 0)
      return 1;
    g.out = (char *)sp;
    g.c_dt = g.o_dt = p.kind == GK_I8 ? FHIP_INT32 : FHIP_FLOAT;
    g.o_sm = pitch;
    g.n_store = pitch;
    g.o_sn = 1;
    g.o_vec = 1;
    g.epi = DevEpilogue{};
    g.epi.rank = 3;
    g.outer = p.ksplit;
    g.o_outer = p.M * pitch;
    g.kt_split = (int32_t)(p.K * fhip_dtype_size(d->a.dtype) / kTileKBytes / p.ksplit);
    gemm_fill_linear(fhip_epilogue{}, g);
    const int rc = launch();
    if (rc != 0)
      return rc;
    GemmSumArgs sa{};
    sa.part = (const float *)sp;
    sa.out = out;
    sa.part_stride = p.M * pitch;
    sa.pitch = (int32_t)pitch;
    sa.mn4 = p.M * p.N / 4;
    sa.o_sm = p.o_sm;
    sa.N = (int32_t)p.N;
    sa.parts = p.ksplit;
    sa.rank = r;
    sa.c_dt = d->c.dtype;
    sa.o_dt = d->out.dtype;
    sa.ints = p.kind == GK_I8;
    sa.epi = epi;
    hipLaunchKernelGGL(gemm_splitk_sum_kernel, dim3((unsigned)((sa.mn4 + 255) / 256)),
                       dim3(256), 0, ctx->stream, sa);
    FHIP_HIP_CHECK(ctx, hipGetLastError());
    return 0;
  }
  gemm_fill_linear(d->epilogue, g);
  switch (p.kind) {
  case GK_BF16:
    return gemm_launch_bf16(ctx, p, g);
  case GK_F16:
    return gemm_launch_f16(ctx, p, g);
  case GK_I8:
    return gemm_launch_i8(ctx, p, g);
  case GK_FP8E4M3:
    return gemm_launch_fp8e4m3(ctx, p, g);
  default:
    return gemm_launch_fp8e5m2(ctx, p, g);
  }
}
