// Convolution forward as implicit GEMM on MFMA.
//
// For channels-last tensors (X [N,H,W,C], W [K,R,S,C], OUT [N,P,Q,K]) the
// convolution is the GEMM  OUT[m, k] = sum_j A[m, j] * Wt[k, j]  with
// m = (n, p, q) and j = (r, s, c).  A is never built: the GEMM kernel's
// A-loader gathers each 128-byte run of channels of tap (r, s) straight from
// X (zeros outside the image), so HBM sees X once per filter tap through L2
// and the filter once per row tile; bias / activation chains are applied from
// the accumulators before the single NHWC store.
//
// Reference semantics: aten.convolution, groups = 1 here (reference
// support/asm_emitter.h:690-701, node/conv_node.h:38-56).
#include "common.h"
#include "fast_paths.h"
#include "gemm_kernel.h"

#include <cstdlib>

namespace {

struct ConvPlan {
  bool ok = false;
  int kind = 0;
  int64_t M = 0, N = 0, K = 0;
  ConvGeom geom{};
  int bm = 256, bn = 128;
  bool halo = false;
  int tile_rows = 0; // halo mode: rows per M tile (<= bm)
  // grouped convolution: one GEMM per group (the kernel's outer batch dim)
  // over the group's channel runs of X, its rows of W and its columns of OUT;
  // N and K are a group's
  int groups = 1;
  int64_t channels_out = 0; // of all groups
  // gather mode, one group, few tiles: the reduction is cut into ksplit parts
  // on workgroups of their own, whose f32 results a second kernel adds (and
  // applies the epilogue to); needs the context's scratch
  int ksplit = 1;
};

// strides equal the dense channels-last strides of dims (unit dims are free)
bool is_channels_last(const fhip_tensor_desc &t) {
  int64_t expect = 1;
  // order: dim 1 fastest, then spatial dims right to left, dim 0 slowest
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

// Strides `st` of an operand over the output dims [n, k, spatial...]: do the
// pixel dims (n, p, q) collapse to one stride `sm` per flattened pixel index?
bool pixel_stride(const int64_t *st, const int64_t *dim, int sp, int64_t *sm) {
  int pix_dims[FHIP_MAX_RANK]; // fastest first: last spatial dim .. first, then n
  int np = 0;
  for (int i = 1 + sp; i >= 2; --i)
    pix_dims[np++] = i;
  pix_dims[np++] = 0;
  int64_t mult = 1;
  bool have = false;
  *sm = 0;
  for (int i = 0; i < np; ++i) {
    const int dd = pix_dims[i];
    if (dim[dd] != 1) {
      if (!have) {
        if (st[dd] % mult != 0)
          return false;
        *sm = st[dd] / mult;
        have = true;
      } else if (st[dd] != *sm * mult) {
        return false;
      }
    }
    mult *= dim[dd];
  }
  return true;
}

void set_channels_last(fhip_tensor_desc &t, int dtype, int64_t d0, int64_t d1,
                       int64_t d2, int64_t d3) {
  t.rank = 4;
  t.dtype = dtype;
  t.dim[0] = d0, t.dim[1] = d1, t.dim[2] = d2, t.dim[3] = d3;
  t.stride[1] = 1;
  t.stride[3] = d1;
  t.stride[2] = d1 * d3;
  t.stride[0] = d1 * d3 * d2;
}

// A 3-D convolution whose filter is 1 x 1 in H and W (unit strides, no padding
// there) over dense channels-last tensors is the 2-D convolution of
// [N, C, D, H * W] images with an [fd, 1] filter: `f` receives that problem
// (geometry only -- the fused operands keep the original descriptor's shape).
bool fold_3d(const fhip_conv_desc *d, fhip_conv_desc *f) {
  if (d->spatial_rank != 3 || d->x.rank != 5)
    return false;
  if (d->w.dim[3] != 1 || d->w.dim[4] != 1 || d->stride[1] != 1 ||
      d->stride[2] != 1 || d->padding[1] != 0 || d->padding[2] != 0)
    return false;
  if (!is_channels_last(d->x) || !is_channels_last(d->w) ||
      !is_channels_last(d->out) || !is_channels_last(d->y))
    return false;
  *f = *d;
  const int64_t hw = d->x.dim[3] * d->x.dim[4];
  set_channels_last(f->x, d->x.dtype, d->x.dim[0], d->x.dim[1], d->x.dim[2], hw);
  set_channels_last(f->w, d->w.dtype, d->w.dim[0], d->w.dim[1], d->w.dim[2], 1);
  set_channels_last(f->y, d->y.dtype, d->y.dim[0], d->y.dim[1], d->y.dim[2], hw);
  set_channels_last(f->out, d->out.dtype, d->out.dim[0], d->out.dim[1],
                    d->out.dim[2], hw);
  f->spatial_rank = 2;
  f->padding[1] = 0, f->stride[1] = 1, f->dilation[1] = 1;
  f->padding[2] = 0, f->stride[2] = 1, f->dilation[2] = 1;
  return true;
}

// `d` is the geometry that runs (possibly folded and channel-padded); the
// fused operands are described over `orig`'s output dims.
ConvPlan make_plan(const fhip_conv_desc *d, const fhip_conv_desc *orig = nullptr,
                   bool allow_scratch = true) {
  ConvPlan p;
  if (!orig)
    orig = d;
  if (d->spatial_rank != 2 && d->spatial_rank != 1)
    return p;
  if (d->x.dtype != d->w.dtype)
    return p;
  if (d->x.dtype == FHIP_BFLOAT16)
    p.kind = GK_BF16;
  else if (d->x.dtype == FHIP_HALF)
    p.kind = GK_F16;
  else
    return p;
  const int elem = 2;
  const int sp = d->spatial_rank;
  const int64_t Call = d->x.dim[1];
  const int64_t C = d->w.dim[1]; // channels of one group
  if (C <= 0 || Call % C != 0 || d->w.dim[0] % (Call / C) != 0)
    return p;
  p.groups = (int)(Call / C);
  if ((C * elem) % kTileKBytes != 0)
    return p;
  if (!is_channels_last(d->x) || !is_channels_last(d->w) ||
      !is_channels_last(d->out))
    return p;
  auto f = [](int dt) {
    return dt == FHIP_FLOAT || dt == FHIP_BFLOAT16 || dt == FHIP_HALF;
  };
  if (!f(d->y.dtype) || !f(d->out.dtype) || !fhip_epilogue_is_fast(d->epilogue))
    return p;
  ConvGeom &g = p.geom;
  const int h = sp == 2 ? 0 : -1; // index of the H dim among spatial dims
  g.H = sp == 2 ? (int32_t)d->x.dim[2] : 1;
  g.W = (int32_t)d->x.dim[1 + sp];
  g.C = (int32_t)C;
  g.P = sp == 2 ? (int32_t)d->y.dim[2] : 1;
  g.Q = (int32_t)d->y.dim[1 + sp];
  const int64_t R = sp == 2 ? d->w.dim[2] : 1;
  g.S = (int32_t)d->w.dim[1 + sp];
  g.pad_h = h == 0 ? (int32_t)d->padding[0] : 0;
  g.str_h = h == 0 ? (int32_t)d->stride[0] : 1;
  g.dil_h = h == 0 ? (int32_t)d->dilation[0] : 1;
  g.pad_w = (int32_t)d->padding[sp - 1];
  g.str_w = (int32_t)d->stride[sp - 1];
  g.dil_w = (int32_t)d->dilation[sp - 1];
  g.x_pitch = (int32_t)(Call * elem);
  g.slices_per_tap = (int32_t)(C * elem / kTileKBytes);
  p.M = d->x.dim[0] * g.P * g.Q;
  p.channels_out = d->w.dim[0];
  p.N = d->w.dim[0] / p.groups;
  p.K = R * g.S * C;
  // 32-bit byte offsets in the gather; one validity bit per filter row and
  // one per filter column
  const int64_t x_bytes = d->x.dim[0] * (int64_t)g.H * g.W * Call * elem;
  if (x_bytes >= (1ll << 31) || p.M >= (1ll << 31) || R > 16 || g.S > 16 ||
      p.K * elem >= (1ll << 23) || p.groups > 65535)
    return p;
  g.x_bytes = (uint32_t)x_bytes;
  g.R = (int32_t)R;
  g.magic_q = conv_magic(g.Q);
  g.magic_p = conv_magic(g.P);
  g.magic_s = conv_magic(g.S);
  g.magic_spt = conv_magic(g.slices_per_tap);
  // Fused operands must be addressable as base + m * sm + k * sk: either
  // constant over pixels (a per-channel vector) or laid out like OUT.
  for (int i = 0; i < d->epilogue.count; ++i) {
    const fhip_epilogue_op &o = d->epilogue.op[i];
    if (o.operand_kind != FHIP_OPERAND_TENSOR)
      continue;
    if (!f(o.operand.dtype))
      return p;
    int64_t st[FHIP_MAX_RANK];
    if (!fhip_broadcast_strides(o.operand, orig->y.rank, orig->y.dim, st))
      return p;
    int64_t sm;
    if (!pixel_stride(st, orig->y.dim, orig->spatial_rank, &sm))
      return p;
  }
  p.bn = p.N > 128 ? 256 : 128;
  p.bm = p.M >= 256 ? 256 : 128;
  // 128-wide outputs run as 128 x 128 tiles on two stages: two workgroups
  // share a compute unit and cover each other's prologue and epilogue
  if (p.bn == 128 || p.bm == 128)
    p.bm = p.bn = 128;
  // Few output pixels (the 14 x 14 and 7 x 7 layers of a ResNet): 256 x 256
  // tiles would leave most of the 256 compute units idle, so the tile shrinks
  // until three quarters of them have one (N32 C256 14 x 14 -> K256: 25 tiles
  // 127 us, 98 tiles of 128 x 128 33 us).
  if (p.bm == 256 && p.bn == 256) {
    auto tiles = [&](int bm, int bn) {
      return ((p.M + bm - 1) / bm) * ((p.N + bn - 1) / bn) * p.groups;
    };
    if (tiles(256, 256) < 192)
      p.bn = 128;
    // (both run on eight wavefronts in two phases at the same rate per
    // output; the 128 x 128 tiles share a compute unit in pairs)
    if (p.bn == 128 && tiles(256, 128) < 192)
      p.bm = 128;
  }
  const FhipKnobs &knobs = fhip_knobs();
  if (knobs.conv_tile_bm) {
    const int bm = knobs.conv_tile_bm, bn = knobs.conv_tile_bn;
    if ((bm == 128 || bm == 256 || (bm == 512 && bn == 128)) &&
        (bn == 128 || bn == 256) && bm >= bn)
      p.bm = bm, p.bn = bn;
  }
  // Halo mode (the slab of input pixels stays in LDS for all taps): unit
  // stride, output extent == input extent, and a slab small enough that two
  // workgroups still share a compute unit.  FUSILLI_HIP_CONV_HALO=0 / 1
  // overrides the size rule (tests, tuning).
  p.halo = false;
  if (g.str_h == 1 && g.str_w == 1 && g.P == g.H && g.Q == g.W) {
    const int64_t reach = (int64_t)(R - 1) * g.dil_h * g.W +
                          (int64_t)(g.S - 1) * g.dil_w;
    auto slab_of = [&](int bm) {
      const int64_t rows = (bm + reach + 7) / 8 * 8;
      return rows * g.slices_per_tap * kTileKBytes + kTileKBytes;
    };
    const int want = knobs.conv_halo; // 0 off, 128 / 256 tile, else auto
    // 64-wide column tiles: half the filter ring (FUSILLI_HIP_CONV_BN=64
    // forces them for wider outputs: tuning)
    const bool narrow = p.N <= 64 || knobs.conv_bn == 64;
    const int ring128 = narrow ? HaloShape<128, 64>::kRingBytes
                               : HaloShape<128>::kRingBytes;
    const int ring256 = narrow ? HaloShape<256, 64>::kRingBytes
                               : HaloShape<256>::kRingBytes;
    const bool fits128 = slab_of(128) + ring128 <= 160 * 1024;
    const bool small128 = slab_of(128) + ring128 <= 80 * 1024;
    const bool small256 = slab_of(256) + ring256 <= 80 * 1024;
    // 256-row tiles when the output has enough pixels to give every slot
    // (two workgroups per compute unit) a tile of at least 160 rows
    const int64_t slots = 2 * 256;
    const bool big = p.M * ((p.N + 127) / 128) >= 160 * slots;
    int bm = 0;
    if (want == 0)
      bm = 0;
    else if (want == 256)
      bm = small256 ? 256 : 0;
    else if (want > 0)
      bm = fits128 ? 128 : 0;
    else // a slab past 80 KB (one workgroup per compute unit) still beats
         // the gather: 55.6 vs 74 us for C = K = 128, 56 x 56; 24 vs 32 us for
         // C = K = 256, 14 x 14 at N = 32 and 46 vs 52 us at N = 128
      bm = small256 && big ? 256 : (fits128 ? 128 : 0);
    // ... unless the gather would run its 128 x 128 tiles (eight wavefronts,
    // two workgroups per compute unit) over two rounds of the machine or more:
    // C256 -> K64 1 x 1 at 56 x 56 24.8 -> 18.0 us, C = K = 128 3 x 3 at 56 x 56
    // and N = 64 98 -> 84 us (C = K = 128 at 28 x 28, 196 tiles: halo 16.2, gather 20.7)
    if (want < 0 && bm == 128 && p.bm == 128 && p.bn == 128 &&
        ((p.M + 127) / 128) * ((p.N + 127) / 128) * p.groups >= 512)
      bm = 0;
    // a single tap has nothing to reuse in the slab (C128 -> K512 at 28 x 28:
    // halo 19.6, gather 12.9 us; C256 -> K1024 at 14 x 14: 13.9, 11.4 us);
    // with one K slice in all the halo kernel's shorter set-up still wins
    // (C64 -> K256 at 56 x 56: 17.7 against 19.3 us)
    if (want < 0 && reach == 0 && g.slices_per_tap >= 2)
      bm = 0;
    if (bm) {
      p.halo = true;
      p.bm = bm;
      p.bn = narrow ? 64 : 128;
      const int64_t rows = (bm + reach + 7) / 8 * 8;
      g.halo_rows = (int32_t)rows;
      g.slab_bytes = (uint32_t)slab_of(bm);
      // Tile height that spreads the pixels evenly over whole rounds of the
      // machine's slots (C3: 100352 pixels -> 512 tiles of 196 rows).
      p.tile_rows = bm;
      if (bm == 256) {
        const int64_t tn = (p.N + 127) / 128;
        const int64_t per_round = slots / tn > 0 ? slots / tn : 1;
        const int64_t rounds = (p.M + 256 * per_round - 1) / (256 * per_round);
        const int64_t tiles = rounds * per_round;
        p.tile_rows = (int)((p.M + tiles - 1) / tiles);
      }
    }
  }
  if (!p.halo && p.groups == 1 && allow_scratch && p.N % 4 == 0) {
    // (C512 7 x 7 -> K512 at N32: 52 tiles of 72 K slices 73 us; 4 x 52
    // workgroups of 18 slices and the sum 27 us)
    const int64_t tiles = ((p.M + p.bm - 1) / p.bm) * ((p.N + p.bn - 1) / p.bn);
    const int64_t slices = p.K * elem / kTileKBytes;
    // (128 x 128 tiles: two workgroups per compute unit, 512 slots)
    const int64_t slots = p.bm == 128 && p.bn == 128 ? 512 : 256;
    if (tiles < slots / 2 && slices >= 16) {
      int64_t want = slots / tiles;
      want = want > 8 ? 8 : want;
      for (int64_t sk = want; sk >= 2; --sk)
        if (slices % sk == 0 && slices / sk >= 6) {
          p.ksplit = (int)sk;
          break;
        }
    }
  }
  p.ok = true;
  return p;
}

// The problem that the MFMA kernel runs for descriptor `d`: `d` itself, its
// 2-D fold, and / or a copy with the channels zero-padded to a multiple of 64
// (the kernel's K slices are 128 bytes of one filter tap).
struct ConvResolved {
  ConvPlan plan;
  fhip_conv_desc run;  // geometry of the launch
  bool padded = false; // X and W are first copied into the context's scratch
  int64_t C = 0, Cp = 0, x_pixels = 0, w_pixels = 0;
  size_t x_bytes = 0, w_bytes = 0;
};

ConvResolved resolve(const fhip_conv_desc *d, bool allow_scratch = true) {
  ConvResolved r;
  fhip_conv_desc folded;
  const fhip_conv_desc *g = fold_3d(d, &folded) ? &folded : d;
  r.run = *g;
  r.plan = make_plan(g, d, allow_scratch);
  if (r.plan.ok || !allow_scratch)
    return r;
  // channel padding: 16-bit channels-last tensors, whole 16-byte chunks
  const int64_t C = g->x.dim[1];
  if ((g->spatial_rank != 2 && g->spatial_rank != 1) || g->x.rank != 2 + g->spatial_rank)
    return r;
  if (g->x.dtype != g->w.dtype ||
      (g->x.dtype != FHIP_BFLOAT16 && g->x.dtype != FHIP_HALF))
    return r;
  if (g->w.dim[1] != C || C % 8 != 0 || C % 64 == 0)
    return r;
  if (!is_channels_last(g->x) || !is_channels_last(g->w))
    return r;
  const int64_t Cp = (C + 63) / 64 * 64;
  fhip_conv_desc pd = *g;
  auto widen = [&](fhip_tensor_desc &t) {
    // channels-last strides of the same dims with Cp channels
    t.dim[1] = Cp;
    int64_t expect = Cp;
    for (int i = t.rank - 1; i >= 2; --i) {
      t.stride[i] = expect;
      expect *= t.dim[i];
    }
    t.stride[0] = expect;
    t.stride[1] = 1;
  };
  widen(pd.x);
  widen(pd.w);
  r.plan = make_plan(&pd, d);
  if (!r.plan.ok)
    return r;
  r.run = pd;
  r.padded = true;
  r.C = C, r.Cp = Cp;
  r.x_pixels = fhip_desc_volume(g->x) / C;
  r.w_pixels = fhip_desc_volume(g->w) / C;
  r.x_bytes = ((size_t)(r.x_pixels * Cp * 2) + 255) / 256 * 256;
  r.w_bytes = ((size_t)(r.w_pixels * Cp * 2) + 255) / 256 * 256;
  return r;
}

// dst[pixel][0 .. Cp) = src[pixel][0 .. C), zeros behind; one 16-byte chunk per thread
// Both operands in one launch: the chunks of X's copy, then those of W's.
__global__ void conv_pad_channels_kernel(const uint4 *x, uint4 *xp, int64_t x_pixels,
                                         const uint4 *w, uint4 *wp, int64_t w_pixels,
                                         int32_t c8, int32_t cp8) {
  int64_t lin = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const uint4 *src = x;
  uint4 *dst = xp;
  if (lin >= x_pixels * cp8) {
    lin -= x_pixels * cp8;
    if (lin >= w_pixels * cp8)
      return;
    src = w;
    dst = wp;
  }
  const int64_t pixel = lin / cp8;
  const int32_t chunk = (int32_t)(lin - pixel * cp8);
  dst[lin] = chunk < c8 ? src[pixel * c8 + chunk] : make_uint4(0, 0, 0, 0);
}

struct SplitSumArgs {
  const float *part; // [parts][M][pitch]: rows padded to whole column tiles
  void *out;         // [M][N], dense
  int64_t mn4;       // M * N / 4
  int64_t part_stride; // M * pitch
  int32_t N, pitch, parts;
  int32_t y_dt, o_dt;
  DevEpilogue epi;   // rank 3: strides {0, per pixel, per channel} over (0, m, n)
};

// OUT[m][n] = epilogue(round(sum over the parts)), four columns per thread
__global__ void conv_splitk_sum_kernel(SplitSumArgs a) {
  const int64_t lin = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (lin >= a.mn4)
    return;
  const int64_t e = lin * 4;
  const int64_t m = e / a.N;
  const int n0 = (int)(e - m * a.N);
  const float *src = a.part + m * a.pitch + n0;
  float4 acc = *(const float4 *)src;
  for (int z = 1; z < a.parts; ++z) {
    const float4 v = *(const float4 *)(src + (int64_t)z * a.part_stride);
    acc.x += v.x, acc.y += v.y, acc.z += v.z, acc.w += v.w;
  }
  // fused operands are addressed as base + m * pixel step + n * channel step,
  // whatever the rank of the convolution (a folded 3-D problem included)
  int64_t coord[FHIP_MAX_RANK] = {};
  coord[1] = m;
  float v[4] = {acc.x, acc.y, acc.z, acc.w};
  int64_t cols[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    cols[i] = n0 + i;
    v[i] = fhip_round_through<float>(a.y_dt, v[i]);
  }
  fhip_apply_epilogue_many<float, 4>(a.epi, v, coord, 2, cols);
#pragma unroll
  for (int i = 0; i < 4; ++i)
    fhip_store<float>(a.out, a.o_dt, e + i, v[i]);
}

} // namespace

int conv_launch_bf16(fhip_ctx *ctx, int bm, int bn, const GemmArgs &g) {
  return conv_launch_kind<GK_BF16>(ctx, bm, bn, g);
}
template <int KIND>
int conv_launch_halo_bm(fhip_ctx *ctx, int bm, int bn, const GemmArgs &g) {
  if (bn == 64)
    return bm == 256 ? conv_launch_halo<KIND, 256, 64>(ctx, g)
                     : conv_launch_halo<KIND, 128, 64>(ctx, g);
  return bm == 256 ? conv_launch_halo<KIND, 256>(ctx, g)
                   : conv_launch_halo<KIND, 128>(ctx, g);
}
int conv_launch_f16(fhip_ctx *ctx, int bm, int bn, const GemmArgs &g) {
  return conv_launch_kind<GK_F16>(ctx, bm, bn, g);
}

bool fhip_fast_conv_applicable(const fhip_conv_desc *d, bool allow_scratch) {
  return fhip_fast_conv_rf_applicable(d) || resolve(d, allow_scratch).plan.ok;
}

int fhip_fast_conv(fhip_ctx *ctx, const fhip_conv_desc *d, const void *x,
                   const void *w, const DevEpilogue &epi, void *out,
                   bool *handled, bool allow_scratch) {
  if (handled)
    *handled = true;
  bool taken = false;
  if (fhip_fast_conv_rf(ctx, d, x, w, epi, out, &taken) != 0)
    return 1;
  if (taken)
    return 0;
  const ConvResolved res = resolve(d, allow_scratch);
  const ConvPlan &p = res.plan;
  if (handled) {
    *handled = p.ok;
    if (!p.ok)
      return 0;
  }
  FHIP_REQUIRE(ctx, p.ok, "conv: descriptor not supported by the MFMA kernel");
  FHIP_REQUIRE(ctx, ((uintptr_t)x & 15) == 0 && ((uintptr_t)w & 15) == 0,
               "conv: X and W must be 16-byte aligned");
  // the context's scratch: zero-padded copies of X and W, then the parts of a
  // split reduction
  const size_t pad_bytes = res.padded ? res.x_bytes + res.w_bytes : 0;
  // (rows of the parts are padded to whole column tiles, which are stored
  // whole: every cache line of the parts is written by one workgroup)
  const int64_t part_pitch = (p.N + p.bn - 1) / p.bn * p.bn;
  const size_t part_bytes =
      p.ksplit > 1 ? (size_t)p.ksplit * (size_t)(p.M * part_pitch) * sizeof(float) : 0;
  char *scratch = nullptr;
  if (pad_bytes + part_bytes > 0) {
    void *sp = nullptr;
    if (fhip_ctx_scratch(ctx, pad_bytes + part_bytes, &sp) != 0)
      return 1;
    scratch = (char *)sp;
  }
  if (res.padded) {
    // channel counts that are no multiple of 64: zero-padded copies of X and W
    char *xp = scratch, *wp = xp + res.x_bytes;
    const int32_t c8 = (int32_t)(res.C / 8), cp8 = (int32_t)(res.Cp / 8);
    const int64_t xt = res.x_pixels * cp8, wt = res.w_pixels * cp8;
    hipLaunchKernelGGL(conv_pad_channels_kernel, dim3((unsigned)((xt + wt + 255) / 256)),
                       dim3(256), 0, ctx->stream, (const uint4 *)x, (uint4 *)xp, res.x_pixels,
                       (const uint4 *)w, (uint4 *)wp, res.w_pixels, c8, cp8);
    FHIP_HIP_CHECK(ctx, hipGetLastError());
    x = xp;
    w = wp;
  }
  const int sp = d->spatial_rank; // of the descriptor the fused operands follow
  GemmArgs g{};
  g.conv = p.geom;
  g.a = (const char *)x;
  g.b = (const char *)w;
  g.out = (char *)out;
  g.M = p.M;
  g.N = p.N;
  g.K = p.K;
  g.a_ld = 0;
  g.b_ld = p.K; // filter rows are R*S*C contiguous elements
  g.o_sm = p.channels_out; // OUT is dense channels-last: pixels are all groups' channels apart
  g.o_sn = 1;
  g.o_batch = 0;
  if (p.groups > 1) {
    g.outer = p.groups;
    g.a_outer = p.geom.C;  // a group's first input channel
    g.b_outer = p.N * p.K; // its filter rows
    g.o_outer = p.N;       // its first output channel,
    g.epi_n_outer = p.N;   // which fused per-channel operands see as well
  }
  g.c_dt = d->y.dtype;
  g.o_dt = d->out.dtype;
  g.tile_rows = p.halo ? p.tile_rows : p.bm;
  g.tiles_m = (int)((p.M + g.tile_rows - 1) / g.tile_rows);
  g.tiles_n = (int)((p.N + p.bn - 1) / p.bn);
  g.o_vec = (p.N * fhip_dtype_size(d->out.dtype)) % 16 == 0 &&
            (p.channels_out * fhip_dtype_size(d->out.dtype)) % 16 == 0 &&
            ((uintptr_t)out & 15) == 0;
  g.epi = epi;
  g.epi.rank = 3;
  for (int i = 0; i < epi.count; ++i) {
    const DevEpiOp &s = epi.op[i];
    DevEpiOp &o = g.epi.op[i];
    int64_t st[FHIP_MAX_RANK], sm = 0;
    for (int k = 0; k < d->y.rank; ++k)
      st[k] = s.stride[k];
    if (s.kind == FHIP_OPERAND_TENSOR)
      FHIP_REQUIRE(ctx, pixel_stride(st, d->y.dim, sp, &sm),
                   "conv: fused operand layout not supported");
    o.stride[0] = 0;
    o.stride[1] = sm;          // per-pixel step (0 for channel vectors)
    o.stride[2] = s.stride[1]; // per-channel step
  }
  // A single tap at unit stride without padding is the matrix product
  // X[pixels][C] . W[K][C]^T of dense operands: the GEMM entry takes them as
  // they lie (no pixel decode per K slice, its own tile and split choice).
  // N32: C1024 -> K256 at 14 x 14 20.5 -> 13.4 us, C512 -> K128 at 28 x 28
  // 12.5 -> 9.8, C256 -> K128 at 56 x 56 20.1 -> 17.9, C64 -> K256 17.6 -> 16.7.
  {
    const ConvGeom &cg = p.geom;
    const FhipKnobs &knobs = fhip_knobs();
    const int64_t elem = fhip_dtype_size(d->x.dtype);
    if (allow_scratch && !res.padded && p.groups == 1 && cg.R == 1 && cg.S == 1 &&
        cg.str_h == 1 && cg.str_w == 1 && cg.pad_h == 0 && cg.pad_w == 0 && cg.P == cg.H &&
        cg.Q == cg.W && cg.x_pitch == cg.C * elem && p.channels_out == p.N &&
        knobs.conv_tile_bm == 0 && knobs.conv_halo < 0) {
      fhip_matmul_desc md{};
      auto mat = [](fhip_tensor_desc &t, int64_t rows, int64_t cols, int64_t s_row, int64_t s_col,
                    int dt) {
        t.rank = 3;
        t.dim[0] = 1, t.dim[1] = rows, t.dim[2] = cols;
        t.stride[0] = rows * cols, t.stride[1] = s_row, t.stride[2] = s_col;
        t.dtype = dt;
      };
      mat(md.a, p.M, p.K, p.K, 1, d->x.dtype);
      mat(md.b, p.K, p.N, 1, p.K, d->w.dtype); // filter rows are B's columns
      mat(md.c, p.M, p.N, p.N, 1, d->y.dtype);
      mat(md.out, p.M, p.N, p.N, 1, d->out.dtype);
      md.out_dtype = d->out.dtype;
      md.epilogue = d->epilogue;
      if (fhip_fast_matmul_applicable(&md)) {
        if (fhip_fast_matmul(ctx, &md, x, w, g.epi, out) != 0)
          return 1;
        char inner[sizeof(ctx->last_kernel)];
        std::snprintf(inner, sizeof(inner), "%s", ctx->last_kernel);
        fhip_note_kernel(ctx, "conv_igemm as %s", inner);
        return 0;
      }
    }
  }
  if (p.ksplit > 1) {
    // every part writes plain f32 sums; rounding and the fused operations
    // follow in the kernel that adds them
    const DevEpilogue by_pixel = g.epi; // the remapped (0, pixel, channel) strides
    float *part = (float *)(scratch + pad_bytes);
    g.out = (char *)part;
    g.c_dt = g.o_dt = FHIP_FLOAT;
    g.o_sm = part_pitch;
    g.n_store = part_pitch;
    g.o_vec = 1;
    g.epi = DevEpilogue{};
    g.epi.rank = 3;
    g.outer = p.ksplit;
    g.o_outer = p.M * part_pitch;
    g.kt_split = (int32_t)(p.K * 2 / kTileKBytes / p.ksplit);
    gemm_fill_linear(fhip_epilogue{}, g);
    const int rc = p.kind == GK_BF16 ? conv_launch_bf16(ctx, p.bm, p.bn, g)
                                     : conv_launch_f16(ctx, p.bm, p.bn, g);
    if (rc != 0)
      return rc;
    SplitSumArgs a{};
    a.part = part;
    a.out = out;
    a.part_stride = p.M * part_pitch;
    a.pitch = (int32_t)part_pitch;
    a.mn4 = p.M * p.N / 4;
    a.N = (int32_t)p.N;
    a.parts = p.ksplit;
    a.y_dt = d->y.dtype;
    a.o_dt = d->out.dtype;
    a.epi = by_pixel;
    hipLaunchKernelGGL(conv_splitk_sum_kernel, dim3((unsigned)((a.mn4 + 255) / 256)),
                       dim3(256), 0, ctx->stream, a);
    FHIP_HIP_CHECK(ctx, hipGetLastError());
    fhip_note_kernel(ctx, "conv_igemm gather %dx%d split=%d padded=%d groups=%d", p.bm, p.bn,
                     p.ksplit, (int)res.padded, (int)p.groups);
    return 0;
  }
  gemm_fill_linear(d->epilogue, g);
  fhip_note_kernel(ctx, "conv_igemm %s %dx%d split=1 padded=%d groups=%d",
                   p.halo ? "halo" : "gather", p.bm, p.bn, (int)res.padded, (int)p.groups);
  if (p.halo)
    return p.kind == GK_BF16 ? conv_launch_halo_bm<GK_BF16>(ctx, p.bm, p.bn, g)
                             : conv_launch_halo_bm<GK_F16>(ctx, p.bm, p.bn, g);
  if (p.kind == GK_BF16)
    return conv_launch_bf16(ctx, p.bm, p.bn, g);
  return conv_launch_f16(ctx, p.bm, p.bn, g);
}

// ---------------------------------------------------------------------------
// Data gradient on the same kernels.  With one group and (first) unit strides
//   DX[n, c, i] = sum_{k, f} DY[n, k, i + pad - f * dil] * W[k, c, f]
// is the forward convolution of DY (K channels) with the filter
//   W'[c, k, f'] = W[k, c, F - 1 - f']   (taps mirrored, channel roles swapped)
// under padding' = dil * (F - 1) - pad.  W' is small (the filter's size); it is
// rebuilt in the caller's workspace on every call, channels-last, by a
// transposing copy, and the forward kernel does the rest.  Strides above one:
// DY is spread over a zero grid first (DY(p, q) at (p * stride, q * stride)),
// which is the unit-stride case again at stride^2 times the MFMA work.
// (Reference node/conv_node.h:428-598; aten.convolution_backward, input
// gradient.)
// ---------------------------------------------------------------------------
namespace {

struct DgradPlan {
  bool ok = false;
  fhip_conv_desc fwd; // the equivalent forward problem
  size_t filter_bytes = 0;
  // strides above one: DY is first spread over a zero grid of the unit-stride
  // output extent (element (p, q) at (p * stride, q * stride)), in workspace
  // behind the mirrored filter
  bool spread = false;
  size_t spread_bytes = 0;
};

DgradPlan make_dgrad_plan(const fhip_conv_desc *d, bool allow_scratch = true) {
  DgradPlan p;
  const int sp = d->spatial_rank;
  if (sp != 1 && sp != 2)
    return p;
  // groups: the forward problem is grouped the same way (a group's K / groups
  // gradient channels in, its C / groups channels out)
  const int64_t Cg = d->w.dim[1];
  if (Cg < 1 || d->x.dim[1] % Cg != 0 || d->w.dim[0] % (d->x.dim[1] / Cg) != 0)
    return p;
  const int64_t groups = d->x.dim[1] / Cg;
  if (d->y.dtype != d->w.dtype)
    return p;
  fhip_conv_desc &f = p.fwd;
  std::memset(&f, 0, sizeof(f));
  f.spatial_rank = sp;
  for (int i = 0; i < sp; ++i) {
    if (d->stride[i] != 1)
      p.spread = true;
    const int64_t pad = d->dilation[i] * (d->w.dim[2 + i] - 1) - d->padding[i];
    if (pad < 0)
      return p;
    f.padding[i] = pad;
    f.stride[i] = 1;
    f.dilation[i] = d->dilation[i];
  }
  f.x = d->y; // DY plays the input
  if (p.spread) {
    // dense channels-last grid [N, K, unit-stride output extent]
    int64_t st = f.x.dim[1];
    f.x.stride[1] = 1;
    for (int i = sp - 1; i >= 0; --i) {
      f.x.dim[2 + i] = d->x.dim[2 + i] + 2 * d->padding[i] -
                       d->dilation[i] * (d->w.dim[2 + i] - 1);
      if (f.x.dim[2 + i] < (d->y.dim[2 + i] - 1) * d->stride[i] + 1)
        return p;
      f.x.stride[2 + i] = st;
      st *= f.x.dim[2 + i];
    }
    f.x.stride[0] = st;
    if (!is_channels_last(d->y) || (d->y.dim[1] * 2) % 16 != 0)
      return p;
    p.spread_bytes = (size_t)(st * f.x.dim[0]) * 2;
  }
  f.y = d->x; // DX plays the output
  f.out = d->x;
  f.out_dtype = d->x.dtype;
  // W' [C, K / groups, F...], dense channels-last
  f.w.rank = d->w.rank;
  f.w.dtype = d->w.dtype;
  f.w.dim[0] = d->x.dim[1];
  f.w.dim[1] = d->w.dim[0] / groups;
  int64_t st = f.w.dim[1];
  f.w.stride[1] = 1;
  for (int i = sp - 1; i >= 0; --i) {
    f.w.dim[2 + i] = d->w.dim[2 + i];
    f.w.stride[2 + i] = st;
    st *= f.w.dim[2 + i];
  }
  f.w.stride[0] = st;
  if (!fhip_fast_conv_applicable(&f, allow_scratch))
    return p;
  p.filter_bytes =
      ((size_t)(st * f.w.dim[0]) * fhip_dtype_size(f.w.dtype) + 255) / 256 * 256;
  p.ok = true;
  return p;
}

struct SpreadArgs {
  int64_t P, Q, Hd, Wd, cpp; // DY extent, grid extent, 16-byte chunks per pixel
  int64_t sh, sw;            // convolution strides
  int64_t total;             // chunks of the grid
};

// grid[n][h][w][:] = DY[n][h / sh][w / sw][:] where both divisions are exact
// and inside DY, zeros elsewhere (both channels-last, 16-bit)
__global__ void conv_spread_kernel(SpreadArgs a, const uint4 *src, uint4 *dst) {
  const int64_t lin = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (lin >= a.total)
    return;
  const int64_t chunk = lin % a.cpp;
  int64_t pixel = lin / a.cpp;
  const int64_t w = pixel % a.Wd;
  pixel /= a.Wd;
  const int64_t h = pixel % a.Hd;
  const int64_t n = pixel / a.Hd;
  const int64_t p = h / a.sh, q = w / a.sw;
  uint4 v = make_uint4(0, 0, 0, 0);
  if (p * a.sh == h && q * a.sw == w && p < a.P && q < a.Q)
    v = src[((n * a.P + p) * a.Q + q) * a.cpp + chunk];
  dst[lin] = v;
}

struct FlipArgs {
  int64_t K, C, R, S;         // of one group; R = 1 for one spatial dim
  int64_t sk, sc, sr, ss;     // element strides of W [groups * K, C, R, S]
};

// dst[g * C + c][r'][s'][k] = src[g * K + k][c][R - 1 - r'][S - 1 - s'], 16-bit
// elements
__global__ void conv_flip_filter_kernel(FlipArgs a, const uint16_t *src,
                                        uint16_t *dst, int64_t total) {
  const int64_t lin = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (lin >= total)
    return;
  const int64_t k = lin % a.K;
  int64_t rem = lin / a.K;
  const int64_t s2 = rem % a.S;
  rem /= a.S;
  const int64_t r2 = rem % a.R;
  const int64_t gc = rem / a.R;
  const int64_t grp = gc / a.C, c = gc - grp * a.C;
  dst[lin] = src[(grp * a.K + k) * a.sk + c * a.sc + (a.R - 1 - r2) * a.sr +
                 (a.S - 1 - s2) * a.ss];
}

} // namespace

// Scratch of the entry point that allocates nothing (fhip_conv_dgrad_static):
// the mirrored filter and, with strides above one, DY spread over its zero
// grid live here instead of in caller workspace.  Every device that loads the
// library holds its own copy at its own address until the process ends; the
// address is resolved once per device by fhip_conv_dgrad_static_setup and kept
// in the context.  In host code the array's name is only a handle for that
// query, never a pointer to pass on.
static __device__ __align__(256) unsigned char
    dgrad_static_scratch[FHIP_CONV_DGRAD_STATIC_MAX_BYTES];

int fhip_conv_dgrad_static_setup(fhip_ctx *ctx) {
  // one slot per device ordinal; written under the context-creation lock
  constexpr int kMaxDevices = 64;
  static void *per_device[kMaxDevices] = {};
  FHIP_REQUIRE(ctx, ctx->device >= 0 && ctx->device < kMaxDevices,
               "device ordinal %d beyond the static scratch table", ctx->device);
  if (!per_device[ctx->device]) {
    void *ptr = nullptr;
    FHIP_HIP_CHECK(ctx, hipGetSymbolAddress(&ptr, HIP_SYMBOL(dgrad_static_scratch)));
    FHIP_REQUIRE(ctx, ptr != nullptr && ((uintptr_t)ptr & 255) == 0,
                 "static scratch address not resolved");
    per_device[ctx->device] = ptr;
  }
  ctx->dgrad_static_scratch = per_device[ctx->device];
  return 0;
}

// the forward kernel's name, marked as the data gradient's
static void dgrad_note(fhip_ctx *ctx, const char *prefix) {
  char inner[sizeof(ctx->last_kernel)];
  std::snprintf(inner, sizeof(inner), "%s", ctx->last_kernel);
  fhip_note_kernel(ctx, "%s%s", prefix, inner);
}

bool fhip_fast_conv_dgrad_applicable(const fhip_conv_desc *d,
                                     size_t *workspace_bytes, bool allow_scratch) {
  const DgradPlan p = make_dgrad_plan(d, allow_scratch);
  if (workspace_bytes)
    *workspace_bytes = p.ok ? p.filter_bytes + p.spread_bytes : 0;
  return p.ok;
}

int fhip_fast_conv_dgrad(fhip_ctx *ctx, const fhip_conv_desc *d, const void *dy,
                         const void *w, void *dx, void *workspace, bool allow_scratch) {
  const DgradPlan p = make_dgrad_plan(d, allow_scratch);
  FHIP_REQUIRE(ctx, p.ok, "conv dgrad: descriptor not supported by the MFMA kernel");
  // the register-filter kernel needs neither the mirrored filter nor workspace
  if (fhip_fast_conv_dgrad_rf_applicable(d) &&
      (((uintptr_t)dy | (uintptr_t)w | (uintptr_t)dx) & 15) == 0)
    return fhip_fast_conv_dgrad_rf(ctx, d, dy, w, dx);
  FHIP_REQUIRE(ctx, ((uintptr_t)workspace & 15) == 0,
               "conv dgrad: workspace must be 16-byte aligned");
  const int sp = d->spatial_rank;
  FlipArgs a;
  const int64_t groups = d->x.dim[1] / d->w.dim[1];
  a.K = d->w.dim[0] / groups;
  a.C = d->w.dim[1];
  a.R = sp == 2 ? d->w.dim[2] : 1;
  a.S = d->w.dim[1 + sp];
  a.sk = d->w.dim[0] == 1 ? 0 : d->w.stride[0];
  a.sc = d->w.dim[1] == 1 ? 0 : d->w.stride[1];
  a.sr = sp == 2 ? d->w.stride[2] : 0;
  a.ss = d->w.stride[1 + sp];
  const int64_t total = groups * a.K * a.C * a.R * a.S;
  hipLaunchKernelGGL(conv_flip_filter_kernel,
                     dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                     ctx->stream, a, (const uint16_t *)w, (uint16_t *)workspace,
                     total);
  FHIP_HIP_CHECK(ctx, hipGetLastError());
  DevEpilogue epi{};
  if (p.spread) {
    char *grid = (char *)workspace + p.filter_bytes;
    SpreadArgs sa;
    sa.P = sp == 2 ? d->y.dim[2] : 1;
    sa.Q = d->y.dim[1 + sp];
    sa.Hd = sp == 2 ? p.fwd.x.dim[2] : 1;
    sa.Wd = p.fwd.x.dim[1 + sp];
    sa.cpp = d->y.dim[1] * 2 / 16;
    sa.sh = sp == 2 ? d->stride[0] : 1;
    sa.sw = d->stride[sp - 1];
    sa.total = (int64_t)(p.spread_bytes / 16);
    FHIP_REQUIRE(ctx, ((uintptr_t)dy & 15) == 0, "conv dgrad: DY must be 16-byte aligned");
    hipLaunchKernelGGL(conv_spread_kernel,
                       dim3((unsigned)((sa.total + 255) / 256)), dim3(256), 0,
                       ctx->stream, sa, (const uint4 *)dy, (uint4 *)grid);
    FHIP_HIP_CHECK(ctx, hipGetLastError());
    const int rc = fhip_fast_conv(ctx, &p.fwd, grid, workspace, epi, dx, nullptr, allow_scratch);
    dgrad_note(ctx, "dgrad spread + ");
    return rc;
  }
  const int rc = fhip_fast_conv(ctx, &p.fwd, dy, workspace, epi, dx, nullptr, allow_scratch);
  dgrad_note(ctx, "dgrad ");
  return rc;
}
