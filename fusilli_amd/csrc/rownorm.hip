// RMSNorm / LayerNorm forward for rows that are dense in memory: the whole row
// is held in registers (one 16-byte load per lane per 1 KiB of row), statistics
// are reduced with wavefront shuffles, and the normalised row, the optional
// scale/bias and the fused pointwise chain are applied before a single 16-byte
// store per lane.  HBM traffic is the compulsory read of X plus write of OUT.
//
// Reference semantics: aten.rms_norm / aten.layer_norm over all dims except
// dim 0 (reference support/asm_emitter.h:1592-1626, 1427-1503;
// node/norm_utils.h:27-99).
#include "common.h"
#include "fast_paths.h"
#include "rownorm_kernel.h"

#include <algorithm>
#include <cstdlib>
#include <type_traits>
#include <utility>
#include <vector>

namespace {

// Inner dims (1..rank-1) of `t` that have extent > 1, ordered by stride.
struct InnerLayout {
  bool dense = false;
  int64_t inner = 1;
};

InnerLayout inner_layout(const fhip_tensor_desc &t) {
  InnerLayout r;
  std::vector<std::pair<int64_t, int64_t>> ds; // (stride, dim)
  for (int i = 1; i < t.rank; ++i) {
    r.inner *= t.dim[i];
    if (t.dim[i] > 1)
      ds.emplace_back(t.stride[i], t.dim[i]);
  }
  std::sort(ds.begin(), ds.end());
  int64_t expect = 1;
  for (auto &p : ds) {
    if (p.first != expect)
      return r;
    expect *= p.second;
  }
  r.dense = true;
  return r;
}

// `t` walks the row exactly like `x` (same stride on every inner dim > 1).
bool same_inner_strides(const fhip_tensor_desc &x, const int64_t *strides) {
  for (int i = 1; i < x.rank; ++i)
    if (x.dim[i] > 1 && strides[i] != x.stride[i])
      return false;
  return true;
}

bool zero_inner_strides(const fhip_tensor_desc &x, const int64_t *strides) {
  for (int i = 1; i < x.rank; ++i)
    if (x.dim[i] > 1 && strides[i] != 0)
      return false;
  return true;
}

bool fast_dtype(int dt) {
  return dt == FHIP_BFLOAT16 || dt == FHIP_HALF || dt == FHIP_FLOAT;
}

// Picks (chunks per lane, wavefronts per row) for a row of `inner` elements:
// the first instantiated pair that covers the row.  FUSILLI_HIP_ROWNORM_SHAPE
// ("wpr,chunks") overrides the choice for tuning runs.
bool pick_shape(int64_t inner, int vec, int *chunks, int *wpr) {
  const int64_t per_wave_chunk = 64 * (int64_t)vec;
  const int64_t need = (inner + per_wave_chunk - 1) / per_wave_chunk;
  {
    const int w = fhip_knobs().rownorm_shape_w, c = fhip_knobs().rownorm_shape_c;
    if (w > 0 && (int64_t)w * c >= need) {
      for (const RowNormShape &sh : kRowNormShapes)
        if (sh.wpr == w && sh.chunks == c) {
          *wpr = w;
          *chunks = c;
          return true;
        }
    }
  }
  for (const RowNormShape &sh : kRowNormShapes) {
    if ((int64_t)sh.wpr * sh.chunks >= need) {
      *wpr = sh.wpr;
      *chunks = sh.chunks;
      return true;
    }
  }
  return false;
}

} // namespace

bool fhip_fast_norm_applicable(const fhip_norm_desc *d) {
  const fhip_tensor_desc &x = d->x;
  if (!fast_dtype(x.dtype) || d->out.dtype != x.dtype)
    return false;
  if (!fast_dtype(d->y.dtype) || !fhip_epilogue_is_fast(d->epilogue))
    return false;
  for (int i = 0; i < d->epilogue.count; ++i)
    if (fhip_pw_is_transcendental(d->epilogue.op[i].mode))
      return false;
  const InnerLayout lay = inner_layout(x);
  if (!lay.dense)
    return false;
  const int vec = 16 / fhip_dtype_size(x.dtype);
  if (lay.inner % vec != 0)
    return false;
  // rows that do not fit the register-resident kernels go to the long-row
  // kernels (no fused pointwise chain there)
  int chunks, wpr;
  if (!pick_shape(lay.inner, vec, &chunks, &wpr) && !fhip_norm_long_applicable(d))
    return false;
  const int64_t xrs = x.dim[0] > 1 ? x.stride[0] : lay.inner;
  const int64_t ors = d->out.dim[0] > 1 ? d->out.stride[0] : lay.inner;
  if (xrs < lay.inner || ors < lay.inner || xrs % vec || ors % vec)
    return false;
  if (!same_inner_strides(x, d->out.stride))
    return false;
  auto operand_dtype_ok = [&](int dt) {
    return dt == x.dtype || dt == FHIP_FLOAT;
  };
  if (d->scale.rank && (!same_inner_strides(x, d->scale.stride) ||
                        !operand_dtype_ok(d->scale.dtype)))
    return false;
  if (d->bias.rank && (!same_inner_strides(x, d->bias.stride) ||
                       !operand_dtype_ok(d->bias.dtype)))
    return false;
  if (d->emit_stats && !fast_dtype(d->stats_dtype))
    return false;
  for (int i = 0; i < d->epilogue.count; ++i) {
    const fhip_epilogue_op &o = d->epilogue.op[i];
    if (o.operand_kind != FHIP_OPERAND_TENSOR)
      continue;
    int64_t st[FHIP_MAX_RANK];
    if (!fhip_broadcast_strides(o.operand, x.rank, x.dim, st) ||
        !operand_dtype_ok(o.operand.dtype))
      return false;
    if (!same_inner_strides(x, st) && !zero_inner_strides(x, st))
      return false;
    if (same_inner_strides(x, st) && st[0] % vec != 0)
      return false;
  }
  return true;
}

int fhip_fast_norm(fhip_ctx *ctx, const fhip_norm_desc *d, const void *x,
                   const void *scale, const void *bias, const DevEpilogue &epi,
                   void *out, void *mean, void *inv_variance) {
  const InnerLayout lay = inner_layout(d->x);
  const int vec = 16 / fhip_dtype_size(d->x.dtype);
  int chunks = 1, wpr = 1;
  if (!pick_shape(lay.inner, vec, &chunks, &wpr))
    return fhip_norm_long(ctx, d, lay.inner, x, scale, bias, out, mean,
                          inv_variance);
  RowNormArgs g{};
  g.x = x;
  g.scale = scale;
  g.bias = bias;
  g.out = out;
  g.mean = mean;
  g.rstd = inv_variance;
  g.rows = d->x.dim[0];
  g.inner = lay.inner;
  g.x_row_stride = d->x.dim[0] > 1 ? d->x.stride[0] : lay.inner;
  g.out_row_stride = d->out.dim[0] > 1 ? d->out.stride[0] : lay.inner;
  g.scale_dt = d->scale.dtype;
  g.bias_dt = d->bias.dtype;
  g.y_dt = d->y.dtype;
  g.stats_dt = d->stats_dtype;
  g.is_layernorm = d->is_layernorm;
  g.emit_stats = d->emit_stats;
  g.eps = d->epsilon;
  g.epi_count = epi.count;
  for (int i = 0; i < epi.count; ++i) {
    const DevEpiOp &s = epi.op[i];
    FastEpiOp &o = g.epi[i];
    o.mode = s.mode;
    o.kind = s.kind;
    o.acc_is_in1 = s.acc_is_in1;
    o.result_dtype = s.result_dtype;
    o.operand_dtype = s.operand_dtype;
    o.scalar = s.scalar;
    o.params = s.params;
    o.ptr = s.ptr;
    o.row_stride = s.stride[0];
    o.col_unit = (s.kind == FHIP_OPERAND_TENSOR &&
                  same_inner_strides(d->x, s.stride) && lay.inner > 1)
                     ? 1
                     : 0;
  }
  // 16-byte alignment of every vector-accessed base pointer.
  auto aligned = [](const void *p) { return ((uintptr_t)p & 15u) == 0; };
  FHIP_REQUIRE(ctx, aligned(x) && aligned(out) && aligned(scale) &&
                        aligned(bias),
               "rownorm: tensor base pointers must be 16-byte aligned");
  for (int i = 0; i < epi.count; ++i)
    FHIP_REQUIRE(ctx, g.epi[i].col_unit == 0 || aligned(g.epi[i].ptr),
                 "rownorm: epilogue operand must be 16-byte aligned");
  // Choose the compile-time specialisation that matches this call exactly.
  int variant = RN_GENERAL;
  const bool scale_same = scale && d->scale.dtype == d->x.dtype;
  const bool bias_same = bias && d->bias.dtype == d->x.dtype;
  if (!d->is_layernorm && scale_same && !bias) {
    if (epi.count == 0) {
      variant = RN_RMS_SCALE;
    } else if (epi.count == 1 && g.epi[0].mode == FHIP_PW_MUL) {
      if (g.epi[0].kind == FHIP_OPERAND_SCALAR)
        variant = RN_RMS_SCALE_MULS;
      else if (g.epi[0].kind == FHIP_OPERAND_TENSOR && g.epi[0].col_unit &&
               g.epi[0].operand_dtype == d->x.dtype)
        variant = RN_RMS_SCALE_MULT;
    }
  } else if (d->is_layernorm && scale_same && bias_same && epi.count == 0) {
    variant = RN_LN_SCALE_BIAS;
  }
  if (fhip_knobs().rownorm_general)
    variant = RN_GENERAL; // tuning / test hook: force the general kernel
  bool launched;
  switch (d->x.dtype) {
  case FHIP_BFLOAT16:
    launched = rownorm_launch_bf16(chunks, wpr, variant, g.rows, ctx->num_cus, ctx->stream, g);
    break;
  case FHIP_HALF:
    launched = rownorm_launch_f16(chunks, wpr, variant, g.rows, ctx->num_cus, ctx->stream, g);
    break;
  default:
    launched = rownorm_launch_f32(chunks, wpr, variant, g.rows, ctx->num_cus, ctx->stream, g);
    break;
  }
  FHIP_REQUIRE(ctx, launched, "rownorm: no kernel for shape (%d, %d)", wpr,
               chunks);
  FHIP_HIP_CHECK(ctx, hipGetLastError());
  fhip_note_kernel(ctx, "rownorm chunks=%d waves_per_row=%d variant=%d", chunks, wpr, variant);
  return 0;
}
