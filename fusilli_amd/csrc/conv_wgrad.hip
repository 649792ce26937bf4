// Convolution weight gradient on the MFMA GEMM kernel.
//
//   DW[k, r, s, c] = sum over n, p, q of DY[n, p, q, k] * X[n, p + r*dil - pad_h, q + s - pad_w, c]
//
// (channels-last tensors, one group, unit dilation along W; written here for
// unit strides, equal strides in both dims work the same way, see the plan).
// Both operands are first copied into zero-padded grids of the same geometry,
// [N][rows = H + 2 pad_h][pitch >= W + 2 pad_w] pixels with pitch a multiple of
// 64: X shifted by the padding, DY in the top-left corner.  With m the flat
// pixel index of that grid, tap (r, s) of X is pixel m + r * dil * pitch + s,
// whatever m: image borders need no case distinction because DY is zero
// wherever the shifted pixel would leave the image.  For one filter row r the
// S taps of a pixel are S * C consecutive elements, so
//   partial[r][n][k][s * C + c] = sum_m DYp[n][m][k] * Xp[n][m + r * dil * pitch][s * C + c]
// is one batched GEMM per filter row, all rows in one launch (A = DYp, M-contiguous; B = Xp with
// overlapping rows of S * C elements, row stride C; reduction over the 64-pixel
// K slices of an image, or of an equal share of it; batch = image x share),
// and DW is the sum of the partial results over the batch.
//
// Reference semantics: node/conv_node.h:255-426 (ConvWGradNode),
// aten.convolution_backward, weight gradient.
#include "common.h"
#include "fast_paths.h"

namespace {

struct WgradPlan {
  bool ok = false;
  int64_t N = 0, H = 0, W = 0, C = 0, K = 0, P = 0, Q = 0, R = 0, S = 0;
  int64_t Kp = 0; // channels of the padded DY grid: K, or 128 for narrower outputs
  int64_t pad_h = 0, pad_w = 0, dil_h = 1;
  int64_t rows = 0, pitch = 0, pix = 0; // padded grid
  int64_t split = 1; // GEMM batches per image (more workgroups, shorter K)
  int64_t str = 1;   // convolution stride (same in both dims)
  int64_t rows_y = 0, pix_y = 0; // DY's grid: rows / str rows of the same pitch
  size_t xp_bytes = 0, dyp_bytes = 0, part_bytes = 0;
  fhip_matmul_desc mm; // one filter row
};

bool wg_channels_last(const fhip_tensor_desc &t) {
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

size_t wg_align(size_t b) { return (b + 255) / 256 * 256; }

WgradPlan make_wgrad_plan(const fhip_conv_desc *d) {
  WgradPlan p;
  if (d->spatial_rank != 2)
    return p;
  const int dt = d->x.dtype;
  if (dt != FHIP_BFLOAT16 && dt != FHIP_HALF)
    return p;
  if (d->y.dtype != dt)
    return p;
  const int wdt = d->w.dtype;
  if (wdt != FHIP_BFLOAT16 && wdt != FHIP_HALF && wdt != FHIP_FLOAT)
    return p;
  if (d->w.dim[1] != d->x.dim[1]) // groups
    return p;
  if (d->stride[0] != d->stride[1] || d->dilation[1] != 1)
    return p;
  p.str = d->stride[0];
  if (!wg_channels_last(d->x) || !wg_channels_last(d->y))
    return p;
  p.N = d->x.dim[0], p.C = d->x.dim[1], p.H = d->x.dim[2], p.W = d->x.dim[3];
  p.K = d->w.dim[0], p.R = d->w.dim[2], p.S = d->w.dim[3];
  // the padding copies move whole 16-byte chunks of a pixel's channels
  if (p.C % 8 != 0 || p.K % 8 != 0)
    return p;
  // the GEMM's tiles want at least 128 rows: narrower gradients are zero-padded
  p.Kp = p.K < 128 ? 128 : p.K;
  p.P = d->y.dim[2], p.Q = d->y.dim[3];
  p.pad_h = d->padding[0], p.pad_w = d->padding[1], p.dil_h = d->dilation[0];
  // Strides: output pixel (p, q) reads input pixel (p * str + r * dil, q * str
  // + s); with DY on a grid of the SAME pitch and rows / str rows, DY pixel m
  // pairs with X pixel str * m + shift: B's row stride becomes str * C.
  p.rows = (p.H + 2 * p.pad_h + p.str - 1) / p.str * p.str;
  p.pitch = (p.W + 2 * p.pad_w + 63) / 64 * 64;
  p.pix = p.rows * p.pitch;
  p.rows_y = p.rows / p.str;
  p.pix_y = p.rows_y * p.pitch;
  if (p.P > p.rows_y || (p.Q - 1) * p.str + p.S > p.pitch)
    return p;
  // guard behind the last image: the furthest tap of the last pixel
  const int64_t guard = (p.R - 1) * p.dil_h * p.pitch * p.C + p.S * p.C;
  p.xp_bytes = wg_align((size_t)(p.N * p.pix * p.C + guard) * 2);
  p.dyp_bytes = wg_align((size_t)(p.N * p.pix_y * p.Kp) * 2);
  // An image's pixels are cut into `split` equal runs of whole 64-pixel
  // slices, each a batch entry of its own: the largest cut that keeps at
  // least 8 slices per run and at most ~1024 workgroups per launch.
  {
    const int64_t slices = p.pix_y / 64;
    const int64_t col_tiles = (p.S * p.C + 127) / 128, row_tiles = (p.K + 127) / 128;
    for (int64_t f = 1; f <= slices; ++f)
      if (slices % f == 0 && slices / f >= 8 &&
          p.N * f * col_tiles * row_tiles <= 1024)
        p.split = f;
  }
  p.part_bytes = wg_align((size_t)(p.R * p.N * p.split * p.Kp * p.S * p.C) * 4);
  if (p.xp_bytes >= (1ull << 32) || p.dyp_bytes >= (1ull << 32))
    return p;
  fhip_matmul_desc &m = p.mm;
  std::memset(&m, 0, sizeof(m));
  auto set = [](fhip_tensor_desc &t, int dtype, int64_t d0, int64_t d1, int64_t d2,
                int64_t s0, int64_t s1, int64_t s2) {
    t.rank = 3;
    t.dtype = dtype;
    t.dim[0] = d0, t.dim[1] = d1, t.dim[2] = d2;
    t.stride[0] = s0, t.stride[1] = s1, t.stride[2] = s2;
  };
  const int64_t nb = p.N * p.split, run = p.pix_y / p.split;
  set(m.a, dt, nb, p.Kp, run, run * p.Kp, 1, p.Kp);
  set(m.b, dt, nb, run, p.S * p.C, p.str * run * p.C, p.str * p.C, 1);
  set(m.c, FHIP_FLOAT, nb, p.Kp, p.S * p.C, p.Kp * p.S * p.C, p.S * p.C, 1);
  m.out = m.c;
  m.out_dtype = FHIP_FLOAT;
  if (!fhip_fast_matmul_applicable(&m))
    return p;
  p.ok = true;
  return p;
}

struct PadArgs {
  int64_t N, rows, pitch, ch;  // destination grid, channels per pixel
  int64_t src_ch;              // channels per source pixel (<= ch: the rest is zero)
  int64_t h, w;                // source extent
  int64_t off_h, off_w;        // destination position of source pixel (0, 0)
  int64_t total;               // 16-byte chunks of the destination
};

// dst[n][row][col][:] = src[n][row - off_h][col - off_w][:] inside the source,
// zeros elsewhere; one 16-byte chunk (8 channels) per thread.
__global__ void conv_pad_grid_kernel(PadArgs a, const uint4 *src, uint4 *dst) {
  const int64_t lin = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (lin >= a.total)
    return;
  const int64_t cpp = a.ch / 8; // chunks per pixel
  const int64_t chunk = lin % cpp;
  int64_t pixel = lin / cpp;
  const int64_t col = pixel % a.pitch;
  pixel /= a.pitch;
  const int64_t row = pixel % a.rows;
  const int64_t n = pixel / a.rows;
  const int64_t sr = row - a.off_h, sc = col - a.off_w;
  uint4 v = make_uint4(0, 0, 0, 0);
  const int64_t scpp = a.src_ch / 8;
  if (n < a.N && sr >= 0 && sr < a.h && sc >= 0 && sc < a.w && chunk < scpp)
    v = src[((n * a.h + sr) * a.w + sc) * scpp + chunk];
  dst[lin] = v;
}

struct WgradSumArgs {
  int64_t N, K, R, S, C;
  int64_t Kp; // rows of a partial result (K, or 128 for narrower gradients)
  int64_t sk, sc, sr, ss; // element strides of DW [K, C, R, S]
  int32_t dt;
};

// DW[k][c][r][s] = sum over the N batch entries of partial[r][n][k][s * C + c]
__global__ void conv_wgrad_sum_kernel(WgradSumArgs a, const float *part,
                                      void *dw, int64_t total) {
  const int64_t lin = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (lin >= total)
    return;
  const int64_t sc = a.S * a.C;
  const int64_t j = lin % sc; // s * C + c
  int64_t rem = lin / sc;
  const int64_t k = rem % a.K;
  const int64_t r = rem / a.K;
  const float *src = part + (r * a.N * a.Kp + k) * sc + j;
  float acc = 0.f;
#pragma unroll 8 // independent loads: several in flight
  for (int64_t n = 0; n < a.N; ++n)
    acc += src[n * a.Kp * sc];
  const int64_t s = j / a.C, c = j - s * a.C;
  fhip_store<float>(dw, a.dt, k * a.sk + c * a.sc + r * a.sr + s * a.ss, acc);
}

} // namespace

bool fhip_fast_conv_wgrad_applicable(const fhip_conv_desc *d,
                                     size_t *workspace_bytes) {
  if (fhip_fast_conv_wgrad_direct_applicable(d, workspace_bytes))
    return true;
  const WgradPlan p = make_wgrad_plan(d);
  if (workspace_bytes)
    *workspace_bytes = p.ok ? p.xp_bytes + p.dyp_bytes + p.part_bytes : 0;
  return p.ok;
}

int fhip_fast_conv_wgrad(fhip_ctx *ctx, const fhip_conv_desc *d, const void *dy,
                         const void *x, void *dw, void *workspace) {
  if (fhip_fast_conv_wgrad_direct_applicable(d, nullptr))
    return fhip_fast_conv_wgrad_direct(ctx, d, dy, x, dw, workspace);
  const WgradPlan p = make_wgrad_plan(d);
  FHIP_REQUIRE(ctx, p.ok, "conv wgrad: descriptor not supported by the MFMA path");
  FHIP_REQUIRE(ctx, ((uintptr_t)workspace & 255) == 0 && ((uintptr_t)x & 15) == 0 &&
                        ((uintptr_t)dy & 15) == 0,
               "conv wgrad: workspace must be 256-byte and tensors 16-byte aligned");
  char *xp = (char *)workspace;
  char *dyp = xp + p.xp_bytes;
  float *part = (float *)(dyp + p.dyp_bytes);
  // X into its padded grid (the guard behind the last image included: the
  // grid is extended by whole zero images' worth of chunks up to the buffer's
  // end), DY into the top-left corner of the same grid
  PadArgs ax{p.N, p.rows, p.pitch, p.C, p.C, p.H, p.W, p.pad_h, p.pad_w,
             (int64_t)(p.xp_bytes / 16)};
  hipLaunchKernelGGL(conv_pad_grid_kernel, dim3((unsigned)((ax.total + 255) / 256)),
                     dim3(256), 0, ctx->stream, ax, (const uint4 *)x, (uint4 *)xp);
  PadArgs ay{p.N, p.rows_y, p.pitch, p.Kp, p.K, p.P, p.Q, 0, 0,
             (int64_t)(p.N * p.pix_y * p.Kp * 2 / 16)};
  hipLaunchKernelGGL(conv_pad_grid_kernel, dim3((unsigned)((ay.total + 255) / 256)),
                     dim3(256), 0, ctx->stream, ay, (const uint4 *)dy, (uint4 *)dyp);
  FHIP_HIP_CHECK(ctx, hipGetLastError());
  DevEpilogue epi{};
  // all filter rows in one launch: the outer batch dim steps B by one filter
  // row of pixels and the output by one block of partial results
  if (fhip_fast_matmul_outer(ctx, &p.mm, dyp, xp, epi, part, (int)p.R, 0,
                             p.dil_h * p.pitch * p.C,
                             p.N * p.split * p.Kp * p.S * p.C) != 0)
    return 1;
  WgradSumArgs as;
  as.N = p.N * p.split, as.K = p.K, as.R = p.R, as.S = p.S, as.C = p.C;
  as.Kp = p.Kp;
  as.sk = d->w.dim[0] == 1 ? 0 : d->w.stride[0];
  as.sc = d->w.dim[1] == 1 ? 0 : d->w.stride[1];
  as.sr = d->w.dim[2] == 1 ? 0 : d->w.stride[2];
  as.ss = d->w.dim[3] == 1 ? 0 : d->w.stride[3];
  as.dt = d->w.dtype;
  const int64_t total = p.R * p.K * p.S * p.C;
  hipLaunchKernelGGL(conv_wgrad_sum_kernel, dim3((unsigned)((total + 255) / 256)),
                     dim3(256), 0, ctx->stream, as, part, dw, total);
  FHIP_HIP_CHECK(ctx, hipGetLastError());
  fhip_note_kernel(ctx, "conv_wgrad batched gemm");
  return 0;
}
