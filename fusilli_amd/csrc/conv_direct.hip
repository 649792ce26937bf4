// Register-blocked direct convolution, data gradient and weight gradient for
// any layout, dtype, group count and 1 - 3 spatial dims: the path of every
// convolution the MFMA kernels do not take (few channels, NCHW, f32, groups).
//
// All three kernels put one output PIXEL on a thread (consecutive threads are
// consecutive pixels of the innermost spatial dim, so NCHW tensors are read and
// written in contiguous runs) and a block of channels in its registers:
//   * forward: 8 output channels per thread; the workgroup's slice of the
//     filter sits in LDS as f32 ([channel][tap][8]) and every X value loaded
//     feeds 8 multiply-adds against two 16-byte broadcast reads;
//   * data gradient: 8 input channels per thread, the filter slice in LDS as
//     [output channel][tap][8]; the taps' validity (inside DY, divisible by the
//     stride) is decided once per tap, outside the channel loop;
//   * weight gradient: a thread accumulates a 4 (output channels) x 32 (filter
//     channel, tap) block of DW over its pixels in registers; the workgroup's
//     256 partial blocks are added through LDS in a fixed order and the
//     workgroups' sums by a second kernel -- no atomics.
// Spatial dims are padded to three on the host (leading dims of extent 1), so
// the kernels have one loop nest.
//
// Reference semantics: aten.convolution / aten.convolution_backward
// (reference support/asm_emitter.h:690-701, 868-873, 1030-1035;
// node/conv_node.h:38-56, 255-598).
#include "common.h"
#include "fast_paths.h"

#include <type_traits>

namespace {

constexpr int kDcT = 8;       // channels per thread (forward, data gradient)
constexpr int kDcLds = 8192;  // floats of staged filter
constexpr int kWgK = 4;       // weight gradient: output channels per thread
constexpr int kWgJ = 32;      // weight gradient: (filter channel, tap) pairs

struct DcArgs {
  int32_t N, groups, fC, kpg; // filter channels / output channels per group
  int32_t xd[3], yd[3], fd[3], pad[3], str[3], dil[3];
  int64_t xs[5], ws[5], ys[5], os[5]; // [n or k, channel, 3 spatial]; os = OUT
  int32_t x_dt, w_dt, y_dt, o_dt;
  int32_t sp;    // spatial rank of the caller's tensors (epilogue coordinates)
  int32_t chunk; // channels staged per pass
  DevEpilogue epi;
};

// DT >= 0: every tensor of the call has this dtype (the switch folds away)
template <int DT>
__device__ __forceinline__ float dc_load(const void *p, int dt, int64_t i) {
  return fhip_load<float>(p, DT >= 0 ? DT : dt, i);
}

template <int DT>
__global__ __launch_bounds__(256) void direct_conv_fprop_kernel(
    DcArgs g, const void *x, const void *w, void *out) {
  __shared__ __attribute__((aligned(16))) float wl[kDcLds];
  const int tid = threadIdx.x;
  const int fvol = g.fd[0] * g.fd[1] * g.fd[2];
  const int kblocks = (g.kpg + kDcT - 1) / kDcT;
  const int grp = blockIdx.y / kblocks;
  const int kb = (blockIdx.y - grp * kblocks) * kDcT;
  const int kvalid = g.kpg - kb < kDcT ? g.kpg - kb : kDcT;
  const int k0 = grp * g.kpg + kb;
  const uint32_t total = (uint32_t)g.N * g.yd[0] * g.yd[1] * g.yd[2];
  const uint32_t p = blockIdx.x * 256u + tid;
  const bool live = p < total;
  uint32_t r = live ? p : 0;
  const int o2 = r % (uint32_t)g.yd[2];
  r /= (uint32_t)g.yd[2];
  const int o1 = r % (uint32_t)g.yd[1];
  r /= (uint32_t)g.yd[1];
  const int o0 = r % (uint32_t)g.yd[0];
  const int n = r / (uint32_t)g.yd[0];
  const int i0 = o0 * g.str[0] - g.pad[0], i1 = o1 * g.str[1] - g.pad[1],
            i2 = o2 * g.str[2] - g.pad[2];
  const int64_t xb = n * g.xs[0] + (int64_t)grp * g.fC * g.xs[1];
  float acc[kDcT];
#pragma unroll
  for (int t = 0; t < kDcT; ++t)
    acc[t] = 0.f;
  for (int c0 = 0; c0 < g.fC; c0 += g.chunk) {
    const int cnt = g.fC - c0 < g.chunk ? g.fC - c0 : g.chunk;
    __syncthreads();
    for (int e = tid; e < cnt * fvol * kDcT; e += 256) {
      const int kt = e % kDcT;
      const int t = e / kDcT;
      const int f = t % fvol, cl = t / fvol;
      const int f2 = f % g.fd[2], q = f / g.fd[2];
      const int f1 = q % g.fd[1], f0 = q / g.fd[1];
      float v = 0.f;
      if (kt < kvalid)
        v = dc_load<DT>(w, g.w_dt,
                        (k0 + kt) * g.ws[0] + (c0 + cl) * g.ws[1] +
                            f0 * g.ws[2] + f1 * g.ws[3] + f2 * g.ws[4]);
      wl[e] = v;
    }
    __syncthreads();
    if (!live)
      continue;
    for (int cl = 0; cl < cnt; ++cl) {
      const int64_t xc = xb + (c0 + cl) * g.xs[1];
      const float *wc = wl + cl * fvol * kDcT;
      for (int f0 = 0; f0 < g.fd[0]; ++f0) {
        const int a0 = i0 + f0 * g.dil[0];
        if ((unsigned)a0 >= (unsigned)g.xd[0])
          continue;
        for (int f1 = 0; f1 < g.fd[1]; ++f1) {
          const int a1 = i1 + f1 * g.dil[1];
          if ((unsigned)a1 >= (unsigned)g.xd[1])
            continue;
          const int64_t xr = xc + a0 * g.xs[2] + a1 * g.xs[3];
          const float *wr = wc + (f0 * g.fd[1] + f1) * g.fd[2] * kDcT;
          for (int f2 = 0; f2 < g.fd[2]; ++f2) {
            const int a2 = i2 + f2 * g.dil[2];
            if ((unsigned)a2 >= (unsigned)g.xd[2])
              continue;
            const float xv = dc_load<DT>(x, g.x_dt, xr + a2 * g.xs[4]);
            const float *wp = wr + f2 * kDcT;
#pragma unroll
            for (int t = 0; t < kDcT; ++t)
              acc[t] = __builtin_fmaf(xv, wp[t], acc[t]);
          }
        }
      }
    }
  }
  if (!live)
    return;
  int64_t coord[FHIP_MAX_RANK];
  coord[0] = n;
  const int o[3] = {o0, o1, o2};
  for (int i = 0; i < g.sp; ++i)
    coord[2 + i] = o[3 - g.sp + i];
  const int64_t ob = n * g.os[0] + o0 * g.os[2] + o1 * g.os[3] + o2 * g.os[4];
  // (the channels of a thread together: a fused operand's values are fetched
  // as one batch of loads)
  float v[kDcT];
  int64_t chans[kDcT];
#pragma unroll
  for (int t = 0; t < kDcT; ++t) {
    chans[t] = k0 + (t < kvalid ? t : kvalid - 1);
    v[t] = fhip_round_through<float>(g.y_dt, acc[t]);
  }
  if (g.epi.count > 0)
    fhip_apply_epilogue_many<float, kDcT>(g.epi, v, coord, 1, chans);
#pragma unroll
  for (int t = 0; t < kDcT; ++t) {
    if (t >= kvalid)
      break;
    fhip_store<float>(out, g.o_dt, ob + (k0 + t) * g.os[1], v[t]);
  }
}

// ---- channels-last groups of 1, 2, 4 or 8 channels (depthwise, ResNeXt) ------
// 16-bit channels-last X, W and OUT (f32 OUT too) with as many output as input
// channels per group.  A thread owns one output pixel and 8 consecutive
// channels -- whole groups -- so that every tap is ONE 16-byte load of X (the
// lanes of a pixel are consecutive chunks: coalesced) feeding 8 x CG
// multiply-adds, and the 8 results leave as one 16-byte store.  A workgroup is
// 16 pixels x 16 channel blocks; it keeps the f32 filter of its 128 channels in
// LDS as [block][tap][8][CG] (blocks 4 words past a multiple of 64 apart: the
// 16 blocks of a wavefront read different banks, its 4 pixels the same words)
// and four groups of 16 pixels (a thread's four pixels go tap by tap together).
constexpr int kDcClPix = 4; // pixels per thread

struct DcClArgs {
  int32_t N, H, W, C, K, P, Q, R, S;
  int32_t pad_h, pad_w, str_h, str_w, dil_h, dil_w;
  int32_t cbs;     // 8-channel blocks of a pixel
  int32_t stride;  // LDS words between the blocks' filters
  int32_t y_dt, o_dt, sp;
  uint32_t pixels;
  uint32_t x_bytes;
  DevEpilogue epi;
};

template <bool BF16, int CG>
__global__ __launch_bounds__(256) void direct_conv_fprop_cl_kernel(
    DcClArgs g, const void *x, const void *w, void *out) {
  extern __shared__ __attribute__((aligned(16))) float wcl[];
  const int tid = threadIdx.x;
  const int cbl = tid & 15, pl = tid >> 4;
  const int cb0 = blockIdx.y * 16;
  const int fvol = g.R * g.S;
  const int per_block = fvol * 8 * CG;
  auto to_f32 = [](uint32_t h) __attribute__((always_inline)) {
    if constexpr (BF16)
      return __builtin_bit_cast(float, h << 16);
    else
      return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
  };
  for (int e = tid; e < 16 * per_block; e += 256) {
    const int b = e / per_block, rest = e - b * per_block; // rest = (tap * 8 + k) * CG + j
    const int j = rest % CG, tk = rest / CG;
    const int k = tk & 7, tap = tk >> 3;
    const int kg = (cb0 + b) * 8 + k;
    float v = 0.f;
    if (kg < g.K)
      v = to_f32(((const uint16_t *)w)[((int64_t)kg * fvol + tap) * CG + j]);
    wcl[b * g.stride + rest] = v;
  }
  __syncthreads();
  const int cb = cb0 + cbl;
  if (cb >= g.cbs)
    return;
  const float *wl = wcl + cbl * g.stride;
  // kDcClPix pixels per thread, 16 apart, tap by tap together: their loads are
  // in flight at the same time and a tap's filter is read from LDS once for
  // all of them.
  const uint32_t first = blockIdx.x * (uint32_t)(16 * kDcClPix) + (uint32_t)pl;
  // Per pixel: the byte offset of tap (0, 0) and one bit per filter row and
  // column that lies inside the image; a tap's own offset is the same for
  // every lane.  X is read through a buffer descriptor, so a tap outside the
  // image (offset 2^31) reads zeros.
  uint32_t base[kDcClPix], rmask[kDcClPix], cmask[kDcClPix];
  float acc[kDcClPix][8];
  const uint32_t chan = (uint32_t)cb * 8u;
#pragma unroll
  for (int u = 0; u < kDcClPix; ++u) {
    const uint32_t pix = first + (uint32_t)u * 16u;
    const bool live = pix < g.pixels;
    const uint32_t px = live ? pix : 0u;
    const int q = px % (uint32_t)g.Q;
    const uint32_t t = px / (uint32_t)g.Q;
    const int p = t % (uint32_t)g.P;
    const int n = (int)(t / (uint32_t)g.P);
    const int ih0 = p * g.str_h - g.pad_h, iw0 = q * g.str_w - g.pad_w;
    // (modulo 2^32: taps above or left of the image are masked)
    base[u] = ((uint32_t)((n * g.H + ih0) * g.W + iw0) * (uint32_t)g.C + chan) * 2u;
    uint32_t rm = 0, cm = 0;
    for (int r = 0; r < g.R; ++r)
      rm |= (uint32_t)(live && (unsigned)(ih0 + r * g.dil_h) < (unsigned)g.H) << r;
    for (int s2 = 0; s2 < g.S; ++s2)
      cm |= (uint32_t)((unsigned)(iw0 + s2 * g.dil_w) < (unsigned)g.W) << s2;
    rmask[u] = rm;
    cmask[u] = cm;
#pragma unroll
    for (int k = 0; k < 8; ++k)
      acc[u][k] = 0.f;
  }
  const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<void *>(x), 0, (int)g.x_bytes, 0x00020000);
  for (int r = 0; r < g.R; ++r)
    for (int s = 0; s < g.S; ++s) {
      const int toff = ((r * g.dil_h * g.W + s * g.dil_w) * g.C) * 2;
      typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
      u32x4 xv[kDcClPix];
#pragma unroll
      for (int u = 0; u < kDcClPix; ++u) {
        const bool in = (rmask[u] >> r) & (cmask[u] >> s) & 1u;
        // (the sum, not a scalar offset: the range check sees only the lane's
        // offset, and base alone may lie before the tensor)
        xv[u] = __builtin_amdgcn_raw_buffer_load_b128(
            rx, in ? (int)(base[u] + (uint32_t)toff) : (int)0x80000000, 0, 0);
      }
      // (16-byte aligned: the blocks' distance and a tap's 8 * CG words are
      // multiples of 4 words)
      const float4 *wt4 = (const float4 *)(wl + (r * g.S + s) * 8 * CG);
      float wt[8 * CG];
#pragma unroll
      for (int i = 0; i < 2 * CG; ++i) {
        const float4 v = wt4[i];
        wt[4 * i] = v.x, wt[4 * i + 1] = v.y, wt[4 * i + 2] = v.z, wt[4 * i + 3] = v.w;
      }
#pragma unroll
      for (int u = 0; u < kDcClPix; ++u) {
        const uint32_t xw[4] = {xv[u].x, xv[u].y, xv[u].z, xv[u].w};
        float xf[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          xf[2 * i] = to_f32(xw[i] & 0xffffu);
          xf[2 * i + 1] = to_f32(xw[i] >> 16);
        }
#pragma unroll
        for (int k = 0; k < 8; ++k)
#pragma unroll
          for (int j = 0; j < CG; ++j)
            acc[u][k] = __builtin_fmaf(xf[k / CG * CG + j], wt[k * CG + j], acc[u][k]);
      }
    }
#pragma unroll
  for (int u = 0; u < kDcClPix; ++u) {
    const uint32_t pix = first + (uint32_t)u * 16u;
    if (pix >= g.pixels)
      break;
    float y[8];
#pragma unroll
    for (int k = 0; k < 8; ++k)
      y[k] = g.y_dt == FHIP_FLOAT ? acc[u][k] : fhip_round_through<float>(g.y_dt, acc[u][k]);
    if (g.epi.count > 0) {
      const int q = pix % (uint32_t)g.Q;
      const uint32_t t = pix / (uint32_t)g.Q;
      int64_t coord[FHIP_MAX_RANK];
      coord[0] = t / (uint32_t)g.P;
      if (g.sp == 2) {
        coord[2] = t % (uint32_t)g.P;
        coord[3] = q;
      } else {
        coord[2] = q;
      }
      int64_t chans[8];
#pragma unroll
      for (int k = 0; k < 8; ++k)
        chans[k] = cb * 8 + k;
      fhip_apply_epilogue_many<float, 8>(g.epi, y, coord, 1, chans);
    }
    // (OUT has fewer than 2^31 elements)
    const uint32_t ob = pix * (uint32_t)g.K + chan;
    if (g.o_dt == FHIP_FLOAT) {
      float4 *o = (float4 *)((float *)out + ob);
      o[0] = make_float4(y[0], y[1], y[2], y[3]);
      o[1] = make_float4(y[4], y[5], y[6], y[7]);
    } else {
      uint32_t ow[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        uint32_t lo, hi;
        if (g.o_dt == FHIP_BFLOAT16) {
          lo = __builtin_bit_cast(uint16_t, (__bf16)y[2 * i]);
          hi = __builtin_bit_cast(uint16_t, (__bf16)y[2 * i + 1]);
        } else {
          lo = __builtin_bit_cast(uint16_t, (_Float16)y[2 * i]);
          hi = __builtin_bit_cast(uint16_t, (_Float16)y[2 * i + 1]);
        }
        ow[i] = lo | (hi << 16);
      }
      *(uint4 *)((uint16_t *)out + ob) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
    }
  }
}

// ---- depthwise 3 x 3, unit stride and dilation, channels-last ------------------
// A thread owns a strip of kDwQ consecutive output pixels of one row and 8
// consecutive channels.  Its 9 x 8 filter values stay in registers (72 floats,
// loaded as nine 16-byte vectors: the 8 channels' taps are contiguous in W),
// and the strip's 3 x (kDwQ + 2) input vectors are loaded once -- each feeds up
// to three output pixels -- so a pixel costs 4.5 loads instead of 9 and no LDS
// at all.  Lanes run over the channel blocks first (a pixel's chunks are
// coalesced), then over the strips.  Taps outside the image read zeros through
// the buffer descriptor's range check.
constexpr int kDwQ = 4;

template <bool BF16>
__global__ __launch_bounds__(256) void depthwise3x3_cl_kernel(DcClArgs g, const void *x,
                                                              const void *w, void *out,
                                                              uint32_t strips, uint32_t strips_q) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  auto to_f32 = [](uint32_t h) __attribute__((always_inline)) {
    if constexpr (BF16)
      return __builtin_bit_cast(float, h << 16);
    else
      return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
  };
  const int cb = blockIdx.y * 16 + (threadIdx.x & 15);
  const uint32_t strip = blockIdx.x * 16u + (threadIdx.x >> 4);
  if (cb >= g.cbs || strip >= strips)
    return;
  const uint32_t chan = (uint32_t)cb * 8u;
  // filter: wt[tap][k] = W[chan + k][tap]
  float wt[9][8];
  {
    const u32x4 *wp = (const u32x4 *)((const uint16_t *)w + (size_t)chan * 9);
    uint32_t raw[36];
#pragma unroll
    for (int i = 0; i < 9; ++i) {
      const u32x4 v = wp[i];
      raw[4 * i] = v.x, raw[4 * i + 1] = v.y, raw[4 * i + 2] = v.z, raw[4 * i + 3] = v.w;
    }
#pragma unroll
    for (int k = 0; k < 8; ++k)
#pragma unroll
      for (int t = 0; t < 9; ++t) {
        const int e = k * 9 + t;
        wt[t][k] = to_f32((e & 1) ? raw[e >> 1] >> 16 : raw[e >> 1] & 0xffffu);
      }
  }
  const uint32_t qs = strip % strips_q;
  const uint32_t t1 = strip / strips_q;
  const int p = (int)(t1 % (uint32_t)g.P);
  const int n = (int)(t1 / (uint32_t)g.P);
  const int q0 = (int)qs * kDwQ;
  const int ih0 = p - g.pad_h, iw0 = q0 - g.pad_w;
  const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<void *>(x), 0, (int)g.x_bytes, 0x00020000);
  u32x4 xv[3][kDwQ + 2];
#pragma unroll
  for (int r = 0; r < 3; ++r) {
    const int ih = ih0 + r;
    const bool row_in = (unsigned)ih < (unsigned)g.H;
#pragma unroll
    for (int c = 0; c < kDwQ + 2; ++c) {
      const int iw = iw0 + c;
      const bool in = row_in && (unsigned)iw < (unsigned)g.W;
      const uint32_t off = ((uint32_t)((n * g.H + ih) * g.W + iw) * (uint32_t)g.C + chan) * 2u;
      xv[r][c] = __builtin_amdgcn_raw_buffer_load_b128(rx, in ? (int)off : (int)0x80000000, 0, 0);
    }
  }
  float acc[kDwQ][8];
#pragma unroll
  for (int u = 0; u < kDwQ; ++u)
#pragma unroll
    for (int k = 0; k < 8; ++k)
      acc[u][k] = 0.f;
#pragma unroll
  for (int r = 0; r < 3; ++r)
#pragma unroll
    for (int c = 0; c < kDwQ + 2; ++c) {
      const uint32_t xw[4] = {xv[r][c].x, xv[r][c].y, xv[r][c].z, xv[r][c].w};
      float xf[8];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        xf[2 * i] = to_f32(xw[i] & 0xffffu);
        xf[2 * i + 1] = to_f32(xw[i] >> 16);
      }
      // input column c is tap s = c - u of output pixel u (taps in filter order
      // per pixel: r ascending, then s ascending -- the order of the other kernels)
#pragma unroll
      for (int u = 0; u < kDwQ; ++u) {
        const int sx = c - u;
        if (sx < 0 || sx > 2)
          continue;
#pragma unroll
        for (int k = 0; k < 8; ++k)
          acc[u][k] = __builtin_fmaf(xf[k], wt[r * 3 + sx][k], acc[u][k]);
      }
    }
#pragma unroll
  for (int u = 0; u < kDwQ; ++u) {
    const int qq = q0 + u;
    if (qq >= g.Q)
      break;
    float y[8];
#pragma unroll
    for (int k = 0; k < 8; ++k)
      y[k] = g.y_dt == FHIP_FLOAT ? acc[u][k] : fhip_round_through<float>(g.y_dt, acc[u][k]);
    if (g.epi.count > 0) {
      int64_t coord[FHIP_MAX_RANK];
      coord[0] = n;
      coord[2] = p;
      coord[3] = qq;
      int64_t chans[8];
#pragma unroll
      for (int k = 0; k < 8; ++k)
        chans[k] = cb * 8 + k;
      fhip_apply_epilogue_many<float, 8>(g.epi, y, coord, 1, chans);
    }
    // (OUT has fewer than 2^31 elements)
    const uint32_t ob = ((uint32_t)((n * g.P + p) * g.Q + qq)) * (uint32_t)g.K + chan;
    if (g.o_dt == FHIP_FLOAT) {
      float4 *o = (float4 *)((float *)out + ob);
      o[0] = make_float4(y[0], y[1], y[2], y[3]);
      o[1] = make_float4(y[4], y[5], y[6], y[7]);
    } else {
      uint32_t ow[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        uint32_t lo, hi;
        if (g.o_dt == FHIP_BFLOAT16) {
          lo = __builtin_bit_cast(uint16_t, (__bf16)y[2 * i]);
          hi = __builtin_bit_cast(uint16_t, (__bf16)y[2 * i + 1]);
        } else {
          lo = __builtin_bit_cast(uint16_t, (_Float16)y[2 * i]);
          hi = __builtin_bit_cast(uint16_t, (_Float16)y[2 * i + 1]);
        }
        ow[i] = lo | (hi << 16);
      }
      *(uint4 *)((uint16_t *)out + ob) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
    }
  }
}

// dense channels-last strides of dims [d0, C, spatial...] (unit dims are free)
bool dc_channels_last(const fhip_tensor_desc &t) {
  int64_t expect = t.dim[1];
  if (t.dim[1] != 1 && t.stride[1] != 1)
    return false;
  for (int i = t.rank - 1; i >= 2; --i) {
    if (t.dim[i] != 1 && t.stride[i] != expect)
      return false;
    expect *= t.dim[i];
  }
  return t.dim[0] == 1 || t.stride[0] == expect;
}

constexpr int kDcClLds = 64 * 1024;

bool make_cl_args(const fhip_conv_desc *d, DcClArgs &g) {
  const int sp = d->spatial_rank;
  if ((sp != 1 && sp != 2) || d->x.rank != 2 + sp)
    return false;
  if (d->x.dtype != d->w.dtype ||
      (d->x.dtype != FHIP_BFLOAT16 && d->x.dtype != FHIP_HALF))
    return false;
  if (d->out.dtype != FHIP_BFLOAT16 && d->out.dtype != FHIP_HALF &&
      d->out.dtype != FHIP_FLOAT)
    return false;
  const int64_t C = d->x.dim[1], K = d->w.dim[0], CG = d->w.dim[1];
  if (C != K || C % 8 != 0 || (CG != 1 && CG != 2 && CG != 4 && CG != 8))
    return false;
  if (!dc_channels_last(d->x) || !dc_channels_last(d->w) || !dc_channels_last(d->out) ||
      d->out.rank != d->y.rank)
    return false;
  const int64_t lim = 1ll << 30;
  const int64_t pixels = fhip_desc_volume(d->y) / (K > 0 ? K : 1);
  if (fhip_desc_volume(d->x) >= lim || fhip_desc_volume(d->y) >= lim * 2 || pixels < 1)
    return false;
  g.N = (int32_t)d->x.dim[0];
  g.C = (int32_t)C;
  g.K = (int32_t)K;
  g.H = sp == 2 ? (int32_t)d->x.dim[2] : 1;
  g.W = (int32_t)d->x.dim[1 + sp];
  g.P = sp == 2 ? (int32_t)d->y.dim[2] : 1;
  g.Q = (int32_t)d->y.dim[1 + sp];
  g.R = sp == 2 ? (int32_t)d->w.dim[2] : 1;
  g.S = (int32_t)d->w.dim[1 + sp];
  g.pad_h = sp == 2 ? (int32_t)d->padding[0] : 0;
  g.str_h = sp == 2 ? (int32_t)d->stride[0] : 1;
  g.dil_h = sp == 2 ? (int32_t)d->dilation[0] : 1;
  g.pad_w = (int32_t)d->padding[sp - 1];
  g.str_w = (int32_t)d->stride[sp - 1];
  g.dil_w = (int32_t)d->dilation[sp - 1];
  if (d->padding[sp - 1] >= lim || d->stride[sp - 1] >= lim || d->dilation[sp - 1] >= lim ||
      (sp == 2 && (d->padding[0] >= lim || d->stride[0] >= lim || d->dilation[0] >= lim)))
    return false;
  const int64_t per_block = (int64_t)g.R * g.S * 8 * CG;
  // blocks 4 words past a multiple of 64 apart
  const int64_t stride = (per_block + 59) / 64 * 64 + 4;
  if (16 * stride * 4 > kDcClLds)
    return false;
  g.stride = (int32_t)stride;
  g.cbs = (int32_t)(C / 8);
  if ((g.cbs + 15) / 16 > 65535)
    return false;
  g.pixels = (uint32_t)pixels;
  g.x_bytes = (uint32_t)(fhip_desc_volume(d->x) * 2);
  if (g.R > 32 || g.S > 32) // one validity bit per filter row and column
    return false;
  g.y_dt = d->y.dtype;
  g.o_dt = d->out.dtype;
  g.sp = sp;
  g.epi.count = 0;
  g.epi.rank = 0;
  return true;
}

// DX[n, c, i..] = sum over the k of c's group and the taps f with
// i + pad - f * dil = o * stride:  DY[n, k, o..] * W[k, c % fC, f..]
template <int DT>
__global__ __launch_bounds__(256) void direct_conv_dgrad_kernel(
    DcArgs g, const void *dy, const void *w, void *dx) {
  __shared__ __attribute__((aligned(16))) float wl[kDcLds];
  const int tid = threadIdx.x;
  const int fvol = g.fd[0] * g.fd[1] * g.fd[2];
  const int cblocks = (g.fC + kDcT - 1) / kDcT;
  const int grp = blockIdx.y / cblocks;
  const int cb = (blockIdx.y - grp * cblocks) * kDcT;
  const int cvalid = g.fC - cb < kDcT ? g.fC - cb : kDcT;
  const uint32_t total = (uint32_t)g.N * g.xd[0] * g.xd[1] * g.xd[2];
  const uint32_t p = blockIdx.x * 256u + tid;
  const bool live = p < total;
  uint32_t r = live ? p : 0;
  const int i2 = r % (uint32_t)g.xd[2];
  r /= (uint32_t)g.xd[2];
  const int i1 = r % (uint32_t)g.xd[1];
  r /= (uint32_t)g.xd[1];
  const int i0 = r % (uint32_t)g.xd[0];
  const int n = r / (uint32_t)g.xd[0];
  const int64_t yn = n * g.ys[0] + (int64_t)grp * g.kpg * g.ys[1];
  float acc[kDcT];
#pragma unroll
  for (int t = 0; t < kDcT; ++t)
    acc[t] = 0.f;
  // output position along one dim for tap f, or -1
  auto source = [](int i, int pad, int f, int dil, int str, int extent) {
    const int t = i + pad - f * dil;
    if (t < 0)
      return -1;
    const int o = str == 1 ? t : t / str;
    return o * str == t && o < extent ? o : -1;
  };
  for (int kk0 = 0; kk0 < g.kpg; kk0 += g.chunk) {
    const int cnt = g.kpg - kk0 < g.chunk ? g.kpg - kk0 : g.chunk;
    __syncthreads();
    for (int e = tid; e < cnt * fvol * kDcT; e += 256) {
      const int ct = e % kDcT;
      const int t = e / kDcT;
      const int f = t % fvol, kl = t / fvol;
      const int f2 = f % g.fd[2], q = f / g.fd[2];
      const int f1 = q % g.fd[1], f0 = q / g.fd[1];
      float v = 0.f;
      if (ct < cvalid)
        v = dc_load<DT>(w, g.w_dt,
                        (int64_t)(grp * g.kpg + kk0 + kl) * g.ws[0] +
                            (cb + ct) * g.ws[1] + f0 * g.ws[2] + f1 * g.ws[3] +
                            f2 * g.ws[4]);
      wl[e] = v;
    }
    __syncthreads();
    if (!live)
      continue;
    const int64_t yk = yn + kk0 * g.ys[1];
    for (int f0 = 0; f0 < g.fd[0]; ++f0) {
      const int s0 = source(i0, g.pad[0], f0, g.dil[0], g.str[0], g.yd[0]);
      if (s0 < 0)
        continue;
      for (int f1 = 0; f1 < g.fd[1]; ++f1) {
        const int s1 = source(i1, g.pad[1], f1, g.dil[1], g.str[1], g.yd[1]);
        if (s1 < 0)
          continue;
        for (int f2 = 0; f2 < g.fd[2]; ++f2) {
          const int s2 = source(i2, g.pad[2], f2, g.dil[2], g.str[2], g.yd[2]);
          if (s2 < 0)
            continue;
          const int64_t yb = yk + s0 * g.ys[2] + s1 * g.ys[3] + s2 * g.ys[4];
          const float *wf = wl + ((f0 * g.fd[1] + f1) * g.fd[2] + f2) * kDcT;
          for (int kl = 0; kl < cnt; ++kl) {
            const float yv = dc_load<DT>(dy, g.y_dt, yb + kl * g.ys[1]);
            const float *wp = wf + kl * fvol * kDcT;
#pragma unroll
            for (int t = 0; t < kDcT; ++t)
              acc[t] = __builtin_fmaf(yv, wp[t], acc[t]);
          }
        }
      }
    }
  }
  if (!live)
    return;
  const int64_t xb = n * g.xs[0] + i0 * g.xs[2] + i1 * g.xs[3] + i2 * g.xs[4] +
                     (int64_t)(grp * g.fC + cb) * g.xs[1];
#pragma unroll
  for (int t = 0; t < kDcT; ++t) {
    if (t >= cvalid)
      break;
    fhip_store<float>(dx, g.x_dt, xb + t * g.xs[1], acc[t]);
  }
}

// DW[k, fc, f..] = sum over n, o..:  DY[n, k, o..] * X[n, c, o * stride - pad +
// f * dil].  Workgroup (run, k block, pair block): pixels [run * per_run, ...)
// of output channels k0 .. k0 + 3 against 32 (filter channel, tap) pairs; its
// sums go to partial[run][k][pair].
template <int DT>
__global__ __launch_bounds__(256) void direct_conv_wgrad_kernel(
    DcArgs g, const void *dy, const void *x, float *partial, uint32_t per_run,
    uint32_t total) {
  __shared__ int pd[kWgJ][4];      // tap displacement per dim, pair in range
  __shared__ int64_t poff[kWgJ];   // X offset of the pair (channel and tap)
  __shared__ float red[kWgJ][257]; // one accumulator row of all threads
  __shared__ float red2[8][kWgJ];
  const int tid = threadIdx.x;
  const int fvol = g.fd[0] * g.fd[1] * g.fd[2];
  const int npairs = g.fC * fvol;
  const int kblocks = (g.kpg + kWgK - 1) / kWgK;
  const int grp = blockIdx.y / kblocks;
  const int kb = (blockIdx.y - grp * kblocks) * kWgK;
  const int kvalid = g.kpg - kb < kWgK ? g.kpg - kb : kWgK;
  const int k0 = grp * g.kpg + kb;
  const int j0 = blockIdx.z * kWgJ;
  if (tid < kWgJ) {
    const int j = j0 + tid;
    const bool in = j < npairs;
    const int jj = in ? j : 0;
    // pairs are numbered tap-major, channel-minor: a thread's 32 X values of
    // a pixel are neighbouring channels where the layout is channels-last
    const int fc = jj % g.fC, f = jj / g.fC;
    const int f2 = f % g.fd[2], q = f / g.fd[2];
    const int f1 = q % g.fd[1], f0 = q / g.fd[1];
    pd[tid][0] = f0 * g.dil[0];
    pd[tid][1] = f1 * g.dil[1];
    pd[tid][2] = f2 * g.dil[2];
    pd[tid][3] = in ? 1 : 0;
    poff[tid] = (int64_t)(grp * g.fC + fc) * g.xs[1] +
                (int64_t)(f0 * g.dil[0]) * g.xs[2] +
                (int64_t)(f1 * g.dil[1]) * g.xs[3] +
                (int64_t)(f2 * g.dil[2]) * g.xs[4];
  }
  __syncthreads();
  float acc[kWgK][kWgJ];
#pragma unroll
  for (int t = 0; t < kWgK; ++t)
#pragma unroll
    for (int j = 0; j < kWgJ; ++j)
      acc[t][j] = 0.f;
  const uint32_t first = blockIdx.x * per_run;
  const uint32_t last = first + per_run < total ? first + per_run : total;
  for (uint32_t p = first + tid; p < last; p += 256) {
    uint32_t r = p;
    const int o2 = r % (uint32_t)g.yd[2];
    r /= (uint32_t)g.yd[2];
    const int o1 = r % (uint32_t)g.yd[1];
    r /= (uint32_t)g.yd[1];
    const int o0 = r % (uint32_t)g.yd[0];
    const int n = r / (uint32_t)g.yd[0];
    const int64_t yb = n * g.ys[0] + o0 * g.ys[2] + o1 * g.ys[3] +
                       o2 * g.ys[4] + (int64_t)k0 * g.ys[1];
    float gy[kWgK];
#pragma unroll
    for (int t = 0; t < kWgK; ++t)
      gy[t] = t < kvalid ? dc_load<DT>(dy, g.y_dt, yb + t * g.ys[1]) : 0.f;
    const int b0 = o0 * g.str[0] - g.pad[0], b1 = o1 * g.str[1] - g.pad[1],
              b2 = o2 * g.str[2] - g.pad[2];
    const int64_t xb =
        n * g.xs[0] + b0 * g.xs[2] + b1 * g.xs[3] + b2 * g.xs[4];
#pragma unroll
    for (int j = 0; j < kWgJ; ++j) {
      const bool ok = pd[j][3] != 0 &&
                      (unsigned)(b0 + pd[j][0]) < (unsigned)g.xd[0] &&
                      (unsigned)(b1 + pd[j][1]) < (unsigned)g.xd[1] &&
                      (unsigned)(b2 + pd[j][2]) < (unsigned)g.xd[2];
      float xv = 0.f;
      if (ok)
        xv = dc_load<DT>(x, g.x_dt, xb + poff[j]);
#pragma unroll
      for (int t = 0; t < kWgK; ++t)
        acc[t][j] = __builtin_fmaf(gy[t], xv, acc[t][j]);
    }
  }
  // sum over the workgroup, one output channel at a time: thread (part, j)
  // adds 32 threads' values of pair j, then 32 threads add the 8 parts
  const int rj = tid & 31, part = tid >> 5;
#pragma unroll
  for (int t = 0; t < kWgK; ++t) {
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kWgJ; ++j)
      red[j][tid] = acc[t][j];
    __syncthreads();
    float s = 0.f;
    for (int i = 0; i < 32; ++i)
      s += red[rj][part * 32 + i];
    red2[part][rj] = s;
    __syncthreads();
    if (tid < kWgJ && t < kvalid && j0 + tid < npairs) {
      float sum = 0.f;
#pragma unroll
      for (int q = 0; q < 8; ++q)
        sum += red2[q][tid];
      const int64_t K = (int64_t)g.groups * g.kpg;
      partial[((int64_t)blockIdx.x * K + (k0 + t)) * npairs + j0 + tid] = sum;
    }
  }
}

// DW = sum of the runs' partial sums in run order; one thread per element.
__global__ __launch_bounds__(256) void direct_conv_wgrad_sum_kernel(
    DcArgs g, const float *partial, void *dw, int64_t elems, int runs) {
  const int64_t lin = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (lin >= elems)
    return;
  float sum = 0.f;
#pragma unroll 8
  for (int r = 0; r < runs; ++r)
    sum += partial[(int64_t)r * elems + lin];
  const int fvol = g.fd[0] * g.fd[1] * g.fd[2];
  const int64_t npairs = (int64_t)g.fC * fvol;
  const int64_t k = lin / npairs;
  const int j = (int)(lin - k * npairs);
  const int fc = j % g.fC, f = j / g.fC;
  const int f2 = f % g.fd[2], q = f / g.fd[2];
  const int f1 = q % g.fd[1], f0 = q / g.fd[1];
  fhip_store<float>(dw, g.w_dt,
                    k * g.ws[0] + fc * g.ws[1] + f0 * g.ws[2] + f1 * g.ws[3] +
                        f2 * g.ws[4],
                    sum);
}

// Spatial dims padded to three with leading unit dims.
bool make_args(const fhip_conv_desc *d, DcArgs &g) {
  const int sp = d->spatial_rank;
  if (sp < 1 || sp > 3)
    return false;
  const int64_t lim = 1ll << 30;
  g.N = (int32_t)d->x.dim[0];
  g.fC = (int32_t)d->w.dim[1];
  if (d->x.dim[0] >= lim || d->x.dim[1] >= lim || d->w.dim[0] >= lim ||
      d->w.dim[1] < 1)
    return false;
  g.groups = (int32_t)(d->x.dim[1] / d->w.dim[1]);
  g.kpg = (int32_t)(d->w.dim[0] / g.groups);
  auto st = [](const fhip_tensor_desc &t, int i) {
    return t.dim[i] == 1 ? (int64_t)0 : t.stride[i];
  };
  for (int i = 0; i < 2; ++i) {
    g.xs[i] = st(d->x, i);
    g.ws[i] = st(d->w, i);
    g.ys[i] = st(d->y, i);
    g.os[i] = st(d->out, i);
  }
  int64_t fvol = 1, xvol = d->x.dim[0], yvol = d->x.dim[0];
  for (int i = 0; i < 3; ++i) {
    const int j = i - (3 - sp);
    if (j < 0) {
      g.xd[i] = g.yd[i] = g.fd[i] = 1;
      g.pad[i] = 0;
      g.str[i] = g.dil[i] = 1;
      g.xs[2 + i] = g.ws[2 + i] = g.ys[2 + i] = g.os[2 + i] = 0;
      continue;
    }
    if (d->x.dim[2 + j] >= lim || d->y.dim[2 + j] >= lim ||
        d->w.dim[2 + j] >= lim || d->padding[j] >= lim || d->stride[j] >= lim ||
        d->dilation[j] >= lim ||
        d->dilation[j] * (d->w.dim[2 + j] - 1) + d->padding[j] +
                d->stride[j] * d->y.dim[2 + j] >=
            lim)
      return false;
    g.xd[i] = (int32_t)d->x.dim[2 + j];
    g.yd[i] = (int32_t)d->y.dim[2 + j];
    g.fd[i] = (int32_t)d->w.dim[2 + j];
    g.pad[i] = (int32_t)d->padding[j];
    g.str[i] = (int32_t)d->stride[j];
    g.dil[i] = (int32_t)d->dilation[j];
    g.xs[2 + i] = st(d->x, 2 + j);
    g.ws[2 + i] = st(d->w, 2 + j);
    g.ys[2 + i] = st(d->y, 2 + j);
    g.os[2 + i] = d->out.rank == d->y.rank ? st(d->out, 2 + j) : 0;
    fvol *= d->w.dim[2 + j];
    xvol *= d->x.dim[2 + j];
    yvol *= d->y.dim[2 + j];
    if (fvol >= lim || xvol >= lim || yvol >= lim)
      return false;
  }
  // a filter row of one channel block fits the staging buffer
  if (fvol * kDcT > kDcLds || fvol * d->w.dim[1] >= lim)
    return false;
  g.chunk = (int32_t)(kDcLds / (fvol * kDcT));
  g.x_dt = d->x.dtype;
  g.w_dt = d->w.dtype;
  g.y_dt = d->y.dtype;
  g.o_dt = d->out.dtype;
  g.sp = sp;
  g.epi.count = 0;
  g.epi.rank = 0;
  return true;
}

// the dtype the three tensors share (a compile-time path), or -1
int common_dtype(int a, int b, int c) {
  if (a == b && b == c &&
      (a == FHIP_FLOAT || a == FHIP_BFLOAT16 || a == FHIP_HALF))
    return a;
  return -1;
}

template <typename F> void by_dtype(int dt, F &&f) {
  switch (dt) {
  case FHIP_FLOAT:
    f(std::integral_constant<int, FHIP_FLOAT>{});
    break;
  case FHIP_BFLOAT16:
    f(std::integral_constant<int, FHIP_BFLOAT16>{});
    break;
  case FHIP_HALF:
    f(std::integral_constant<int, FHIP_HALF>{});
    break;
  default:
    f(std::integral_constant<int, -1>{});
    break;
  }
}

} // namespace

bool fhip_direct_conv_applicable(const fhip_conv_desc *d) {
  DcArgs g{};
  if (!make_args(d, g))
    return false;
  // grid limits: channel blocks in y (and pair blocks in z for the weight
  // gradient)
  const int64_t kblocks = (int64_t)g.groups * ((g.kpg + kWgK - 1) / kWgK);
  const int64_t cblocks = (int64_t)g.groups * ((g.fC + kDcT - 1) / kDcT);
  const int64_t fvol = (int64_t)g.fd[0] * g.fd[1] * g.fd[2];
  return kblocks <= 65535 && cblocks <= 65535 &&
         (g.fC * fvol + kWgJ - 1) / kWgJ <= 65535;
}

bool fhip_direct_conv_cl_applicable(const fhip_conv_desc *d) {
  DcClArgs g{};
  // (tensors that are not 16-byte aligned run on the general kernel)
  return make_cl_args(d, g) && fhip_direct_conv_applicable(d);
}

int fhip_direct_conv_fprop(fhip_ctx *ctx, const fhip_conv_desc *d,
                           const void *x, const void *w, const DevEpilogue &epi,
                           void *out) {
  {
    DcClArgs c{};
    if (make_cl_args(d, c) && (((uintptr_t)x | (uintptr_t)w | (uintptr_t)out) & 15) == 0) {
      c.epi = epi;
      // depthwise 3 x 3 at unit stride and dilation: the strip kernel
      if (d->w.dim[1] == 1 && c.sp == 2 && c.R == 3 && c.S == 3 && c.str_h == 1 && c.str_w == 1 &&
          c.dil_h == 1 && c.dil_w == 1 && fhip_knobs().conv_depthwise_strips) {
        const uint32_t strips_q = (uint32_t)((c.Q + kDwQ - 1) / kDwQ);
        const uint32_t strips = strips_q * (uint32_t)c.P * (uint32_t)c.N;
        const dim3 sgrid((strips + 15u) / 16u, (unsigned)((c.cbs + 15) / 16));
        if (d->x.dtype == FHIP_BFLOAT16)
          hipLaunchKernelGGL((depthwise3x3_cl_kernel<true>), sgrid, dim3(256), 0, ctx->stream, c, x,
                             w, out, strips, strips_q);
        else
          hipLaunchKernelGGL((depthwise3x3_cl_kernel<false>), sgrid, dim3(256), 0, ctx->stream, c,
                             x, w, out, strips, strips_q);
        FHIP_HIP_CHECK(ctx, hipGetLastError());
        fhip_note_kernel(ctx, "conv_depthwise3x3 channels_last strip=%d", kDwQ);
        return 0;
      }
      const dim3 grid((unsigned)((c.pixels + 16u * kDcClPix - 1) / (16u * kDcClPix)),
                      (unsigned)((c.cbs + 15) / 16));
      const size_t lds = (size_t)16 * c.stride * 4;
      const bool bf16 = d->x.dtype == FHIP_BFLOAT16;
      auto go = [&](auto cg) {
        constexpr int CG = decltype(cg)::value;
        if (bf16)
          hipLaunchKernelGGL((direct_conv_fprop_cl_kernel<true, CG>), grid, dim3(256), lds,
                             ctx->stream, c, x, w, out);
        else
          hipLaunchKernelGGL((direct_conv_fprop_cl_kernel<false, CG>), grid, dim3(256), lds,
                             ctx->stream, c, x, w, out);
      };
      switch ((int)d->w.dim[1]) {
      case 1:
        go(std::integral_constant<int, 1>{});
        break;
      case 2:
        go(std::integral_constant<int, 2>{});
        break;
      case 4:
        go(std::integral_constant<int, 4>{});
        break;
      default:
        go(std::integral_constant<int, 8>{});
        break;
      }
      FHIP_HIP_CHECK(ctx, hipGetLastError());
      fhip_note_kernel(ctx, "conv_direct channels_last group_width=%d", (int)d->w.dim[1]);
      return 0;
    }
  }
  fhip_note_kernel(ctx, "conv_direct");
  DcArgs g{};
  FHIP_REQUIRE(ctx, make_args(d, g),
               "conv: descriptor not supported by the direct kernel");
  g.epi = epi;
  const int64_t pixels = (int64_t)g.N * g.yd[0] * g.yd[1] * g.yd[2];
  if (pixels == 0 || d->w.dim[0] == 0)
    return 0;
  const dim3 grid((unsigned)((pixels + 255) / 256),
                  (unsigned)(g.groups * ((g.kpg + kDcT - 1) / kDcT)));
  by_dtype(common_dtype(g.x_dt, g.w_dt, g.x_dt), [&](auto dt) {
    hipLaunchKernelGGL(direct_conv_fprop_kernel<decltype(dt)::value>, grid,
                       dim3(256), 0, ctx->stream, g, x, w, out);
  });
  FHIP_HIP_CHECK(ctx, hipGetLastError());
  return 0;
}

int fhip_direct_conv_dgrad(fhip_ctx *ctx, const fhip_conv_desc *d,
                           const void *dy, const void *w, void *dx) {
  fhip_note_kernel(ctx, "conv_direct_dgrad");
  DcArgs g{};
  FHIP_REQUIRE(ctx, make_args(d, g),
               "conv: descriptor not supported by the direct kernel");
  // output channels staged per pass
  const int64_t pixels = (int64_t)g.N * g.xd[0] * g.xd[1] * g.xd[2];
  if (pixels == 0 || d->x.dim[1] == 0)
    return 0;
  const dim3 grid((unsigned)((pixels + 255) / 256),
                  (unsigned)(g.groups * ((g.fC + kDcT - 1) / kDcT)));
  by_dtype(common_dtype(g.y_dt, g.w_dt, g.y_dt), [&](auto dt) {
    hipLaunchKernelGGL(direct_conv_dgrad_kernel<decltype(dt)::value>, grid,
                       dim3(256), 0, ctx->stream, g, dy, w, dx);
  });
  FHIP_HIP_CHECK(ctx, hipGetLastError());
  return 0;
}

int fhip_direct_conv_wgrad(fhip_ctx *ctx, const fhip_conv_desc *d,
                           const void *dy, const void *x, void *dw) {
  fhip_note_kernel(ctx, "conv_direct_wgrad");
  DcArgs g{};
  FHIP_REQUIRE(ctx, make_args(d, g),
               "conv: descriptor not supported by the direct kernel");
  const int64_t elems = fhip_desc_volume(d->w);
  if (elems == 0)
    return 0;
  const int64_t pixels = (int64_t)g.N * g.yd[0] * g.yd[1] * g.yd[2];
  const int64_t fvol = (int64_t)g.fd[0] * g.fd[1] * g.fd[2];
  const int64_t gy = (int64_t)g.groups * ((g.kpg + kWgK - 1) / kWgK);
  const int64_t gz = (g.fC * fvol + kWgJ - 1) / kWgJ;
  // pixel runs: about two workgroups per compute unit, at least 256 pixels each
  const int64_t cus = ctx->num_cus > 0 ? ctx->num_cus : 256;
  int64_t runs = (2 * cus + gy * gz - 1) / (gy * gz);
  const int64_t most = (pixels + 255) / 256;
  runs = runs < most ? runs : most;
  runs = runs < 1024 ? runs : 1024;
  runs = runs < 1 ? 1 : runs;
  int64_t per_run = (pixels + runs - 1) / runs;
  per_run = per_run < 1 ? 1 : per_run;
  runs = pixels > 0 ? (pixels + per_run - 1) / per_run : 1;
  void *scratch = nullptr;
  if (fhip_ctx_scratch(ctx, (size_t)(runs * elems) * sizeof(float), &scratch) != 0)
    return 1;
  const dim3 grid((unsigned)runs, (unsigned)gy, (unsigned)gz);
  by_dtype(common_dtype(g.x_dt, g.y_dt, g.x_dt), [&](auto dt) {
    hipLaunchKernelGGL(direct_conv_wgrad_kernel<decltype(dt)::value>, grid,
                       dim3(256), 0, ctx->stream, g, dy, x, (float *)scratch,
                       (uint32_t)per_run, (uint32_t)pixels);
  });
  hipLaunchKernelGGL(direct_conv_wgrad_sum_kernel,
                     dim3((unsigned)((elems + 255) / 256)), dim3(256), 0,
                     ctx->stream, g, (const float *)scratch, dw, elems,
                     (int)runs);
  FHIP_HIP_CHECK(ctx, hipGetLastError());
  return 0;
}
