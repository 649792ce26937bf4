/*
 * fusilli_oracle.c — CPU restatement of the reference's operator semantics.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the product (fusilli_amd/, include/)
 * links, loads or calls this file; it is the checker used by tests/, by the
 * smoke test and by the CPU-baseline leg of the benchmark.
 *
 * The reference holds no arithmetic of its own: Graph::emitAsm lowers each
 * node to one torch-dialect op and the IREE compiler/runtime (pinned
 * iree-3.12.0rc20260515, version.json:3; not vendored) executes it.  Each
 * function below restates the published definition of the aten op the
 * reference emits, citing the emitter line that selects it and, where the
 * reference's samples carry a CPU formula, that formula.
 *
 * All tensors here are dense, in the op's logical dim order (NCHW, KCRS,
 * [B,H,S,D], [..,M,K]); the Python wrapper (oracle/oracle.py) applies the
 * TensorAttr dim/stride layout rules before and after.  Inputs are the exact
 * values of the quantised storage type widened to f32; accumulation is in
 * f64; results are f64 (int32 for the integer matmul).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>

/* ---- element conversions ------------------------------------------------ */

/* bfloat16: top 16 bits of an IEEE f32, round to nearest even
 * (reference support/float_types.h:89-103 `bf16 = __bf16`). */
uint16_t oracle_f32_to_bf16(float f) {
  union {
    float f;
    uint32_t u;
  } v = {f};
  if ((v.u & 0x7fffffffu) > 0x7f800000u)
    return (uint16_t)((v.u >> 16) | 0x0040u); /* quiet NaN */
  const uint32_t lsb = (v.u >> 16) & 1u;
  v.u += 0x7fffu + lsb;
  return (uint16_t)(v.u >> 16);
}

float oracle_bf16_to_f32(uint16_t h) {
  union {
    float f;
    uint32_t u;
  } v;
  v.u = (uint32_t)h << 16;
  return v.f;
}

/* OCP 8-bit floats (OCP 8-bit Floating Point Specification v1.0):
 * e4m3fn: 4 exponent bits, bias 7, no infinities, S.1111.111 = NaN, max 448;
 * e5m2  : 5 exponent bits, bias 15, IEEE-style inf/NaN, max 57344.
 * Decoding is exact.  Encoding rounds to nearest even on the fp8 grid and
 * saturates finite overflow to the largest finite value. */
static float fp8_decode(uint8_t v, int ebits) {
  const int mbits = 7 - ebits;
  const int bias = (1 << (ebits - 1)) - 1;
  const int sign = v >> 7;
  const int e = (v >> mbits) & ((1 << ebits) - 1);
  const int m = v & ((1 << mbits) - 1);
  double r;
  if (ebits == 4 && e == 15 && m == 7)
    return NAN;
  if (ebits == 5 && e == 31)
    return m ? NAN : (sign ? -INFINITY : INFINITY);
  if (e == 0)
    r = ldexp((double)m, 1 - bias - mbits);
  else
    r = ldexp((double)((1 << mbits) | m), e - bias - mbits);
  return (float)(sign ? -r : r);
}

static uint8_t fp8_encode(float f, int ebits) {
  const int mbits = 7 - ebits;
  const int bias = (1 << (ebits - 1)) - 1;
  const uint8_t maxfinite = ebits == 4 ? 0x7e : 0x7b;
  const uint8_t sign = signbit(f) ? 0x80 : 0;
  if (isnan(f))
    return (uint8_t)(sign | (ebits == 4 ? 0x7f : 0x7e));
  double a = fabs((double)f);
  if (isinf(f))
    return (uint8_t)(sign | (ebits == 4 ? maxfinite : 0x7c));
  if (a == 0.0)
    return sign;
  int ex;
  (void)frexp(a, &ex); /* a = m * 2^ex, m in [0.5, 1) */
  int e = ex - 1;      /* a in [2^e, 2^(e+1)) */
  if (e < 1 - bias)
    e = 1 - bias; /* subnormal grid */
  /* units of the grid at this exponent */
  const double q = ldexp(a, mbits - e);
  double r = nearbyint(q); /* default rounding mode: nearest even */
  uint32_t code;
  if (r >= (double)(2 << mbits)) { /* rounded up into the next binade */
    r /= 2.0;
    e += 1;
  }
  if (r < (double)(1 << mbits))
    code = (uint32_t)r; /* subnormal (or zero) */
  else
    code = ((uint32_t)(e + bias) << mbits) | ((uint32_t)r & ((1u << mbits) - 1u));
  if (code > maxfinite)
    code = maxfinite;
  return (uint8_t)(sign | code);
}

float oracle_fp8e4m3_to_f32(uint8_t v) { return fp8_decode(v, 4); }
float oracle_fp8e5m2_to_f32(uint8_t v) { return fp8_decode(v, 5); }
uint8_t oracle_f32_to_fp8e4m3(float f) { return fp8_encode(f, 4); }
uint8_t oracle_f32_to_fp8e5m2(float f) { return fp8_encode(f, 5); }

void oracle_f32_to_bf16_n(const float *in, uint16_t *out, int64_t n) {
  for (int64_t i = 0; i < n; ++i)
    out[i] = oracle_f32_to_bf16(in[i]);
}
void oracle_bf16_to_f32_n(const uint16_t *in, float *out, int64_t n) {
  for (int64_t i = 0; i < n; ++i)
    out[i] = oracle_bf16_to_f32(in[i]);
}
void oracle_f32_to_fp8_n(const float *in, uint8_t *out, int64_t n, int ebits) {
  for (int64_t i = 0; i < n; ++i)
    out[i] = fp8_encode(in[i], ebits);
}
void oracle_fp8_to_f32_n(const uint8_t *in, float *out, int64_t n, int ebits) {
  for (int64_t i = 0; i < n; ++i)
    out[i] = fp8_decode(in[i], ebits);
}

/* ---- matmul: aten.matmul (reference support/asm_emitter.h:1669-1696;
 *      shape rule node/matmul_node.h:40-66).  C[b,m,n] = sum_k A[b,m,k]*B[b,k,n]
 *      with the batch already broadcast by the caller. ------------------- */
void oracle_matmul_f32(const float *a, const float *b, double *c, int64_t batch,
                       int64_t m, int64_t k, int64_t n) {
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t bi = 0; bi < batch; ++bi)
    for (int64_t i = 0; i < m; ++i) {
      const float *ar = a + (bi * m + i) * k;
      double *cr = c + (bi * m + i) * n;
      for (int64_t j = 0; j < n; ++j)
        cr[j] = 0.0;
      for (int64_t kk = 0; kk < k; ++kk) {
        const double av = ar[kk];
        const float *br = b + (bi * k + kk) * n;
        for (int64_t j = 0; j < n; ++j)
          cr[j] += av * (double)br[j];
      }
    }
}

/* Integer matmul: si8 x si8 -> si32, exact (|acc| <= K * 127^2 < 2^31 for
 * K <= 133 000). */
void oracle_matmul_i8_i32(const int8_t *a, const int8_t *b, int32_t *c,
                          int64_t batch, int64_t m, int64_t k, int64_t n) {
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t bi = 0; bi < batch; ++bi)
    for (int64_t i = 0; i < m; ++i) {
      const int8_t *ar = a + (bi * m + i) * k;
      int32_t *cr = c + (bi * m + i) * n;
      for (int64_t j = 0; j < n; ++j)
        cr[j] = 0;
      for (int64_t kk = 0; kk < k; ++kk) {
        const int32_t av = ar[kk];
        const int8_t *br = b + (bi * k + kk) * n;
        for (int64_t j = 0; j < n; ++j)
          cr[j] += av * (int32_t)br[j];
      }
    }
}

/* Selected rows of an integer matmul (for full-size checks where the whole
 * product is too slow on the host). rows[i] indexes into m. */
void oracle_matmul_i8_i32_rows(const int8_t *a, const int8_t *b, int32_t *c,
                               const int64_t *rows, int64_t nrows, int64_t k,
                               int64_t n) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < nrows; ++r) {
    const int8_t *ar = a + rows[r] * k;
    int32_t *cr = c + r * n;
    for (int64_t j = 0; j < n; ++j)
      cr[j] = 0;
    for (int64_t kk = 0; kk < k; ++kk) {
      const int32_t av = ar[kk];
      const int8_t *br = b + kk * n;
      for (int64_t j = 0; j < n; ++j)
        cr[j] += av * (int32_t)br[j];
    }
  }
}

void oracle_matmul_f32_rows(const float *a, const float *b, double *c,
                            const int64_t *rows, int64_t nrows, int64_t k,
                            int64_t n) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < nrows; ++r) {
    const float *ar = a + rows[r] * k;
    double *cr = c + r * n;
    for (int64_t j = 0; j < n; ++j)
      cr[j] = 0.0;
    for (int64_t kk = 0; kk < k; ++kk) {
      const double av = ar[kk];
      const float *br = b + kk * n;
      for (int64_t j = 0; j < n; ++j)
        cr[j] += av * (double)br[j];
    }
  }
}

/* ---- convolution forward: aten.convolution, transposed = false, no bias
 *      (reference support/asm_emitter.h:690-701): cross-correlation with
 *      symmetric zero padding, stride, dilation; groups = C / fC; output
 *      extent 1 + (H + 2p - d(R-1) - 1)/s (node/conv_node.h:38-56).
 *      x [N,C,D1..], w [K,fC,F1..], y [N,K,O1..]; spatial rank 1..3, given
 *      as 3 extents with leading 1s. ------------------------------------- */
void oracle_conv_fprop(const float *x, const float *w, double *y, int64_t N,
                       int64_t C, int64_t K, int64_t fC, const int64_t *xd,
                       const int64_t *fd, const int64_t *od, const int64_t *pad,
                       const int64_t *str, const int64_t *dil) {
  const int64_t groups = C / fC;
  const int64_t kpg = K / groups;
  const int64_t xvol = xd[0] * xd[1] * xd[2];
  const int64_t fvol = fd[0] * fd[1] * fd[2];
  const int64_t ovol = od[0] * od[1] * od[2];
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t n = 0; n < N; ++n)
    for (int64_t k = 0; k < K; ++k) {
      const int64_t g = k / kpg;
      for (int64_t o0 = 0; o0 < od[0]; ++o0)
        for (int64_t o1 = 0; o1 < od[1]; ++o1)
          for (int64_t o2 = 0; o2 < od[2]; ++o2) {
            double acc = 0.0;
            for (int64_t fc = 0; fc < fC; ++fc) {
              const float *xc = x + (n * C + g * fC + fc) * xvol;
              const float *wc = w + (k * fC + fc) * fvol;
              for (int64_t f0 = 0; f0 < fd[0]; ++f0) {
                const int64_t i0 = o0 * str[0] - pad[0] + f0 * dil[0];
                if (i0 < 0 || i0 >= xd[0])
                  continue;
                for (int64_t f1 = 0; f1 < fd[1]; ++f1) {
                  const int64_t i1 = o1 * str[1] - pad[1] + f1 * dil[1];
                  if (i1 < 0 || i1 >= xd[1])
                    continue;
                  for (int64_t f2 = 0; f2 < fd[2]; ++f2) {
                    const int64_t i2 = o2 * str[2] - pad[2] + f2 * dil[2];
                    if (i2 < 0 || i2 >= xd[2])
                      continue;
                    acc += (double)xc[(i0 * xd[1] + i1) * xd[2] + i2] *
                           (double)wc[(f0 * fd[1] + f1) * fd[2] + f2];
                  }
                }
              }
            }
            y[(n * K + k) * ovol + (o0 * od[1] + o1) * od[2] + o2] = acc;
          }
    }
}

/* ---- convolution backward (reference node/conv_node.h:255-598; both nodes
 *      emit aten.convolution_backward): the adjoints of the forward above.
 *      Written as the forward loop nest run once more, scattering
 *      dY[n,k,o] into dX (times W) or into dW (times X) -- the same index
 *      arithmetic as oracle_conv_fprop, so a gather formulation in a kernel
 *      is checked against a different derivation.  f64 accumulation. ------ */
void oracle_conv_dgrad(const float *dy, const float *w, double *dx, int64_t N,
                       int64_t C, int64_t K, int64_t fC, const int64_t *xd,
                       const int64_t *fd, const int64_t *od, const int64_t *pad,
                       const int64_t *str, const int64_t *dil) {
  const int64_t groups = C / fC;
  const int64_t kpg = K / groups;
  const int64_t xvol = xd[0] * xd[1] * xd[2];
  const int64_t fvol = fd[0] * fd[1] * fd[2];
  const int64_t ovol = od[0] * od[1] * od[2];
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < N; ++n) {
    for (int64_t i = 0; i < C * xvol; ++i)
      dx[n * C * xvol + i] = 0.0;
    for (int64_t k = 0; k < K; ++k) {
      const int64_t g = k / kpg;
      for (int64_t o0 = 0; o0 < od[0]; ++o0)
        for (int64_t o1 = 0; o1 < od[1]; ++o1)
          for (int64_t o2 = 0; o2 < od[2]; ++o2) {
            const double gy =
                dy[(n * K + k) * ovol + (o0 * od[1] + o1) * od[2] + o2];
            for (int64_t fc = 0; fc < fC; ++fc) {
              double *xc = dx + (n * C + g * fC + fc) * xvol;
              const float *wc = w + (k * fC + fc) * fvol;
              for (int64_t f0 = 0; f0 < fd[0]; ++f0) {
                const int64_t i0 = o0 * str[0] - pad[0] + f0 * dil[0];
                if (i0 < 0 || i0 >= xd[0])
                  continue;
                for (int64_t f1 = 0; f1 < fd[1]; ++f1) {
                  const int64_t i1 = o1 * str[1] - pad[1] + f1 * dil[1];
                  if (i1 < 0 || i1 >= xd[1])
                    continue;
                  for (int64_t f2 = 0; f2 < fd[2]; ++f2) {
                    const int64_t i2 = o2 * str[2] - pad[2] + f2 * dil[2];
                    if (i2 < 0 || i2 >= xd[2])
                      continue;
                    xc[(i0 * xd[1] + i1) * xd[2] + i2] +=
                        gy * (double)wc[(f0 * fd[1] + f1) * fd[2] + f2];
                  }
                }
              }
            }
          }
    }
  }
}

void oracle_conv_wgrad(const float *dy, const float *x, double *dw, int64_t N,
                       int64_t C, int64_t K, int64_t fC, const int64_t *xd,
                       const int64_t *fd, const int64_t *od, const int64_t *pad,
                       const int64_t *str, const int64_t *dil) {
  const int64_t groups = C / fC;
  const int64_t kpg = K / groups;
  const int64_t xvol = xd[0] * xd[1] * xd[2];
  const int64_t fvol = fd[0] * fd[1] * fd[2];
  const int64_t ovol = od[0] * od[1] * od[2];
#pragma omp parallel for schedule(static)
  for (int64_t k = 0; k < K; ++k) {
    const int64_t g = k / kpg;
    for (int64_t i = 0; i < fC * fvol; ++i)
      dw[k * fC * fvol + i] = 0.0;
    for (int64_t n = 0; n < N; ++n)
      for (int64_t o0 = 0; o0 < od[0]; ++o0)
        for (int64_t o1 = 0; o1 < od[1]; ++o1)
          for (int64_t o2 = 0; o2 < od[2]; ++o2) {
            const double gy =
                dy[(n * K + k) * ovol + (o0 * od[1] + o1) * od[2] + o2];
            for (int64_t fc = 0; fc < fC; ++fc) {
              const float *xc = x + (n * C + g * fC + fc) * xvol;
              double *wc = dw + (k * fC + fc) * fvol;
              for (int64_t f0 = 0; f0 < fd[0]; ++f0) {
                const int64_t i0 = o0 * str[0] - pad[0] + f0 * dil[0];
                if (i0 < 0 || i0 >= xd[0])
                  continue;
                for (int64_t f1 = 0; f1 < fd[1]; ++f1) {
                  const int64_t i1 = o1 * str[1] - pad[1] + f1 * dil[1];
                  if (i1 < 0 || i1 >= xd[1])
                    continue;
                  for (int64_t f2 = 0; f2 < fd[2]; ++f2) {
                    const int64_t i2 = o2 * str[2] - pad[2] + f2 * dil[2];
                    if (i2 < 0 || i2 >= xd[2])
                      continue;
                    wc[(f0 * fd[1] + f1) * fd[2] + f2] +=
                        gy * (double)xc[(i0 * xd[1] + i1) * xd[2] + i2];
                  }
                }
              }
            }
          }
  }
}

/* ---- SDPA: aten.scaled_dot_product_attention (reference
 *      support/asm_emitter.h:2409-2468; CPU formula
 *      samples/sdpa_utils.cpp:49-102):
 *      O = softmax(Q K^T * scale + mask, causal: -inf where sk > sq) V,
 *      scale default 1/sqrt(D); GQA: query head h reads K/V head
 *      h / (Hq/Hkv).  mask is NULL or a dense additive [B,Hq,Sq,Skv]. ------ */
void oracle_sdpa(const float *q, const float *k, const float *v,
                 const float *mask, double *o, int64_t B, int64_t Hq,
                 int64_t Hkv, int64_t Sq, int64_t Skv, int64_t D, int64_t Dv,
                 int causal, double scale) {
  const int64_t rep = Hq / Hkv;
#pragma omp parallel for collapse(3) schedule(dynamic, 8)
  for (int64_t b = 0; b < B; ++b)
    for (int64_t h = 0; h < Hq; ++h)
      for (int64_t sq = 0; sq < Sq; ++sq) {
        const int64_t hk = h / rep;
        const float *qr = q + ((b * Hq + h) * Sq + sq) * D;
        double *s = (double *)malloc(sizeof(double) * (size_t)Skv);
        double mx = -INFINITY;
        for (int64_t sk = 0; sk < Skv; ++sk) {
          const float *kr = k + ((b * Hkv + hk) * Skv + sk) * D;
          double d = 0.0;
          for (int64_t e = 0; e < D; ++e)
            d += (double)qr[e] * (double)kr[e];
          d *= scale;
          if (mask)
            d += (double)mask[((b * Hq + h) * Sq + sq) * Skv + sk];
          if (causal && sk > sq)
            d = -INFINITY;
          s[sk] = d;
          if (d > mx)
            mx = d;
        }
        double sum = 0.0;
        for (int64_t sk = 0; sk < Skv; ++sk) {
          s[sk] = exp(s[sk] - mx);
          sum += s[sk];
        }
        double *orow = o + ((b * Hq + h) * Sq + sq) * Dv;
        for (int64_t e = 0; e < Dv; ++e)
          orow[e] = 0.0;
        for (int64_t sk = 0; sk < Skv; ++sk) {
          const double p = s[sk] / sum;
          if (p == 0.0)
            continue;
          const float *vr = v + ((b * Hkv + hk) * Skv + sk) * Dv;
          for (int64_t e = 0; e < Dv; ++e)
            orow[e] += p * (double)vr[e];
        }
        free(s);
      }
}

/* ---- RMSNorm: aten.rms_norm over all dims but dim 0 (reference
 *      support/asm_emitter.h:1592-1626, node/norm_utils.h:27-36; CPU formula
 *      samples/rmsnorm/rmsnorm_utils.h:26-66):
 *      y = x / sqrt(mean(x^2) + eps) * scale. ---------------------------- */
void oracle_rmsnorm(const float *x, const float *scale, double eps, double *y,
                    int64_t rows, int64_t inner) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    const float *xr = x + r * inner;
    double ss = 0.0;
    for (int64_t i = 0; i < inner; ++i)
      ss += (double)xr[i] * (double)xr[i];
    const double inv = 1.0 / sqrt(ss / (double)inner + eps);
    for (int64_t i = 0; i < inner; ++i)
      y[r * inner + i] =
          (double)xr[i] * inv * (scale ? (double)scale[i] : 1.0);
  }
}

/* Single-precision, storage-type-in / storage-type-out variant used as the
 * CPU baseline of the bandwidth benchmark: bf16 row in, f32 accumulate,
 * bf16 out, then one fused multiply by a scalar. */
void oracle_rmsnorm_bf16_baseline(const uint16_t *x, const uint16_t *scale,
                                  float eps, float mul, uint16_t *y,
                                  int64_t rows, int64_t inner) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    const uint16_t *xr = x + r * inner;
    float ss = 0.f;
    for (int64_t i = 0; i < inner; ++i) {
      const float f = oracle_bf16_to_f32(xr[i]);
      ss += f * f;
    }
    const float inv = 1.0f / sqrtf(ss / (float)inner + eps);
    for (int64_t i = 0; i < inner; ++i)
      y[r * inner + i] = oracle_f32_to_bf16(oracle_bf16_to_f32(xr[i]) * inv *
                                            oracle_bf16_to_f32(scale[i]) * mul);
  }
}

/* ---- LayerNorm: aten.layer_norm / aten.native_layer_norm over all dims but
 *      dim 0 (reference support/asm_emitter.h:1427-1503; CPU formula
 *      samples/layernorm/layernorm_utils.h:25-82): biased variance;
 *      y = (x - mean) * rstd * scale + bias; also returns mean and rstd. -- */
void oracle_layernorm(const float *x, const float *scale, const float *bias,
                      double eps, double *y, double *mean, double *rstd,
                      int64_t rows, int64_t inner) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    const float *xr = x + r * inner;
    double s = 0.0;
    for (int64_t i = 0; i < inner; ++i)
      s += (double)xr[i];
    const double mu = s / (double)inner;
    double ss = 0.0;
    for (int64_t i = 0; i < inner; ++i) {
      const double d = (double)xr[i] - mu;
      ss += d * d;
    }
    const double inv = 1.0 / sqrt(ss / (double)inner + eps);
    if (mean)
      mean[r] = mu;
    if (rstd)
      rstd[r] = inv;
    for (int64_t i = 0; i < inner; ++i)
      y[r * inner + i] = ((double)xr[i] - mu) * inv *
                             (scale ? (double)scale[i] : 1.0) +
                         (bias ? (double)bias[i] : 0.0);
  }
}
