// Shared host/device helpers of the gfx950 backend: context, error reporting,
// element-type load/store, pointwise math and the fused-epilogue evaluator.
#ifndef FUSILLI_AMD_CSRC_COMMON_H
#define FUSILLI_AMD_CSRC_COMMON_H

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <atomic>
#include <string>

#include "../../include/fusilli_hip.h"

// ---------------------------------------------------------------------------
// Context
// ---------------------------------------------------------------------------
struct fhip_ctx {
  int device = 0;
  hipStream_t stream = nullptr;
  bool owns_stream = false;
  int num_cus = 0;
  // this device's copy of the data gradient's static scratch array
  void *dgrad_static_scratch = nullptr;
  // device memory for kernels' partial results, owned by the context (one
  // stream: its users are ordered); grown on demand, freed with the context
  void *scratch = nullptr;
  size_t scratch_bytes = 0;
  std::string err;
  // name and shape parameters of the kernel variant that the last operator
  // call on this context chose (fhip_last_kernel)
  char last_kernel[96] = {0};
};
// Records the variant the running call has chosen; a call that launches
// helpers around one main kernel names the main kernel.
inline void fhip_note_kernel(fhip_ctx *ctx, const char *fmt, ...) {
  if (!ctx)
    return;
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(ctx->last_kernel, sizeof(ctx->last_kernel), fmt, ap);
  va_end(ap);
}
// At least `bytes` of 256-byte aligned scratch in *out.  Growing it allocates
// (after the stream has drained): not for callers under graph capture.
int fhip_ctx_scratch(fhip_ctx *ctx, size_t bytes, void **out);

// Tuning / test knobs from the environment, parsed once per process (and again
// on fhip_tuning_reload) instead of on every launch.
struct FhipKnobs {
  bool has_rownorm_wgs = false;
  int rownorm_wgs_per_cu = 0;       // FUSILLI_HIP_ROWNORM_WGS_PER_CU
  int pointwise_wgs_per_cu = 0;     // FUSILLI_HIP_POINTWISE_WGS_PER_CU (0: built-in)
  int rownorm_shape_w = 0, rownorm_shape_c = 0; // FUSILLI_HIP_ROWNORM_SHAPE "w,c"
  bool rownorm_general = false;     // FUSILLI_HIP_ROWNORM_GENERAL
  int conv_tile_bm = 0, conv_tile_bn = 0; // FUSILLI_HIP_CONV_TILE "bm,bn"
  int conv_halo = -1;               // FUSILLI_HIP_CONV_HALO (-1: unset)
  int conv_bn = 0;                  // FUSILLI_HIP_CONV_BN
  int conv_rows = -1;               // FUSILLI_HIP_CONV_ROWS (-1: unset)
  int gemm_tile_bm = 0, gemm_tile_bn = 0; // FUSILLI_HIP_GEMM_TILE "bm,bn"
  bool conv_depthwise_strips = true; // FUSILLI_HIP_CONV_DEPTHWISE_STRIPS=0: the general small-group kernel
  int gemm_split = 0;               // FUSILLI_HIP_GEMM_SPLIT (parts of a split reduction; 0: planner, 1: none)
  int conv_slices = 0;              // FUSILLI_HIP_CONV_SLICES (channel slices per workgroup of the register-filter kernel: 2 or 4; 0: planner)
  int wgrad_direct = -1;            // FUSILLI_HIP_WGRAD_DIRECT (-1: unset, 0: off)
  int dgrad_rf = -1;                // FUSILLI_HIP_DGRAD_ROWS (-1: unset, 0: off, n: rows per
                                    // tile, + 100 x column tiles per row of tiles)
};
const FhipKnobs &fhip_knobs();

// "Done once per device" flag for per-kernel set-up such as
// hipFuncSetAttribute: one bit per device ordinal, safe to test and set from
// several threads (the set-up itself is idempotent).
struct FhipOncePerDevice {
  std::atomic<uint64_t> bits{0};
  bool done(int device) const {
    return (bits.load(std::memory_order_acquire) >> (device & 63)) & 1;
  }
  void mark(int device) {
    bits.fetch_or(1ull << (device & 63), std::memory_order_release);
  }
};

struct fhip_event {
  hipEvent_t ev;
};

std::string &fhip_tls_error();
int fhip_fail(fhip_ctx *ctx, const char *fmt, ...);

#define FHIP_HIP_CHECK(ctx, expr)                                              \
  do {                                                                         \
    hipError_t e_ = (expr);                                                    \
    if (e_ != hipSuccess)                                                      \
      return fhip_fail((ctx), "%s failed: %s (%s:%d)", #expr,                  \
                       hipGetErrorString(e_), __FILE__, __LINE__);             \
  } while (0)

#define FHIP_REQUIRE(ctx, cond, ...)                                           \
  do {                                                                         \
    if (!(cond))                                                               \
      return fhip_fail((ctx), __VA_ARGS__);                                    \
  } while (0)

// ---------------------------------------------------------------------------
// Element types
// ---------------------------------------------------------------------------
__host__ __device__ inline int fhip_dtype_size(int dt) {
  switch (dt) {
  case FHIP_HALF:
  case FHIP_BFLOAT16:
  case FHIP_INT16:
    return 2;
  case FHIP_FLOAT:
  case FHIP_INT32:
    return 4;
  case FHIP_DOUBLE:
  case FHIP_INT64:
    return 8;
  case FHIP_UINT8:
  case FHIP_INT8:
  case FHIP_BOOLEAN:
  case FHIP_FP8E5M2:
  case FHIP_FP8E4M3:
    return 1;
  default:
    return 0;
  }
}

__host__ __device__ inline bool fhip_dtype_is_float(int dt) {
  return dt == FHIP_HALF || dt == FHIP_BFLOAT16 || dt == FHIP_FLOAT ||
         dt == FHIP_DOUBLE || dt == FHIP_FP8E5M2 || dt == FHIP_FP8E4M3;
}

__host__ __device__ inline bool fhip_dtype_is_int(int dt) {
  return dt == FHIP_UINT8 || dt == FHIP_INT8 || dt == FHIP_INT16 ||
         dt == FHIP_INT32 || dt == FHIP_INT64 || dt == FHIP_BOOLEAN;
}

// Software fp8 conversions (OCP e4m3fn: bias 7, no inf, max 448; e5m2: bias 15,
// IEEE-like).  Round to nearest even; finite overflow saturates to the largest
// finite value (matches the v_cvt_pk_fp8_f32 saturating mode used on gfx950).
__host__ __device__ inline float fhip_fp8_to_float(uint8_t v, int ebits) {
  const int mbits = 7 - ebits;
  const int bias = (1 << (ebits - 1)) - 1;
  const uint32_t sign = (v >> 7) & 1u;
  const uint32_t e = (v >> mbits) & ((1u << ebits) - 1u);
  const uint32_t m = v & ((1u << mbits) - 1u);
  float r;
  if (ebits == 4) {
    if (e == 15 && m == 7) {
      uint32_t nanbits = 0x7fc00000u | (sign << 31);
      float f;
      memcpy(&f, &nanbits, 4);
      return f;
    }
  } else {
    if (e == 31) {
      uint32_t bits = (sign << 31) | (m ? 0x7fc00000u : 0x7f800000u);
      float f;
      memcpy(&f, &bits, 4);
      return f;
    }
  }
  if (e == 0) {
    r = (float)m * (1.0f / (float)(1 << mbits));
    // 2^(1-bias)
    float sc = 1.0f;
    for (int i = 0; i < bias - 1; ++i)
      sc *= 0.5f;
    r *= sc;
  } else {
    uint32_t bits = ((e - bias + 127) << 23) | (m << (23 - mbits));
    memcpy(&r, &bits, 4);
  }
  return sign ? -r : r;
}

__host__ __device__ inline uint8_t fhip_float_to_fp8(float f, int ebits) {
  const int mbits = 7 - ebits;
  const int bias = (1 << (ebits - 1)) - 1;
  uint32_t bits;
  memcpy(&bits, &f, 4);
  const uint8_t sign = (uint8_t)((bits >> 24) & 0x80u);
  const uint32_t absbits = bits & 0x7fffffffu;
  const uint8_t maxfinite = (ebits == 4) ? 0x7e : 0x7b;
  if (absbits > 0x7f800000u) // NaN
    return (uint8_t)(sign | ((ebits == 4) ? 0x7f : 0x7e));
  if (absbits == 0x7f800000u)
    return (uint8_t)(sign | ((ebits == 4) ? maxfinite : 0x7c));
  int e = (int)(absbits >> 23) - 127;
  uint32_t man = (absbits & 0x7fffffu) | 0x800000u; // 24-bit significand
  if (absbits < 0x00800000u)
    return sign; // f32 denormals are far below fp8 range
  const int emin = 1 - bias;
  int shift = 23 - mbits; // bits dropped for a normal result
  if (e < emin)
    shift += emin - e;
  if (shift > 25)
    return sign;
  uint32_t q = man >> shift;
  const uint32_t rem = man & ((1u << shift) - 1u);
  const uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1u)))
    q += 1;
  // q holds significand (with hidden bit when normal) in units of 2^-mbits.
  uint32_t outv;
  if (e < emin) {
    outv = q; // subnormal (q may carry into exponent 1 when == 1<<mbits)
  } else {
    if (q >= (2u << mbits)) {
      q >>= 1;
      e += 1;
    }
    outv = ((uint32_t)(e + bias) << mbits) | (q & ((1u << mbits) - 1u));
  }
  if (outv > maxfinite)
    outv = maxfinite;
  return (uint8_t)(sign | outv);
}

#if defined(__HIPCC__)

// Load element `idx` of a tensor of runtime dtype as CT (float or double).
template <typename CT>
__device__ __forceinline__ CT fhip_load(const void *p, int dt, int64_t idx) {
  switch (dt) {
  case FHIP_HALF:
    return (CT)(float)((const _Float16 *)p)[idx];
  case FHIP_BFLOAT16:
    return (CT)(float)((const __bf16 *)p)[idx];
  case FHIP_FLOAT:
    return (CT)((const float *)p)[idx];
  case FHIP_DOUBLE:
    return (CT)((const double *)p)[idx];
  case FHIP_UINT8:
    return (CT)((const uint8_t *)p)[idx];
  case FHIP_BOOLEAN:
    return (CT)(((const uint8_t *)p)[idx] != 0);
  case FHIP_INT8:
    return (CT)((const int8_t *)p)[idx];
  case FHIP_INT16:
    return (CT)((const int16_t *)p)[idx];
  case FHIP_INT32:
    return (CT)((const int32_t *)p)[idx];
  case FHIP_INT64:
    return (CT)((const int64_t *)p)[idx];
  case FHIP_FP8E5M2:
    return (CT)fhip_fp8_to_float(((const uint8_t *)p)[idx], 5);
  case FHIP_FP8E4M3:
    return (CT)fhip_fp8_to_float(((const uint8_t *)p)[idx], 4);
  default:
    return (CT)0;
  }
}

template <typename CT>
__device__ __forceinline__ void fhip_store(void *p, int dt, int64_t idx, CT v) {
  switch (dt) {
  case FHIP_HALF:
    ((_Float16 *)p)[idx] = (_Float16)(float)v;
    break;
  case FHIP_BFLOAT16:
    ((__bf16 *)p)[idx] = (__bf16)(float)v;
    break;
  case FHIP_FLOAT:
    ((float *)p)[idx] = (float)v;
    break;
  case FHIP_DOUBLE:
    ((double *)p)[idx] = (double)v;
    break;
  case FHIP_UINT8:
    ((uint8_t *)p)[idx] = (uint8_t)(int64_t)v;
    break;
  case FHIP_BOOLEAN:
    ((uint8_t *)p)[idx] = (v != (CT)0) ? 1 : 0;
    break;
  case FHIP_INT8:
    ((int8_t *)p)[idx] = (int8_t)(int64_t)v;
    break;
  case FHIP_INT16:
    ((int16_t *)p)[idx] = (int16_t)(int64_t)v;
    break;
  case FHIP_INT32:
    ((int32_t *)p)[idx] = (int32_t)(int64_t)v;
    break;
  case FHIP_INT64:
    ((int64_t *)p)[idx] = (int64_t)v;
    break;
  case FHIP_FP8E5M2:
    ((uint8_t *)p)[idx] = fhip_float_to_fp8((float)v, 5);
    break;
  case FHIP_FP8E4M3:
    ((uint8_t *)p)[idx] = fhip_float_to_fp8((float)v, 4);
    break;
  default:
    break;
  }
}

// Round a compute-type value through a storage dtype (the rounding point of a
// virtual tensor between fused nodes).
template <typename CT>
__device__ __forceinline__ CT fhip_round_through(int dt, CT v) {
  switch (dt) {
  case FHIP_HALF:
    return (CT)(float)(_Float16)(float)v;
  case FHIP_BFLOAT16:
    return (CT)(float)(__bf16)(float)v;
  case FHIP_FLOAT:
    return (CT)(float)v;
  case FHIP_FP8E5M2:
    return (CT)fhip_fp8_to_float(fhip_float_to_fp8((float)v, 5), 5);
  case FHIP_FP8E4M3:
    return (CT)fhip_fp8_to_float(fhip_float_to_fp8((float)v, 4), 4);
  case FHIP_UINT8:
    return (CT)(uint8_t)(int64_t)v;
  case FHIP_INT8:
    return (CT)(int8_t)(int64_t)v;
  case FHIP_INT16:
    return (CT)(int16_t)(int64_t)v;
  case FHIP_INT32:
    return (CT)(int32_t)(int64_t)v;
  case FHIP_INT64:
    return (CT)(int64_t)v;
  case FHIP_BOOLEAN:
    return (CT)(v != (CT)0);
  default:
    return v;
  }
}

// ---------------------------------------------------------------------------
// Pointwise math (reference semantics: support/asm_emitter.h:1806-2122)
// ---------------------------------------------------------------------------
template <typename CT> __device__ __forceinline__ CT fhip_sigmoid(CT x) {
  return (CT)1 / ((CT)1 + exp(-x));
}

template <typename CT>
__device__ __forceinline__ CT fhip_pw_unary(int mode, CT x,
                                            const fhip_pointwise_params &p) {
  switch (mode) {
  case FHIP_PW_ABS:
    return fabs(x);
  case FHIP_PW_CEIL:
    return ceil(x);
  case FHIP_PW_FLOOR:
    return floor(x);
  case FHIP_PW_ELU_FWD:
    return x > (CT)0 ? x : (CT)p.elu_alpha * (exp(x) - (CT)1);
  case FHIP_PW_ERF:
    return erf(x);
  case FHIP_PW_EXP:
    return exp(x);
  case FHIP_PW_GELU_FWD:
    return (CT)0.5 * x * ((CT)1 + erf(x * (CT)0.70710678118654752440));
  case FHIP_PW_GELU_APPROX_TANH_FWD: {
    const CT k = (CT)0.79788456080286535588; // sqrt(2/pi)
    return (CT)0.5 * x *
           ((CT)1 + tanh(k * (x + (CT)0.044715 * x * x * x)));
  }
  case FHIP_PW_IDENTITY:
    return x;
  case FHIP_PW_LOG:
    return log(x);
  case FHIP_PW_LOGICAL_NOT:
    return (CT)(x == (CT)0);
  case FHIP_PW_NEG:
    return -x;
  case FHIP_PW_RECIPROCAL:
    return (CT)1 / x;
  case FHIP_PW_RELU_FWD:
    return x > (CT)0 ? x : (x != x ? x : (CT)0);
  case FHIP_PW_RSQRT:
    return (CT)1 / sqrt(x);
  case FHIP_PW_SIGMOID_FWD:
    return fhip_sigmoid(x);
  case FHIP_PW_SIN:
    return sin(x);
  case FHIP_PW_SOFTPLUS_FWD: {
    const CT bx = x * (CT)p.softplus_beta;
    return bx > (CT)p.softplus_threshold
               ? x
               : log1p(exp(bx)) / (CT)p.softplus_beta;
  }
  case FHIP_PW_SQRT:
    return sqrt(x);
  case FHIP_PW_SWISH_FWD:
    return x * fhip_sigmoid(x * (CT)p.swish_beta);
  case FHIP_PW_TAN:
    return tan(x);
  case FHIP_PW_TANH_FWD:
    return tanh(x);
  default:
    return x;
  }
}

template <typename CT>
__device__ __forceinline__ CT fhip_pw_binary(int mode, CT a, CT b,
                                             const fhip_pointwise_params &p) {
  switch (mode) {
  case FHIP_PW_ADD:
    return a + b;
  case FHIP_PW_ADD_SQUARE:
    return a + b * b;
  case FHIP_PW_SUB:
    return a - b;
  case FHIP_PW_MUL:
    return a * b;
  case FHIP_PW_DIV:
    return a / b;
  case FHIP_PW_MAX_OP:
    return (a != a || b != b) ? (a != a ? a : b) : (a > b ? a : b);
  case FHIP_PW_MIN_OP:
    return (a != a || b != b) ? (a != a ? a : b) : (a < b ? a : b);
  case FHIP_PW_CMP_EQ:
    return (CT)(a == b);
  case FHIP_PW_CMP_NEQ:
    return (CT)(a != b);
  case FHIP_PW_CMP_LT:
    return (CT)(a < b);
  case FHIP_PW_CMP_LE:
    return (CT)(a <= b);
  case FHIP_PW_CMP_GT:
    return (CT)(a > b);
  case FHIP_PW_CMP_GE:
    return (CT)(a >= b);
  case FHIP_PW_LOGICAL_AND:
    return (CT)((a != (CT)0) && (b != (CT)0));
  case FHIP_PW_LOGICAL_OR:
    return (CT)((a != (CT)0) || (b != (CT)0));
  // Backward modes: IN_0 = incoming gradient, IN_1 = forward input.
  case FHIP_PW_RELU_BWD:
    return b > (CT)0 ? a : (CT)0;
  case FHIP_PW_TANH_BWD: {
    const CT y = tanh(b);
    return a * ((CT)1 - y * y);
  }
  case FHIP_PW_GELU_BWD: {
    const CT cdf = (CT)0.5 * ((CT)1 + erf(b * (CT)0.70710678118654752440));
    const CT pdf =
        (CT)0.39894228040143267794 * exp((CT)-0.5 * b * b); // 1/sqrt(2pi)
    return a * (cdf + b * pdf);
  }
  case FHIP_PW_GELU_APPROX_TANH_BWD: {
    const CT k = (CT)0.79788456080286535588;
    const CT c = (CT)0.044715;
    const CT inner = k * (b + c * b * b * b);
    const CT t = tanh(inner);
    const CT dinner = k * ((CT)1 + (CT)3 * c * b * b);
    return a * ((CT)0.5 * ((CT)1 + t) +
                (CT)0.5 * b * ((CT)1 - t * t) * dinner);
  }
  case FHIP_PW_SWISH_BWD: {
    const CT bx = b * (CT)p.swish_beta;
    const CT s = fhip_sigmoid(bx);
    return a * (s + bx * s * ((CT)1 - s));
  }
  default:
    return a;
  }
}

// Modes the tuned kernels evaluate inline in their epilogues (cheap, and
// branch-uniform across the wavefront).  Chains with any other mode run on the
// generic kernels.
__host__ __device__ inline bool fhip_pw_is_fast(int mode) {
  switch (mode) {
  case FHIP_PW_ADD:
  case FHIP_PW_SUB:
  case FHIP_PW_MUL:
  case FHIP_PW_DIV:
  case FHIP_PW_MAX_OP:
  case FHIP_PW_MIN_OP:
  case FHIP_PW_RELU_FWD:
  case FHIP_PW_IDENTITY:
  case FHIP_PW_NEG:
  case FHIP_PW_ABS:
  case FHIP_PW_SIGMOID_FWD:
  case FHIP_PW_SWISH_FWD:
  case FHIP_PW_TANH_FWD:
  case FHIP_PW_GELU_FWD:
  case FHIP_PW_GELU_APPROX_TANH_FWD:
    return true;
  default:
    return false;
  }
}

#if defined(__HIPCC__)
// TRANSCENDENTAL = false drops tanh / erf based modes (callers must then keep
// such chains off the kernel).
template <bool TRANSCENDENTAL = true>
__device__ __forceinline__ float fhip_pw_fast_unary(int mode, float x,
                                                    float swish_beta) {
  if constexpr (TRANSCENDENTAL) {
    switch (mode) {
    case FHIP_PW_TANH_FWD:
      return tanhf(x);
    case FHIP_PW_GELU_FWD:
      return 0.5f * x * (1.f + erff(x * 0.70710678118654752440f));
    case FHIP_PW_GELU_APPROX_TANH_FWD:
      return 0.5f * x *
             (1.f + tanhf(0.79788456080286535588f *
                          (x + 0.044715f * x * x * x)));
    default:
      break;
    }
  }
  switch (mode) {
  case FHIP_PW_RELU_FWD:
    return x > 0.f ? x : (x != x ? x : 0.f);
  case FHIP_PW_NEG:
    return -x;
  case FHIP_PW_ABS:
    return fabsf(x);
  case FHIP_PW_SIGMOID_FWD:
    return 1.f / (1.f + expf(-x));
  case FHIP_PW_SWISH_FWD:
    return x / (1.f + expf(-x * swish_beta));
  default:
    return x;
  }
}

// Vector forms: one uniform branch per call, straight-line code per case.
// (Per-element mode dispatch costs a scalar branch per element and dominates
// bandwidth-bound kernels.)
template <bool TRANSCENDENTAL, int N>
__device__ __forceinline__ void fhip_pw_fast_unary_vec(int mode, float (&y)[N],
                                                       float swish_beta) {
#define FHIP_VEC_CASE(MODE)                                                    \
  case MODE:                                                                   \
    _Pragma("unroll") for (int i = 0; i < N; ++i) y[i] =                       \
        fhip_pw_fast_unary<TRANSCENDENTAL>(MODE, y[i], swish_beta);            \
    break;
  switch (mode) {
    FHIP_VEC_CASE(FHIP_PW_RELU_FWD)
    FHIP_VEC_CASE(FHIP_PW_NEG)
    FHIP_VEC_CASE(FHIP_PW_ABS)
    FHIP_VEC_CASE(FHIP_PW_SIGMOID_FWD)
    FHIP_VEC_CASE(FHIP_PW_SWISH_FWD)
  default:
    if constexpr (TRANSCENDENTAL) {
      switch (mode) {
        FHIP_VEC_CASE(FHIP_PW_TANH_FWD)
        FHIP_VEC_CASE(FHIP_PW_GELU_FWD)
        FHIP_VEC_CASE(FHIP_PW_GELU_APPROX_TANH_FWD)
      default:
        break;
      }
    }
    break;
  }
#undef FHIP_VEC_CASE
}

template <int N>
__device__ __forceinline__ void
fhip_pw_fast_binary_vec(int mode, bool acc_is_in1, float (&y)[N],
                        const float (&o)[N]) {
#define FHIP_VEC_CASE(MODE)                                                    \
  case MODE:                                                                   \
    if (acc_is_in1) {                                                          \
      _Pragma("unroll") for (int i = 0; i < N; ++i) y[i] =                     \
          fhip_pw_fast_binary(MODE, o[i], y[i]);                               \
    } else {                                                                   \
      _Pragma("unroll") for (int i = 0; i < N; ++i) y[i] =                     \
          fhip_pw_fast_binary(MODE, y[i], o[i]);                               \
    }                                                                          \
    break;
  switch (mode) {
    FHIP_VEC_CASE(FHIP_PW_ADD)
    FHIP_VEC_CASE(FHIP_PW_SUB)
    FHIP_VEC_CASE(FHIP_PW_MUL)
    FHIP_VEC_CASE(FHIP_PW_DIV)
    FHIP_VEC_CASE(FHIP_PW_MAX_OP)
    FHIP_VEC_CASE(FHIP_PW_MIN_OP)
  default:
    break;
  }
#undef FHIP_VEC_CASE
}

template <int N>
__device__ __forceinline__ void fhip_round_fast_vec(int dt, float (&y)[N]) {
  if (dt == FHIP_BFLOAT16) {
#pragma unroll
    for (int i = 0; i < N; ++i)
      y[i] = (float)(__bf16)y[i];
  } else if (dt == FHIP_HALF) {
#pragma unroll
    for (int i = 0; i < N; ++i)
      y[i] = (float)(_Float16)y[i];
  }
}

__host__ __device__ inline bool fhip_pw_is_transcendental(int mode) {
  return mode == FHIP_PW_TANH_FWD || mode == FHIP_PW_GELU_FWD ||
         mode == FHIP_PW_GELU_APPROX_TANH_FWD;
}

// Rounding through f16 / bf16 / f32 only (the intermediate types tuned kernels
// accept).
__device__ __forceinline__ float fhip_round_fast(int dt, float v) {
  if (dt == FHIP_BFLOAT16)
    return (float)(__bf16)v;
  if (dt == FHIP_HALF)
    return (float)(_Float16)v;
  return v;
}

__device__ __forceinline__ float fhip_pw_fast_binary(int mode, float a,
                                                     float b) {
  switch (mode) {
  case FHIP_PW_ADD:
    return a + b;
  case FHIP_PW_SUB:
    return a - b;
  case FHIP_PW_MUL:
    return a * b;
  case FHIP_PW_DIV:
    return a / b;
  case FHIP_PW_MAX_OP:
    return (a != a || b != b) ? (a != a ? a : b) : (a > b ? a : b);
  case FHIP_PW_MIN_OP:
    return (a != a || b != b) ? (a != a ? a : b) : (a < b ? a : b);
  default:
    return a;
  }
}
#endif

__host__ __device__ inline int fhip_pw_arity(int mode) {
  switch (mode) {
  case FHIP_PW_BINARY_SELECT:
    return 3;
  case FHIP_PW_ADD:
  case FHIP_PW_ADD_SQUARE:
  case FHIP_PW_CMP_EQ:
  case FHIP_PW_CMP_GE:
  case FHIP_PW_CMP_GT:
  case FHIP_PW_CMP_LE:
  case FHIP_PW_CMP_LT:
  case FHIP_PW_CMP_NEQ:
  case FHIP_PW_DIV:
  case FHIP_PW_GELU_APPROX_TANH_BWD:
  case FHIP_PW_GELU_BWD:
  case FHIP_PW_LOGICAL_AND:
  case FHIP_PW_LOGICAL_OR:
  case FHIP_PW_MAX_OP:
  case FHIP_PW_MIN_OP:
  case FHIP_PW_MUL:
  case FHIP_PW_RELU_BWD:
  case FHIP_PW_SUB:
  case FHIP_PW_SWISH_BWD:
  case FHIP_PW_TANH_BWD:
    return 2;
  default:
    return 1;
  }
}

// ---------------------------------------------------------------------------
// Fused epilogue, device form.  Strides are expressed on the producer's
// logical output coordinates (stride 0 where the operand broadcasts).
// ---------------------------------------------------------------------------
struct DevEpiOp {
  int32_t mode;
  int32_t kind; // FHIP_OPERAND_*
  int32_t acc_is_in1;
  int32_t result_dtype;
  int32_t operand_dtype;
  float scalar;
  fhip_pointwise_params params;
  const void *ptr;
  int64_t stride[FHIP_MAX_RANK];
};

struct DevEpilogue {
  int32_t count;
  int32_t rank; // rank of the coordinate vector the strides refer to
  DevEpiOp op[FHIP_MAX_EPILOGUE];
};

template <typename CT>
__device__ __forceinline__ CT fhip_apply_epilogue(const DevEpilogue &e, CT v,
                                                  const int64_t *coord) {
  for (int i = 0; i < e.count; ++i) {
    const DevEpiOp &o = e.op[i];
    if (o.kind == FHIP_OPERAND_NONE) {
      v = fhip_pw_unary<CT>(o.mode, v, o.params);
    } else {
      CT other;
      if (o.kind == FHIP_OPERAND_SCALAR) {
        other = (CT)o.scalar;
      } else {
        int64_t off = 0;
        for (int r = 0; r < e.rank; ++r)
          off += coord[r] * o.stride[r];
        other = fhip_load<CT>(o.ptr, o.operand_dtype, off);
      }
      v = o.acc_is_in1 ? fhip_pw_binary<CT>(o.mode, other, v, o.params)
                       : fhip_pw_binary<CT>(o.mode, v, other, o.params);
    }
    v = fhip_round_through<CT>(o.result_dtype, v);
  }
  return v;
}

// The helpers below handle several values of a thread.  Their rare cases (an
// element type or mode outside the common ones) run the per-value helper --
// a switch over every type / mode -- in a loop that is NOT unrolled: inlined
// once per value those switches are most of a kernel's code (the 64 x 64-tile
// f32 matmul kernel was 267 KB, refetched by every compute unit a small grid
// lands on), and an out-of-line call would cost every kernel that contains
// one its register budget.
// N values to a tensor of runtime dtype (element n at idx[n] when bit n of
// `live` is set): one switch for all.
template <typename CT, int N>
__device__ __forceinline__ void fhip_store_many(void *p, int dt, const int64_t (&idx)[N],
                                                const CT (&v)[N], uint32_t live) {
  switch (dt) {
  case FHIP_FLOAT:
#pragma unroll
    for (int n = 0; n < N; ++n)
      if ((live >> n) & 1)
        ((float *)p)[idx[n]] = (float)v[n];
    break;
  case FHIP_BFLOAT16:
#pragma unroll
    for (int n = 0; n < N; ++n)
      if ((live >> n) & 1)
        ((__bf16 *)p)[idx[n]] = (__bf16)(float)v[n];
    break;
  case FHIP_HALF:
#pragma unroll
    for (int n = 0; n < N; ++n)
      if ((live >> n) & 1)
        ((_Float16 *)p)[idx[n]] = (_Float16)(float)v[n];
    break;
  default:
#pragma clang loop unroll(disable)
    for (int n = 0; n < N; ++n)
      if ((live >> n) & 1)
        fhip_store<CT>(p, dt, idx[n], v[n]);
  }
}

// N elements of a tensor of runtime dtype at once: one switch for all, so the
// loads are issued back to back (N calls of fhip_load each wait for their
// value before the next address is even formed).
template <typename CT, int N>
__device__ __forceinline__ void fhip_load_many(const void *p, int dt, const int64_t (&idx)[N],
                                               CT (&out)[N]) {
  switch (dt) {
  case FHIP_FLOAT:
#pragma unroll
    for (int n = 0; n < N; ++n)
      out[n] = (CT)((const float *)p)[idx[n]];
    break;
  case FHIP_BFLOAT16:
#pragma unroll
    for (int n = 0; n < N; ++n)
      out[n] = (CT)(float)((const __bf16 *)p)[idx[n]];
    break;
  case FHIP_HALF:
#pragma unroll
    for (int n = 0; n < N; ++n)
      out[n] = (CT)(float)((const _Float16 *)p)[idx[n]];
    break;
  default:
#pragma clang loop unroll(disable)
    for (int n = 0; n < N; ++n)
      out[n] = fhip_load<CT>(p, dt, idx[n]);
  }
}

// The chain on N values whose coordinates differ in one dim only (`var_dim`,
// where value n sits at vals[n]; coord[var_dim] is ignored).  Same results as N
// calls of fhip_apply_epilogue; an operand's N values are fetched together.
// Callers pass a valid coordinate also for values they will not store.
template <typename CT, int N>
__device__ __forceinline__ void fhip_apply_epilogue_many(const DevEpilogue &e, CT (&v)[N],
                                                         const int64_t *coord, int var_dim,
                                                         const int64_t (&vals)[N]) {
  for (int i = 0; i < e.count; ++i) {
    const DevEpiOp &o = e.op[i];
    // (f32 chains of the common modes: the mode is chosen once for the N
    // values, not per value -- a switch over every mode, inlined N times, is
    // most of such a kernel's code)
    constexpr bool kF32 = std::is_same<CT, float>::value;
    const bool fast = kF32 && fhip_pw_is_fast(o.mode);
    if (o.kind == FHIP_OPERAND_NONE) {
      if constexpr (kF32) {
        if (fast) {
          fhip_pw_fast_unary_vec<true, N>(o.mode, v, o.params.swish_beta);
        } else {
#pragma clang loop unroll(disable)
          for (int n = 0; n < N; ++n)
            v[n] = fhip_pw_unary<CT>(o.mode, v[n], o.params);
        }
      } else {
#pragma clang loop unroll(disable)
        for (int n = 0; n < N; ++n)
          v[n] = fhip_pw_unary<CT>(o.mode, v[n], o.params);
      }
    } else {
      CT other[N];
      if (o.kind == FHIP_OPERAND_SCALAR) {
#pragma unroll
        for (int n = 0; n < N; ++n)
          other[n] = (CT)o.scalar;
      } else {
        int64_t base = 0;
        for (int r = 0; r < e.rank; ++r)
          base += r == var_dim ? 0 : coord[r] * o.stride[r];
        int64_t off[N];
#pragma unroll
        for (int n = 0; n < N; ++n)
          off[n] = base + vals[n] * o.stride[var_dim];
        fhip_load_many<CT, N>(o.ptr, o.operand_dtype, off, other);
      }
      bool done = false;
      if constexpr (kF32) {
        if (fast) {
          fhip_pw_fast_binary_vec<N>(o.mode, o.acc_is_in1 != 0, v, other);
          done = true;
        }
      }
      if (!done) {
#pragma clang loop unroll(disable)
        for (int n = 0; n < N; ++n)
          v[n] = o.acc_is_in1 ? fhip_pw_binary<CT>(o.mode, other[n], v[n], o.params)
                              : fhip_pw_binary<CT>(o.mode, v[n], other[n], o.params);
      }
    }
    const int rd = o.result_dtype;
    if (kF32 && (rd == FHIP_FLOAT || rd == FHIP_BFLOAT16 || rd == FHIP_HALF)) {
      if constexpr (kF32)
        fhip_round_fast_vec<N>(rd, v);
    } else {
#pragma clang loop unroll(disable)
      for (int n = 0; n < N; ++n)
        v[n] = fhip_round_through<CT>(rd, v[n]);
    }
  }
}

#endif // __HIPCC__

// ---------------------------------------------------------------------------
// Host-side descriptor helpers
// ---------------------------------------------------------------------------
inline int64_t fhip_desc_volume(const fhip_tensor_desc &t) {
  int64_t v = 1;
  for (int i = 0; i < t.rank; ++i)
    v *= t.dim[i];
  return v;
}

// True when strides describe the dense row-major layout of dims (unit dims may
// carry any stride).
inline bool fhip_desc_is_contiguous(const fhip_tensor_desc &t) {
  int64_t expect = 1;
  for (int i = t.rank - 1; i >= 0; --i) {
    if (t.dim[i] != 1 && t.stride[i] != expect)
      return false;
    expect *= t.dim[i];
  }
  return true;
}

bool fhip_check_desc(fhip_ctx *ctx, const fhip_tensor_desc &t,
                     const char *what);
// True when every step of the chain is one the tuned kernels evaluate inline
// and every rounding point is f16 / bf16 / f32.
inline bool fhip_epilogue_is_fast(const fhip_epilogue &e) {
  for (int i = 0; i < e.count; ++i) {
    const int rd = e.op[i].result_dtype;
    if (!fhip_pw_is_fast(e.op[i].mode) ||
        !(rd == FHIP_FLOAT || rd == FHIP_BFLOAT16 || rd == FHIP_HALF))
      return false;
  }
  return true;
}
// Right-aligned broadcast of `operand` against an output of out_rank/out_dims;
// writes per-output-dim strides (0 where broadcast).  Returns false when the
// shapes are not broadcast-compatible.
bool fhip_broadcast_strides(const fhip_tensor_desc &operand, int out_rank,
                            const int64_t *out_dims, int64_t *strides);
#if defined(__HIPCC__)
// Builds the device epilogue for a producer whose logical output is
// (out_rank, out_dims).  Returns non-zero (and sets the error) when invalid.
int fhip_build_epilogue(fhip_ctx *ctx, const fhip_epilogue &e, int out_rank,
                        const int64_t *out_dims,
                        const void *const *operand_ptrs, DevEpilogue *out);
#endif

#endif // FUSILLI_AMD_CSRC_COMMON_H
