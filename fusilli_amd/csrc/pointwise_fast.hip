// Bandwidth-bound standalone pointwise kernel (reference:
// include/fusilli/node/pointwise_node.h:44-169 and the emitted
// linalg.generic of include/fusilli/support/asm_emitter.h:1806-2122).
//
// Covers dense outputs of f32 / bf16 / f16 whose inputs have the same dtype
// and are dense tensors of the same shape, scalars, trailing-dimension vectors
// broadcast over the leading dimensions (bias rows) or leading-dimension
// tensors broadcast over the trailing ones (per-row values).  Every lane moves 8 consecutive elements
// per step with 16-byte accesses and evaluates them with the same per-element
// functions as the strided kernel, so both produce the same bits.  The common
// modes are compiled as kernels of their own.
#include "common.h"
#include "fast_paths.h"

#include <hip/hip_runtime.h>

namespace {

enum { IN_FULL = 0, IN_SCALAR = 1, IN_ROW = 2, IN_COL = 3 };

struct PwFastArgs {
  const void *in[3];
  void *out;
  int64_t nvec;       // 8-element vectors in the output (< 2^31)
  int32_t span[3];    // IN_ROW: vectors of the repeated block;
                      // IN_COL: output vectors per input element
  uint32_t magic[3];  // floor(2^32 / span)
  float scalar[3];
  int32_t kind[3];
  int32_t o_dt;
  int32_t mode;
  int32_t num_inputs;
  int32_t hoist_rows; // IN_ROW operands are the same for every chunk of a
                      // thread: load them once
  fhip_pointwise_params params;
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

// DT: 0 f32, 1 bf16, 2 f16 -- the one dtype of every tensor of the call.
template <int DT> struct PwType;
template <> struct PwType<0> { static constexpr int kBytes = 4; };
template <> struct PwType<1> { static constexpr int kBytes = 2; };
template <> struct PwType<2> { static constexpr int kBytes = 2; };

// 8 elements as loaded: two 16-byte words for f32, one otherwise.
struct Raw {
  u32x4 lo, hi;
};

// n / d for 0 <= n < 2^31 with magic = floor(2^32 / d), d > 1: the estimate
// is at most one too small.
__device__ __forceinline__ int32_t div_magic(int32_t n, int32_t d,
                                             uint32_t magic) {
  int32_t q = (int32_t)__umulhi((uint32_t)n, magic);
  if (n - q * d >= d)
    ++q;
  return d == 1 ? n : q;
}

// Issues the loads of input i for output vector `vec` and nothing else, so
// that the loads of all inputs and unrolled vectors go out back to back.
template <int DT>
__device__ __forceinline__ void fetch_raw(const PwFastArgs &g, int i,
                                          int32_t vec, Raw &raw) {
  constexpr int ES = PwType<DT>::kBytes;
  const int kind = g.kind[i];
  const char *base = (const char *)g.in[i];
  if (kind == IN_FULL || kind == IN_ROW) {
    int32_t rv = vec;
    if (kind == IN_ROW)
      rv = vec - div_magic(vec, g.span[i], g.magic[i]) * g.span[i];
    const char *p = base + (int64_t)rv * (8 * ES);
    // (plain loads: nontemporal ones measured the same)
    raw.lo = *(const u32x4 *)p;
    if constexpr (ES == 4)
      raw.hi = *(const u32x4 *)(p + 16);
  } else if (kind == IN_COL) {
    const char *p =
        base + (int64_t)div_magic(vec, g.span[i], g.magic[i]) * ES;
    if constexpr (ES == 4)
      raw.lo.x = *(const uint32_t *)p;
    else
      raw.lo.x = *(const uint16_t *)p;
  }
}

template <int DT>
__device__ __forceinline__ float widen(uint32_t bits) {
  if constexpr (DT == 0)
    return __builtin_bit_cast(float, bits);
  else if constexpr (DT == 1)
    return __builtin_bit_cast(float, bits << 16);
  else
    return (float)__builtin_bit_cast(_Float16, (uint16_t)bits);
}

template <int DT>
__device__ __forceinline__ void expand(const PwFastArgs &g, int i,
                                       const Raw &raw, float (&v)[8]) {
  const int kind = g.kind[i];
  if (kind == IN_FULL || kind == IN_ROW) {
    const uint32_t w[8] = {raw.lo.x, raw.lo.y, raw.lo.z, raw.lo.w,
                           raw.hi.x, raw.hi.y, raw.hi.z, raw.hi.w};
    if constexpr (DT == 0) {
#pragma unroll
      for (int c = 0; c < 8; ++c)
        v[c] = __builtin_bit_cast(float, w[c]);
    } else {
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        v[2 * c] = widen<DT>(w[c] & 0xffffu);
        v[2 * c + 1] = widen<DT>(w[c] >> 16);
      }
    }
  } else {
    const float s = kind == IN_COL ? widen<DT>(raw.lo.x) : g.scalar[i];
#pragma unroll
    for (int c = 0; c < 8; ++c)
      v[c] = s;
  }
}

// Streaming (nontemporal) stores: the output is not read again by this
// kernel, and keeping it out of the caches' way measurably helps the reads.
template <int DT>
__device__ __forceinline__ void store8(void *out, int32_t vec,
                                       const float (&v)[8]) {
  if constexpr (DT == 0) {
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    f32x4 *p = (f32x4 *)((char *)out + (int64_t)vec * 32);
    __builtin_nontemporal_store(f32x4{v[0], v[1], v[2], v[3]}, p);
    __builtin_nontemporal_store(f32x4{v[4], v[5], v[6], v[7]}, p + 1);
  } else if constexpr (DT == 1) {
    bf16x8 a;
#pragma unroll
    for (int i = 0; i < 8; ++i)
      a[i] = (__bf16)v[i];
    __builtin_nontemporal_store(a, (bf16x8 *)((char *)out + (int64_t)vec * 16));
  } else {
    f16x8 a;
#pragma unroll
    for (int i = 0; i < 8; ++i)
      a[i] = (_Float16)v[i];
    __builtin_nontemporal_store(a, (f16x8 *)((char *)out + (int64_t)vec * 16));
  }
}

#define PW_UNARY_MODES(X)                                                      \
  X(FHIP_PW_ABS) X(FHIP_PW_CEIL) X(FHIP_PW_ELU_FWD) X(FHIP_PW_ERF)             \
  X(FHIP_PW_EXP) X(FHIP_PW_FLOOR) X(FHIP_PW_GELU_APPROX_TANH_FWD)              \
  X(FHIP_PW_GELU_FWD) X(FHIP_PW_IDENTITY) X(FHIP_PW_LOG)                       \
  X(FHIP_PW_LOGICAL_NOT) X(FHIP_PW_NEG) X(FHIP_PW_RECIPROCAL)                  \
  X(FHIP_PW_RELU_FWD) X(FHIP_PW_RSQRT) X(FHIP_PW_SIGMOID_FWD) X(FHIP_PW_SIN)   \
  X(FHIP_PW_SOFTPLUS_FWD) X(FHIP_PW_SQRT) X(FHIP_PW_SWISH_FWD) X(FHIP_PW_TAN)  \
  X(FHIP_PW_TANH_FWD)
#define PW_BINARY_MODES(X)                                                     \
  X(FHIP_PW_ADD) X(FHIP_PW_ADD_SQUARE) X(FHIP_PW_CMP_EQ) X(FHIP_PW_CMP_GE)     \
  X(FHIP_PW_CMP_GT) X(FHIP_PW_CMP_LE) X(FHIP_PW_CMP_LT) X(FHIP_PW_CMP_NEQ)     \
  X(FHIP_PW_DIV) X(FHIP_PW_GELU_APPROX_TANH_BWD) X(FHIP_PW_GELU_BWD)           \
  X(FHIP_PW_LOGICAL_AND) X(FHIP_PW_LOGICAL_OR) X(FHIP_PW_MAX_OP)               \
  X(FHIP_PW_MIN_OP) X(FHIP_PW_MUL) X(FHIP_PW_RELU_BWD) X(FHIP_PW_SUB)          \
  X(FHIP_PW_SWISH_BWD) X(FHIP_PW_TANH_BWD)

// erf-based GELU for 16-bit outputs: erf by Abramowitz & Stegun 7.1.26
// (|error| <= 1.5e-7, far below bf16 / f16 resolution) on the hardware's
// exp2 and reciprocal.  With w = (1 - erf(|x| / sqrt 2)) / 2 = p(t) t e / 2 the
// result is x (1 - w) for x >= 0 and x w below, i.e. max(x, 0) - |x| w: eleven
// multiply-adds and the two transcendentals per element, no cancellation on
// the negative side.
__device__ __forceinline__ float gelu_erf_16bit(float x) {
  const float ax = __builtin_fabsf(x);
  // t = 1 / (1 + 0.3275911 |x| / sqrt 2)
  const float t = __builtin_amdgcn_rcpf(__builtin_fmaf(0.23164189f, ax, 1.f));
  // half of the polynomial's coefficients
  float p = __builtin_fmaf(0.5307027145f, t, -0.7265760135f);
  p = __builtin_fmaf(p, t, 0.7107068705f);
  p = __builtin_fmaf(p, t, -0.142248368f);
  p = __builtin_fmaf(p, t, 0.127414796f);
  // e = exp(-x^2 / 2) = exp2(-(|x| sqrt(log2(e) / 2))^2)
  const float u = ax * 0.84932180028801904272f;
  const float e = __builtin_amdgcn_exp2f(-u * u);
  const float w = p * t * e;
  return __builtin_fmaf(-ax, w, __builtin_fmaxf(x, 0.f));
}

// One lane evaluates 8 elements.  MODE >= 0 fixes the mode at compile time;
// MODE < 0 branches on the runtime mode once per 8 elements, each arm with the
// mode folded in (a per-element switch would dominate the kernel).
template <int NIN, int MODE, int DT>
__device__ __forceinline__ void evaluate(const PwFastArgs &g,
                                         const float (&a)[8],
                                         const float (&b)[8],
                                         const float (&c)[8], float (&r)[8]) {
  if constexpr (NIN == 3) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
      r[i] = a[i] != 0.f ? b[i] : c[i];
  } else if constexpr (MODE == FHIP_PW_GELU_FWD && DT != 0) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
      r[i] = gelu_erf_16bit(a[i]);
  } else if constexpr (MODE >= 0) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
      r[i] = NIN == 1 ? fhip_pw_unary<float>(MODE, a[i], g.params)
                      : fhip_pw_binary<float>(MODE, a[i], b[i], g.params);
  } else if constexpr (NIN == 1) {
#define PW_ARM(M)                                                              \
  case M:                                                                      \
    _Pragma("unroll") for (int i = 0; i < 8; ++i) r[i] =                       \
        fhip_pw_unary<float>(M, a[i], g.params);                               \
    break;
    switch (g.mode) {
      PW_UNARY_MODES(PW_ARM)
    default:
      break;
    }
#undef PW_ARM
  } else {
#define PW_ARM(M)                                                              \
  case M:                                                                      \
    _Pragma("unroll") for (int i = 0; i < 8; ++i) r[i] =                       \
        fhip_pw_binary<float>(M, a[i], b[i], g.params);                        \
    break;
    switch (g.mode) {
      PW_BINARY_MODES(PW_ARM)
    default:
      break;
    }
#undef PW_ARM
  }
}

// A workgroup walks chunks of UNROLL * 256 consecutive vectors; all loads of
// a chunk are issued before the first value is used.  When the distance
// between a workgroup's chunks is a multiple of a broadcast row's length
// (hoist_rows), a thread meets the same row elements in every chunk and keeps
// them in registers.
template <int NIN, int MODE, int DT, int UNROLL>
__global__ __launch_bounds__(256) void pointwise_fast_kernel(PwFastArgs g) {
  const int32_t nvec = (int32_t)g.nvec;
  const int32_t chunks = (nvec + 256 * UNROLL - 1) / (256 * UNROLL);
  const bool hoist = g.hoist_rows != 0;
  Raw rows[UNROLL][NIN];
  if (hoist) {
    const int32_t v0 = (int32_t)blockIdx.x * (256 * UNROLL) + threadIdx.x;
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int32_t v = v0 + u * 256 < nvec ? v0 + u * 256 : nvec - 1;
#pragma unroll
      for (int i = 0; i < NIN; ++i)
        if (g.kind[i] == IN_ROW)
          fetch_raw<DT>(g, i, v, rows[u][i]);
    }
  }
  for (int32_t ch = blockIdx.x; ch < chunks; ch += gridDim.x) {
    const int32_t v0 = ch * (256 * UNROLL) + threadIdx.x;
    Raw raw[UNROLL][NIN];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      // lanes past the end re-read the last vector and store nothing
      const int32_t v = v0 + u * 256 < nvec ? v0 + u * 256 : nvec - 1;
#pragma unroll
      for (int i = 0; i < NIN; ++i) {
        if (hoist && g.kind[i] == IN_ROW)
          raw[u][i] = rows[u][i];
        else
          fetch_raw<DT>(g, i, v, raw[u][i]);
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int32_t v = v0 + u * 256;
      float a[8], b[8], c[8], r[8];
      expand<DT>(g, 0, raw[u][0], a);
      if constexpr (NIN >= 2)
        expand<DT>(g, 1, raw[u][1], b);
      if constexpr (NIN >= 3)
        expand<DT>(g, 2, raw[u][2], c);
      evaluate<NIN, MODE, DT>(g, a, b, c, r);
      if (v < nvec)
        store8<DT>(g.out, v, r);
    }
  }
}

// Two vectors per lane and chunk and up to 32 workgroups per compute unit
// measured best on 8192 x 4096 bf16 (ADD of a bias row 24.7 -> 23.7-24.1 us,
// GELU 25.9 -> 24.6 us against four vectors and 8 workgroups).
constexpr int kUnroll = 2;
constexpr int kWgsPerCu = 32;

int64_t pw_gcd(int64_t a, int64_t b) {
  while (b) {
    const int64_t t = a % b;
    a = b;
    b = t;
  }
  return a;
}

template <int NIN, int MODE, int DT>
void launch_dt(fhip_ctx *ctx, const PwFastArgs &g0) {
  PwFastArgs g = g0;
  // a bounded number of workgroups per compute unit, each walking several
  // chunks of a large tensor
  const int64_t chunk = 256 * kUnroll;
  int64_t blocks = (g.nvec + chunk - 1) / chunk;
  const int knob = fhip_knobs().pointwise_wgs_per_cu;
  const int64_t cap = 256 * (knob > 0 ? knob : kWgsPerCu);
  if (blocks > cap)
    blocks = cap;
  // broadcast rows: a grid that is a multiple of `need` workgroups puts every
  // thread on the same row elements in all of its chunks
  int64_t need = 1;
  bool has_row = false;
  for (int i = 0; i < g.num_inputs; ++i)
    if (g.kind[i] == IN_ROW) {
      has_row = true;
      const int64_t n = g.span[i] / pw_gcd(g.span[i], chunk);
      need = need / pw_gcd(need, n) * n;
    }
  if (has_row && need <= blocks) {
    blocks = blocks / need * need;
    g.hoist_rows = 1;
  }
  hipLaunchKernelGGL((pointwise_fast_kernel<NIN, MODE, DT, kUnroll>),
                     dim3((unsigned)blocks), dim3(256), 0, ctx->stream, g);
}

template <int NIN, int MODE>
void launch_mode(fhip_ctx *ctx, const PwFastArgs &g) {
  if (g.o_dt == FHIP_FLOAT)
    launch_dt<NIN, MODE, 0>(ctx, g);
  else if (g.o_dt == FHIP_BFLOAT16)
    launch_dt<NIN, MODE, 1>(ctx, g);
  else
    launch_dt<NIN, MODE, 2>(ctx, g);
}

bool float_like(int dt) {
  return dt == FHIP_FLOAT || dt == FHIP_BFLOAT16 || dt == FHIP_HALF;
}

// Row-major dense strides of `dims`, or false.
bool dense_row_major(const fhip_tensor_desc &t) {
  int64_t expect = 1;
  for (int i = t.rank - 1; i >= 0; --i) {
    if (t.dim[i] != 1 && t.stride[i] != expect)
      return false;
    expect *= t.dim[i];
  }
  return true;
}

struct PwPlan {
  bool ok = false;
  PwFastArgs g{};
};

PwPlan make_plan(const fhip_pointwise_desc *d) {
  PwPlan p;
  const fhip_tensor_desc &o = d->out;
  if (!float_like(o.dtype) || !dense_row_major(o))
    return p;
  const int64_t total = fhip_desc_volume(o);
  if (total <= 0 || total % 8 != 0 || total / 8 >= (1ll << 31))
    return p;
  int64_t ostride[FHIP_MAX_RANK];
  {
    int64_t s = 1;
    for (int i = o.rank - 1; i >= 0; --i) {
      ostride[i] = s;
      s *= o.dim[i];
    }
  }
  PwFastArgs &g = p.g;
  g.nvec = total / 8;
  g.o_dt = o.dtype;
  g.mode = d->mode;
  g.num_inputs = d->num_inputs;
  g.params = d->params;
  for (int i = 0; i < d->num_inputs; ++i) {
    g.span[i] = 1;
    g.magic[i] = 0;
    if (d->in_is_scalar[i]) {
      g.kind[i] = IN_SCALAR;
      g.scalar[i] = (float)d->in_scalar[i];
      continue;
    }
    if (d->in[i].dtype != o.dtype)
      return p;
    int64_t st[FHIP_MAX_RANK];
    if (!fhip_broadcast_strides(d->in[i], o.rank, o.dim, st))
      return p;
    // split point k: dims [k, rank) against dims [0, k)
    bool matched = false;
    for (int k = 0; k <= o.rank && !matched; ++k) {
      bool lead_zero = true, lead_dense = true, trail_zero = true,
           trail_dense = true;
      int64_t inner = 1;
      for (int j = k; j < o.rank; ++j)
        inner *= o.dim[j];
      for (int j = 0; j < o.rank; ++j) {
        if (o.dim[j] == 1)
          continue;
        if (j < k) {
          lead_zero = lead_zero && st[j] == 0;
          lead_dense = lead_dense && st[j] * inner == ostride[j];
        } else {
          trail_zero = trail_zero && st[j] == 0;
          trail_dense = trail_dense && st[j] == ostride[j];
        }
      }
      if (k == 0 && trail_dense) {
        g.kind[i] = IN_FULL;
        matched = true;
      } else if (k > 0 && k < o.rank && lead_zero && trail_dense &&
                 inner % 8 == 0) {
        g.kind[i] = IN_ROW;
        g.span[i] = (int32_t)(inner / 8);
        g.magic[i] = (uint32_t)((1ull << 32) / (uint32_t)g.span[i]);
        matched = true;
      } else if (k > 0 && k < o.rank && lead_dense && trail_zero &&
                 inner % 8 == 0) {
        g.kind[i] = IN_COL;
        g.span[i] = (int32_t)(inner / 8);
        g.magic[i] = (uint32_t)((1ull << 32) / (uint32_t)g.span[i]);
        matched = true;
      }
    }
    if (!matched)
      return p;
  }
  p.ok = true;
  return p;
}

} // namespace

bool fhip_fast_pointwise_applicable(const fhip_pointwise_desc *d) {
  return make_plan(d).ok;
}

int fhip_fast_pointwise(fhip_ctx *ctx, const fhip_pointwise_desc *d,
                        const void *in0, const void *in1, const void *in2,
                        void *out) {
  PwPlan p = make_plan(d);
  FHIP_REQUIRE(ctx, p.ok, "fhip_fast_pointwise: descriptor not supported");
  PwFastArgs &g = p.g;
  g.in[0] = in0, g.in[1] = in1, g.in[2] = in2;
  g.out = out;
  fhip_note_kernel(ctx, "pointwise_fast inputs=%d mode=%d", (int)d->num_inputs, (int)d->mode);
  // the common modes get kernels of their own
#define PW_CASE(NIN, MODE)                                                     \
  case MODE:                                                                   \
    launch_mode<NIN, MODE>(ctx, g);                                            \
    break;
  if (d->num_inputs == 1) {
    switch (d->mode) {
      PW_CASE(1, FHIP_PW_IDENTITY)
      PW_CASE(1, FHIP_PW_RELU_FWD)
      PW_CASE(1, FHIP_PW_GELU_FWD)
      PW_CASE(1, FHIP_PW_GELU_APPROX_TANH_FWD)
      PW_CASE(1, FHIP_PW_SIGMOID_FWD)
      PW_CASE(1, FHIP_PW_SWISH_FWD)
      PW_CASE(1, FHIP_PW_TANH_FWD)
      PW_CASE(1, FHIP_PW_EXP)
      PW_CASE(1, FHIP_PW_NEG)
    default:
      launch_mode<1, -1>(ctx, g);
      break;
    }
  } else if (d->num_inputs == 2) {
    switch (d->mode) {
      PW_CASE(2, FHIP_PW_ADD)
      PW_CASE(2, FHIP_PW_SUB)
      PW_CASE(2, FHIP_PW_MUL)
      PW_CASE(2, FHIP_PW_DIV)
      PW_CASE(2, FHIP_PW_MAX_OP)
      PW_CASE(2, FHIP_PW_MIN_OP)
    default:
      launch_mode<2, -1>(ctx, g);
      break;
    }
  } else {
    launch_mode<3, -1>(ctx, g);
  }
#undef PW_CASE
  FHIP_HIP_CHECK(ctx, hipGetLastError());
  return 0;
}
