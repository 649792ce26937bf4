// Context, memory, stream and event entry points of the C ABI, plus the
// host-side descriptor helpers shared by the op entry points.
#include "common.h"
#include "fast_paths.h"

#include <mutex>

namespace {
std::mutex g_knob_mu;
FhipKnobs g_knobs;
std::atomic<bool> g_knobs_ready{false};

FhipKnobs parse_knobs() {
  FhipKnobs k;
  if (const char *e = getenv("FUSILLI_HIP_ROWNORM_WGS_PER_CU")) {
    k.has_rownorm_wgs = true;
    k.rownorm_wgs_per_cu = atoi(e);
  }
  if (const char *e = getenv("FUSILLI_HIP_CONV_DEPTHWISE_STRIPS"))
    k.conv_depthwise_strips = atoi(e) != 0;
  if (const char *e = getenv("FUSILLI_HIP_GEMM_SPLIT"))
    k.gemm_split = atoi(e);
  if (const char *e = getenv("FUSILLI_HIP_CONV_SLICES"))
    k.conv_slices = atoi(e);
  if (const char *e = getenv("FUSILLI_HIP_POINTWISE_WGS_PER_CU"))
    k.pointwise_wgs_per_cu = atoi(e);
  if (const char *e = getenv("FUSILLI_HIP_ROWNORM_SHAPE"))
    if (sscanf(e, "%d,%d", &k.rownorm_shape_w, &k.rownorm_shape_c) != 2)
      k.rownorm_shape_w = k.rownorm_shape_c = 0;
  k.rownorm_general = getenv("FUSILLI_HIP_ROWNORM_GENERAL") != nullptr;
  if (const char *e = getenv("FUSILLI_HIP_CONV_TILE"))
    if (sscanf(e, "%d,%d", &k.conv_tile_bm, &k.conv_tile_bn) != 2)
      k.conv_tile_bm = k.conv_tile_bn = 0;
  if (const char *e = getenv("FUSILLI_HIP_CONV_HALO"))
    k.conv_halo = atoi(e);
  if (const char *e = getenv("FUSILLI_HIP_CONV_BN"))
    k.conv_bn = atoi(e);
  if (const char *e = getenv("FUSILLI_HIP_CONV_ROWS"))
    k.conv_rows = atoi(e);
  if (const char *e = getenv("FUSILLI_HIP_WGRAD_DIRECT"))
    k.wgrad_direct = atoi(e);
  if (const char *e = getenv("FUSILLI_HIP_DGRAD_ROWS"))
    k.dgrad_rf = atoi(e);
  if (const char *e = getenv("FUSILLI_HIP_GEMM_TILE"))
    if (sscanf(e, "%d,%d", &k.gemm_tile_bm, &k.gemm_tile_bn) != 2)
      k.gemm_tile_bm = k.gemm_tile_bn = 0;
  return k;
}
} // namespace

const FhipKnobs &fhip_knobs() {
  if (!g_knobs_ready.load(std::memory_order_acquire)) {
    std::lock_guard<std::mutex> lock(g_knob_mu);
    if (!g_knobs_ready.load(std::memory_order_relaxed)) {
      g_knobs = parse_knobs();
      g_knobs_ready.store(true, std::memory_order_release);
    }
  }
  return g_knobs;
}

int fhip_tuning_reload(void) {
  std::lock_guard<std::mutex> lock(g_knob_mu);
  g_knobs = parse_knobs();
  g_knobs_ready.store(true, std::memory_order_release);
  return 0;
}

std::string &fhip_tls_error() {
  static thread_local std::string s;
  return s;
}

int fhip_fail(fhip_ctx *ctx, const char *fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  if (ctx)
    ctx->err = buf;
  fhip_tls_error() = buf;
  return 1;
}

int fhip_ctx_scratch(fhip_ctx *ctx, size_t bytes, void **out) {
  if (bytes > ctx->scratch_bytes) {
    FHIP_HIP_CHECK(ctx, hipSetDevice(ctx->device));
    if (ctx->scratch) {
      FHIP_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));
      FHIP_HIP_CHECK(ctx, hipFree(ctx->scratch));
      ctx->scratch = nullptr;
      ctx->scratch_bytes = 0;
    }
    const size_t want = bytes < (64u << 10) ? (64u << 10) : bytes;
    FHIP_HIP_CHECK(ctx, hipMalloc(&ctx->scratch, want));
    ctx->scratch_bytes = want;
  }
  *out = ctx->scratch;
  return 0;
}

bool fhip_check_desc(fhip_ctx *ctx, const fhip_tensor_desc &t,
                     const char *what) {
  if (t.rank < 1 || t.rank > FHIP_MAX_RANK) {
    fhip_fail(ctx, "%s: rank %d outside [1, %d]", what, t.rank, FHIP_MAX_RANK);
    return false;
  }
  if (fhip_dtype_size(t.dtype) == 0) {
    fhip_fail(ctx, "%s: unsupported element type %d", what, t.dtype);
    return false;
  }
  for (int i = 0; i < t.rank; ++i) {
    if (t.dim[i] < 1 || t.stride[i] < 0) {
      fhip_fail(ctx, "%s: dim[%d]=%lld stride[%d]=%lld invalid", what, i,
                (long long)t.dim[i], i, (long long)t.stride[i]);
      return false;
    }
  }
  return true;
}

bool fhip_broadcast_strides(const fhip_tensor_desc &operand, int out_rank,
                            const int64_t *out_dims, int64_t *strides) {
  if (operand.rank > out_rank)
    return false;
  const int shift = out_rank - operand.rank;
  for (int i = 0; i < out_rank; ++i)
    strides[i] = 0;
  for (int i = 0; i < operand.rank; ++i) {
    const int64_t od = out_dims[i + shift];
    if (operand.dim[i] == od)
      strides[i + shift] = (od == 1) ? 0 : operand.stride[i];
    else if (operand.dim[i] == 1)
      strides[i + shift] = 0;
    else
      return false;
  }
  return true;
}

int fhip_build_epilogue(fhip_ctx *ctx, const fhip_epilogue &e, int out_rank,
                        const int64_t *out_dims,
                        const void *const *operand_ptrs, DevEpilogue *out) {
  memset(out, 0, sizeof(*out));
  FHIP_REQUIRE(ctx, e.count >= 0 && e.count <= FHIP_MAX_EPILOGUE,
               "epilogue: count %d outside [0, %d]", e.count,
               FHIP_MAX_EPILOGUE);
  out->count = e.count;
  out->rank = out_rank;
  for (int i = 0; i < e.count; ++i) {
    const fhip_epilogue_op &s = e.op[i];
    DevEpiOp &d = out->op[i];
    FHIP_REQUIRE(ctx, s.mode > FHIP_PW_NOT_SET && s.mode < FHIP_PW_MODE_COUNT,
                 "epilogue[%d]: invalid pointwise mode %d", i, s.mode);
    const int arity = fhip_pw_arity(s.mode);
    FHIP_REQUIRE(ctx, arity <= 2,
                 "epilogue[%d]: ternary modes cannot be fused", i);
    FHIP_REQUIRE(ctx,
                 (arity == 1) == (s.operand_kind == FHIP_OPERAND_NONE),
                 "epilogue[%d]: mode %d takes %d inputs but operand_kind is %d",
                 i, s.mode, arity, s.operand_kind);
    FHIP_REQUIRE(ctx, fhip_dtype_size(s.result_dtype) != 0,
                 "epilogue[%d]: unsupported result dtype %d", i,
                 s.result_dtype);
    d.mode = s.mode;
    d.kind = s.operand_kind;
    d.acc_is_in1 = s.acc_is_in1;
    d.result_dtype = s.result_dtype;
    d.scalar = s.scalar;
    d.params = s.params;
    if (s.operand_kind == FHIP_OPERAND_TENSOR) {
      FHIP_REQUIRE(ctx, operand_ptrs != nullptr,
                   "epilogue[%d]: operand pointer array is null", i);
      FHIP_REQUIRE(ctx,
                   s.operand_index >= 0 && s.operand_index < FHIP_MAX_EPILOGUE,
                   "epilogue[%d]: operand_index %d out of range", i,
                   s.operand_index);
      d.ptr = operand_ptrs[s.operand_index];
      FHIP_REQUIRE(ctx, d.ptr != nullptr, "epilogue[%d]: operand pointer null",
                   i);
      if (!fhip_check_desc(ctx, s.operand, "epilogue operand"))
        return 1;
      d.operand_dtype = s.operand.dtype;
      FHIP_REQUIRE(ctx,
                   fhip_broadcast_strides(s.operand, out_rank, out_dims,
                                          d.stride),
                   "epilogue[%d]: operand dims do not broadcast to the "
                   "producer's output",
                   i);
    }
  }
  return 0;
}

extern "C" {

int fhip_abi_version(void) { return FHIP_ABI_VERSION; }

int fhip_device_count(int *count) {
  FHIP_REQUIRE(nullptr, count != nullptr, "fhip_device_count: null out");
  FHIP_HIP_CHECK(nullptr, hipGetDeviceCount(count));
  return 0;
}

int fhip_device_arch(int device_id, char *buf, size_t buf_len) {
  FHIP_REQUIRE(nullptr, buf && buf_len > 0, "fhip_device_arch: null buffer");
  hipDeviceProp_t prop;
  FHIP_HIP_CHECK(nullptr, hipGetDeviceProperties(&prop, device_id));
  snprintf(buf, buf_len, "%s", prop.gcnArchName);
  return 0;
}

int fhip_ctx_create(int device_id, void *external_stream, fhip_ctx **out) {
  FHIP_REQUIRE(nullptr, out != nullptr, "fhip_ctx_create: null out");
  *out = nullptr;
  static std::mutex mu; // serialises first-touch runtime initialisation
  std::lock_guard<std::mutex> lock(mu);
  int n = 0;
  FHIP_HIP_CHECK(nullptr, hipGetDeviceCount(&n));
  FHIP_REQUIRE(nullptr, device_id >= 0 && device_id < n,
               "fhip_ctx_create: device %d not present (%d visible)", device_id,
               n);
  FHIP_HIP_CHECK(nullptr, hipSetDevice(device_id));
  hipDeviceProp_t prop;
  FHIP_HIP_CHECK(nullptr, hipGetDeviceProperties(&prop, device_id));
  FHIP_REQUIRE(nullptr, strncmp(prop.gcnArchName, "gfx950", 6) == 0,
               "fhip_ctx_create: device %d is %s; this backend holds gfx950 "
               "code only",
               device_id, prop.gcnArchName);
  fhip_ctx *c = new fhip_ctx();
  c->device = device_id;
  c->num_cus = prop.multiProcessorCount;
  if (external_stream) {
    c->stream = (hipStream_t)external_stream;
    c->owns_stream = false;
  } else {
    hipError_t e = hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking);
    if (e != hipSuccess) {
      delete c;
      return fhip_fail(nullptr, "hipStreamCreate failed: %s",
                       hipGetErrorString(e));
    }
    c->owns_stream = true;
  }
  if (fhip_conv_dgrad_static_setup(c) != 0) {
    fhip_tls_error() = c->err;
    if (c->owns_stream)
      (void)hipStreamDestroy(c->stream);
    delete c;
    return 1;
  }
  *out = c;
  return 0;
}

int fhip_ctx_destroy(fhip_ctx *ctx) {
  if (!ctx)
    return 0;
  (void)hipSetDevice(ctx->device);
  if (ctx->owns_stream && ctx->stream) {
    (void)hipStreamSynchronize(ctx->stream);
    (void)hipStreamDestroy(ctx->stream);
  }
  if (ctx->scratch)
    (void)hipFree(ctx->scratch);
  delete ctx;
  return 0;
}

const char *fhip_last_error(fhip_ctx *ctx) {
  return ctx ? ctx->err.c_str() : fhip_tls_error().c_str();
}

void *fhip_ctx_stream(fhip_ctx *ctx) { return ctx ? (void *)ctx->stream : nullptr; }
int fhip_ctx_device(fhip_ctx *ctx) { return ctx ? ctx->device : -1; }

const char *fhip_last_kernel(fhip_ctx *ctx) { return ctx ? ctx->last_kernel : ""; }

int fhip_malloc(fhip_ctx *ctx, size_t bytes, void **out) {
  FHIP_REQUIRE(ctx, ctx && out, "fhip_malloc: null argument");
  *out = nullptr;
  FHIP_HIP_CHECK(ctx, hipSetDevice(ctx->device));
  FHIP_HIP_CHECK(ctx, hipMalloc(out, bytes ? bytes : 1));
  return 0;
}

int fhip_free(fhip_ctx *ctx, void *ptr) {
  FHIP_REQUIRE(ctx, ctx != nullptr, "fhip_free: null context");
  if (!ptr)
    return 0;
  FHIP_HIP_CHECK(ctx, hipSetDevice(ctx->device));
  FHIP_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));
  FHIP_HIP_CHECK(ctx, hipFree(ptr));
  return 0;
}

int fhip_memcpy_h2d(fhip_ctx *ctx, void *dst, const void *src, size_t bytes) {
  FHIP_REQUIRE(ctx, ctx && (bytes == 0 || (dst && src)),
               "fhip_memcpy_h2d: null argument");
  if (bytes == 0)
    return 0;
  FHIP_HIP_CHECK(ctx, hipSetDevice(ctx->device));
  FHIP_HIP_CHECK(ctx, hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice,
                                     ctx->stream));
  // Pageable source memory may be reused by the caller as soon as we return.
  FHIP_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));
  return 0;
}

int fhip_memcpy_d2h(fhip_ctx *ctx, void *dst, const void *src, size_t bytes) {
  FHIP_REQUIRE(ctx, ctx && (bytes == 0 || (dst && src)),
               "fhip_memcpy_d2h: null argument");
  FHIP_HIP_CHECK(ctx, hipSetDevice(ctx->device));
  if (bytes)
    FHIP_HIP_CHECK(ctx, hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost,
                                       ctx->stream));
  FHIP_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));
  return 0;
}

int fhip_memcpy_d2d(fhip_ctx *ctx, void *dst, const void *src, size_t bytes) {
  FHIP_REQUIRE(ctx, ctx && (bytes == 0 || (dst && src)),
               "fhip_memcpy_d2d: null argument");
  if (bytes == 0)
    return 0;
  FHIP_HIP_CHECK(ctx, hipSetDevice(ctx->device));
  FHIP_HIP_CHECK(ctx, hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice,
                                     ctx->stream));
  return 0;
}

__global__ void fhip_fill_bytes_kernel(uint8_t *dst, uint8_t v, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t step = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += step)
    dst[i] = v;
}

int fhip_memset(fhip_ctx *ctx, void *dst, int byte_value, size_t bytes) {
  FHIP_REQUIRE(ctx, ctx && (bytes == 0 || dst), "fhip_memset: null argument");
  if (bytes == 0)
    return 0;
  FHIP_HIP_CHECK(ctx, hipSetDevice(ctx->device));
  // A fill kernel rather than a memset node, so callers may capture it.
  size_t blocks = (bytes + 255) / 256;
  if (blocks > 4096)
    blocks = 4096;
  hipLaunchKernelGGL(fhip_fill_bytes_kernel, dim3((unsigned)blocks), dim3(256),
                     0, ctx->stream, (uint8_t *)dst, (uint8_t)byte_value,
                     bytes);
  FHIP_HIP_CHECK(ctx, hipGetLastError());
  return 0;
}

int fhip_stream_sync(fhip_ctx *ctx) {
  FHIP_REQUIRE(ctx, ctx != nullptr, "fhip_stream_sync: null context");
  FHIP_HIP_CHECK(ctx, hipSetDevice(ctx->device));
  FHIP_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));
  return 0;
}

int fhip_event_create(fhip_ctx *ctx, fhip_event **out) {
  FHIP_REQUIRE(ctx, ctx && out, "fhip_event_create: null argument");
  FHIP_HIP_CHECK(ctx, hipSetDevice(ctx->device));
  fhip_event *e = new fhip_event();
  hipError_t r = hipEventCreate(&e->ev);
  if (r != hipSuccess) {
    delete e;
    return fhip_fail(ctx, "hipEventCreate failed: %s", hipGetErrorString(r));
  }
  *out = e;
  return 0;
}

int fhip_event_record(fhip_ctx *ctx, fhip_event *ev) {
  FHIP_REQUIRE(ctx, ctx && ev, "fhip_event_record: null argument");
  FHIP_HIP_CHECK(ctx, hipEventRecord(ev->ev, ctx->stream));
  return 0;
}

int fhip_event_elapsed_ms(fhip_ctx *ctx, fhip_event *start, fhip_event *stop,
                          float *ms) {
  FHIP_REQUIRE(ctx, ctx && start && stop && ms,
               "fhip_event_elapsed_ms: null argument");
  FHIP_HIP_CHECK(ctx, hipEventSynchronize(stop->ev));
  FHIP_HIP_CHECK(ctx, hipEventElapsedTime(ms, start->ev, stop->ev));
  return 0;
}

int fhip_event_destroy(fhip_ctx *ctx, fhip_event *ev) {
  if (!ev)
    return 0;
  (void)hipEventDestroy(ev->ev);
  delete ev;
  (void)ctx;
  return 0;
}

} // extern "C"
