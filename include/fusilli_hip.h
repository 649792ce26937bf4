/*
 * fusilli_hip.h — C ABI of the MI355X (gfx950) execution backend.
 *
 * This is the boundary that replaces everything the reference does below
 * Graph::emitAsm(): torch-MLIR emission, iree-compile and the IREE runtime
 * (reference: include/fusilli/backend/runtime.h:242-315 createVmContext,
 * :383-529 Graph::execute → iree_vm_invoke; backend/compile_session.h:489-570).
 * The C++ front end (include/fusilli.h) and any other host (ctypes, cgo, JNI)
 * bind exactly these entry points.  Plain C: opaque context pointer, raw device
 * pointers, sizes, POD descriptors.  No torch, no IREE, no C++ types.
 *
 * Conventions
 *   - every function returns 0 on success, non-zero on failure; the text of the
 *     last failure on a context is fhip_last_error(ctx) (ctx == NULL: the
 *     calling thread's last context-less failure);
 *   - the caller owns all device memory; a context owns its stream only when
 *     it created it (external_stream == NULL);
 *   - all kernel entry points are asynchronous and ordered on the context's
 *     stream; fhip_memcpy_d2h and fhip_stream_sync are the sync points
 *     (reference: Buffer::read, backend/runtime.h:646-674);
 *   - tensors are described like the reference's TensorAttr: logical dims in
 *     the op's fixed logical order (NCHW / KCRS / [B,H,S,D] / [..,M,K]) plus
 *     element strides that define the physical layout
 *     (reference: attributes/tensor_attributes.h:374-809);
 *   - a context is not thread-safe; creating contexts concurrently is
 *     (reference: tests/test_handle.cpp:47-85).
 */
#ifndef FUSILLI_HIP_H
#define FUSILLI_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FHIP_MAX_RANK 8
#define FHIP_MAX_EPILOGUE 4
#define FHIP_ABI_VERSION 1

/* Element types.  Values 0..12 equal the reference's DataType enum
 * (attributes/types.h:27-45); FP8E4M3 (OCP e4m3fn, the gfx950 hardware format)
 * is an extension the reference lacks. */
typedef enum {
  FHIP_NOT_SET = 0,
  FHIP_HALF = 1,
  FHIP_BFLOAT16 = 2,
  FHIP_FLOAT = 3,
  FHIP_DOUBLE = 4,
  FHIP_UINT8 = 5,
  FHIP_INT4 = 6, /* unsupported by every kernel; reserved for numbering */
  FHIP_INT8 = 7,
  FHIP_INT16 = 8,
  FHIP_INT32 = 9,
  FHIP_INT64 = 10,
  FHIP_BOOLEAN = 11, /* one byte per element, 0 or 1 */
  FHIP_FP8E5M2 = 12,
  FHIP_FP8E4M3 = 13
} fhip_dtype;

/* Pointwise modes.  Values equal the reference's PointwiseAttr::Mode
 * (attributes/pointwise_attributes.h:27-84, NOT_SET = 0). */
typedef enum {
  FHIP_PW_NOT_SET = 0,
  FHIP_PW_ABS,
  FHIP_PW_ADD,
  FHIP_PW_ADD_SQUARE,
  FHIP_PW_BINARY_SELECT,
  FHIP_PW_CEIL,
  FHIP_PW_CMP_EQ,
  FHIP_PW_CMP_GE,
  FHIP_PW_CMP_GT,
  FHIP_PW_CMP_LE,
  FHIP_PW_CMP_LT,
  FHIP_PW_CMP_NEQ,
  FHIP_PW_DIV,
  FHIP_PW_ELU_FWD,
  FHIP_PW_ERF,
  FHIP_PW_EXP,
  FHIP_PW_FLOOR,
  FHIP_PW_GELU_APPROX_TANH_BWD,
  FHIP_PW_GELU_APPROX_TANH_FWD,
  FHIP_PW_GELU_BWD,
  FHIP_PW_GELU_FWD,
  FHIP_PW_IDENTITY,
  FHIP_PW_LOG,
  FHIP_PW_LOGICAL_AND,
  FHIP_PW_LOGICAL_NOT,
  FHIP_PW_LOGICAL_OR,
  FHIP_PW_MAX_OP,
  FHIP_PW_MIN_OP,
  FHIP_PW_MUL,
  FHIP_PW_NEG,
  FHIP_PW_RECIPROCAL,
  FHIP_PW_RELU_BWD,
  FHIP_PW_RELU_FWD,
  FHIP_PW_RSQRT,
  FHIP_PW_SIGMOID_FWD,
  FHIP_PW_SIN,
  FHIP_PW_SOFTPLUS_FWD,
  FHIP_PW_SQRT,
  FHIP_PW_SUB,
  FHIP_PW_SWISH_BWD,
  FHIP_PW_SWISH_FWD,
  FHIP_PW_TAN,
  FHIP_PW_TANH_BWD,
  FHIP_PW_TANH_FWD,
  FHIP_PW_MODE_COUNT
} fhip_pointwise_mode;

/* Reduction modes.  Values equal the reference's ReductionAttr::Mode
 * (attributes/reduction_attributes.h:27-38). */
typedef enum {
  FHIP_RED_NOT_SET = 0,
  FHIP_RED_ADD,
  FHIP_RED_SUM,
  FHIP_RED_MUL,
  FHIP_RED_MIN,
  FHIP_RED_MAX,
  FHIP_RED_AMAX,
  FHIP_RED_AVG,
  FHIP_RED_NORM1,
  FHIP_RED_NORM2,
  FHIP_RED_MUL_NO_ZEROS
} fhip_reduction_mode;

/* Logical dims + element strides + element type: the information a validated
 * TensorAttr carries (attributes/tensor_attributes.h:374-443).  A stride of 0
 * on an input marks a broadcast dim. */
typedef struct {
  int32_t rank;
  int32_t dtype; /* fhip_dtype */
  int64_t dim[FHIP_MAX_RANK];
  int64_t stride[FHIP_MAX_RANK];
} fhip_tensor_desc;

/* Float parameters of the parameterised pointwise modes
 * (attributes/pointwise_attributes.h:190-194 defaults: 1, 1, 20, 1). */
typedef struct {
  float elu_alpha;
  float softplus_beta;
  float softplus_threshold;
  float swish_beta;
} fhip_pointwise_params;

/* One fused pointwise step applied to a producer's result before it is
 * stored.  The running value `v` (f32, or int32 for integer matmul) takes the
 * place of IN_0 (acc_is_in1 == 0) or IN_1 (acc_is_in1 == 1) of the reference's
 * PointwiseNode (node/pointwise_node.h:44-169); the other operand, for binary
 * modes, is either a tensor broadcastable to the producer's output
 * (operand_kind FHIP_OPERAND_TENSOR, pointer passed in the entry point's
 * epilogue pointer array at index operand_index) or an inlined scalar constant
 * (FHIP_OPERAND_SCALAR; reference: scalar TensorAttr inlined as a constant,
 * support/asm_emitter.h:241-276).  result_dtype is the dtype of the pointwise
 * node's OUT_0; the value is rounded through it (the reference materialises
 * that type between ops). */
enum { FHIP_OPERAND_NONE = 0, FHIP_OPERAND_TENSOR = 1, FHIP_OPERAND_SCALAR = 2 };
typedef struct {
  int32_t mode; /* fhip_pointwise_mode, unary or binary */
  int32_t operand_kind;
  int32_t operand_index;
  int32_t acc_is_in1;
  int32_t result_dtype; /* fhip_dtype */
  float scalar;
  fhip_pointwise_params params;
  fhip_tensor_desc operand; /* logical dims right-aligned-broadcastable to the
                               producer's output; strides as given by caller */
} fhip_epilogue_op;

typedef struct {
  int32_t count;
  fhip_epilogue_op op[FHIP_MAX_EPILOGUE];
} fhip_epilogue;

/* ---- context, memory, stream (replaces Handle / Buffer internals:
 *      backend/handle.h:35-176, backend/buffer.h:31-81,
 *      backend/runtime.h:81-231, :531-674) -------------------------------- */
typedef struct fhip_ctx fhip_ctx;

int fhip_abi_version(void);
int fhip_device_count(int *count);
/* gcnArchName of the device into buf (e.g. "gfx950:sramecc+:xnack-"). */
int fhip_device_arch(int device_id, char *buf, size_t buf_len);
/* external_stream: a hipStream_t the caller owns, or NULL for a stream the
 * context creates (handle.h:89-112). */
/* Tuning knobs (environment variables FUSILLI_HIP_*: tile shapes, grid caps)
 * are parsed once per process, not per launch.  fhip_tuning_reload parses them
 * again; call it only while no other thread is inside the library.  It has no
 * counterpart in the reference, whose flags travel through
 * FUSILLI_EXTRA_COMPILER_FLAGS at compile time (backend/backend.h:226-297). */
int fhip_tuning_reload(void);
int fhip_ctx_create(int device_id, void *external_stream, fhip_ctx **out);
int fhip_ctx_destroy(fhip_ctx *ctx);
const char *fhip_last_error(fhip_ctx *ctx);
/* Name of the kernel variant that the last operator call on this context
 * launched, with its shape parameters (e.g. "conv_rf rows=7",
 * "gemm_mfma 256x256 w8", "sdpa_fwd d=128 causal=1 mask=0"); "" before the
 * first call.  The string lives in the context and is overwritten by the next
 * call.  It has no counterpart in the reference, where one IREE dispatch list
 * serves every shape: here several tuned kernels stand behind one operator,
 * and tests and benchmarks assert that the one they mean to cover has run. */
const char *fhip_last_kernel(fhip_ctx *ctx);
void *fhip_ctx_stream(fhip_ctx *ctx);
int fhip_ctx_device(fhip_ctx *ctx);

int fhip_malloc(fhip_ctx *ctx, size_t bytes, void **out);
int fhip_free(fhip_ctx *ctx, void *ptr);
int fhip_memcpy_h2d(fhip_ctx *ctx, void *dst, const void *src, size_t bytes);
int fhip_memcpy_d2h(fhip_ctx *ctx, void *dst, const void *src, size_t bytes);
int fhip_memcpy_d2d(fhip_ctx *ctx, void *dst, const void *src, size_t bytes);
int fhip_memset(fhip_ctx *ctx, void *dst, int byte_value, size_t bytes);
int fhip_stream_sync(fhip_ctx *ctx);

/* Stream-ordered timers for harnesses (the reference measures from outside with
 * rocprofv3, benchmarks/run_benchmark.py:41-119; these bracket launches on the
 * context's own stream). */
typedef struct fhip_event fhip_event;
int fhip_event_create(fhip_ctx *ctx, fhip_event **out);
int fhip_event_record(fhip_ctx *ctx, fhip_event *ev);
int fhip_event_elapsed_ms(fhip_ctx *ctx, fhip_event *start, fhip_event *stop,
                          float *ms); /* synchronises on `stop` */
int fhip_event_destroy(fhip_ctx *ctx, fhip_event *ev);

/* ---- matmul (node/matmul_node.h:72-253; aten.matmul,
 *      support/asm_emitter.h:1669-1696) ---------------------------------- */
typedef struct {
  fhip_tensor_desc a; /* [..., M, K] */
  fhip_tensor_desc b; /* [..., K, N] */
  fhip_tensor_desc c; /* [..., M, N]; dtype = result type of the matmul node */
  fhip_epilogue epilogue;
  int32_t out_dtype; /* dtype actually stored = last epilogue result_dtype,
                        or c.dtype when the epilogue is empty */
  fhip_tensor_desc out; /* layout of the stored tensor (== c when no epilogue) */
} fhip_matmul_desc;

int fhip_matmul_workspace_size(const fhip_matmul_desc *d, size_t *bytes);
/* 0 = unsupported, 1 = generic strided kernel, 2 = MFMA fast path */
int fhip_matmul_supported(const fhip_matmul_desc *d);
int fhip_matmul(fhip_ctx *ctx, const fhip_matmul_desc *d, const void *a,
                const void *b, const void *const *epilogue_operands, void *out,
                void *workspace, size_t workspace_bytes);

/* ---- convolution forward (node/conv_node.h:62-253; aten.convolution,
 *      support/asm_emitter.h:690-701) ------------------------------------ */
typedef struct {
  fhip_tensor_desc x; /* [N, C, spatial...]  */
  fhip_tensor_desc w; /* [K, C/groups, filter spatial...] */
  fhip_tensor_desc y; /* [N, K, out spatial...] */
  int32_t spatial_rank; /* 1, 2 or 3 */
  int64_t padding[3];
  int64_t stride[3];
  int64_t dilation[3];
  fhip_epilogue epilogue;
  int32_t out_dtype;
  fhip_tensor_desc out;
} fhip_conv_desc;

int fhip_conv_fprop_workspace_size(const fhip_conv_desc *d, size_t *bytes);
int fhip_conv_fprop_supported(const fhip_conv_desc *d);
int fhip_conv_fprop(fhip_ctx *ctx, const fhip_conv_desc *d, const void *x,
                    const void *w, const void *const *epilogue_operands,
                    void *out, void *workspace, size_t workspace_bytes);

/* ---- convolution backward: data gradient (node/conv_node.h:428-598,
 *      ConvDGradNode) and weight gradient (node/conv_node.h:255-426,
 *      ConvWGradNode); both lower to aten.convolution_backward in the
 *      reference.  The descriptor names the forward problem: `x` describes DX
 *      (dgrad output) or X (wgrad input), `w` describes W (dgrad input) or DW
 *      (wgrad output), `y` describes DY.  `epilogue` must be empty; `out` and
 *      `out_dtype` are not read.  f32 accumulation, one rounding to the
 *      gradient's dtype.  fhip_conv_dgrad_supported returns 2 where the MFMA
 *      kernel takes the problem (16-bit channels-last tensors, one group):
 *      it then needs fhip_conv_dgrad_workspace_size bytes of 256-byte aligned
 *      workspace (a mirrored copy of the filter; with strides above one also
 *      DY spread over a zero grid) and fails without them.  fhip_conv_wgrad_supported returns 2 for 16-bit
 *      channels-last X and DY with equal strides, one group, K >= 128 and
 *      S * C >= 128 (batched MFMA GEMMs over zero-padded copies of both
 *      operands; 256-byte aligned workspace of
 *      fhip_conv_wgrad_workspace_size bytes). ----------------------------- */
int fhip_conv_dgrad_workspace_size(const fhip_conv_desc *d, size_t *bytes);
int fhip_conv_dgrad_supported(const fhip_conv_desc *d);
int fhip_conv_dgrad(fhip_ctx *ctx, const fhip_conv_desc *d, const void *dy,
                    const void *w, void *dx, void *workspace,
                    size_t workspace_bytes);
/* fhip_conv_dgrad without any allocation and without caller workspace.  It has
 * no counterpart in the reference; it exists for callers that cannot allocate
 * device memory around the call (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  The mirrored filter (and DY's zero
 * grid for strides above one) live in a per-device static array of
 * FHIP_CONV_DGRAD_STATIC_MAX_BYTES inside the library; descriptors whose
 * fhip_conv_dgrad_workspace_size exceeds that fail with a message.  It plans
 * without the context's growable scratch: descriptors that fhip_conv_dgrad
 * runs on zero-padded channel copies or with a split reduction take the
 * direct (slower) kernels here, 1 x 1 filters at unit stride (which
 * fhip_conv_dgrad hands to the matrix-product kernels, whose planner may use
 * the scratch) stay on the convolution kernel, and the results of both may
 * differ from fhip_conv_dgrad's in the last bit (another summation order);
 * every other
 * descriptor runs the same kernel with bit-identical results.  All calls on
 * one GPU share the array: calls that overlap on one GPU (two streams, two
 * contexts) race. */
#define FHIP_CONV_DGRAD_STATIC_MAX_BYTES (8u << 20)
int fhip_conv_dgrad_static(fhip_ctx *ctx, const fhip_conv_desc *d,
                           const void *dy, const void *w, void *dx);
int fhip_conv_wgrad_workspace_size(const fhip_conv_desc *d, size_t *bytes);
int fhip_conv_wgrad_supported(const fhip_conv_desc *d);
int fhip_conv_wgrad(fhip_ctx *ctx, const fhip_conv_desc *d, const void *dy,
                    const void *x, void *dw, void *workspace,
                    size_t workspace_bytes);

/* ---- scaled dot-product attention forward (node/sdpa_node.h:36-236;
 *      aten.scaled_dot_product_attention, support/asm_emitter.h:2409-2468) */
typedef struct {
  fhip_tensor_desc q; /* [B, Hq, Sq, D]   */
  fhip_tensor_desc k; /* [B, Hkv, Skv, D] */
  fhip_tensor_desc v; /* [B, Hkv, Skv, Dv] */
  fhip_tensor_desc mask; /* rank 0 = absent; additive float mask or boolean
                            mask broadcastable to [B, Hq, Sq, Skv] */
  fhip_tensor_desc o; /* [B, Hq, Sq, Dv] */
  int32_t is_causal; /* key position > query position is masked (top-left) */
  int32_t has_scale;
  float scale; /* used when has_scale; else 1/sqrt(D) */
} fhip_sdpa_desc;

int fhip_sdpa_fwd_workspace_size(const fhip_sdpa_desc *d, size_t *bytes);
int fhip_sdpa_fwd_supported(const fhip_sdpa_desc *d);
int fhip_sdpa_fwd(fhip_ctx *ctx, const fhip_sdpa_desc *d, const void *q,
                  const void *k, const void *v, const void *mask, void *o,
                  void *workspace, size_t workspace_bytes);

/* ---- RMSNorm / LayerNorm forward (node/rmsnorm_node.h:38-219,
 *      node/layernorm_node.h:38-264, node/norm_utils.h:27-99;
 *      aten.rms_norm / aten.(native_)layer_norm,
 *      support/asm_emitter.h:1592-1626, 1427-1503).
 *      Normalises over every dim except dim 0. -------------------------- */
typedef struct {
  fhip_tensor_desc x;
  fhip_tensor_desc scale; /* rank 0 = absent; dims = x dims with dim0 = 1 */
  fhip_tensor_desc bias;  /* layernorm only; rank 0 = absent */
  fhip_tensor_desc y;     /* dtype of the norm node's Y */
  float epsilon;
  int32_t is_layernorm;  /* 0 = RMSNorm, 1 = LayerNorm */
  int32_t emit_stats;    /* layernorm TRAINING: store mean and inv_variance,
                            [B,1,...,1] contiguous, dtype stats_dtype */
  int32_t stats_dtype;
  fhip_epilogue epilogue;
  int32_t out_dtype;
  fhip_tensor_desc out;
} fhip_norm_desc;

int fhip_norm_fwd_workspace_size(const fhip_norm_desc *d, size_t *bytes);
int fhip_norm_fwd_supported(const fhip_norm_desc *d);
int fhip_norm_fwd(fhip_ctx *ctx, const fhip_norm_desc *d, const void *x,
                  const void *scale, const void *bias,
                  const void *const *epilogue_operands, void *out, void *mean,
                  void *inv_variance, void *workspace, size_t workspace_bytes);

/* ---- batch normalisation forward (node/batchnorm_node.h:33-245;
 *      aten.native_batch_norm, support/asm_emitter.h:1066-1290).  Statistics
 *      are per channel (dim 1) over batch and space.  SCALE, BIAS, the
 *      running statistics and the saved statistics are dense vectors of C
 *      elements.  Inference (training = 0) normalises with the running mean
 *      and variance; training computes the batch mean and biased variance,
 *      normalises with them and stores mean and 1 / sqrt(var + eps).  The
 *      reference's MOMENTUM operand does not influence any of these outputs
 *      (the op returns no updated running statistics) and has no field. --- */
typedef struct {
  fhip_tensor_desc x; /* [N, C, spatial...] */
  fhip_tensor_desc y; /* same dims */
  int32_t training;
  int32_t has_scale, has_bias;
  int32_t scale_dtype, bias_dtype;
  int32_t running_dtype; /* MEAN and VAR (inference) */
  int32_t stats_dtype;   /* SAVED_MEAN and SAVED_INV_VARIANCE (training) */
  float epsilon;
} fhip_batchnorm_desc;

int fhip_batchnorm_fwd_workspace_size(const fhip_batchnorm_desc *d,
                                      size_t *bytes);
int fhip_batchnorm_fwd_supported(const fhip_batchnorm_desc *d);
int fhip_batchnorm_fwd(fhip_ctx *ctx, const fhip_batchnorm_desc *d,
                       const void *x, const void *scale, const void *bias,
                       const void *running_mean, const void *running_var,
                       void *y, void *saved_mean, void *saved_inv_variance,
                       void *workspace, size_t workspace_bytes);

/* ---- reduction (node/reduction_node.h:31-146;
 *      support/asm_emitter.h:2165-2322).  Keep-dim: y has x's rank; a dim is
 *      reduced where y.dim == 1 and x.dim > 1. --------------------------- */
typedef struct {
  fhip_tensor_desc x;
  fhip_tensor_desc y;
  int32_t mode; /* fhip_reduction_mode */
} fhip_reduce_desc;

int fhip_reduce_workspace_size(const fhip_reduce_desc *d, size_t *bytes);
int fhip_reduce_supported(const fhip_reduce_desc *d);
int fhip_reduce(fhip_ctx *ctx, const fhip_reduce_desc *d, const void *x,
                void *y, void *workspace, size_t workspace_bytes);

/* ---- standalone pointwise (node/pointwise_node.h:44-169;
 *      support/asm_emitter.h:1806-2122).  Inputs broadcast right-aligned to
 *      out's dims (attributes/tensor_attributes.h:334-372).  An input with
 *      in_is_scalar[i] != 0 has no pointer; its value is in_scalar[i]. ------ */
typedef struct {
  int32_t mode; /* fhip_pointwise_mode */
  int32_t num_inputs;
  fhip_tensor_desc in[3];
  int32_t in_is_scalar[3];
  double in_scalar[3];
  fhip_tensor_desc out;
  fhip_pointwise_params params;
} fhip_pointwise_desc;

int fhip_pointwise_supported(const fhip_pointwise_desc *d);
int fhip_pointwise(fhip_ctx *ctx, const fhip_pointwise_desc *d,
                   const void *in0, const void *in1, const void *in2,
                   void *out);

#ifdef __cplusplus
} /* extern "C" */
#endif

#endif /* FUSILLI_HIP_H */
