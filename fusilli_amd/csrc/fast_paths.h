// Tuned gfx950 kernels behind the op entry points.  Each op has a predicate
// (does the tuned kernel accept this descriptor?) and a launcher.  Launchers
// assume the descriptor passed the entry point's validation.
#ifndef FUSILLI_AMD_CSRC_FAST_PATHS_H
#define FUSILLI_AMD_CSRC_FAST_PATHS_H

#include "common.h"

bool fhip_fast_matmul_applicable(const fhip_matmul_desc *d);
int fhip_fast_matmul(fhip_ctx *ctx, const fhip_matmul_desc *d, const void *a,
                     const void *b, const DevEpilogue &epi, void *out);

// The same with an outer batch dim of `outer` entries around the descriptor's
// own (element strides per operand, 16-byte multiples; empty epilogue).
int fhip_fast_matmul_outer(fhip_ctx *ctx, const fhip_matmul_desc *d,
                           const void *a, const void *b, const DevEpilogue &epi,
                           void *out, int outer, int64_t a_outer,
                           int64_t b_outer, int64_t o_outer);

// `allow_scratch` false: only plans that leave the context's scratch alone
// (no zero-padded channel copies, no split reduction) -- for the entry point
// that must not allocate.
bool fhip_fast_conv_applicable(const fhip_conv_desc *d, bool allow_scratch = true);
// With `handled` the call plans once and reports whether a tuned kernel was
// launched; a descriptor that none takes is then no error.
int fhip_fast_conv(fhip_ctx *ctx, const fhip_conv_desc *d, const void *x,
                   const void *w, const DevEpilogue &epi, void *out,
                   bool *handled = nullptr, bool allow_scratch = true);

// The same problem on the register-filter kernel (unit stride and dilation,
// 3 x 3 x 64 filters, K a multiple of 128, 16-bit output, linear epilogue that
// may end in a ReLU); fhip_fast_conv tries it first.
bool fhip_fast_conv_rf_applicable(const fhip_conv_desc *d);
// With `handled` the call plans once and reports whether it launched; a
// descriptor it does not take is then no error.
int fhip_fast_conv_rf(fhip_ctx *ctx, const fhip_conv_desc *d, const void *x,
                      const void *w, const DevEpilogue &epi, void *out,
                      bool *handled = nullptr);

// Data gradient through the forward kernel (unit strides, one group); needs
// `*workspace_bytes` of 16-byte aligned workspace for the mirrored filter.
bool fhip_fast_conv_dgrad_applicable(const fhip_conv_desc *d,
                                     size_t *workspace_bytes,
                                     bool allow_scratch = true);
int fhip_fast_conv_dgrad(fhip_ctx *ctx, const fhip_conv_desc *d, const void *dy,
                         const void *w, void *dx, void *workspace,
                         bool allow_scratch = true);

// Data gradient of 3 x 3 convolutions over 128 output channels with the filter
// in registers (conv_rf_dgrad.hip): one kernel, W read as it lies, no
// workspace.  fhip_fast_conv_dgrad takes it where it applies.
bool fhip_fast_conv_dgrad_rf_applicable(const fhip_conv_desc *d);
int fhip_fast_conv_dgrad_rf(fhip_ctx *ctx, const fhip_conv_desc *d,
                            const void *dy, const void *w, void *dx);

// Resolves this device's address of the static scratch array behind
// fhip_conv_dgrad_static into the context (device current, creation lock held).
int fhip_conv_dgrad_static_setup(fhip_ctx *ctx);

// Weight gradient as batched GEMMs over zero-padded copies of X and DY
// (channels-last 16-bit tensors, equal strides, one group); needs
// `*workspace_bytes` of 256-byte aligned workspace.
bool fhip_fast_conv_wgrad_applicable(const fhip_conv_desc *d,
                                     size_t *workspace_bytes);
int fhip_fast_conv_wgrad(fhip_ctx *ctx, const fhip_conv_desc *d, const void *dy,
                         const void *x, void *dw, void *workspace);

// Weight gradient of 3 x 3, padding-1, unit-stride convolutions straight from
// X and DY (no operand copies): one MFMA kernel plus the sum of its partial
// results; `*workspace_bytes` of 256-byte aligned workspace hold those.
bool fhip_fast_conv_wgrad_direct_applicable(const fhip_conv_desc *d,
                                            size_t *workspace_bytes);
int fhip_fast_conv_wgrad_direct(fhip_ctx *ctx, const fhip_conv_desc *d,
                                const void *dy, const void *x, void *dw,
                                void *workspace);

// Register-blocked direct kernels for any layout, dtype, group count and 1 - 3
// spatial dims (conv_direct.hip): the path of the convolutions the MFMA
// kernels do not take.  The weight gradient keeps its partial sums in the
// context's scratch buffer.
bool fhip_direct_conv_applicable(const fhip_conv_desc *d);
// forward: the channels-last kernel for groups of 1, 2, 4 or 8 channels
bool fhip_direct_conv_cl_applicable(const fhip_conv_desc *d);
int fhip_direct_conv_fprop(fhip_ctx *ctx, const fhip_conv_desc *d,
                           const void *x, const void *w, const DevEpilogue &epi,
                           void *out);
int fhip_direct_conv_dgrad(fhip_ctx *ctx, const fhip_conv_desc *d,
                           const void *dy, const void *w, void *dx);
int fhip_direct_conv_wgrad(fhip_ctx *ctx, const fhip_conv_desc *d,
                           const void *dy, const void *x, void *dw);

bool fhip_fast_sdpa_applicable(const fhip_sdpa_desc *d);
int fhip_fast_sdpa(fhip_ctx *ctx, const fhip_sdpa_desc *d, const void *q,
                   const void *k, const void *v, const void *mask, void *o);

bool fhip_fast_norm_applicable(const fhip_norm_desc *d);
int fhip_fast_norm(fhip_ctx *ctx, const fhip_norm_desc *d, const void *x,
                   const void *scale, const void *bias, const DevEpilogue &epi,
                   void *out, void *mean, void *inv_variance);

// Rows too long for the register-resident kernels (rownorm_long.hip); the
// layout conditions are the caller's (rownorm.hip).
bool fhip_norm_long_applicable(const fhip_norm_desc *d);
int fhip_norm_long(fhip_ctx *ctx, const fhip_norm_desc *d, int64_t inner,
                   const void *x, const void *scale, const void *bias, void *out,
                   void *mean, void *inv_variance);

bool fhip_fast_reduce_applicable(const fhip_reduce_desc *d);
int fhip_fast_reduce(fhip_ctx *ctx, const fhip_reduce_desc *d, const void *x,
                     void *y);

// Batch normalisation of dense channels-last tensors (column statistics with
// whole pixel vectors per load); everything else runs on the generic kernels.
bool fhip_fast_batchnorm_applicable(const fhip_batchnorm_desc *d);
int fhip_fast_batchnorm(fhip_ctx *ctx, const fhip_batchnorm_desc *d, const void *x,
                        const void *scale, const void *bias, const void *running_mean,
                        const void *running_var, void *y, void *saved_mean,
                        void *saved_inv_variance);

bool fhip_fast_pointwise_applicable(const fhip_pointwise_desc *d);
int fhip_fast_pointwise(fhip_ctx *ctx, const fhip_pointwise_desc *d,
                        const void *in0, const void *in1, const void *in2,
                        void *out);

#endif // FUSILLI_AMD_CSRC_FAST_PATHS_H
