#include "common.h"
#include "fast_paths.h"
bool fhip_fast_conv_applicable(const fhip_conv_desc *) { return false; }
int fhip_fast_conv(fhip_ctx *ctx, const fhip_conv_desc *, const void *, const void *, const DevEpilogue &, void *) { return fhip_fail(ctx, "no fast conv"); }
