#include "common.h"
#include "fast_paths.h"
bool fhip_fast_reduce_applicable(const fhip_reduce_desc *) { return false; }
int fhip_fast_reduce(fhip_ctx *ctx, const fhip_reduce_desc *, const void *, void *) { return fhip_fail(ctx, "no fast reduce"); }
