#include "common.h"
#include "fast_paths.h"
bool fhip_fast_sdpa_applicable(const fhip_sdpa_desc *) { return false; }
int fhip_fast_sdpa(fhip_ctx *ctx, const fhip_sdpa_desc *, const void *, const void *, const void *, void *) { return fhip_fail(ctx, "no fast sdpa"); }
