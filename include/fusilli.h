// Umbrella header of the graph API (namespace fusilli), source-compatible
// with programs written against the reference's <fusilli.h>
// (reference include/fusilli.h:16-70) apart from the IREE types that leaked
// through it: buffers take std::vector<size_t> shapes, and Buffer::import
// takes a raw device pointer.  Link with -lfusilli_hip.
#ifndef FUSILLI_H
#define FUSILLI_H

#include "fusilli/backend.h"
#include "fusilli/errors.h"
#include "fusilli/graph.h"
#include "fusilli/nodes.h"
#include "fusilli/op_attrs.h"
#include "fusilli/plan.h"
#include "fusilli/tensor_attr.h"
#include "fusilli/types.h"

#endif // FUSILLI_H
