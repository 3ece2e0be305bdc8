/* Forwarding header: a caller written against the reference includes this
 * path (reference include/ops/causal_softmax/causal_softmax.h:13-25) and finds here the four CausalSoftmax entry points.  Everything is declared in
 * infiniop.h. */
#ifndef INFINIOP_AMD_FWD_OPS_CAUSAL_SOFTMAX_CAUSAL_SOFTMAX_H
#define INFINIOP_AMD_FWD_OPS_CAUSAL_SOFTMAX_CAUSAL_SOFTMAX_H
#include "../../infiniop.h"
#include "../../export.h"
#endif
