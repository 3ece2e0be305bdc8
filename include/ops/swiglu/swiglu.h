/* Forwarding header: a caller written against the reference includes this
 * path (reference include/ops/swiglu/swiglu.h:13-25) and finds here the three SwiGLU entry points.  Everything is declared in
 * infiniop.h. */
#ifndef INFINIOP_AMD_FWD_OPS_SWIGLU_SWIGLU_H
#define INFINIOP_AMD_FWD_OPS_SWIGLU_SWIGLU_H
#include "../../infiniop.h"
#include "../../export.h"
#endif
