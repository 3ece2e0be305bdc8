/* Forwarding header: a caller written against the reference includes this
 * path (reference include/ops/mlp/mlp.h:15-35) and finds here the four MLP entry points.  Everything is declared in
 * infiniop.h. */
#ifndef INFINIOP_AMD_FWD_OPS_MLP_MLP_H
#define INFINIOP_AMD_FWD_OPS_MLP_MLP_H
#include "../../infiniop.h"
#include "../../export.h"
#endif
