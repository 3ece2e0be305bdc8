/* Forwarding header: a caller written against the reference includes this
 * path (reference include/ops/matmul/matmul.h:13-31) and finds here the four Matmul entry points.  Everything is declared in
 * infiniop.h. */
#ifndef INFINIOP_AMD_FWD_OPS_MATMUL_MATMUL_H
#define INFINIOP_AMD_FWD_OPS_MATMUL_MATMUL_H
#include "../../infiniop.h"
#include "../../export.h"
#endif
