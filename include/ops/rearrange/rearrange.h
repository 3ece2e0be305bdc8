/* Forwarding header: a caller written against the reference includes this
 * path (reference include/ops/rearrange/rearrange.h:12-19) and finds here the three Rearrange entry points.  Everything is declared in
 * infiniop.h. */
#ifndef INFINIOP_AMD_FWD_OPS_REARRANGE_REARRANGE_H
#define INFINIOP_AMD_FWD_OPS_REARRANGE_REARRANGE_H
#include "../../infiniop.h"
#include "../../export.h"
#endif
