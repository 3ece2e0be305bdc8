/* Forwarding header for the fused Add + RMSNorm entry points, laid out like
 * the reference's per-operator headers (pattern of reference
 * include/ops/rms_norm/rms_norm.h); the operator itself has no counterpart in
 * the reference.  Everything is declared in infiniop.h. */
#ifndef INFINIOP_AMD_FWD_OPS_ADD_RMS_NORM_H
#define INFINIOP_AMD_FWD_OPS_ADD_RMS_NORM_H
#include "../../infiniop.h"
#include "../../export.h"
#endif
