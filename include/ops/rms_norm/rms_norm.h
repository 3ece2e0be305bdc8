/* Forwarding header: a caller written against the reference includes this
 * path (reference include/ops/rms_norm/rms_norm.h:13-26) and finds here the four RMSNorm entry points.  Everything is declared in
 * infiniop.h. */
#ifndef INFINIOP_AMD_FWD_OPS_RMS_NORM_RMS_NORM_H
#define INFINIOP_AMD_FWD_OPS_RMS_NORM_RMS_NORM_H
#include "../../infiniop.h"
#include "../../export.h"
#endif
