/* Forwarding header: a caller written against the reference includes this
 * path (reference include/ops/attention/attention.h:15-38) and finds here the four Attention entry points.  Everything is declared in
 * infiniop.h. */
#ifndef INFINIOP_AMD_FWD_OPS_ATTENTION_ATTENTION_H
#define INFINIOP_AMD_FWD_OPS_ATTENTION_ATTENTION_H
#include "../../infiniop.h"
#include "../../export.h"
#endif
