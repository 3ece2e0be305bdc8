/* Forwarding header: a caller written against the reference includes this
 * path (reference include/ops/rotary_embedding/rotary_embedding.h:10-30) and finds here the four RoPE entry points.  Everything is declared in
 * infiniop.h. */
#ifndef INFINIOP_AMD_FWD_OPS_ROTARY_EMBEDDING_ROTARY_EMBEDDING_H
#define INFINIOP_AMD_FWD_OPS_ROTARY_EMBEDDING_ROTARY_EMBEDDING_H
#include "../../infiniop.h"
#include "../../export.h"
#endif
