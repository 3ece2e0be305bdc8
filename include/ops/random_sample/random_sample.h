/* Forwarding header: a caller written against the reference includes this
 * path (reference include/ops/random_sample/random_sample.h:14-29) and finds here the four RandomSample entry points.  Everything is declared in
 * infiniop.h. */
#ifndef INFINIOP_AMD_FWD_OPS_RANDOM_SAMPLE_RANDOM_SAMPLE_H
#define INFINIOP_AMD_FWD_OPS_RANDOM_SAMPLE_RANDOM_SAMPLE_H
#include "../../infiniop.h"
#include "../../export.h"
#endif
