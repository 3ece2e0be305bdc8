/* Forwarding header: a caller written against the reference includes this
 * path (reference include/status.h:4-14) and finds here infiniopStatus_t.  Everything is declared in
 * infiniop.h. */
#ifndef INFINIOP_AMD_FWD_STATUS_H
#define INFINIOP_AMD_FWD_STATUS_H
#include "infiniop.h"
#include "export.h"
#endif
