/* Forwarding header: a caller written against the reference includes this
 * path (reference include/ops/add/add.h:13-25) and finds here infiniopCreateAddDescriptor, infiniopAdd, infiniopDestroyAddDescriptor.  Everything is declared in
 * infiniop.h. */
#ifndef INFINIOP_AMD_FWD_OPS_ADD_ADD_H
#define INFINIOP_AMD_FWD_OPS_ADD_ADD_H
#include "../../infiniop.h"
#include "../../export.h"
#endif
