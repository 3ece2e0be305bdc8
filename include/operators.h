/* Forwarding header: a caller written against the reference includes this
 * path (reference include/operators.h:1-9) and finds here the core types: Device, infiniopStatus_t, DataLayout, TensorDescriptor, HandleStruct.  Everything is declared in
 * infiniop.h. */
#ifndef INFINIOP_AMD_FWD_OPERATORS_H
#define INFINIOP_AMD_FWD_OPERATORS_H
#include "infiniop.h"
#include "export.h"
#endif
