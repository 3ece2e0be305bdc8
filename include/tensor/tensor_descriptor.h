/* Forwarding header: a caller written against the reference includes this
 * path (reference include/tensor/tensor_descriptor.h:8-10) and finds here infiniopCreateTensorDescriptor, infiniopDestroyTensorDescriptor.  Everything is declared in
 * infiniop.h. */
#ifndef INFINIOP_AMD_FWD_TENSOR_TENSOR_DESCRIPTOR_H
#define INFINIOP_AMD_FWD_TENSOR_TENSOR_DESCRIPTOR_H
#include "../infiniop.h"
#include "../export.h"
#endif
