/* Forwarding header: a caller written against the reference includes this
 * path (reference include/tensor.h:7-18) and finds here struct TensorDescriptor, infiniopTensorDescriptor_t.  Everything is declared in
 * infiniop.h. */
#ifndef INFINIOP_AMD_FWD_TENSOR_H
#define INFINIOP_AMD_FWD_TENSOR_H
#include "infiniop.h"
#include "export.h"
#endif
