/* Forwarding header: a caller written against the reference includes this
 * path (reference include/data_type.h:4-46) and finds here DataLayout / DT and the element-type constants.  Everything is declared in
 * infiniop.h. */
#ifndef INFINIOP_AMD_FWD_DATA_TYPE_H
#define INFINIOP_AMD_FWD_DATA_TYPE_H
#include "infiniop.h"
#include "export.h"
#endif
