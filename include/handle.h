/* Forwarding header: a caller written against the reference includes this
 * path (reference include/handle.h:6-10) and finds here HandleStruct, infiniopHandle_t.  Everything is declared in
 * infiniop.h. */
#ifndef INFINIOP_AMD_FWD_HANDLE_H
#define INFINIOP_AMD_FWD_HANDLE_H
#include "infiniop.h"
#include "export.h"
#endif
