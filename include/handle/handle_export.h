/* Forwarding header: a caller written against the reference includes this
 * path (reference include/handle/handle_export.h:8-10) and finds here infiniopCreateHandle, infiniopDestroyHandle.  Everything is declared in
 * infiniop.h. */
#ifndef INFINIOP_AMD_FWD_HANDLE_HANDLE_EXPORT_H
#define INFINIOP_AMD_FWD_HANDLE_HANDLE_EXPORT_H
#include "../infiniop.h"
#endif
