/* Forwarding header: a caller written against the reference includes this
 * path (reference include/device.h:4-9) and finds here enum DeviceEnum / Device, with DevAmdGpu = 4 appended.  Everything is declared in
 * infiniop.h. */
#ifndef INFINIOP_AMD_FWD_DEVICE_H
#define INFINIOP_AMD_FWD_DEVICE_H
#include "infiniop.h"
#include "export.h"
#endif
