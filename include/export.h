/* The two macros every operator header of the reference starts from
 * (reference include/export.h:4-16): `__export` marks an entry point as
 * visible outside the shared library, `__C` gives it C linkage.  A caller or
 * binding copied from the reference may use them in its own declarations;
 * here they are the names infiniop.h uses for the same two things. */
#ifndef INFINIOP_AMD_FWD_EXPORT_H
#define INFINIOP_AMD_FWD_EXPORT_H
#include "infiniop.h"
#ifndef __export
#define __export INFINIOP_EXPORT
#endif
#ifndef __C
#define __C INFINIOP_C
#endif
#endif
