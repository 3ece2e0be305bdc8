/* Source-compatible umbrella: callers of the reference include this name
 * (reference include/infini_operators.h:1-19). */
#include "infiniop.h"
