/* Forwarding header: programs written against oneDNN include "dnnl_debug.h" from the
 * top of the include directory (reference: include/dnnl_debug.h). */
#ifndef DNNL_DEBUG_H
#define DNNL_DEBUG_H

#include "oneapi/dnnl/dnnl_debug.h"

#endif /* DNNL_DEBUG_H */
