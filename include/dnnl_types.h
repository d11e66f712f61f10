/* Forwarding header: programs written against oneDNN include "dnnl_types.h" from the
 * top of the include directory (reference: include/dnnl_types.h). */
#ifndef DNNL_TYPES_H
#define DNNL_TYPES_H

#include "oneapi/dnnl/dnnl_types.h"

#endif /* DNNL_TYPES_H */
