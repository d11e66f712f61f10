/* Forwarding header: programs written against oneDNN include "dnnl.h" from the
 * top of the include directory (reference: include/dnnl.h). */
#ifndef DNNL_H
#define DNNL_H

#include "oneapi/dnnl/dnnl.h"

#endif /* DNNL_H */
