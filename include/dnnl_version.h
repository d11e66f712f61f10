/* Forwarding header: programs written against oneDNN include "dnnl_version.h" from the
 * top of the include directory (reference: include/dnnl_version.h). */
#ifndef DNNL_VERSION_H
#define DNNL_VERSION_H

#include "oneapi/dnnl/dnnl_version.h"

#endif /* DNNL_VERSION_H */
