/* Forwarding header: programs written against oneDNN include "dnnl_config.h" from the
 * top of the include directory (reference: include/dnnl_config.h). */
#ifndef DNNL_CONFIG_H
#define DNNL_CONFIG_H

#include "oneapi/dnnl/dnnl_config.h"

#endif /* DNNL_CONFIG_H */
