/* Forwarding header: programs written against oneDNN include "dnnl.hpp" from the
 * top of the include directory (reference: include/dnnl.hpp). */
#ifndef DNNL_HPP
#define DNNL_HPP

#include "oneapi/dnnl/dnnl.hpp"

#endif /* DNNL_HPP */
