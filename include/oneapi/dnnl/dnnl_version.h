#ifndef ONEAPI_DNNL_DNNL_VERSION_H
#define ONEAPI_DNNL_DNNL_VERSION_H
/* API level this library follows (reference CMakeLists.txt:55) */
#define DNNL_VERSION_MAJOR 3
#define DNNL_VERSION_MINOR 8
#define DNNL_VERSION_PATCH 0
#endif
