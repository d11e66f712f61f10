/* Build configuration of the MI355X-native quantized-matmul library.
 * Stands where the reference generates include/oneapi/dnnl/dnnl_config.h.in. */
#ifndef ONEAPI_DNNL_DNNL_CONFIG_H
#define ONEAPI_DNNL_DNNL_CONFIG_H

#define DNNL_RUNTIME_NONE 0u
#define DNNL_RUNTIME_SEQ 1u
#define DNNL_RUNTIME_OMP 2u
#define DNNL_RUNTIME_TBB 4u
#define DNNL_RUNTIME_THREADPOOL 8u
#define DNNL_RUNTIME_OCL 256u
#define DNNL_RUNTIME_SYCL 512u
#define DNNL_RUNTIME_DPCPP DNNL_RUNTIME_SYCL
/* not in the reference: a GPU engine driven directly through HIP streams */
#define DNNL_RUNTIME_HIP 1024u

#define DNNL_CPU_THREADING_RUNTIME DNNL_RUNTIME_NONE
#define DNNL_CPU_RUNTIME DNNL_RUNTIME_NONE
#define DNNL_GPU_RUNTIME DNNL_RUNTIME_HIP
#define DNNL_GPU_VENDOR_AMD 4u
#define DNNL_GPU_VENDOR DNNL_GPU_VENDOR_AMD

#if defined(_WIN32)
#define DNNL_API
#else
#define DNNL_API __attribute__((visibility("default")))
#endif

#endif
