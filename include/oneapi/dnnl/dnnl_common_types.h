/* Common C types of the dnnl API subset served by the MI355X quantized-matmul
 * library. Names and numeric values follow the reference's
 * include/oneapi/dnnl/dnnl_common_types.h (status :45-68, data types :76-115,
 * fpmath :134-145, accumulation :154-169, engine kinds :177-184, stream flags
 * :203-213) so that binaries and bindings written against it keep working. */
#ifndef ONEAPI_DNNL_DNNL_COMMON_TYPES_H
#define ONEAPI_DNNL_DNNL_COMMON_TYPES_H

#include <stddef.h>
#include <stdint.h>

#include "oneapi/dnnl/dnnl_config.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    dnnl_success = 0,
    dnnl_out_of_memory = 1,
    dnnl_invalid_arguments = 2,
    dnnl_unimplemented = 3,
    dnnl_last_impl_reached = 4,
    dnnl_runtime_error = 5,
    dnnl_not_required = 6,
    dnnl_invalid_graph = 7,
    dnnl_invalid_graph_op = 8,
    dnnl_invalid_shape = 9,
    dnnl_invalid_data_type = 10,
} dnnl_status_t;

typedef enum {
    dnnl_data_type_undef = 0,
    dnnl_f16 = 1,
    dnnl_bf16 = 2,
    dnnl_f32 = 3,
    dnnl_s32 = 4,
    dnnl_s8 = 5,
    dnnl_u8 = 6,
    dnnl_f64 = 7,
    dnnl_boolean = 8,
    dnnl_f8_e5m2 = 9,
    dnnl_f8_e4m3 = 10,
    dnnl_s4 = 11,
    dnnl_u4 = 12,
    dnnl_e8m0 = 13,
    dnnl_f4_e2m1 = 14,
    dnnl_f4_e3m0 = 15,
    dnnl_data_type_max = 0x7fff,
} dnnl_data_type_t;

#define DNNL_MAX_NDIMS 12
typedef int64_t dnnl_dim_t;
typedef dnnl_dim_t dnnl_dims_t[DNNL_MAX_NDIMS];

typedef enum {
    dnnl_fpmath_mode_strict,
    dnnl_fpmath_mode_bf16,
    dnnl_fpmath_mode_f16,
    dnnl_fpmath_mode_any,
    dnnl_fpmath_mode_tf32,
} dnnl_fpmath_mode_t;

typedef enum {
    dnnl_accumulation_mode_strict,
    dnnl_accumulation_mode_relaxed,
    dnnl_accumulation_mode_any,
    dnnl_accumulation_mode_s32,
    dnnl_accumulation_mode_f32,
    dnnl_accumulation_mode_f16
} dnnl_accumulation_mode_t;

typedef enum {
    dnnl_any_engine,
    dnnl_cpu,
    dnnl_gpu,
} dnnl_engine_kind_t;

struct dnnl_engine;
typedef struct dnnl_engine *dnnl_engine_t;

struct dnnl_stream;
typedef struct dnnl_stream *dnnl_stream_t;
typedef const struct dnnl_stream *const_dnnl_stream_t;

typedef enum {
    dnnl_stream_in_order = 0x1U,
    dnnl_stream_out_of_order = 0x2U,
    dnnl_stream_default_flags = dnnl_stream_in_order,
} dnnl_stream_flags_t;

typedef struct {
    int major, minor, patch;
    const char *hash;
    unsigned cpu_runtime, gpu_runtime;
} dnnl_version_t;

#define DNNL_MEMORY_NONE (NULL)
#define DNNL_MEMORY_ALLOCATE ((void *)(size_t)-1)

#ifdef __cplusplus
}
#endif
#endif
