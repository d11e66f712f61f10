/*
 * Scaled dot-product attention, the reference's internal primitive: not part
 * of its public headers, but exported by its library and declared by its
 * tests (tests/gtests/internals/sdpa_internal.hpp:36-44, defined in
 * src/common/sdpa_test_iface.cpp:27-44). Same name, arguments and execute
 * argument ids (src/common/sdpa_types.hpp:32-35) here.
 *
 *   dst = softmax(scale * Q x K + mask) x V
 *
 * query [.., Q, D], key [.., D, S], value [.., S, D], dst [.., Q, D];
 * mask_desc may be NULL; scale_dt is dnnl_data_type_undef when no scale tensor
 * is passed; invert_scale divides by the scale; kv_head_number is the number
 * of key / value heads (grouped-query attention); causal_mask masks key index
 * > query index. kq_attr / vs_attr carry the scales and zero points of a
 * quantized key / value cache (DNNL_ARG_WEIGHTS entries).
 *
 * Execute arguments: DNNL_ARG_QUERIES, DNNL_ARG_KEYS, DNNL_ARG_VALUES,
 * DNNL_ARG_DST, DNNL_ARG_SCALE, DNNL_ARG_ATTN_MASK and
 * DNNL_ARG_ATTR_SCALES / DNNL_ARG_ATTR_ZERO_POINTS | DNNL_ARG_KEYS / _VALUES.
 */
#ifndef SDPA_INTERNAL_H
#define SDPA_INTERNAL_H

#include <stdbool.h>

#include "oneapi/dnnl/dnnl.h"

#define DNNL_ARG_QUERIES DNNL_ARG_SRC_0
#define DNNL_ARG_KEYS DNNL_ARG_SRC_1
#define DNNL_ARG_VALUES DNNL_ARG_SRC_2
#define DNNL_ARG_ATTN_MASK DNNL_ARG_SHIFT

/* src/common/c_types_map.hpp:1981-1983 */
#define DNNL_PRIMITIVE_KIND_SDPA ((dnnl_primitive_kind_t)((1 << 12) + 1))

#ifdef __cplusplus
extern "C" {
#endif

dnnl_status_t DNNL_API sdpa_primitive_desc_create(
        dnnl_primitive_desc_t *primitive_desc_iface, dnnl_engine_t engine,
        const_dnnl_memory_desc_t query_desc, const_dnnl_memory_desc_t key_desc,
        const_dnnl_memory_desc_t value_desc, const_dnnl_memory_desc_t dst_desc,
        const_dnnl_memory_desc_t mask_desc, dnnl_data_type_t scale_dt,
        bool invert_scale, dnnl_dim_t kv_head_number, bool causal_mask,
        const_dnnl_primitive_attr_t attr, const_dnnl_primitive_attr_t kq_attr,
        const_dnnl_primitive_attr_t vs_attr);

#ifdef __cplusplus
}
#endif
#endif
