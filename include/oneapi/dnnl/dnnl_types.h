/* C types of the dnnl API subset served by the MI355X quantized-matmul library:
 * memory descriptors, attributes, post-ops, the matmul and reorder primitives.
 * Enumerator names and values follow the reference's
 * include/oneapi/dnnl/dnnl_types.h (format kinds :45-58, format tags :165-230
 * and aliases :1056-1180, primitive kinds :1995-2044, algorithm kinds
 * :2046-2200, scratchpad/rounding modes :2396-2416, DNNL_RUNTIME_* :2279-2304,
 * DNNL_ARG_* :2476-2700, dnnl_exec_arg_t :2704-2707, queries :2712-2790).
 * Only plain (strided) format tags are named here; the blocked tags of the
 * reference describe CPU/Xe register layouts that this backend does not use -
 * prepacked weights are described by an opaque descriptor obtained through
 * format_tag any. */
#ifndef ONEAPI_DNNL_DNNL_TYPES_H
#define ONEAPI_DNNL_DNNL_TYPES_H

#include <stddef.h>
#include <stdint.h>

#include "oneapi/dnnl/dnnl_common_types.h"
#include "oneapi/dnnl/dnnl_config.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    dnnl_format_kind_undef = 0,
    dnnl_format_kind_any,
    dnnl_blocked,
    dnnl_format_kind_opaque,
    dnnl_format_kind_max = 0x7fff,
} dnnl_format_kind_t;

typedef enum {
    dnnl_format_tag_undef = 0,
    dnnl_format_tag_any = 1,
    dnnl_a = 2,
    dnnl_ab = 3,
    dnnl_abc = 4,
    dnnl_abcd = 5,
    dnnl_abcde = 6,
    dnnl_abcdef = 7,
    dnnl_abcdefg = 8,
    dnnl_abcdefgh = 9,
    dnnl_abcdefghi = 10,
    dnnl_abcdefghij = 11,
    dnnl_abcdefghijk = 12,
    dnnl_abcdefghijkl = 13,
    dnnl_ba = 14,
    dnnl_acb = 15,
    dnnl_bac = 16,
    dnnl_bca = 17,
    dnnl_cab = 18,
    dnnl_cba = 19,
    dnnl_abdc = 20,
    dnnl_acbd = 21,
    dnnl_acdb = 22,
    dnnl_adbc = 23,
    dnnl_adcb = 24,
    dnnl_bacd = 25,
    dnnl_bcda = 26,
    dnnl_cdab = 27,
    dnnl_cdba = 28,
    dnnl_dcab = 29,
    dnnl_abced = 30,
    dnnl_abdec = 31,
    dnnl_acbde = 32,
    dnnl_acdeb = 33,
    dnnl_adecb = 34,
    dnnl_bacde = 35,
    dnnl_bcdea = 36,
    dnnl_cdeab = 37,
    dnnl_cdeba = 38,
    dnnl_decab = 39,
    dnnl_abcdfe = 40,
    dnnl_abdefc = 41,
    dnnl_abdfce = 42,
    dnnl_acbdef = 43,
    dnnl_adefcb = 44,
    dnnl_defcab = 45,
    dnnl_abcdegf = 46,
    dnnl_abcdefhg = 47,
    dnnl_abcdefgih = 48,
    dnnl_abcdefghji = 49,
    dnnl_abcdefghikj = 50,
    dnnl_abcdefghijlk = 51,
    /* one past the last tag of oneDNN v3.8's full list (its blocked tags are not
     * part of this subset): the same value as there */
    dnnl_format_tag_last = 847,
    dnnl_x = dnnl_a,
    dnnl_nc = dnnl_ab,
    dnnl_cn = dnnl_ba,
    dnnl_tn = dnnl_ab,
    dnnl_nt = dnnl_ba,
    dnnl_ncw = dnnl_abc,
    dnnl_nwc = dnnl_acb,
    dnnl_nchw = dnnl_abcd,
    dnnl_nhwc = dnnl_acdb,
    dnnl_chwn = dnnl_bcda,
    dnnl_ncdhw = dnnl_abcde,
    dnnl_ndhwc = dnnl_acdeb,
    dnnl_oi = dnnl_ab,
    dnnl_io = dnnl_ba,
    dnnl_tnc = dnnl_abc,
    dnnl_ntc = dnnl_bac,
} dnnl_format_tag_t;

typedef enum {
    dnnl_prop_kind_undef = 0,
    dnnl_forward_training = 64,
    dnnl_forward_inference = 96,
    dnnl_forward = dnnl_forward_training,
} dnnl_prop_kind_t;

typedef enum {
    dnnl_undefined_primitive,
    dnnl_reorder,
    dnnl_shuffle,
    dnnl_concat,
    dnnl_sum,
    dnnl_convolution,
    dnnl_deconvolution,
    dnnl_eltwise,
    dnnl_lrn,
    dnnl_batch_normalization,
    dnnl_inner_product,
    dnnl_rnn,
    dnnl_gemm,
    dnnl_binary,
    dnnl_matmul,
    dnnl_resampling,
    dnnl_pooling,
    dnnl_reduction,
    dnnl_prelu,
    dnnl_softmax,
    dnnl_layer_normalization,
    dnnl_group_normalization,
    dnnl_primitive_kind_max = 0x7fff,
} dnnl_primitive_kind_t;

typedef enum {
    dnnl_alg_kind_undef = 0,
    dnnl_eltwise_relu = 0x20,
    dnnl_eltwise_tanh = 0x21,
    dnnl_eltwise_elu = 0x22,
    dnnl_eltwise_square = 0x23,
    dnnl_eltwise_abs = 0x24,
    dnnl_eltwise_sqrt = 0x25,
    dnnl_eltwise_linear = 0x26,
    dnnl_eltwise_soft_relu = 0x27,
    dnnl_eltwise_hardsigmoid = 0x28,
    dnnl_eltwise_logistic = 0x29,
    dnnl_eltwise_exp = 0x2a,
    dnnl_eltwise_gelu_tanh = 0x2b,
    dnnl_eltwise_swish = 0x2c,
    dnnl_eltwise_log = 0x2d,
    dnnl_eltwise_clip = 0x2e,
    dnnl_eltwise_clip_v2 = 0x2f,
    dnnl_eltwise_pow = 0x30,
    dnnl_eltwise_gelu_erf = 0x31,
    dnnl_eltwise_round = 0x32,
    dnnl_eltwise_mish = 0x33,
    dnnl_eltwise_hardswish = 0x34,
    dnnl_eltwise_relu_use_dst_for_bwd = 0x100,
    dnnl_eltwise_tanh_use_dst_for_bwd = 0x101,
    dnnl_eltwise_elu_use_dst_for_bwd = 0x102,
    dnnl_eltwise_sqrt_use_dst_for_bwd = 0x103,
    dnnl_eltwise_logistic_use_dst_for_bwd = 0x104,
    dnnl_eltwise_exp_use_dst_for_bwd = 0x105,
    dnnl_eltwise_clip_v2_use_dst_for_bwd = 0x106,
    dnnl_binary_add = 0x1fff0,
    dnnl_binary_mul = 0x1fff1,
    dnnl_binary_max = 0x1fff2,
    dnnl_binary_min = 0x1fff3,
    dnnl_binary_div = 0x1fff4,
    dnnl_binary_sub = 0x1fff5,
    dnnl_binary_ge = 0x1fff6,
    dnnl_binary_gt = 0x1fff7,
    dnnl_binary_le = 0x1fff8,
    dnnl_binary_lt = 0x1fff9,
    dnnl_binary_eq = 0x1fffa,
    dnnl_binary_ne = 0x1fffb,
    dnnl_binary_select = 0x1fffc,
    dnnl_softmax_accurate = 0x30000,
    dnnl_softmax_log,
} dnnl_alg_kind_t;

typedef enum {
    dnnl_scratchpad_mode_library,
    dnnl_scratchpad_mode_user,
} dnnl_scratchpad_mode_t;

typedef enum {
    dnnl_rounding_mode_environment,
    dnnl_rounding_mode_stochastic,
} dnnl_rounding_mode_t;

struct dnnl_memory_desc;
typedef struct dnnl_memory_desc *dnnl_memory_desc_t;
typedef const struct dnnl_memory_desc *const_dnnl_memory_desc_t;
struct dnnl_memory;
typedef struct dnnl_memory *dnnl_memory_t;
typedef const struct dnnl_memory *const_dnnl_memory_t;
struct dnnl_primitive_desc;
typedef struct dnnl_primitive_desc *dnnl_primitive_desc_t;
typedef const struct dnnl_primitive_desc *const_dnnl_primitive_desc_t;
struct dnnl_primitive_attr;
typedef struct dnnl_primitive_attr *dnnl_primitive_attr_t;
typedef const struct dnnl_primitive_attr *const_dnnl_primitive_attr_t;
struct dnnl_post_ops;
typedef struct dnnl_post_ops *dnnl_post_ops_t;
typedef const struct dnnl_post_ops *const_dnnl_post_ops_t;
struct dnnl_primitive;
typedef struct dnnl_primitive *dnnl_primitive_t;
typedef const struct dnnl_primitive *const_dnnl_primitive_t;

#define DNNL_RUNTIME_DIM_VAL INT64_MIN
#define DNNL_RUNTIME_SIZE_VAL ((size_t)DNNL_RUNTIME_DIM_VAL)
static const union {
    unsigned u;
    float f;
} DNNL_RUNTIME_F32_VAL_REP = {0x7fc000d0};
#define DNNL_RUNTIME_F32_VAL (DNNL_RUNTIME_F32_VAL_REP.f)
static const int DNNL_RUNTIME_S32_VAL_REP = INT32_MIN;
#define DNNL_RUNTIME_S32_VAL DNNL_RUNTIME_S32_VAL_REP

#define DNNL_ARG_UNDEF 0
#define DNNL_ARG_SRC_0 1
#define DNNL_ARG_SRC DNNL_ARG_SRC_0
#define DNNL_ARG_FROM DNNL_ARG_SRC_0
#define DNNL_ARG_SRC_1 2
#define DNNL_ARG_SRC_2 3
#define DNNL_ARG_SCALE 51
#define DNNL_ARG_SHIFT 52
#define DNNL_ARG_DST_0 17
#define DNNL_ARG_DST DNNL_ARG_DST_0
#define DNNL_ARG_TO DNNL_ARG_DST_0
#define DNNL_ARG_WEIGHTS_0 33
#define DNNL_ARG_WEIGHTS DNNL_ARG_WEIGHTS_0
#define DNNL_ARG_BIAS 41
#define DNNL_ARG_SCRATCHPAD 80
#define DNNL_ARG_DIFF_SRC_0 129
#define DNNL_ARG_DIFF_SRC DNNL_ARG_DIFF_SRC_0
#define DNNL_ARG_DIFF_WEIGHTS_0 161
#define DNNL_ARG_DIFF_WEIGHTS DNNL_ARG_DIFF_WEIGHTS_0
#define DNNL_ARG_ATTR_ROUNDING_SEED 508
#define DNNL_ARG_ATTR_DROPOUT_MASK 509
#define DNNL_ARG_ATTR_DROPOUT_PROBABILITY 510
#define DNNL_ARG_ATTR_DROPOUT_SEED 511
#define DNNL_ARG_ATTR_SCALES 4096
#define DNNL_ARG_ATTR_ZERO_POINTS 8192
#define DNNL_ARG_ATTR_MULTIPLE_POST_OP_BASE 32768
#define DNNL_ARG_ATTR_MULTIPLE_POST_OP(idx) \
    (DNNL_ARG_ATTR_MULTIPLE_POST_OP_BASE * ((idx) + 1))

typedef struct {
    int arg;
    dnnl_memory_t memory;
} dnnl_exec_arg_t;

typedef enum {
    dnnl_query_undef = 0,
    dnnl_query_engine,
    dnnl_query_primitive_kind,
    dnnl_query_num_of_inputs_s32,
    dnnl_query_num_of_outputs_s32,
    dnnl_query_time_estimate_f64,
    dnnl_query_memory_consumption_s64,
    dnnl_query_scratchpad_engine,
    dnnl_query_impl_info_str,
    dnnl_query_reorder_src_engine,
    dnnl_query_reorder_dst_engine,
    dnnl_query_prop_kind,
    dnnl_query_cache_blob_id_size_s64,
    dnnl_query_cache_blob_id,
    dnnl_query_strides,
    dnnl_query_dilations,
    dnnl_query_padding_l,
    dnnl_query_padding_r,
    dnnl_query_epsilon_f32,
    dnnl_query_flags,
    dnnl_query_alg_kind,
    dnnl_query_alpha_f32,
    dnnl_query_beta_f32,
    dnnl_query_axis_s32,
    dnnl_query_local_size_s64,
    dnnl_query_k_f32,
    dnnl_query_p_f32,
    dnnl_query_factors,
    dnnl_query_cell_kind,
    dnnl_query_direction,
    dnnl_query_activation_kind,
    dnnl_query_kernel,
    dnnl_query_group_size_s64,
    dnnl_query_some_md = 128,
    dnnl_query_src_md,
    dnnl_query_diff_src_md,
    dnnl_query_weights_md,
    dnnl_query_diff_weights_md,
    dnnl_query_dst_md,
    dnnl_query_diff_dst_md,
    dnnl_query_workspace_md,
    dnnl_query_scratchpad_md,
    dnnl_query_exec_arg_md = 255,
    dnnl_query_ndims_s32,
    dnnl_query_dims,
    dnnl_query_data_type,
    dnnl_query_submemory_offset_s64,
    dnnl_query_padded_dims,
    dnnl_query_padded_offsets,
    dnnl_query_format_kind,
    dnnl_query_inner_nblks_s32,
    dnnl_query_inner_blks,
    dnnl_query_inner_idxs,
    dnnl_query_max = 0x7fff,
} dnnl_query_t;

#ifdef __cplusplus
}
#endif
#endif
