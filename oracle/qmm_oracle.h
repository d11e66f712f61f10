/*
 * CPU oracle for the quantized matmul path -- TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C restatement of the reference library's scalar matmul, reorder and
 * type-conversion semantics. Nothing in the shipped library links, loads or
 * calls this code: only the test-suite, the smoke check and the benchmark's
 * CPU-baseline leg do, and only as the checker.
 *
 * Enum values are the reference's public ones
 * (include/oneapi/dnnl/dnnl_common_types.h:76-115, dnnl_types.h:2048-2171).
 */
#ifndef QMM_ORACLE_H
#define QMM_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    ORC_DT_UNDEF = 0,
    ORC_F16 = 1,
    ORC_BF16 = 2,
    ORC_F32 = 3,
    ORC_S32 = 4,
    ORC_S8 = 5,
    ORC_U8 = 6,
    ORC_F8_E5M2 = 9,
    ORC_F8_E4M3 = 10,
    ORC_S4 = 11,
    ORC_U4 = 12,
    ORC_E8M0 = 13
};

enum { ORC_PO_SUM = 1, ORC_PO_ELTWISE = 2, ORC_PO_BINARY = 3, ORC_PO_PRELU = 4 };

#define ORC_MAX_NDIMS 12
#define ORC_MAX_PO 32

/* A plain strided tensor; strides are in elements (also for 4-bit types). */
typedef struct {
    int32_t dt;
    int32_t ndims;
    int64_t dims[ORC_MAX_NDIMS];
    int64_t strides[ORC_MAX_NDIMS];
    void *ptr;
} orc_tensor_t;

/* A scales or zero-points attribute entry plus its buffer. */
typedef struct {
    int32_t set; /* 0 = default (scale 1 / zero-point 0) */
    int32_t mask;
    int32_t dt;
    int32_t pad_;
    int64_t g0, g1; /* groups over the tensor's last two dims; 0 = none given */
    const void *ptr;
} orc_quant_t;

typedef struct {
    int32_t kind;
    int32_t alg;
    float alpha, beta, scale;
    int32_t zero_point;
    int32_t sum_dt; /* ORC_DT_UNDEF = same as dst */
    int32_t prelu_mask;
    orc_tensor_t src1; /* binary operand / prelu weights pointer in .ptr */
} orc_postop_t;

enum { ORC_Q_SRC = 0, ORC_Q_WEI = 1, ORC_Q_DST = 2 };

/* How the integer path splits K when a scales / zero-points entry carries no
 * explicit groups. LITERAL follows the v3.8 source to the letter (such an
 * entry counts as group size 1, so products are scaled and summed in f32 one
 * k at a time); WHOLE treats it as one group over all of K (s32 accumulation
 * over the whole group, then the f32 epilogue). See mm_ctx_init(). */
enum { ORC_KGROUP_LITERAL = 0, ORC_KGROUP_WHOLE = 1 };

typedef struct {
    orc_tensor_t src, wei, bias, dst; /* bias.ndims == 0 when absent */
    orc_quant_t scales[3];
    orc_quant_t zps[3];
    int32_t apply_to_int; /* fpmath_mode apply_to_int flag */
    int32_t npo;
    orc_postop_t po[ORC_MAX_PO];
    int32_t nthreads; /* 0 = OpenMP default */
    int32_t k_group_mode; /* ORC_KGROUP_* (integer path only) */
} orc_matmul_t;

/* returns 0 on success, nonzero when the combination is outside what the
 * reference's scalar implementations accept */
int orc_matmul(const orc_matmul_t *p);

/* Exact s32 accumulators of the integer path, before any scaling: one value
 * per (batch, m, n) for a single K group. */
int orc_matmul_s32_acc(const orc_matmul_t *p, int32_t *acc);

/* Reference reorder: dst = sat_round(src_scale*(src - src_zp)/dst_scale + dst_zp)
 * over plain strided tensors; scales/zps follow the same mask/group rules. */
typedef struct {
    orc_tensor_t src, dst;
    orc_quant_t src_scale, dst_scale, src_zp, dst_zp;
} orc_reorder_t;
int orc_reorder(const orc_reorder_t *p);

/* Reference softmax forward over one axis of a plain strided tensor
 * (src/cpu/ref_softmax.cpp:40-312); scales are single values. */
typedef struct {
    orc_tensor_t src, dst;
    int32_t axis;
    int32_t log_softmax; /* 0: softmax_accurate, 1: softmax_log */
    orc_quant_t src_scale, dst_scale;
} orc_softmax_t;
int orc_softmax(const orc_softmax_t *p);

/* scalar conversions */
uint16_t orc_f32_to_bf16(float f);
float orc_bf16_to_f32(uint16_t r);
uint16_t orc_f32_to_f16(float f);
float orc_f16_to_f32(uint16_t r);
uint8_t orc_f16_to_e4m3(uint16_t h);
uint8_t orc_f32_to_e4m3(float f);
uint16_t orc_e4m3_to_f16(uint8_t r);
float orc_e4m3_to_f32(uint8_t r);
uint8_t orc_f16_to_e5m2(uint16_t h);
uint8_t orc_f32_to_e5m2(float f);
float orc_e5m2_to_f32(uint8_t r);
int orc_load_int(int dt, const void *ptr, int64_t idx);
float orc_load_float(int dt, const void *ptr, int64_t idx);
void orc_store_float(int dt, float v, void *ptr, int64_t idx);
float orc_eltwise(int alg, float s, float alpha, float beta);
float orc_binary(int alg, float x, float y);

/* array helpers for the python side */
void orc_cvt_from_f32(int dt, const float *in, void *out, int64_t n);
void orc_cvt_to_f32(int dt, const void *in, float *out, int64_t n);

#ifdef __cplusplus
}
#endif
#endif
