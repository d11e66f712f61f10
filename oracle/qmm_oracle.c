/*
 * CPU oracle for the quantized matmul path -- TEST INFRASTRUCTURE ONLY.
 * See qmm_oracle.h. Build: gcc -O2 -ffp-contract=off -fopenmp -shared -fPIC.
 *
 * Every float operation below is meant to be a separately rounded IEEE
 * binary32 operation (no FMA contraction), as in the reference's scalar C++
 * which is built for an ISA baseline without FMA.
 *
 * Each function cites the reference file:line it restates (paths relative to
 * the reference tree).
 */
#include "qmm_oracle.h"

#include <float.h>
#include <limits.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------------ */
/* bit casts                                                                 */
static inline uint32_t f2u(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
static inline float u2f(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* ------------------------------------------------------------------------ */
/* bf16: src/common/bfloat16.cpp:22-56                                        */
uint16_t orc_f32_to_bf16(float f) {
    uint32_t u = f2u(f);
    uint16_t hi = (uint16_t)(u >> 16);
    switch (fpclassify(f)) {
        case FP_SUBNORMAL:
        case FP_ZERO: return hi & 0x8000; /* denormals flush to signed zero */
        case FP_INFINITE: return hi;
        case FP_NAN: return hi | (1 << 6); /* force quiet */
        default: {
            uint32_t bias = 0x7FFFu + (hi & 1u); /* round to nearest even */
            return (uint16_t)((u + bias) >> 16);
        }
    }
}
float orc_bf16_to_f32(uint16_t r) {
    return u2f((uint32_t)r << 16);
}

/* ------------------------------------------------------------------------ */
/* f16: src/common/float16.hpp:52-127                                         */
uint16_t orc_f32_to_f16(float f) {
    uint32_t i = f2u(f);
    uint32_t s = i >> 31, e = (i >> 23) & 0xFF, m = i & 0x7FFFFF;
    uint32_t mm = m >> 13, r = m & 0x1FFF, ee = 0;
    int32_t eee = (int32_t)e - 127 + 15;
    if (e == 0) {
        ee = 0;
        mm = 0;
    } else if (e == 0xFF) {
        ee = 0x1F;
        if (m != 0) mm |= 0x200;
    } else if (eee > 0 && eee < 0x1F) {
        ee = (uint32_t)eee;
        if (r > (0x1000 - (mm & 1))) {
            mm++;
            if (mm == 0x400) {
                mm = 0;
                ee++;
            }
        }
    } else if (eee >= 0x1F) {
        ee = 0x1F;
        mm = 0;
    } else {
        /* underflow: adding 0.5 lets the f32 adder do the rounding */
        float ff = fabsf(f) + 0.5f;
        ee = 0;
        mm = f2u(ff) & 0x7FF;
    }
    return (uint16_t)((s << 15) | (ee << 10) | mm);
}
float orc_f16_to_f32(uint16_t raw) {
    uint32_t ss = raw >> 15, ee = (raw >> 10) & 0x1F, mm = raw & 0x3FF;
    uint32_t m = mm << 13, e;
    if (ee == 0) {
        if (mm == 0)
            e = 0;
        else
            return (ss ? -1.f : 1.f) * scalbnf((float)mm, -24);
    } else if (ee == 0x1F) {
        e = 0xFF;
        if (m != 0) m |= 0x400000;
    } else
        e = ee - 15 + 127;
    return u2f((ss << 31) | (e << 23) | m);
}

/* ------------------------------------------------------------------------ */
/* f8_e4m3 (OCP: no inf, NaN = s.1111.111): src/common/float8.cpp:93-190      */
uint8_t orc_f16_to_e4m3(uint16_t h) {
    int fraw = h;
    unsigned s8 = (fraw & 0x8000) >> 8;
    fraw &= 0x7fff;
    if (fraw > 0x5f40) return (uint8_t)(s8 | 0x7f); /* > 464, inf, nan */
    if (fraw <= 0x1400) return (uint8_t)s8; /* <= 2^-10 */
    uint16_t shifter = (uint16_t)((fraw & 0x7c00) + 0x1c00);
    int is_denorm = shifter < 0x4000;
    if (is_denorm) shifter = 0x4000;
    /* two separately rounded f16 operations */
    uint16_t rounded = orc_f32_to_f16(
            orc_f16_to_f32((uint16_t)fraw) + orc_f16_to_f32(shifter));
    rounded = orc_f32_to_f16(orc_f16_to_f32(rounded) - orc_f16_to_f32(shifter));
    int e8 = ((rounded & 0x7c00) >> 10) - 8;
    uint8_t m8 = (uint8_t)((rounded & 0x03ff) >> 7);
    if (is_denorm) {
        m8 = (uint8_t)((m8 | 0x8) >> (-e8 + 1));
        e8 = 0;
    }
    return (uint8_t)(s8 | (e8 << 3) | m8);
}
uint8_t orc_f32_to_e4m3(float f) {
    return orc_f16_to_e4m3(orc_f32_to_f16(f));
}
uint16_t orc_e4m3_to_f16(uint8_t r) {
    uint16_t s8 = (r & 0x80) >> 7, e8 = (r & 0x78) >> 3, m8 = r & 0x7;
    uint16_t e16 = e8 + 8, m16 = m8;
    if (e8 == 0 && m8 != 0) {
        uint16_t count = 2;
        count = m8 > 0x1 ? 1 : count;
        count = m8 > 0x3 ? 0 : count;
        e16 -= count;
        m16 = (m16 << (count + 1)) & 0x7;
    } else if (e8 == 0 && m8 == 0) {
        e16 = 0;
    } else if (e8 == 0xf && m8 == 0x7) {
        e16 = 0x1f;
        m16 = 0x4;
    }
    return (uint16_t)((s8 << 15) | (e16 << 10) | (m16 << 7));
}
float orc_e4m3_to_f32(uint8_t r) {
    return orc_f16_to_f32(orc_e4m3_to_f16(r));
}

/* f8_e5m2: src/common/float8.cpp:43-91                                       */
uint8_t orc_f16_to_e5m2(uint16_t fraw) {
    int is_special = (fraw & 0x7c00) == 0x7c00;
    int is_nan = is_special && (fraw & 0x03ff);
    if (is_nan) return (uint8_t)((fraw >> 8) | 0x02);
    if (is_special) return (uint8_t)(fraw >> 8);
    int16_t nudge = 0x007f + ((fraw & 0x0100) >> 8);
    fraw = (uint16_t)(fraw + nudge);
    return (uint8_t)(fraw >> 8);
}
uint8_t orc_f32_to_e5m2(float f) {
    return orc_f16_to_e5m2(orc_f32_to_f16(f));
}
float orc_e5m2_to_f32(uint8_t r) {
    uint8_t raw = ((r & 0x7d) == 0x7d) ? (r | 0x02) : r;
    return orc_f16_to_f32((uint16_t)(raw << 8));
}

/* e8m0: src/common/float8.cpp:28-41                                          */
static float e8m0_to_f32(uint8_t r) {
    if (r == 0xff) return u2f(0xffc00000u);
    return u2f((uint32_t)r << 23);
}

/* ------------------------------------------------------------------------ */
/* typed element access: src/cpu/ref_io_helper.hpp:33-154,                    */
/* 4-bit packing src/common/utils.hpp:835-867, src/common/int4.hpp:28-70      */
static inline int nibble(const void *ptr, int64_t idx) {
    uint8_t b = ((const uint8_t *)ptr)[idx / 2];
    return (idx % 2) ? (b >> 4) & 0xf : b & 0xf; /* even index = low nibble */
}
static inline int s4_value(int nib) {
    return (nib & 0x8) ? -((~nib & 0xf) + 1) : nib;
}

int orc_load_int(int dt, const void *ptr, int64_t idx) {
    switch (dt) {
        case ORC_S32: return ((const int32_t *)ptr)[idx];
        case ORC_S8: return ((const int8_t *)ptr)[idx];
        case ORC_U8: return ((const uint8_t *)ptr)[idx];
        case ORC_S4: return s4_value(nibble(ptr, idx));
        case ORC_U4: return nibble(ptr, idx);
        default: return INT_MAX;
    }
}

float orc_load_float(int dt, const void *ptr, int64_t idx) {
    switch (dt) {
        case ORC_F8_E5M2: return orc_e5m2_to_f32(((const uint8_t *)ptr)[idx]);
        case ORC_F8_E4M3: return orc_e4m3_to_f32(((const uint8_t *)ptr)[idx]);
        case ORC_BF16: return orc_bf16_to_f32(((const uint16_t *)ptr)[idx]);
        case ORC_F16: return orc_f16_to_f32(((const uint16_t *)ptr)[idx]);
        case ORC_F32: return ((const float *)ptr)[idx];
        case ORC_S32: return (float)((const int32_t *)ptr)[idx];
        case ORC_S8: return (float)((const int8_t *)ptr)[idx];
        case ORC_U8: return (float)((const uint8_t *)ptr)[idx];
        case ORC_E8M0: return e8m0_to_f32(((const uint8_t *)ptr)[idx]);
        case ORC_S4: return (float)s4_value(nibble(ptr, idx));
        case ORC_U4: return (float)nibble(ptr, idx);
        default: return NAN;
    }
}

/* saturate + round: src/cpu/simple_q10n.hpp:33-81,
 * s32 upper bound src/common/type_helpers.hpp:219-229.
 * Rounding is nearbyintf under the default mode (ties to even); a NaN passes
 * the clamps and converts like the x86 cvtss2si "integer indefinite". */
static inline int round_sat(float v, float lo, float hi) {
    if (v < lo) v = lo;
    if (v > hi) v = hi;
    if (isnan(v)) return INT_MIN;
    return (int)nearbyintf(v);
}

void orc_store_float(int dt, float v, void *ptr, int64_t idx) {
    switch (dt) {
        case ORC_F8_E5M2: ((uint8_t *)ptr)[idx] = orc_f32_to_e5m2(v); break;
        case ORC_F8_E4M3: ((uint8_t *)ptr)[idx] = orc_f32_to_e4m3(v); break;
        case ORC_BF16: ((uint16_t *)ptr)[idx] = orc_f32_to_bf16(v); break;
        case ORC_F16: ((uint16_t *)ptr)[idx] = orc_f32_to_f16(v); break;
        case ORC_F32: ((float *)ptr)[idx] = v; break;
        case ORC_S32:
            ((int32_t *)ptr)[idx] = round_sat(v, -2147483648.f, 2147483520.f);
            break;
        case ORC_S8:
            ((int8_t *)ptr)[idx] = (int8_t)round_sat(v, -128.f, 127.f);
            break;
        case ORC_U8:
            ((uint8_t *)ptr)[idx] = (uint8_t)round_sat(v, 0.f, 255.f);
            break;
        default: break;
    }
}

void orc_cvt_from_f32(int dt, const float *in, void *out, int64_t n) {
    for (int64_t i = 0; i < n; i++)
        orc_store_float(dt, in[i], out, i);
}
void orc_cvt_to_f32(int dt, const void *in, float *out, int64_t n) {
    for (int64_t i = 0; i < n; i++)
        out[i] = orc_load_float(dt, in, i);
}

/* ------------------------------------------------------------------------ */
/* eltwise forward formulas: src/common/math_utils.hpp:129-416                */
enum {
    ALG_RELU = 0x20,
    ALG_TANH,
    ALG_ELU,
    ALG_SQUARE,
    ALG_ABS,
    ALG_SQRT,
    ALG_LINEAR,
    ALG_SOFT_RELU,
    ALG_HARDSIGMOID,
    ALG_LOGISTIC,
    ALG_EXP,
    ALG_GELU_TANH,
    ALG_SWISH,
    ALG_LOG,
    ALG_CLIP,
    ALG_CLIP_V2,
    ALG_POW,
    ALG_GELU_ERF,
    ALG_ROUND,
    ALG_MISH,
    ALG_HARDSWISH,
    ALG_RELU_DST = 0x100,
    ALG_TANH_DST,
    ALG_ELU_DST,
    ALG_SQRT_DST,
    ALG_LOGISTIC_DST,
    ALG_EXP_DST,
    ALG_CLIP_V2_DST,
    ALG_BIN_ADD = 0x1fff0,
    ALG_BIN_MUL,
    ALG_BIN_MAX,
    ALG_BIN_MIN,
    ALG_BIN_DIV,
    ALG_BIN_SUB,
    ALG_BIN_GE,
    ALG_BIN_GT,
    ALG_BIN_LE,
    ALG_BIN_LT,
    ALG_BIN_EQ,
    ALG_BIN_NE
};

static float logistic_f(float s) { /* :239-245 */
    const float bound = 88.72283172607421875f;
    float in = -s;
    return in < bound ? 1.f / (1.f + expf(in)) : 0.f;
}
static float soft_relu_f(float s, float alpha) { /* :257-262 */
    const float bound = 88.72283172607421875f;
    float in = s * alpha;
    float v = in < bound ? log1pf(expf(in)) : in;
    return v / alpha;
}
static float hardsigmoid_f(float s, float alpha, float beta) { /* :393-397 */
    float v = alpha * s + beta;
    return v <= 0.f ? 0.f : v >= 1.f ? 1.f : v;
}

float orc_eltwise(int alg, float s, float alpha, float beta) {
    switch (alg) {
        case ALG_RELU:
        case ALG_RELU_DST: return s > 0 ? s : s * alpha;
        case ALG_TANH:
        case ALG_TANH_DST: return tanhf(s);
        case ALG_ELU:
        case ALG_ELU_DST: return s > 0 ? s : alpha * expm1f(s);
        case ALG_SQUARE: return s * s;
        case ALG_ABS: return s > 0 ? s : -s;
        case ALG_SQRT:
        case ALG_SQRT_DST: return sqrtf(s);
        case ALG_LINEAR: return alpha * s + beta;
        case ALG_SOFT_RELU: return soft_relu_f(s, alpha);
        case ALG_HARDSIGMOID: return hardsigmoid_f(s, alpha, beta);
        case ALG_LOGISTIC:
        case ALG_LOGISTIC_DST: return logistic_f(s);
        case ALG_EXP:
        case ALG_EXP_DST: return expf(s);
        case ALG_GELU_TANH: { /* :309-314; the last step is in double */
            const float sqrt_2_over_pi = 0.79788458347320556640625f;
            const float fitting_const = 0.044715f;
            float v = tanhf(sqrt_2_over_pi * s * (1 + fitting_const * s * s));
            return (float)(0.5 * s * (1. + v));
        }
        case ALG_SWISH: return s * logistic_f(alpha * s);
        case ALG_LOG: return logf(s);
        case ALG_CLIP: {
            s = s > alpha ? s : alpha;
            return s > beta ? beta : s;
        }
        case ALG_CLIP_V2:
        case ALG_CLIP_V2_DST: {
            s = s > alpha ? s : alpha;
            return s < beta ? s : beta;
        }
        case ALG_POW: return alpha * powf(s, beta);
        case ALG_GELU_ERF: {
            const float sqrt_2_over_2 = 0.707106769084930419921875f;
            float v = s * sqrt_2_over_2;
            return 0.5f * s * (1.f + erff(v));
        }
        case ALG_ROUND: return nearbyintf(s);
        case ALG_MISH: return s * tanhf(soft_relu_f(s, 1.f));
        case ALG_HARDSWISH: return s * hardsigmoid_f(s, alpha, beta);
        default: return NAN;
    }
}

/* src/cpu/primitive_attr_postops.cpp:29-46 */
float orc_binary(int alg, float x, float y) {
    switch (alg) {
        case ALG_BIN_ADD: return x + y;
        case ALG_BIN_DIV: return x / y;
        case ALG_BIN_MAX: return x > y ? x : y; /* nstl::max: (a > b) ? a : b */
        case ALG_BIN_MIN: return x < y ? x : y;
        case ALG_BIN_MUL: return x * y;
        case ALG_BIN_SUB: return x - y;
        case ALG_BIN_GE: return x >= y;
        case ALG_BIN_GT: return x > y;
        case ALG_BIN_LE: return x <= y;
        case ALG_BIN_LT: return x < y;
        case ALG_BIN_EQ: return x == y;
        case ALG_BIN_NE: return x != y;
        default: return NAN;
    }
}

/* ------------------------------------------------------------------------ */
/* indexing helpers                                                           */
static int64_t off_v(const orc_tensor_t *t, const int64_t *idx) {
    int64_t o = 0;
    for (int d = 0; d < t->ndims; d++)
        o += idx[d] * t->strides[d];
    return o;
}

/* src/common/utils.hpp:587-599 */
static void l_dims(int64_t *pos, int64_t l, const int64_t *dims, int nd) {
    for (int d = nd - 1; d >= 0; d--) {
        pos[d] = l % dims[d];
        l /= dims[d];
    }
}

/* src/common/utils.hpp:602-611 */
static int dims_mask(const int64_t *d1, const int64_t *d2, int nd) {
    int mask = 0;
    for (int d = 0; d < nd; d++)
        if (d1[d] == d2[d]) mask |= 1 << d;
    return mask;
}

/* A scales / zero-points tensor is a dense row-major tensor whose dims are the
 * masked dims of the quantized tensor with the last two divided by the groups:
 * src/cpu/matmul/matmul_utils.hpp:156-196 */
typedef struct {
    int nd;
    int mask;
    int64_t g0, g1;
    int64_t dims[ORC_MAX_NDIMS];
    int64_t strides[ORC_MAX_NDIMS];
    int64_t nelems;
    int zero; /* default entry: offset is always 0 */
} qmd_t;

static void qmd_init(qmd_t *q, const orc_quant_t *a, int nd,
        const int64_t *tdims, int64_t g0, int64_t g1) {
    memset(q, 0, sizeof(*q));
    if (g0 <= 0) g0 = 1; /* 0 = no explicit group on that dim */
    if (g1 <= 0) g1 = 1;
    q->nd = nd;
    q->mask = a->mask;
    q->g0 = g0;
    q->g1 = g1;
    if (!a->set || a->dt == ORC_DT_UNDEF || a->mask < 0) {
        q->zero = 1;
        q->nelems = 1;
        return;
    }
    for (int d = 0; d < nd; d++)
        q->dims[d] = (a->mask & (1 << d)) ? tdims[d] : 1;
    if (nd >= 2) {
        q->dims[nd - 1] /= g1;
        q->dims[nd - 2] /= g0;
    }
    int64_t s = 1;
    for (int d = nd - 1; d >= 0; d--) {
        q->strides[d] = s;
        s *= q->dims[d];
    }
    q->nelems = s;
}

static int64_t qmd_off(const qmd_t *q, const int64_t *idx) {
    if (q->zero) return 0;
    int64_t qi[ORC_MAX_NDIMS];
    for (int d = 0; d < q->nd; d++)
        qi[d] = (q->mask & (1 << d)) ? idx[d] : 0;
    if (q->nd >= 2) {
        qi[q->nd - 1] /= q->g1;
        qi[q->nd - 2] /= q->g0;
    }
    int64_t o = 0;
    for (int d = 0; d < q->nd; d++)
        o += qi[d] * q->strides[d];
    return o;
}

static int has_zero_dim(const orc_tensor_t *t) {
    for (int d = 0; d < t->ndims; d++)
        if (t->dims[d] == 0) return 1;
    return 0;
}

/* prelu weights layout: src/cpu/primitive_attr_postops.cpp:196-225 */
static void prelu_tensor(orc_tensor_t *w, const orc_tensor_t *dst, int mask) {
    static const int perm[6][5] = {{0}, {0}, {0, 1}, {0, 2, 1}, {0, 2, 3, 1},
            {0, 2, 3, 4, 1}}; /* a, ab, acb, acdb, acdeb: outer -> inner */
    int nd = dst->ndims;
    w->dt = ORC_F32;
    w->ndims = nd;
    for (int d = 0; d < nd; d++)
        w->dims[d] = (mask & (1 << d)) ? dst->dims[d] : 0;
    int64_t s = 1;
    for (int i = nd - 1; i >= 0; i--) {
        int d = nd <= 5 ? perm[nd][i] : i;
        w->strides[d] = s;
        s *= w->dims[d] > 0 ? w->dims[d] : 1;
    }
}

/* ordered post-op chain: src/cpu/primitive_attr_postops.cpp:278-347 */
static float apply_post_ops(const orc_matmul_t *p, float res, float dst_val,
        int64_t l_offset) {
    const orc_tensor_t *dst = &p->dst;
    for (int i = 0; i < p->npo; i++) {
        const orc_postop_t *e = &p->po[i];
        switch (e->kind) {
            case ORC_PO_SUM:
                res += e->scale * (dst_val - (float)e->zero_point);
                break;
            case ORC_PO_ELTWISE:
                res = orc_eltwise(e->alg, res, e->alpha, e->beta) * e->scale;
                break;
            case ORC_PO_BINARY: {
                int64_t pos[ORC_MAX_NDIMS];
                l_dims(pos, l_offset, dst->dims, dst->ndims);
                int mask = dims_mask(dst->dims, e->src1.dims, dst->ndims);
                for (int d = 0; d < dst->ndims; d++)
                    if (!(mask & (1 << d))) pos[d] = 0;
                float y = orc_load_float(
                        e->src1.dt, e->src1.ptr, off_v(&e->src1, pos));
                res = orc_binary(e->alg, res, y);
                break;
            }
            case ORC_PO_PRELU: {
                if (res >= 0) break;
                orc_tensor_t w;
                prelu_tensor(&w, dst, e->prelu_mask);
                int64_t pos[ORC_MAX_NDIMS];
                l_dims(pos, l_offset, dst->dims, dst->ndims);
                for (int d = 0; d < dst->ndims; d++)
                    if (!(e->prelu_mask & (1 << d))) pos[d] = 0;
                res = ((const float *)e->src1.ptr)[off_v(&w, pos)] * res;
                break;
            }
            default: break;
        }
    }
    return res;
}

static int attr_is_default(const orc_matmul_t *p) {
    for (int i = 0; i < 3; i++)
        if (p->scales[i].set || p->zps[i].set) return 0;
    /* a non-default fpmath mode also makes the attribute non-default, but it
     * changes nothing below unless post-ops / scales are present */
    return p->npo == 0;
}

static int sum_dt_of(const orc_matmul_t *p) {
    for (int i = 0; i < p->npo; i++)
        if (p->po[i].kind == ORC_PO_SUM)
            return p->po[i].sum_dt != ORC_DT_UNDEF ? p->po[i].sum_dt
                                                   : p->dst.dt;
    return p->dst.dt;
}

/* A single-element scale is pre-converted to f32 (and inverted for dst); a
 * multi-element buffer is read element-wise in its own type:
 * src/cpu/cpu_primitive.hpp:32-62 */
/* Destination scales. One value: multiply by its reciprocal
 * (src/cpu/matmul/ref_matmul.cpp:208-209, ref_matmul_int8.cpp:237-238). A mask
 * over M and / or N is accepted for GPU engines only
 * (src/common/matmul.cpp:150-154); the reference's GPU implementation of it
 * divides by the element's entry (src/gpu/intel/ocl/ref_matmul.cl:239-245,
 * mask N); the buffer is dense row-major over the masked dims. */
static float apply_dst_scale(const orc_quant_t *ds, float inv0, float d,
        int64_t m, int64_t n, int64_t N, int nd) {
    if (!ds->set) return d;
    if (ds->mask == 0) return d * inv0;
    const int per_m = (ds->mask >> (nd - 2)) & 1, per_n = (ds->mask >> (nd - 1)) & 1;
    const int64_t i = (per_m ? m * (per_n ? N : 1) : 0) + (per_n ? n : 0);
    return d / orc_load_float(ds->dt, ds->ptr, i);
}

static float single_scale(const orc_quant_t *a, int invert) {
    if (!a->set) return 1.f;
    float s = orc_load_float(a->dt, a->ptr, 0);
    return invert ? 1.f / s : s;
}

/* ------------------------------------------------------------------------ */
typedef struct {
    int nd;
    int64_t M, N, K, batch;
    int src_mask, wei_mask, bia_mask;
    qmd_t q_src_scale, q_wei_scale, q_src_zp, q_wei_zp;
    int64_t ngroups_k, group_k;
} mm_ctx_t;

static void mm_ctx_init(mm_ctx_t *c, const orc_matmul_t *p) {
    int nd = p->dst.ndims;
    c->nd = nd;
    c->M = p->dst.dims[nd - 2];
    c->N = p->dst.dims[nd - 1];
    c->K = p->src.dims[nd - 1];
    c->batch = 1;
    for (int d = 0; d < nd - 2; d++)
        c->batch *= p->dst.dims[d];
    c->src_mask = dims_mask(p->dst.dims, p->src.dims, nd);
    c->wei_mask = dims_mask(p->dst.dims, p->wei.dims, nd);
    c->bia_mask = p->bias.ndims ? dims_mask(p->dst.dims, p->bias.dims, nd) : 0;
    const orc_quant_t *ss = &p->scales[ORC_Q_SRC], *ws = &p->scales[ORC_Q_WEI];
    const orc_quant_t *sz = &p->zps[ORC_Q_SRC], *wz = &p->zps[ORC_Q_WEI];
    /* src entries: group over M is 1, group over K is the second group dim */
    qmd_init(&c->q_src_scale, ss, nd, p->src.dims, 1, ss->g1);
    qmd_init(&c->q_src_zp, sz, nd, p->src.dims, 1, sz->g1);
    qmd_init(&c->q_wei_scale, ws, nd, p->wei.dims, ws->g0, ws->g1);
    qmd_init(&c->q_wei_zp, wz, nd, p->wei.dims, wz->g0, wz->g1);
    /* The kernel's K group is the smallest one over the four entries:
     * src/cpu/matmul/ref_matmul_int8.cpp:139-144. An entry WITHOUT explicit
     * groups reports a group of 1 (quant_entry_t::get_group,
     * src/common/primitive_attr_quant.hpp:83-90), so as written the v3.8
     * reference ends every "group" after a single k and sums the scaled
     * products in f32 (k_group_mode == ORC_KGROUP_LITERAL). With
     * ORC_KGROUP_WHOLE an entry without groups spans all of K, which is the
     * integer accumulation every other implementation of the reference
     * performs (gemm_x8s8s32x_matmul.cpp:165-193, brgemm). */
    int64_t K = c->K, ng = 1, t;
    if (K > 0) {
        const int whole = p->k_group_mode == ORC_KGROUP_WHOLE;
        const int src_kbit = 1 << (nd - 1), wei_kbit = 1 << (nd - 2);
        /* WHOLE: an entry without groups still varies per k when its mask
         * covers the K dim (one value per k: group of 1) */
#define KGROUP(q, g, kbit) \
    ((q)->set && (g) > 0 ? (g) \
                         : (whole && !((q)->set && ((q)->mask & (kbit))) ? K : 1))
        t = K / KGROUP(sz, sz->g1, src_kbit);
        if (t > ng) ng = t;
        t = K / KGROUP(wz, wz->g0, wei_kbit);
        if (t > ng) ng = t;
        t = K / KGROUP(ss, ss->g1, src_kbit);
        if (t > ng) ng = t;
        t = K / KGROUP(ws, ws->g0, wei_kbit);
        if (t > ng) ng = t;
#undef KGROUP
    }
    c->ngroups_k = ng;
    c->group_k = K > 0 ? K / ng : 0;
}

static int is_int_dt(int dt) {
    return dt == ORC_S8 || dt == ORC_U8;
}
static int is_wei_int(int dt) {
    return dt == ORC_S8 || dt == ORC_U8 || dt == ORC_S4 || dt == ORC_U4;
}

/* ---- the group's integer dot product on the host's byte dot-product
 * instruction ------------------------------------------------------------
 * Not another algorithm: the sum over a K group of s * w that the loop of
 * matmul_int8 forms one product at a time, formed 64 products at a time where
 * the CPU has AVX-512 VNNI (vpdpbusd: u8 x s8 -> s32). Integer sums wrap the
 * same in any order, so the result is the scalar loop's bit for bit
 * (tests/test_oracle_matmul.py runs both and compares). Taken for 2-D
 * problems with an s8 or u8 source whose rows are contiguous, s8 weights and
 * no zero points; the weights are copied once per call as [N][K] so that a
 * column's k run is contiguous, with the group sums of every column next to
 * them: an s8 source enters as s + 128 (one flipped bit), and 128 x the
 * column's group sum leaves the product again. QMM_ORACLE_SCALAR=1 in the
 * environment switches it off. This is what makes the oracle usable as a CPU
 * baseline on the GPU box's host cores. */
#if defined(__x86_64__)
#include <immintrin.h>
__attribute__((target("avx512f,avx512bw,avx512vnni")))
static int32_t dot_u8s8(const uint8_t *a, const int8_t *b, int64_t n) {
    __m512i acc = _mm512_setzero_si512();
    int64_t i = 0;
    for (; i + 64 <= n; i += 64)
        acc = _mm512_dpbusd_epi32(acc, _mm512_loadu_si512((const void *)(a + i)),
                _mm512_loadu_si512((const void *)(b + i)));
    if (i < n) {
        const __mmask64 m = (~(uint64_t)0) >> (64 - (n - i));
        acc = _mm512_dpbusd_epi32(acc, _mm512_maskz_loadu_epi8(m, a + i),
                _mm512_maskz_loadu_epi8(m, b + i));
    }
    return _mm512_reduce_add_epi32(acc);
}
static int have_vnni(void) {
    const char *e = getenv("QMM_ORACLE_SCALAR");
    if (e && e[0] == '1') return 0;
    __builtin_cpu_init();
    return __builtin_cpu_supports("avx512f") && __builtin_cpu_supports("avx512bw")
            && __builtin_cpu_supports("avx512vnni");
}
#else
static int32_t dot_u8s8(const uint8_t *a, const int8_t *b, int64_t n) {
    (void)a, (void)b, (void)n;
    return 0;
}
static int have_vnni(void) {
    return 0;
}
#endif

/* integer path: src/cpu/matmul/ref_matmul_int8.cpp:154-261 */
static void matmul_int8(const orc_matmul_t *p, const mm_ctx_t *c,
        int32_t *acc_out) {
    const int nd = c->nd;
    const int non_default = !attr_is_default(p);
    const orc_quant_t *ss = &p->scales[ORC_Q_SRC], *ws = &p->scales[ORC_Q_WEI];
    const orc_quant_t *ds = &p->scales[ORC_Q_DST];
    const orc_quant_t *sz = &p->zps[ORC_Q_SRC], *wz = &p->zps[ORC_Q_WEI];
    const orc_quant_t *dz = &p->zps[ORC_Q_DST];
    const float src_scale0 = single_scale(ss, 0);
    const float wei_scale0 = single_scale(ws, 0);
    const float dst_scale_inv = single_scale(ds, 1);
    const int dst_zp_mult = dz->set && dz->mask > 0;
    const int sum_dt = sum_dt_of(p);
    const int64_t rows = c->batch * c->M;

    /* the fast form of the group's dot product (see dot_u8s8) */
    int8_t *wt = NULL; /* [N][K] */
    int32_t *wsum = NULL; /* [N][groups]: sum of the column's weights per group */
    const int fast = nd == 2 && c->K > 0 && is_int_dt(p->src.dt)
            && p->wei.dt == ORC_S8 && !sz->set && !wz->set
            && p->src.strides[1] == 1 && c->group_k >= 16 && have_vnni();
    if (fast) {
        wt = (int8_t *)malloc((size_t)c->N * c->K);
        wsum = (int32_t *)malloc((size_t)c->N * c->ngroups_k * sizeof(int32_t));
        if (wt && wsum) {
            const int8_t *w = (const int8_t *)p->wei.ptr;
#pragma omp parallel for schedule(static)
            for (int64_t n = 0; n < c->N; n++) {
                for (int64_t k = 0; k < c->K; k++)
                    wt[n * c->K + k]
                            = w[k * p->wei.strides[0] + n * p->wei.strides[1]];
                for (int64_t g = 0; g < c->ngroups_k; g++) {
                    int32_t t = 0;
                    for (int64_t k = 0; k < c->group_k; k++)
                        t += wt[n * c->K + g * c->group_k + k];
                    wsum[n * c->ngroups_k + g] = t;
                }
            }
        }
    }
    const int use_fast = fast && wt && wsum;

    /* rows are taken in blocks so that, in the fast form, a weights column
     * read from memory serves a block's rows (the block's group sums are
     * formed first, column by column, and the loop below picks them up) */
    int64_t RB = 1;
    if (use_fast) {
        RB = 32;
        while (RB > 1 && RB * c->N * c->ngroups_k * 4 > ((int64_t)8 << 20))
            RB /= 2;
    }
    const int64_t nblocks = (rows + RB - 1) / RB;
#pragma omp parallel for schedule(dynamic, 1)
    for (int64_t blk = 0; blk < nblocks; blk++) {
    const int64_t row_lo = blk * RB, row_hi = row_lo + RB < rows ? row_lo + RB : rows;
    uint8_t *urows = NULL; /* the block's rows as unsigned bytes: an s8 source
                              with its top bit flipped */
    int32_t *accb = NULL; /* [row in block][N][group] */
    if (use_fast) {
        urows = (uint8_t *)malloc((size_t)RB * c->K);
        accb = (int32_t *)malloc((size_t)RB * c->N * c->ngroups_k * sizeof(int32_t));
    }
    if (urows && accb) {
        const uint8_t flip = p->src.dt == ORC_S8 ? 0x80 : 0;
        for (int64_t row = row_lo; row < row_hi; row++) {
            const uint8_t *sr = (const uint8_t *)p->src.ptr + row * p->src.strides[0];
            for (int64_t k = 0; k < c->K; k++)
                urows[(row - row_lo) * c->K + k] = sr[k] ^ flip;
        }
        for (int64_t n = 0; n < c->N; n++)
            for (int64_t g = 0; g < c->ngroups_k; g++) {
                const int8_t *wc = wt + n * c->K + g * c->group_k;
                const uint32_t back = p->src.dt == ORC_S8
                        ? 128u * (uint32_t)wsum[n * c->ngroups_k + g]
                        : 0u;
                for (int64_t r = 0; r < row_hi - row_lo; r++)
                    accb[(r * c->N + n) * c->ngroups_k + g] = (int32_t)(
                            (uint32_t)dot_u8s8(urows + r * c->K + g * c->group_k,
                                    wc, c->group_k)
                            - back);
            }
    }
    const int blk_fast = urows && accb;
    for (int64_t row = row_lo; row < row_hi; row++) {
        const int64_t mb = row / c->M, m = row % c->M;
        for (int64_t n = 0; n < c->N; n++) {
            const int64_t l_offset = mb * c->M * c->N + m * c->N + n;
            int64_t di[ORC_MAX_NDIMS], si[ORC_MAX_NDIMS], wi[ORC_MAX_NDIMS];
            l_dims(di, l_offset, p->dst.dims, nd);
            for (int d = 0; d < nd; d++) {
                si[d] = (c->src_mask & (1 << d)) ? di[d] : 0;
                wi[d] = (c->wei_mask & (1 << d)) ? di[d] : 0;
            }
            si[nd - 2] = m;
            wi[nd - 1] = n;
            float d = 0;
            for (int64_t g = 0; g < c->ngroups_k; g++) {
                int32_t acc = 0;
                if (blk_fast) {
                    acc = accb[((row - row_lo) * c->N + n) * c->ngroups_k + g];
                    /* the scale lookups below index by the group's last k */
                    si[nd - 1] = (g + 1) * c->group_k - 1;
                    wi[nd - 2] = (g + 1) * c->group_k - 1;
                }
                for (int64_t k = 0; k < (blk_fast ? 0 : c->group_k); k++) {
                    si[nd - 1] = k + g * c->group_k;
                    wi[nd - 2] = k + g * c->group_k;
                    int s = orc_load_int(p->src.dt, p->src.ptr,
                            off_v(&p->src, si));
                    int w = orc_load_int(p->wei.dt, p->wei.ptr,
                            off_v(&p->wei, wi));
                    if (sz->set)
                        s -= orc_load_int(
                                sz->dt, sz->ptr, qmd_off(&c->q_src_zp, si));
                    if (wz->set)
                        w -= orc_load_int(
                                wz->dt, wz->ptr, qmd_off(&c->q_wei_zp, wi));
                    acc = (int32_t)((uint32_t)acc + (uint32_t)(s * w));
                }
                if (acc_out) {
                    /* exact integer dot product regardless of grouping */
                    acc_out[l_offset] = (int32_t)((uint32_t)(g ? acc_out[l_offset] : 0)
                            + (uint32_t)acc);
                    continue;
                }
                float acc_f = (float)acc;
                if (ss->set)
                    acc_f *= c->q_src_scale.nelems == 1
                            ? src_scale0
                            : orc_load_float(ss->dt, ss->ptr,
                                    qmd_off(&c->q_src_scale, si));
                if (ws->set)
                    acc_f *= c->q_wei_scale.nelems == 1
                            ? wei_scale0
                            : orc_load_float(ws->dt, ws->ptr,
                                    qmd_off(&c->q_wei_scale, wi));
                d += acc_f;
            }
            if (acc_out) continue;
            if (p->bias.ndims) {
                int64_t bi[ORC_MAX_NDIMS];
                for (int dd = 0; dd < nd; dd++)
                    bi[dd] = (c->bia_mask & (1 << dd)) ? di[dd] : 0;
                d += orc_load_float(
                        p->bias.dt, p->bias.ptr, off_v(&p->bias, bi));
            }
            const int64_t dst_off = off_v(&p->dst, di);
            if (non_default) {
                float dst_val = orc_load_float(sum_dt, p->dst.ptr, dst_off);
                d = apply_post_ops(p, d, dst_val, l_offset);
                d = apply_dst_scale(ds, dst_scale_inv, d, m, n, c->N, nd);
                if (dz->set)
                    d += (float)orc_load_int(
                            ORC_S32, dz->ptr, dst_zp_mult * n);
            }
            orc_store_float(p->dst.dt, d, p->dst.ptr, dst_off);
        }
    }
    free(urows);
    free(accb);
    } /* row blocks */
    free(wt);
    free(wsum);
}

/* float / fp8 / weights-decompression path:
 * src/cpu/matmul/ref_matmul.cpp:130-233 */
static void matmul_float(const orc_matmul_t *p, const mm_ctx_t *c) {
    const int nd = c->nd;
    const int non_default = !attr_is_default(p) || p->apply_to_int;
    const orc_quant_t *ss = &p->scales[ORC_Q_SRC], *ws = &p->scales[ORC_Q_WEI];
    const orc_quant_t *ds = &p->scales[ORC_Q_DST];
    const orc_quant_t *wz = &p->zps[ORC_Q_WEI];
    const int decomp = is_wei_int(p->wei.dt) && p->apply_to_int;
    const float src_scale0 = single_scale(ss, 0);
    const float wei_scale0 = single_scale(ws, 0);
    const float dst_scale_inv = single_scale(ds, 1);
    const int64_t wei_scale_stride_n
            = (ws->set && (ws->mask & (1 << (nd - 1)))) ? 1 : 0;
    const int sum_dt = sum_dt_of(p);
    const int64_t rows = c->batch * c->M;

#pragma omp parallel for schedule(static)
    for (int64_t row = 0; row < rows; row++) {
        const int64_t mb = row / c->M, m = row % c->M;
        for (int64_t n = 0; n < c->N; n++) {
            const int64_t l_offset = mb * c->M * c->N + m * c->N + n;
            int64_t di[ORC_MAX_NDIMS], si[ORC_MAX_NDIMS], wi[ORC_MAX_NDIMS];
            l_dims(di, l_offset, p->dst.dims, nd);
            for (int d = 0; d < nd; d++) {
                si[d] = (c->src_mask & (1 << d)) ? di[d] : 0;
                wi[d] = (c->wei_mask & (1 << d)) ? di[d] : 0;
            }
            si[nd - 2] = m;
            wi[nd - 1] = n;
            float acc = 0;
            for (int64_t k = 0; k < c->K; k++) {
                si[nd - 1] = k;
                wi[nd - 2] = k;
                const float s = orc_load_float(
                        p->src.dt, p->src.ptr, off_v(&p->src, si));
                float w = orc_load_float(
                        p->wei.dt, p->wei.ptr, off_v(&p->wei, wi));
                if (decomp) {
                    if (wz->set)
                        w -= (float)orc_load_int(
                                wz->dt, wz->ptr, qmd_off(&c->q_wei_zp, wi));
                    if (ws->set)
                        w *= c->q_wei_scale.nelems == 1
                                ? wei_scale0
                                : orc_load_float(ws->dt, ws->ptr,
                                        qmd_off(&c->q_wei_scale, wi));
                }
                acc += s * w;
            }
            float d = acc;
            if (ss->set) d *= src_scale0;
            if (ws->set && !decomp)
                d *= c->q_wei_scale.nelems == 1
                        ? wei_scale0
                        : orc_load_float(
                                ws->dt, ws->ptr, wei_scale_stride_n * n);
            if (p->bias.ndims) {
                int64_t bi[ORC_MAX_NDIMS];
                for (int dd = 0; dd < nd; dd++)
                    bi[dd] = (c->bia_mask & (1 << dd)) ? di[dd] : 0;
                d += orc_load_float(
                        p->bias.dt, p->bias.ptr, off_v(&p->bias, bi));
            }
            const int64_t dst_off = off_v(&p->dst, di);
            if (non_default) {
                float dst_val = orc_load_float(sum_dt, p->dst.ptr, dst_off);
                d = apply_post_ops(p, d, dst_val, l_offset);
            }
            d = apply_dst_scale(ds, dst_scale_inv, d, m, n, c->N, nd);
            orc_store_float(p->dst.dt, d, p->dst.ptr, dst_off);
        }
    }
}

static int run(const orc_matmul_t *p, int32_t *acc_out) {
    if (p->dst.ndims < 2 || p->dst.ndims > ORC_MAX_NDIMS) return 2;
    if (has_zero_dim(&p->src) || has_zero_dim(&p->wei) || has_zero_dim(&p->dst))
        return 0; /* src/cpu/matmul/ref_matmul_int8.cpp:64-66 */
#ifdef _OPENMP
    if (p->nthreads > 0) omp_set_num_threads(p->nthreads);
#endif
    mm_ctx_t c;
    mm_ctx_init(&c, p);
    if (is_int_dt(p->src.dt)) {
        if (!is_wei_int(p->wei.dt)) return 3;
        matmul_int8(p, &c, acc_out);
    } else {
        if (acc_out) return 3;
        if (p->zps[ORC_Q_SRC].set || p->zps[ORC_Q_DST].set) return 3;
        matmul_float(p, &c);
    }
    return 0;
}

int orc_matmul(const orc_matmul_t *p) {
    return run(p, NULL);
}
int orc_matmul_s32_acc(const orc_matmul_t *p, int32_t *acc) {
    return run(p, acc);
}

/* ------------------------------------------------------------------------ */
/* reorder: src/cpu/reorder/simple_reorder.hpp:2500-2640 (generic reference). */
int orc_reorder(const orc_reorder_t *p) {
    const int nd = p->src.ndims;
    if (has_zero_dim(&p->src)) return 0;
    int64_t n = 1;
    for (int d = 0; d < nd; d++)
        n *= p->src.dims[d];
    qmd_t q_ss, q_ds, q_sz;
    qmd_init(&q_ss, &p->src_scale, nd, p->src.dims, p->src_scale.g0,
            p->src_scale.g1);
    qmd_init(&q_ds, &p->dst_scale, nd, p->src.dims, 1, 1);
    qmd_init(&q_sz, &p->src_zp, nd, p->src.dims, p->src_zp.g0, p->src_zp.g1);
    const float ss0 = single_scale(&p->src_scale, 0);
    const float dst_zp
            = p->dst_zp.set ? (float)orc_load_int(ORC_S32, p->dst_zp.ptr, 0) : 0;
#pragma omp parallel for schedule(static)
    for (int64_t l = 0; l < n; l++) {
        int64_t idx[ORC_MAX_NDIMS];
        l_dims(idx, l, p->src.dims, nd);
        float src_scale = 1.f, dst_scale = 1.f;
        if (p->src_scale.set)
            src_scale = q_ss.nelems == 1
                    ? ss0
                    : orc_load_float(p->src_scale.dt, p->src_scale.ptr,
                            qmd_off(&q_ss, idx));
        if (p->dst_scale.set)
            dst_scale = 1.f
                    / orc_load_float(p->dst_scale.dt, p->dst_scale.ptr,
                            q_ds.nelems == 1 ? 0 : qmd_off(&q_ds, idx));
        int src_zp = 0;
        if (p->src_zp.set)
            src_zp = (int)orc_load_float(
                    p->src_zp.dt, p->src_zp.ptr, qmd_off(&q_sz, idx));
        float in = orc_load_float(p->src.dt, p->src.ptr, off_v(&p->src, idx));
        float d = src_scale * (in - src_zp);
        d = d * dst_scale + dst_zp;
        int64_t o = off_v(&p->dst, idx);
        if (p->dst.dt == ORC_S4 || p->dst.dt == ORC_U4) {
            /* 4-bit stores: src/common/int4.hpp:36-39,53-59 */
            uint8_t *b = (uint8_t *)p->dst.ptr + o / 2;
            uint8_t nib;
            if (p->dst.dt == ORC_U4) {
                float v = d < 0.f ? 0.f : d > 15.f ? 15.f : d;
                nib = (uint8_t)((uint8_t)nearbyintf(v) & 0xf);
            } else {
                float v = d < -8.f ? -8.f : d > 7.f ? 7.f : d;
                int8_t i8 = (int8_t)nearbyintf(v);
                nib = (uint8_t)(i8 & 0xf);
            }
#pragma omp critical
            *b = (o % 2) ? (uint8_t)((*b & 0x0f) | (nib << 4))
                         : (uint8_t)((*b & 0xf0) | nib);
        } else
            orc_store_float(p->dst.dt, d, p->dst.ptr, o);
    }
    return 0;
}

/* ------------------------------------------------------------------------ */
/* softmax forward: src/cpu/ref_softmax.cpp. The reference has two loops and
 * picks by layout (ref_softmax.hpp:137-139): "dense" when the axis is the
 * innermost dim and src and dst are one dense layout AND one data type
 * (memory descriptors compare equal) -- exp(s - max) * (1 / sum),
 * ref_softmax.cpp:40-193 -- and "generic" otherwise -- exp(s - max) / sum,
 * :196-312. Both keep the exponentials in f32 (the default accumulation mode,
 * ref_softmax.hpp:80-92), multiply by the source scale, then by the inverted
 * destination scale (cpu_primitive.hpp:48-56), and convert. */
static int softmax_is_dense(const orc_softmax_t *p) {
    const int nd = p->src.ndims;
    if (p->src.dt != p->dst.dt) return 0;
    if (p->src.strides[p->axis] != 1) return 0;
    for (int d = 0; d < nd; d++)
        if (p->src.strides[d] != p->dst.strides[d]) return 0;
    /* dense: the dims other than the axis, sorted by stride, nest without gaps
     * over rows of `channels` elements */
    int order[ORC_MAX_NDIMS], n = 0;
    for (int d = 0; d < nd; d++)
        if (d != p->axis) order[n++] = d;
    for (int i = 0; i < n; i++)
        for (int j = i + 1; j < n; j++)
            if (p->src.strides[order[j]] < p->src.strides[order[i]]) {
                int t = order[i];
                order[i] = order[j];
                order[j] = t;
            }
    int64_t expect = p->src.dims[p->axis];
    for (int i = 0; i < n; i++) {
        const int k = order[i];
        if (p->src.dims[k] == 1) continue;
        if (p->src.strides[k] != expect) return 0;
        expect *= p->src.dims[k];
    }
    return 1;
}

int orc_softmax(const orc_softmax_t *p) {
    const int nd = p->src.ndims;
    if (nd < 1 || nd > ORC_MAX_NDIMS || p->dst.ndims != nd) return 2;
    if (p->axis < 0 || p->axis >= nd) return 2;
    if (has_zero_dim(&p->src)) return 0;
    const int64_t C = p->src.dims[p->axis];
    const int64_t cs = p->src.strides[p->axis], cd = p->dst.strides[p->axis];
    int64_t odims[ORC_MAX_NDIMS], rows = 1;
    int omap[ORC_MAX_NDIMS], no = 0;
    for (int d = 0; d < nd; d++)
        if (d != p->axis) {
            odims[no] = p->src.dims[d];
            omap[no++] = d;
            rows *= p->src.dims[d];
        }
    const int dense = softmax_is_dense(p);
    const float ss = single_scale(&p->src_scale, 0);
    const float ds = single_scale(&p->dst_scale, 1);
#pragma omp parallel for schedule(static)
    for (int64_t row = 0; row < rows; row++) {
        int64_t so = 0, dof = 0, r = row;
        for (int i = no - 1; i >= 0; i--) {
            const int64_t ix = r % odims[i];
            r /= odims[i];
            so += ix * p->src.strides[omap[i]];
            dof += ix * p->dst.strides[omap[i]];
        }
        float mx = -FLT_MAX;
        for (int64_t c = 0; c < C; c++) {
            const float s = orc_load_float(p->src.dt, p->src.ptr, so + c * cs);
            mx = s > mx ? s : mx;
        }
        float denom = 0.f;
        for (int64_t c = 0; c < C; c++)
            denom += expf(orc_load_float(p->src.dt, p->src.ptr, so + c * cs) - mx);
        float scal;
        if (p->log_softmax)
            scal = logf(denom);
        else if (dense)
            scal = denom ? 1.f / denom : 1.f;
        else
            scal = denom;
        for (int64_t c = 0; c < C; c++) {
            float d = orc_load_float(p->src.dt, p->src.ptr, so + c * cs) - mx;
            if (p->log_softmax)
                d = d - scal;
            else if (dense)
                d = expf(d) * scal;
            else
                d = expf(d) / scal;
            d *= ss;
            d *= ds;
            orc_store_float(p->dst.dt, d, p->dst.ptr, dof + c * cd);
        }
    }
    return 0;
}
