// Device-side scalar layer shared by every kernel of the quantized matmul path:
// typed loads/stores with the reference's conversions, eltwise / binary
// formulas and the ordered epilogue (bias, post-ops, dst scale, dst zero point,
// saturating store).
//
// All float steps here must round separately (the translation units are built
// with -ffp-contract=off): the reference's scalar code is compiled for an ISA
// without FMA, and s8/u8 results are compared bit for bit.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "qmm_hip.h"

namespace qmm {

// dnnl_data_type_t codes (include/oneapi/dnnl/dnnl_common_types.h:76-115)
enum : int {
    dt_undef = 0, dt_f16 = 1, dt_bf16 = 2, dt_f32 = 3, dt_s32 = 4, dt_s8 = 5,
    dt_u8 = 6, dt_f8_e5m2 = 9, dt_f8_e4m3 = 10, dt_s4 = 11, dt_u4 = 12,
    dt_e8m0 = 13
};
// dnnl_primitive_kind_t codes used for post-ops
enum : int { pk_sum = 4, pk_eltwise = 7, pk_binary = 13, pk_prelu = 18 };

#define QMM_HD __host__ __device__ __forceinline__
#define QMM_D __device__ __forceinline__

QMM_HD uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }
QMM_HD float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }

// ---- bf16: src/common/bfloat16.cpp:22-56 ----
QMM_HD uint16_t f32_to_bf16(float f) {
    const uint32_t u = f2u(f);
    const uint32_t e = (u >> 23) & 0xFF;
    const uint16_t hi = (uint16_t)(u >> 16);
    if (e == 0) return hi & 0x8000; // zero and denormals: signed zero
    if (e == 0xFF) return (u & 0x7FFFFF) ? (uint16_t)(hi | 0x40) : hi;
    return (uint16_t)((u + 0x7FFFu + (hi & 1u)) >> 16);
}
QMM_HD float bf16_to_f32(uint16_t r) { return u2f((uint32_t)r << 16); }

// ---- f16: src/common/float16.hpp:52-127 ----
QMM_HD uint16_t f32_to_f16(float f) {
    const uint32_t i = f2u(f);
    const uint32_t s = i >> 31, e = (i >> 23) & 0xFF, m = i & 0x7FFFFF;
    uint32_t mm = m >> 13, ee = 0;
    const uint32_t r = m & 0x1FFF;
    const int32_t eee = (int32_t)e - 127 + 15;
    if (e == 0) {
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
        const float ff = u2f(i & 0x7FFFFFFFu) + 0.5f;
        mm = f2u(ff) & 0x7FF;
    }
    return (uint16_t)((s << 15) | (ee << 10) | mm);
}
QMM_HD float f16_to_f32(uint16_t raw) {
    const uint32_t ss = raw >> 15, ee = (raw >> 10) & 0x1F, mm = raw & 0x3FF;
    uint32_t m = mm << 13, e;
    if (ee == 0) {
        if (mm == 0) return u2f(ss << 31);
        // subnormal half: mm * 2^-24, exact in f32
        const float v = (float)mm * u2f(0x33800000u);
        return ss ? -v : v;
    } else if (ee == 0x1F) {
        e = 0xFF;
        if (m != 0) m |= 0x400000;
    } else
        e = ee - 15 + 127;
    return u2f((ss << 31) | (e << 23) | m);
}

// ---- f8: src/common/float8.cpp:43-190 ----
QMM_HD uint8_t f16_to_e4m3(uint16_t h) {
    int fraw = h;
    const unsigned s8 = (fraw & 0x8000) >> 8;
    fraw &= 0x7fff;
    if (fraw > 0x5f40) return (uint8_t)(s8 | 0x7f);
    if (fraw <= 0x1400) return (uint8_t)s8;
    uint16_t shifter = (uint16_t)((fraw & 0x7c00) + 0x1c00);
    const bool is_denorm = shifter < 0x4000;
    if (is_denorm) shifter = 0x4000;
    uint16_t rounded
            = f32_to_f16(f16_to_f32((uint16_t)fraw) + f16_to_f32(shifter));
    rounded = f32_to_f16(f16_to_f32(rounded) - f16_to_f32(shifter));
    int e8 = ((rounded & 0x7c00) >> 10) - 8;
    uint8_t m8 = (uint8_t)((rounded & 0x03ff) >> 7);
    if (is_denorm) {
        m8 = (uint8_t)((m8 | 0x8) >> (-e8 + 1));
        e8 = 0;
    }
    return (uint8_t)(s8 | (e8 << 3) | m8);
}
QMM_HD uint16_t e4m3_to_f16(uint8_t r) {
    const uint16_t s8 = (r & 0x80) >> 7, e8 = (r & 0x78) >> 3, m8 = r & 0x7;
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
QMM_HD uint8_t f16_to_e5m2(uint16_t fraw) {
    const bool is_special = (fraw & 0x7c00) == 0x7c00;
    const bool is_nan = is_special && (fraw & 0x03ff);
    if (is_nan) return (uint8_t)((fraw >> 8) | 0x02);
    if (is_special) return (uint8_t)(fraw >> 8);
    fraw = (uint16_t)(fraw + 0x007f + ((fraw & 0x0100) >> 8));
    return (uint8_t)(fraw >> 8);
}
QMM_HD float e5m2_to_f32(uint8_t r) {
    const uint8_t raw = ((r & 0x7d) == 0x7d) ? (r | 0x02) : r;
    return f16_to_f32((uint16_t)(raw << 8));
}
QMM_HD float e8m0_to_f32(uint8_t r) {
    return r == 0xff ? u2f(0xffc00000u) : u2f((uint32_t)r << 23);
}

// ---- typed element access: src/cpu/ref_io_helper.hpp:33-154 ----
QMM_HD int nibble_at(const void *p, int64_t idx) {
    const uint8_t b = ((const uint8_t *)p)[idx >> 1];
    return (idx & 1) ? (b >> 4) : (b & 0xf); // even index = low nibble
}
QMM_HD int s4_value(int nib) { return (nib & 8) ? nib - 16 : nib; }

QMM_HD int load_int(int dt, const void *p, int64_t idx) {
    switch (dt) {
        case dt_s32: return ((const int32_t *)p)[idx];
        case dt_s8: return ((const int8_t *)p)[idx];
        case dt_u8: return ((const uint8_t *)p)[idx];
        case dt_s4: return s4_value(nibble_at(p, idx));
        case dt_u4: return nibble_at(p, idx);
        default: return 0x7fffffff;
    }
}

QMM_HD float load_float(int dt, const void *p, int64_t idx) {
    switch (dt) {
        case dt_f32: return ((const float *)p)[idx];
        case dt_bf16: return bf16_to_f32(((const uint16_t *)p)[idx]);
        case dt_f16: return f16_to_f32(((const uint16_t *)p)[idx]);
        case dt_f8_e4m3:
            return f16_to_f32(e4m3_to_f16(((const uint8_t *)p)[idx]));
        case dt_f8_e5m2: return e5m2_to_f32(((const uint8_t *)p)[idx]);
        case dt_s32: return (float)((const int32_t *)p)[idx];
        case dt_s8: return (float)((const int8_t *)p)[idx];
        case dt_u8: return (float)((const uint8_t *)p)[idx];
        case dt_e8m0: return e8m0_to_f32(((const uint8_t *)p)[idx]);
        case dt_s4: return (float)s4_value(nibble_at(p, idx));
        case dt_u4: return (float)nibble_at(p, idx);
        default: return u2f(0x7fc00000u);
    }
}

// clamp then round half to even (src/cpu/simple_q10n.hpp:41-81); a NaN passes
// the clamps and converts to the x86 "integer indefinite" value
QMM_HD int round_sat(float v, float lo, float hi) {
    if (v < lo) v = lo;
    if (v > hi) v = hi;
    if (v != v) return (int)0x80000000;
#if defined(__HIP_DEVICE_COMPILE__)
    return (int)__builtin_rintf(v);
#else
    return (int)__builtin_nearbyintf(v);
#endif
}

QMM_HD void store_float(int dt, float v, void *p, int64_t idx) {
    switch (dt) {
        case dt_f32: ((float *)p)[idx] = v; break;
        case dt_bf16: ((uint16_t *)p)[idx] = f32_to_bf16(v); break;
        case dt_f16: ((uint16_t *)p)[idx] = f32_to_f16(v); break;
        case dt_f8_e4m3:
            ((uint8_t *)p)[idx] = f16_to_e4m3(f32_to_f16(v));
            break;
        case dt_f8_e5m2:
            ((uint8_t *)p)[idx] = f16_to_e5m2(f32_to_f16(v));
            break;
        case dt_s32:
            ((int32_t *)p)[idx] = round_sat(v, -2147483648.f, 2147483520.f);
            break;
        case dt_s8: ((int8_t *)p)[idx] = (int8_t)round_sat(v, -128.f, 127.f); break;
        case dt_u8: ((uint8_t *)p)[idx] = (uint8_t)round_sat(v, 0.f, 255.f); break;
        default: break;
    }
}

// ---- eltwise forward: src/common/math_utils.hpp:129-416 ----
enum : int {
    alg_relu = 0x20, alg_tanh, alg_elu, alg_square, alg_abs, alg_sqrt,
    alg_linear, alg_soft_relu, alg_hardsigmoid, alg_logistic, alg_exp,
    alg_gelu_tanh, alg_swish, alg_log, alg_clip, alg_clip_v2, alg_pow,
    alg_gelu_erf, alg_round, alg_mish, alg_hardswish,
    alg_relu_dst = 0x100, alg_tanh_dst, alg_elu_dst, alg_sqrt_dst,
    alg_logistic_dst, alg_exp_dst, alg_clip_v2_dst,
    alg_bin_add = 0x1fff0, alg_bin_mul, alg_bin_max, alg_bin_min, alg_bin_div,
    alg_bin_sub, alg_bin_ge, alg_bin_gt, alg_bin_le, alg_bin_lt, alg_bin_eq,
    alg_bin_ne
};

QMM_D float logistic_f(float s) {
    const float bound = 88.72283172607421875f;
    const float in = -s;
    return in < bound ? 1.f / (1.f + expf(in)) : 0.f;
}
QMM_D float soft_relu_f(float s, float alpha) {
    const float bound = 88.72283172607421875f;
    const float in = s * alpha;
    const float v = in < bound ? log1pf(expf(in)) : in;
    return v / alpha;
}
QMM_D float hardsigmoid_f(float s, float alpha, float beta) {
    const float v = alpha * s + beta;
    return v <= 0.f ? 0.f : v >= 1.f ? 1.f : v;
}

// One definition per algorithm (eltwise_one / binary_one); the scalar and the
// four-element dispatchers below are generated from the same lists, so they
// cannot drift apart. The *_use_dst_for_bwd aliases compute their base
// algorithm's forward formula.
template <int ALG>
QMM_D float eltwise_one(float s, float alpha, float beta) {
    if constexpr (ALG == alg_relu) {
        return s > 0 ? s : s * alpha;
    } else if constexpr (ALG == alg_tanh) {
        return tanhf(s);
    } else if constexpr (ALG == alg_elu) {
        return s > 0 ? s : alpha * expm1f(s);
    } else if constexpr (ALG == alg_square) {
        return s * s;
    } else if constexpr (ALG == alg_abs) {
        return s > 0 ? s : -s;
    } else if constexpr (ALG == alg_sqrt) {
        return sqrtf(s);
    } else if constexpr (ALG == alg_linear) {
        return alpha * s + beta;
    } else if constexpr (ALG == alg_soft_relu) {
        return soft_relu_f(s, alpha);
    } else if constexpr (ALG == alg_hardsigmoid) {
        return hardsigmoid_f(s, alpha, beta);
    } else if constexpr (ALG == alg_logistic) {
        return logistic_f(s);
    } else if constexpr (ALG == alg_exp) {
        return expf(s);
    } else if constexpr (ALG == alg_gelu_tanh) {
        const float sqrt_2_over_pi = 0.79788458347320556640625f;
        const float fitting_const = 0.044715f;
        const float v = tanhf(sqrt_2_over_pi * s * (1 + fitting_const * s * s));
        return (float)(0.5 * s * (1. + v));
    } else if constexpr (ALG == alg_swish) {
        return s * logistic_f(alpha * s);
    } else if constexpr (ALG == alg_log) {
        return logf(s);
    } else if constexpr (ALG == alg_clip) {
        s = s > alpha ? s : alpha;
        return s > beta ? beta : s;
    } else if constexpr (ALG == alg_clip_v2) {
        s = s > alpha ? s : alpha;
        return s < beta ? s : beta;
    } else if constexpr (ALG == alg_pow) {
        return alpha * powf(s, beta);
    } else if constexpr (ALG == alg_gelu_erf) {
        const float sqrt_2_over_2 = 0.707106769084930419921875f;
        const float v = s * sqrt_2_over_2;
        return 0.5f * s * (1.f + erff(v));
    } else if constexpr (ALG == alg_round) {
        return __builtin_rintf(s);
    } else if constexpr (ALG == alg_mish) {
        return s * tanhf(soft_relu_f(s, 1.f));
    } else {
        static_assert(ALG == alg_hardswish, "unknown eltwise algorithm");
        return s * hardsigmoid_f(s, alpha, beta);
    }
}
// X(algorithm, rows of a four-element group computed by inlined copies): the
// long library routines keep one copy in a loop
#define QMM_ELTWISE_LIST(X) \
    X(alg_relu, 4) X(alg_tanh, 1) X(alg_elu, 1) X(alg_square, 4) X(alg_abs, 4) \
    X(alg_sqrt, 4) X(alg_linear, 4) X(alg_soft_relu, 1) X(alg_hardsigmoid, 4) \
    X(alg_logistic, 4) X(alg_exp, 4) X(alg_gelu_tanh, 1) X(alg_swish, 4) \
    X(alg_log, 1) X(alg_clip, 4) X(alg_clip_v2, 4) X(alg_pow, 1) \
    X(alg_gelu_erf, 1) X(alg_round, 4) X(alg_mish, 1) X(alg_hardswish, 4)

QMM_D int eltwise_base_alg(int alg) {
    switch (alg) {
        case alg_relu_dst: return alg_relu;
        case alg_tanh_dst: return alg_tanh;
        case alg_elu_dst: return alg_elu;
        case alg_sqrt_dst: return alg_sqrt;
        case alg_logistic_dst: return alg_logistic;
        case alg_exp_dst: return alg_exp;
        case alg_clip_v2_dst: return alg_clip_v2;
        default: return alg;
    }
}

QMM_D float eltwise_fwd(int alg, float s, float alpha, float beta) {
    switch (eltwise_base_alg(alg)) {
#define QMM_X(A, U) \
    case A: return eltwise_one<A>(s, alpha, beta);
        QMM_ELTWISE_LIST(QMM_X)
#undef QMM_X
        default: return u2f(0x7fc00000u);
    }
}

// src/cpu/primitive_attr_postops.cpp:29-46
template <int ALG>
QMM_D float binary_one(float x, float y) {
    if constexpr (ALG == alg_bin_add) return x + y;
    else if constexpr (ALG == alg_bin_div) return x / y;
    else if constexpr (ALG == alg_bin_max) return x > y ? x : y;
    else if constexpr (ALG == alg_bin_min) return x < y ? x : y;
    else if constexpr (ALG == alg_bin_mul) return x * y;
    else if constexpr (ALG == alg_bin_sub) return x - y;
    else if constexpr (ALG == alg_bin_ge) return x >= y;
    else if constexpr (ALG == alg_bin_gt) return x > y;
    else if constexpr (ALG == alg_bin_le) return x <= y;
    else if constexpr (ALG == alg_bin_lt) return x < y;
    else if constexpr (ALG == alg_bin_eq) return x == y;
    else {
        static_assert(ALG == alg_bin_ne, "unknown binary algorithm");
        return x != y;
    }
}
#define QMM_BINARY_LIST(X) \
    X(alg_bin_add) X(alg_bin_mul) X(alg_bin_max) X(alg_bin_min) X(alg_bin_div) \
    X(alg_bin_sub) X(alg_bin_ge) X(alg_bin_gt) X(alg_bin_le) X(alg_bin_lt) \
    X(alg_bin_eq) X(alg_bin_ne)

QMM_D float binary_op(int alg, float x, float y) {
    switch (alg) {
#define QMM_X(A) \
    case A: return binary_one<A>(x, y);
        QMM_BINARY_LIST(QMM_X)
#undef QMM_X
        default: return u2f(0x7fc00000u);
    }
}

// ---------------------------------------------------------------------------
// Compact epilogue description used by the tiled kernels. The host folds the
// problem to (batch, m, n) coordinates: every tensor touched after the
// accumulation is addressed as base + b*sb + m*sm + n*sn with zero strides on
// broadcast dims.
struct ep_tensor_t {
    const void *ptr;
    int64_t sb, sm, sn;
    int32_t dt;
    int32_t pad_;
};

struct ep_postop_t {
    int32_t kind, alg;
    float alpha, beta, scale;
    int32_t zero_point;
    ep_tensor_t t; // binary operand, prelu weights (f32) or dst-as-sum_dt
};

constexpr int EP_MAX_PO = 6;

struct epilogue_t {
    ep_tensor_t dst;
    ep_tensor_t bias; // ptr == nullptr: none
    ep_tensor_t src_scale; // per-tensor or per-m (sm != 0); nullptr: none
    ep_tensor_t wei_scale; // per-tensor or per-n (sn != 0); nullptr: none
    const void *dst_scale; // single value, inverted in the kernel
    int32_t dst_scale_dt;
    int32_t npo;
    const int32_t *dst_zp; // s32; index dst_zp_sn * n
    int64_t dst_zp_sn;
    int32_t fast; // EP_FAST_* shape recognised by the host, 0: interpret
    // the shape additionally has a per-column bias, a dst scale / zero point
    // or an f16 / s8 / u8 dst: only epilogue_full4<.., EXT> runs it straight
    int32_t fast_ext;
    ep_postop_t po[EP_MAX_PO];
};

// Epilogue shapes the tiled GEMM handles with straight-line code instead of
// the post-op interpreter: f32 scales (per-tensor / per-m source, per-tensor /
// per-n weights), no bias, no dst scale / zero point, a dense bf16 or f32 dst
// row and at most one post-op of the kinds below.
enum : int {
    EP_FAST_NONE = 0,
    EP_FAST_PLAIN = 1, // no post-op
    EP_FAST_RELU = 2, // eltwise relu(alpha)
    EP_FAST_SWISH = 3, // eltwise swish(alpha)
    EP_FAST_ADD = 4, // binary add with an f32 operand, dense along n
    EP_FAST_SUM = 5, // sum with zero point 0 read in dst's own type
    // shapes only the 256 x 256 kernels run straight-line (fast_ext is set):
    EP_FAST_GELU_ERF = 6,
    EP_FAST_GELU_TANH = 7,
    EP_FAST_BIN32 = 8, // binary add / mul with a dense f32 operand
    EP_FAST_BIN16 = 9 // binary add / mul with a dense f16 / bf16 operand
};

QMM_D float ep_load(const ep_tensor_t &t, int64_t b, int64_t m, int64_t n) {
    return load_float(t.dt, t.ptr, b * t.sb + m * t.sm + n * t.sn);
}

// Ordered tail of the reference kernels, starting after the K reduction:
//   integer path   src/cpu/matmul/ref_matmul_int8.cpp:195-259
//   float path     src/cpu/matmul/ref_matmul.cpp:199-229
// `acc` is (float)s32 for the integer path or the f32 accumulator.
QMM_D void epilogue_apply_store(const epilogue_t &ep, float acc, int64_t b,
        int64_t m, int64_t n) {
    float d = acc;
    if (ep.src_scale.ptr) d *= ep_load(ep.src_scale, b, m, 0);
    if (ep.wei_scale.ptr) d *= ep_load(ep.wei_scale, b, 0, n);
    if (ep.bias.ptr) d += ep_load(ep.bias, b, m, n);
    const int64_t dst_off = b * ep.dst.sb + m * ep.dst.sm + n * ep.dst.sn;
#pragma unroll 1
    for (int i = 0; i < ep.npo; i++) {
        const ep_postop_t &e = ep.po[i];
        if (e.kind == pk_eltwise) {
            d = eltwise_fwd(e.alg, d, e.alpha, e.beta) * e.scale;
        } else if (e.kind == pk_sum) {
            const float old = load_float(e.t.dt, ep.dst.ptr, dst_off);
            d += e.scale * (old - (float)e.zero_point);
        } else if (e.kind == pk_binary) {
            d = binary_op(e.alg, d, ep_load(e.t, b, m, n));
        } else if (e.kind == pk_prelu) {
            if (d < 0) d = ep_load(e.t, b, m, n) * d;
        }
    }
    if (ep.dst_scale) d *= 1.f / load_float(ep.dst_scale_dt, ep.dst_scale, 0);
    if (ep.dst_zp) d += (float)ep.dst_zp[ep.dst_zp_sn * n];
    store_float(ep.dst.dt, d, (void *)ep.dst.ptr, dst_off);
}

// Four elements per dispatch: the algorithm switch is taken once per row piece
// instead of once per element (the kernels are otherwise busy jumping).
#define QMM_PRAGMA(x) _Pragma(#x)
QMM_D void eltwise_fwd4(int alg, float (&d)[4], float alpha, float beta,
        float scale) {
    switch (eltwise_base_alg(alg)) {
#define QMM_X(A, U) \
    case A: \
        QMM_PRAGMA(unroll U) for (int i = 0; i < 4; i++) d[i] \
                = eltwise_one<A>(d[i], alpha, beta) * scale; \
        break;
        QMM_ELTWISE_LIST(QMM_X)
#undef QMM_X
        default:
#pragma unroll
            for (int i = 0; i < 4; i++)
                d[i] = u2f(0x7fc00000u);
            break;
    }
}
QMM_D void binary_op4(int alg, float (&d)[4], const float (&o)[4]) {
    switch (alg) {
#define QMM_X(A) \
    case A: \
        _Pragma("unroll") for (int i = 0; i < 4; i++) d[i] \
                = binary_one<A>(d[i], o[i]); \
        break;
        QMM_BINARY_LIST(QMM_X)
#undef QMM_X
        default:
#pragma unroll
            for (int i = 0; i < 4; i++)
                d[i] = u2f(0x7fc00000u);
            break;
    }
}

// ---- the same tail for four consecutive n at once (n % 4 == 0) -------------
// The tiled kernels hand their results over row-wise: a lane owns 4 neighbouring
// columns of every row it visits. What depends on the column only (weights
// scales, a per-column bias, dst zero points, the inverted dst scale) is
// fetched once per tile into ep_cols_t; row operands (binary / sum / prelu) are
// read as 4-element vectors where the tensor is dense and aligned; f16 results
// are converted by the hardware (round to nearest even, subnormals kept; NaNs
// go through the bit-exact software conversion). The operation order is the
// reference's, as in epilogue_apply_store().
struct ep_cols_t {
    float ws[4], bias[4], zp[4];
    float inv_dst_scale;
    int32_t has_ws, has_bias, bias_per_row, has_ds, has_zp;
    // first post-op's binary operand (EP_FAST_BIN32 / BIN16), at this lane's
    // columns of row 0
    const void *bin_ptr;
    int64_t bin_sm; // elements per row
    int32_t bin_mul, bin_f16;
};

QMM_D void epilogue_cols_load(const epilogue_t &ep, ep_cols_t &c, int64_t b,
        int64_t n, int nvalid) {
    c.has_ws = ep.wei_scale.ptr != nullptr;
    c.has_bias = ep.bias.ptr != nullptr;
    c.bias_per_row = c.has_bias && ep.bias.sm != 0;
    c.has_ds = ep.dst_scale != nullptr;
    c.has_zp = ep.dst_zp != nullptr;
    c.inv_dst_scale
            = c.has_ds ? 1.f / load_float(ep.dst_scale_dt, ep.dst_scale, 0) : 1.f;
    c.bin_ptr = nullptr;
    c.bin_sm = 0;
    c.bin_mul = c.bin_f16 = 0;
    if (ep.fast == EP_FAST_BIN32 || ep.fast == EP_FAST_BIN16) {
        const int64_t off = b * ep.po[0].t.sb + n;
        c.bin_ptr = ep.fast == EP_FAST_BIN32
                ? (const void *)((const float *)ep.po[0].t.ptr + off)
                : (const void *)((const uint16_t *)ep.po[0].t.ptr + off);
        c.bin_sm = ep.po[0].t.sm;
        c.bin_mul = ep.po[0].alg == alg_bin_mul;
        c.bin_f16 = ep.po[0].t.dt == dt_f16;
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        c.ws[i] = 1.f;
        c.bias[i] = 0.f;
        c.zp[i] = 0.f;
        if (i < nvalid) {
            if (c.has_ws) c.ws[i] = ep_load(ep.wei_scale, b, 0, n + i);
            if (c.has_bias && !c.bias_per_row)
                c.bias[i] = ep_load(ep.bias, b, 0, n + i);
            if (c.has_zp) c.zp[i] = (float)ep.dst_zp[ep.dst_zp_sn * (n + i)];
        }
    }
}

QMM_D uint16_t f32_to_f16_hw(float x) {
    return __builtin_bit_cast(uint16_t, (_Float16)x);
}

// four values of a (b, m, n..n+3) tensor operand
QMM_D void ep_load4(const ep_tensor_t &t, int64_t b, int64_t m, int64_t n,
        int nvalid, float (&o)[4]) {
    const int64_t off = b * t.sb + m * t.sm + n * t.sn;
    if (t.sn == 0) {
        const float v = load_float(t.dt, t.ptr, off);
        o[0] = o[1] = o[2] = o[3] = v;
        return;
    }
    if (t.sn == 1 && nvalid == 4) {
        // one vector load at any address (global loads need no alignment)
        if (t.dt == dt_f32) {
            typedef float v4f_any __attribute__((ext_vector_type(4), aligned(4)));
            const v4f_any v = *(const v4f_any *)((const float *)t.ptr + off);
            o[0] = v[0];
            o[1] = v[1];
            o[2] = v[2];
            o[3] = v[3];
            return;
        } else if (t.dt == dt_f16 || t.dt == dt_bf16) {
            typedef unsigned v2u_any __attribute__((ext_vector_type(2), aligned(2)));
            const v2u_any v = *(const v2u_any *)((const uint16_t *)t.ptr + off);
            const uint16_t h[4] = {(uint16_t)v[0], (uint16_t)(v[0] >> 16),
                    (uint16_t)v[1], (uint16_t)(v[1] >> 16)};
#pragma unroll
            for (int i = 0; i < 4; i++)
                o[i] = t.dt == dt_f16 ? (float)__builtin_bit_cast(_Float16, h[i])
                                      : bf16_to_f32(h[i]);
            return;
        }
    }
#pragma unroll
    for (int i = 0; i < 4; i++)
        o[i] = i < nvalid ? load_float(t.dt, t.ptr, off + i * t.sn) : 0.f;
}

QMM_D void epilogue_store4(const epilogue_t &ep, const float (&d)[4],
        int64_t dst_off, int nvalid) {
    void *dst = (void *)ep.dst.ptr;
    const int dt = ep.dst.dt;
    if (nvalid == 4 && ep.dst.sn == 1) {
        if (dt == dt_bf16 || dt == dt_f16) {
            uint16_t *q = (uint16_t *)dst + dst_off;
            uint16_t h[4];
            if (dt == dt_bf16) {
#pragma unroll
                for (int i = 0; i < 4; i++)
                    h[i] = f32_to_bf16(d[i]);
            } else if (d[0] != d[0] || d[1] != d[1] || d[2] != d[2]
                    || d[3] != d[3]) {
#pragma unroll
                for (int i = 0; i < 4; i++)
                    h[i] = f32_to_f16(d[i]);
            } else {
#pragma unroll
                for (int i = 0; i < 4; i++)
                    h[i] = f32_to_f16_hw(d[i]);
            }
            // one 8-byte store whatever the address (rows of odd length start on
            // 2- or 4-byte boundaries; global stores take any address)
            typedef unsigned v2u_any __attribute__((ext_vector_type(2), aligned(2)));
            const uint32_t lo = (uint32_t)h[0] | ((uint32_t)h[1] << 16);
            const uint32_t hi = (uint32_t)h[2] | ((uint32_t)h[3] << 16);
            *(v2u_any *)q = v2u_any {lo, hi};
            return;
        } else if (dt == dt_f32) {
            // (one 16-byte store at any 4-byte address)
            typedef float v4f_any __attribute__((ext_vector_type(4), aligned(4)));
            *(v4f_any *)((float *)dst + dst_off) = v4f_any {d[0], d[1], d[2], d[3]};
            return;
        } else if (dt == dt_s8 || dt == dt_u8) {
            // (one 4-byte store at any address)
            typedef uint32_t u32_any __attribute__((aligned(1)));
            uint32_t w = 0;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int r = dt == dt_s8 ? round_sat(d[i], -128.f, 127.f)
                                          : round_sat(d[i], 0.f, 255.f);
                w |= (uint32_t)(r & 0xff) << (8 * i);
            }
            *(u32_any *)((uint8_t *)dst + dst_off) = w;
            return;
        }
    }
#pragma unroll
    for (int i = 0; i < 4; i++)
        if (i < nvalid) store_float(dt, d[i], dst, dst_off + i * ep.dst.sn);
}

QMM_D void epilogue_post_op4(const epilogue_t &ep, const ep_postop_t &e,
        float (&d)[4], int64_t b, int64_t m, int64_t n, int nvalid) {
    if (e.kind == pk_eltwise) {
        eltwise_fwd4(e.alg, d, e.alpha, e.beta, e.scale);
    } else if (e.kind == pk_sum) {
        ep_tensor_t t = ep.dst;
        t.dt = e.t.dt;
        float old[4];
        ep_load4(t, b, m, n, nvalid, old);
#pragma unroll
        for (int i = 0; i < 4; i++)
            d[i] += e.scale * (old[i] - (float)e.zero_point);
    } else if (e.kind == pk_binary) {
        float y[4];
        ep_load4(e.t, b, m, n, nvalid, y);
        binary_op4(e.alg, d, y);
    } else if (e.kind == pk_prelu) {
        float w[4];
        ep_load4(e.t, b, m, n, nvalid, w);
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (d[i] < 0) d[i] = w[i] * d[i];
    }
}

// d[i]: (float)acc of columns n..n+3 of row m; ss: the row's source scale
QMM_D void epilogue_rows4(const epilogue_t &ep, const ep_cols_t &c,
        float (&d)[4], bool has_ss, float ss, int64_t b, int64_t m, int64_t n,
        int nvalid) {
    // an absent scale is the factor 1.0f: x * 1.0f is x bit for bit, so the
    // multiplications need no branch (has_ss only says where ss came from)
    (void)has_ss;
#pragma unroll
    for (int i = 0; i < 4; i++)
        d[i] = d[i] * ss * c.ws[i];
    if (c.has_bias) {
        if (c.bias_per_row) {
            float bv[4];
            ep_load4(ep.bias, b, m, n, nvalid, bv);
#pragma unroll
            for (int i = 0; i < 4; i++)
                d[i] += bv[i];
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++)
                d[i] += c.bias[i];
        }
    }
    const int64_t dst_off = b * ep.dst.sb + m * ep.dst.sm + n * ep.dst.sn;
    // The first two post-ops are addressed with constant indices: what they
    // read from the parameter block does not depend on the row, so a caller's
    // row loop fetches it once instead of once per row.
    if (ep.npo > 0) epilogue_post_op4(ep, ep.po[0], d, b, m, n, nvalid);
    if (ep.npo > 1) epilogue_post_op4(ep, ep.po[1], d, b, m, n, nvalid);
#pragma unroll 1
    for (int pi = 2; pi < ep.npo; pi++)
        epilogue_post_op4(ep, ep.po[pi], d, b, m, n, nvalid);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        d[i] *= c.inv_dst_scale; // 1.0f when there is no dst scale
        d[i] = c.has_zp ? d[i] + c.zp[i] : d[i];
    }
    epilogue_store4(ep, d, dst_off, nvalid);
}

// one-off form: column operands fetched on the spot
QMM_D void epilogue_apply_store4(const epilogue_t &ep, float (&d)[4],
        int64_t b, int64_t m, int64_t n, int nvalid) {
    ep_cols_t c;
    epilogue_cols_load(ep, c, b, n, nvalid);
    const bool has_ss = ep.src_scale.ptr != nullptr;
    const float ss = has_ss ? ep_load(ep.src_scale, b, m, 0) : 1.f;
    epilogue_rows4(ep, c, d, has_ss, ss, b, m, n, nvalid);
}

// Straight-line epilogue for the EP_FAST_* shapes: d[i] is (float)acc of four
// neighbouring columns n..n+3 of row m. ss / ws are the source and weights
// scales (1.0 when absent is NOT substituted: the flags say whether to
// multiply, so the operation sequence equals the reference's). Everything but
// swish is operation-for-operation the interpreter's arithmetic; swish uses
// the hardware exp2 / rcp (relative error ~4e-7, far inside the 1e-5 / 1 bf16
// ulp bars that any exp implementation other than the reference's libm needs).
QMM_D void epilogue_fast4(const epilogue_t &ep, float (&d)[4], bool has_ss,
        float ss, bool has_ws, const float (&ws)[4], int64_t b, int64_t m,
        int64_t n, int nvalid) {
    if (has_ss) {
#pragma unroll
        for (int i = 0; i < 4; i++)
            d[i] *= ss;
    }
    if (has_ws) {
#pragma unroll
        for (int i = 0; i < 4; i++)
            d[i] *= ws[i];
    }
    const int64_t dst_off = b * ep.dst.sb + m * ep.dst.sm + n;
    const int fast = ep.fast;
    if (fast == EP_FAST_RELU) {
        const float alpha = ep.po[0].alpha;
#pragma unroll
        for (int i = 0; i < 4; i++)
            d[i] = d[i] > 0 ? d[i] : d[i] * alpha;
    } else if (fast == EP_FAST_SWISH) {
        const float na = -ep.po[0].alpha * 1.44269504088896340736f;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float e = __builtin_amdgcn_exp2f(d[i] * na);
            d[i] = d[i] * __builtin_amdgcn_rcpf(1.0f + e);
        }
    } else if (fast == EP_FAST_ADD) {
        const float *q = (const float *)ep.po[0].t.ptr + b * ep.po[0].t.sb
                + m * ep.po[0].t.sm + n;
        if (nvalid == 4 && (((uintptr_t)q) & 15) == 0) {
            const float4 y = *(const float4 *)q;
            d[0] += y.x;
            d[1] += y.y;
            d[2] += y.z;
            d[3] += y.w;
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++)
                if (i < nvalid) d[i] += q[i];
        }
    } else if (fast == EP_FAST_SUM) {
        const float sc = ep.po[0].scale;
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (i < nvalid) {
                const float old = load_float(ep.dst.dt, ep.dst.ptr, dst_off + i);
                d[i] += sc * (old - 0.f);
            }
    }
    if (ep.dst.dt == dt_bf16) {
        uint16_t *q = (uint16_t *)ep.dst.ptr + dst_off;
        uint16_t h[4];
#pragma unroll
        for (int i = 0; i < 4; i++)
            h[i] = f32_to_bf16(d[i]);
        if (nvalid == 4 && (((uintptr_t)q) & 7) == 0) {
            *(uint2 *)q = make_uint2((uint32_t)h[0] | ((uint32_t)h[1] << 16),
                    (uint32_t)h[2] | ((uint32_t)h[3] << 16));
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++)
                if (i < nvalid) q[i] = h[i];
        }
    } else { // f32
        float *q = (float *)ep.dst.ptr + dst_off;
        if (nvalid == 4 && (((uintptr_t)q) & 15) == 0) {
            *(float4 *)q = make_float4(d[0], d[1], d[2], d[3]);
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++)
                if (i < nvalid) q[i] = d[i];
        }
    }
}

// Straight-line epilogue of four neighbouring results of one row when nothing
// has to be checked per lane: the four columns exist, dst (and a binary
// operand) can be accessed as one vector. FAST is the recognised shape, BF16
// the dst type. bf16 results are packed by v_cvt_pk_bf16_f32 (round to nearest
// even); the caller runs with f32 denormals flushed (see
// epilogue_flush_denormals), which reproduces the reference conversion's
// subnormal -> +-0 (src/common/bfloat16.cpp:22-56). Absent scales are passed
// as 1.0, which is exact.
QMM_D void epilogue_flush_denormals() {
    // MODE register, FP_DENORM field for single precision (bits 5:4) = flush
    __builtin_amdgcn_s_setreg(1 | (4 << 6) | (1 << 11), 0);
}

// Straight-line epilogue of the 256 x 256 kernels for full tiles: no control
// flow at all, so that eight rows are in flight at a time. FAST is the post-op
// shape, DSTK the dst type (EP_DST_*); EXT adds what ep.fast_ext announces: a
// per-column bias, the dst scale and dst zero points, each applied through a
// select or as the factor 1.0f so that an absent one changes no bit.
enum : int { EP_DST_F32 = 0, EP_DST_BF16 = 1, EP_DST_F16 = 2,
    EP_DST_Q8 = 3 /* s8 or u8 */ };

// The post-ops that read a second tensor (binary operand, old dst of a sum)
// fetch 8 or 16 bytes per lane and row. The loads cannot be left to the
// compiler's scheduling: it has to assume that the dst store of one row
// aliases the operand load of the next, which leaves one row's load in flight
// at a time. ep_operand_load issues the load on its own, so that a caller can
// request a batch of rows before the first store, and hands the result to
// epilogue_full4<.., PRE = true>.
template <int FAST>
constexpr bool ep_reads_operand() {
    return FAST == EP_FAST_ADD || FAST == EP_FAST_SUM || FAST == EP_FAST_BIN32
            || FAST == EP_FAST_BIN16;
}

template <int FAST, int DSTK>
QMM_D uint4 ep_operand_load(const epilogue_t &ep, const ep_cols_t &c,
        int64_t bz, int64_t m, int64_t en) {
    if constexpr (FAST == EP_FAST_ADD) {
        return *(const uint4 *)((const float *)ep.po[0].t.ptr
                + bz * ep.po[0].t.sb + m * ep.po[0].t.sm + en);
    } else if constexpr (FAST == EP_FAST_BIN32) {
        return *(const uint4 *)((const float *)c.bin_ptr + m * c.bin_sm);
    } else if constexpr (FAST == EP_FAST_BIN16) {
        const uint2 v
                = *(const uint2 *)((const uint16_t *)c.bin_ptr + m * c.bin_sm);
        return make_uint4(v.x, v.y, 0, 0);
    } else if constexpr (FAST == EP_FAST_SUM) {
        const int64_t dst_off = bz * ep.dst.sb + m * ep.dst.sm + en;
        if constexpr (DSTK == EP_DST_F32) {
            return *(const uint4 *)((const float *)ep.dst.ptr + dst_off);
        } else {
            const uint2 v
                    = *(const uint2 *)((const uint16_t *)ep.dst.ptr + dst_off);
            return make_uint4(v.x, v.y, 0, 0);
        }
    } else {
        return make_uint4(0, 0, 0, 0);
    }
}

template <int FAST, int DSTK, bool EXT, bool PRE = false>
QMM_D void epilogue_full4(const epilogue_t &ep, const ep_cols_t &c,
        float (&d)[4], float ss, int64_t bz, int64_t m, int64_t en,
        uint4 pre = make_uint4(0, 0, 0, 0)) {
    if constexpr (!PRE && ep_reads_operand<FAST>())
        pre = ep_operand_load<FAST, DSTK>(ep, c, bz, m, en);
    const float alpha = FAST == EP_FAST_RELU || FAST == EP_FAST_SWISH
            ? ep.po[0].alpha
            : 0.f;
    const float na = -alpha * 1.44269504088896340736f;
    const float sum_scale = FAST == EP_FAST_SUM ? ep.po[0].scale : 0.f;
    // absent scales are 1.0 (exact)
#pragma unroll
    for (int i = 0; i < 4; i++)
        d[i] = d[i] * ss * c.ws[i];
    if constexpr (EXT) {
#pragma unroll
        for (int i = 0; i < 4; i++)
            d[i] = c.has_bias ? d[i] + c.bias[i] : d[i];
    }
    const int64_t dst_off = bz * ep.dst.sb + m * ep.dst.sm + en;
    if constexpr (FAST == EP_FAST_RELU) {
#pragma unroll
        for (int i = 0; i < 4; i++)
            d[i] = d[i] > 0 ? d[i] : d[i] * alpha;
    } else if constexpr (FAST == EP_FAST_SWISH) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float e = __builtin_amdgcn_exp2f(d[i] * na);
            d[i] = d[i] * __builtin_amdgcn_rcpf(1.0f + e);
        }
    } else if constexpr (FAST == EP_FAST_ADD) {
        d[0] += u2f(pre.x);
        d[1] += u2f(pre.y);
        d[2] += u2f(pre.z);
        d[3] += u2f(pre.w);
    } else if constexpr (FAST == EP_FAST_GELU_ERF || FAST == EP_FAST_GELU_TANH) {
#pragma unroll
        for (int i = 0; i < 4; i++)
            d[i] = eltwise_fwd(FAST == EP_FAST_GELU_ERF ? alg_gelu_erf
                                                        : alg_gelu_tanh,
                           d[i], ep.po[0].alpha, ep.po[0].beta)
                    * ep.po[0].scale;
    } else if constexpr (FAST == EP_FAST_BIN32 || FAST == EP_FAST_BIN16) {
        const bool mul = c.bin_mul != 0;
        float y[4];
        if constexpr (FAST == EP_FAST_BIN32) {
            y[0] = u2f(pre.x);
            y[1] = u2f(pre.y);
            y[2] = u2f(pre.z);
            y[3] = u2f(pre.w);
        } else {
            const uint2 v = make_uint2(pre.x, pre.y);
            const uint16_t h[4] = {(uint16_t)v.x, (uint16_t)(v.x >> 16),
                    (uint16_t)v.y, (uint16_t)(v.y >> 16)};
            const bool f16 = c.bin_f16 != 0;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float a = (float)__builtin_bit_cast(_Float16, h[i]);
                const float b = u2f((uint32_t)h[i] << 16);
                y[i] = f16 ? a : b;
            }
        }
#pragma unroll
        for (int i = 0; i < 4; i++)
            d[i] = mul ? d[i] * y[i] : d[i] + y[i];
    } else if constexpr (FAST == EP_FAST_SUM) {
        static_assert(FAST != EP_FAST_SUM || DSTK <= EP_DST_F16, "");
        float o[4];
        if constexpr (DSTK == EP_DST_F32) {
            o[0] = u2f(pre.x);
            o[1] = u2f(pre.y);
            o[2] = u2f(pre.z);
            o[3] = u2f(pre.w);
        } else {
            const uint2 v = make_uint2(pre.x, pre.y);
            if constexpr (DSTK == EP_DST_BF16) {
                o[0] = u2f(v.x << 16);
                o[1] = u2f(v.x & 0xFFFF0000u);
                o[2] = u2f(v.y << 16);
                o[3] = u2f(v.y & 0xFFFF0000u);
            } else {
                o[0] = (float)__builtin_bit_cast(_Float16, (uint16_t)v.x);
                o[1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(v.x >> 16));
                o[2] = (float)__builtin_bit_cast(_Float16, (uint16_t)v.y);
                o[3] = (float)__builtin_bit_cast(_Float16, (uint16_t)(v.y >> 16));
            }
        }
#pragma unroll
        for (int i = 0; i < 4; i++)
            d[i] += sum_scale * (o[i] - 0.f);
    }
    if constexpr (EXT) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            d[i] *= c.inv_dst_scale;
            d[i] = c.has_zp ? d[i] + c.zp[i] : d[i];
        }
    }
    typedef unsigned v2u __attribute__((ext_vector_type(2)));
    if constexpr (DSTK == EP_DST_BF16) {
        if constexpr (EXT) {
            // f32 subnormals convert to +-0 (src/common/bfloat16.cpp:22-56); the
            // kernels that never take this branch get that from the FP mode
#pragma unroll
            for (int i = 0; i < 4; i++)
                d[i] = __builtin_fabsf(d[i]) < 1.17549435e-38f
                        ? __builtin_copysignf(0.f, d[i])
                        : d[i];
        }
        uint32_t h0, h1;
        asm("v_cvt_pk_bf16_f32 %0, %1, %2"
                : "=v"(h0)
                : "v"(d[0]), "v"(d[1]));
        asm("v_cvt_pk_bf16_f32 %0, %1, %2"
                : "=v"(h1)
                : "v"(d[2]), "v"(d[3]));
        *(v2u *)((uint16_t *)ep.dst.ptr + dst_off) = v2u {h0, h1};
    } else if constexpr (DSTK == EP_DST_F16) {
        const uint32_t h0 = (uint32_t)f32_to_f16_hw(d[0])
                | ((uint32_t)f32_to_f16_hw(d[1]) << 16);
        const uint32_t h1 = (uint32_t)f32_to_f16_hw(d[2])
                | ((uint32_t)f32_to_f16_hw(d[3]) << 16);
        *(v2u *)((uint16_t *)ep.dst.ptr + dst_off) = v2u {h0, h1};
    } else if constexpr (DSTK == EP_DST_Q8) {
        const float lo = ep.dst.dt == dt_s8 ? -128.f : 0.f;
        const float hi = ep.dst.dt == dt_s8 ? 127.f : 255.f;
        uint32_t w = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float v = d[i];
            v = v < lo ? lo : v;
            v = v > hi ? hi : v;
            const int r = (int)__builtin_rintf(v); // NaN -> 0, as the reference's low byte
            w |= (uint32_t)(r & 0xff) << (8 * i);
        }
        *(uint32_t *)((uint8_t *)ep.dst.ptr + dst_off) = w;
    } else {
        typedef float v4fl __attribute__((ext_vector_type(4)));
        __builtin_nontemporal_store(v4fl {d[0], d[1], d[2], d[3]},
                (v4fl *)((float *)ep.dst.ptr + dst_off));
    }
}

// wave-uniform test for epilogue_full4: dst rows (and a binary operand's)
// aligned for vector access
QMM_D bool epilogue_full4_ok(const epilogue_t &ep) {
    bool ok = (ep.dst.sm & 3) == 0 && (ep.dst.sb & 3) == 0
            && ((uintptr_t)ep.dst.ptr & 15) == 0 && ep.fast != EP_FAST_NONE;
    if (ep.fast == EP_FAST_ADD || ep.fast == EP_FAST_BIN32
            || ep.fast == EP_FAST_BIN16)
        ok = ok && (ep.po[0].t.sm & 3) == 0 && (ep.po[0].t.sb & 3) == 0
                && ((uintptr_t)ep.po[0].t.ptr & 15) == 0;
    return ok;
}

} // namespace qmm
