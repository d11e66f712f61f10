// hip:gfx950:softmax -- forward softmax / log-softmax over one axis, the step
// between the two matmuls of an attention block (scores -> probabilities).
// Semantics: src/cpu/ref_softmax.cpp:40-193 (axis innermost, src and dst of
// one type and one dense layout, ref_softmax.hpp:137-139: the result is
// exp(s - max) * (1 / sum)) and :196-312 (anything else: exp(s - max) / sum);
// then * src_scale, * (1 / dst_scale), conversion to the destination type.
// All arithmetic in f32; the exponentials stay in registers, so no
// intermediate buffer exists.
//
// Bound: HBM. A row is read once and written once.
#include <hip/hip_runtime.h>

#include <string.h>

#include <string>

#include "qmm_device.hpp"
#include "qmm_hip.h"

namespace qmm {
namespace {

enum { alg_softmax_accurate = 0x30000, alg_softmax_log = 0x30001 }; // dnnl_alg_kind_t

struct softmax_params_t {
    const void *src;
    void *dst;
    const void *src_scale, *dst_scale;
    int32_t src_dt, dst_dt, src_scale_dt, dst_scale_dt;
    int32_t log_softmax;
    int32_t recip; // row kernel: multiply by 1 / sum (else divide by sum)
    int64_t channels; // extent of the softmax axis
    int64_t rows; // product of the other dims (row kernel) / outer * inner
    // row kernel: rows are indexed by the other dims, outermost first
    int32_t nouter, pad2_;
    int64_t odims[QMM_MAX_NDIMS], src_ostr[QMM_MAX_NDIMS],
            dst_ostr[QMM_MAX_NDIMS];
    int64_t src_cstr, dst_cstr; // stride of the softmax axis (generic kernel)
};

QMM_D float wave_max(float v) {
#pragma unroll
    for (int o = 32; o; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}
QMM_D float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

// exp(d) for d <= 0 on the hardware's 2^x: the argument d * log2(e) is formed
// in two parts (the rounded product and its exact remainder plus the part of
// log2(e) a float does not hold), the 2^x of the first is corrected by the
// second, so the error does not grow with |d| (a bare 2^(d * log2e) is off by
// |d| * 2^-24 relative). About 2 ulp; results below the normal range are 0.
QMM_D float exp_nonpos(float d) {
    constexpr float L2E = 1.44269502162933349609375f; // (float)log2(e)
    constexpr float L2E_LO = 1.925963033500011e-08f; // log2(e) - (float)log2(e)
    constexpr float LN2 = 0.693147182464599609375f;
    // below -150 the result is 0 in f32 either way; the clamp keeps -inf (a
    // masked position) out of the remainder arithmetic, where it would turn
    // into inf - inf
    d = fmaxf(d, -150.f);
    const float hi = d * L2E;
    float lo = __builtin_fmaf(d, L2E, -hi);
    lo = __builtin_fmaf(d, L2E_LO, lo);
    const float e = __builtin_amdgcn_exp2f(hi);
    return __builtin_fmaf(e, lo * LN2, e);
}

QMM_D void row_offsets(const softmax_params_t &p, int64_t row, int64_t &so,
        int64_t &dof) {
    so = 0;
    dof = 0;
    for (int d = p.nouter - 1; d >= 0; d--) {
        const int64_t i = row % p.odims[d];
        row /= p.odims[d];
        so += i * p.src_ostr[d];
        dof += i * p.dst_ostr[d];
    }
}

// four consecutive elements of a row as floats (the row start is aligned to
// four elements of its type: checked on the host)
template <int DT>
QMM_D void load4(const void *base, int64_t idx, float (&v)[4]) {
    if constexpr (DT == dt_f32) {
        const float4 x = *(const float4 *)((const float *)base + idx);
        v[0] = x.x, v[1] = x.y, v[2] = x.z, v[3] = x.w;
    } else if constexpr (DT == dt_bf16 || DT == dt_f16) {
        const uint2 x = *(const uint2 *)((const uint16_t *)base + idx);
        const uint16_t h[4] = {(uint16_t)x.x, (uint16_t)(x.x >> 16),
                (uint16_t)x.y, (uint16_t)(x.y >> 16)};
#pragma unroll
        for (int i = 0; i < 4; i++)
            v[i] = DT == dt_bf16 ? bf16_to_f32(h[i]) : f16_to_f32(h[i]);
    } else {
        const uint32_t x = *(const uint32_t *)((const uint8_t *)base + idx);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t b = (x >> (8 * i)) & 0xff;
            v[i] = DT == dt_s8 ? (float)(int8_t)b : (float)b;
        }
    }
}

// Row kernel: the softmax axis is innermost with stride 1 in src and dst. One
// wave per row; the row lives in registers (up to MAXV groups of four elements
// per lane), longer rows are re-read from memory for each of the three passes.
template <int SDT>
__global__ void __launch_bounds__(256)
softmax_rows_kernel(const softmax_params_t p) {
    constexpr int MAXV = 16; // 64 lanes x 16 x 4 = 4096 elements in registers
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= p.rows) return;
    int64_t so, dof;
    row_offsets(p, row, so, dof);
    const int64_t C = p.channels;
    const int64_t C4 = C / 4; // whole groups of four; the tail is scalar
    const bool in_regs = C4 <= 64 * MAXV;
    const size_t ssz = SDT == dt_f32 ? 4 : (SDT == dt_bf16 || SDT == dt_f16) ? 2 : 1;
    const uint8_t *srow = (const uint8_t *)p.src + so * ssz;

    float v[MAXV][4];
    float mx = -3.402823466e+38f;
    if (in_regs) {
        // every load of the row is issued before the first value is used:
        // groups past the row's end re-read its last group and are ignored
#pragma unroll
        for (int g = 0; g < MAXV; g++) {
            if (64 * g < C4) { // wave uniform
                const int64_t q = lane + 64 * g;
                load4<SDT>(srow, (q < C4 ? q : C4 - 1) * 4, v[g]);
            }
        }
#pragma unroll
        for (int g = 0; g < MAXV; g++) {
            if (lane + 64 * g < C4)
                mx = fmaxf(mx, fmaxf(fmaxf(v[g][0], v[g][1]),
                                       fmaxf(v[g][2], v[g][3])));
        }
    } else {
        for (int64_t q = lane; q < C4; q += 64) {
            float t[4];
            load4<SDT>(srow, q * 4, t);
            mx = fmaxf(mx, fmaxf(fmaxf(t[0], t[1]), fmaxf(t[2], t[3])));
        }
    }
    for (int64_t c = C4 * 4 + lane; c < C; c += 64)
        mx = fmaxf(mx, load_float(SDT, srow, c));
    mx = wave_max(mx);

    float sum = 0.f;
    if (in_regs) {
#pragma unroll
        for (int g = 0; g < MAXV; g++) {
            if (lane + 64 * g < C4) {
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float d = v[g][i] - mx;
                    const float e = exp_nonpos(d);
                    sum += e;
                    v[g][i] = p.log_softmax ? d : e;
                }
            }
        }
    } else {
        for (int64_t q = lane; q < C4; q += 64) {
            float t[4];
            load4<SDT>(srow, q * 4, t);
#pragma unroll
            for (int i = 0; i < 4; i++) sum += exp_nonpos(t[i] - mx);
        }
    }
    for (int64_t c = C4 * 4 + lane; c < C; c += 64)
        sum += exp_nonpos(load_float(SDT, srow, c) - mx);
    sum = wave_sum(sum);

    // src/cpu/ref_softmax.cpp:160-182 (src and dst of one type and layout: the
    // reciprocal of the sum is taken once) and :270-290 (otherwise: division)
    const float denom = p.log_softmax
            ? logf(sum)
            : (p.recip ? (sum != 0.f ? 1.f / sum : 1.f) : sum);
    const float ss = p.src_scale ? load_float(p.src_scale_dt, p.src_scale, 0) : 1.f;
    const float ds = p.dst_scale
            ? 1.f / load_float(p.dst_scale_dt, p.dst_scale, 0)
            : 1.f;
    auto finish = [&](float d) {
        float val = p.log_softmax ? d - denom
                                  : (p.recip ? d * denom : d / denom);
        val *= ss;
        val *= ds;
        return val;
    };
    const int ddt = p.dst_dt;
    auto store4 = [&](int64_t idx, const float (&o)[4]) {
        if (ddt == dt_f32) {
            *(float4 *)((float *)p.dst + dof + idx)
                    = make_float4(o[0], o[1], o[2], o[3]);
        } else if (ddt == dt_bf16 || ddt == dt_f16) {
            uint16_t h[4];
#pragma unroll
            for (int i = 0; i < 4; i++)
                h[i] = ddt == dt_bf16
                        ? f32_to_bf16(o[i])
                        // the hardware conversion: round to nearest even,
                        // subnormals kept, as src/common/float16.hpp:52-127
                        : __builtin_bit_cast(uint16_t, (_Float16)o[i]);
            *(uint2 *)((uint16_t *)p.dst + dof + idx) = make_uint2(
                    h[0] | ((uint32_t)h[1] << 16), h[2] | ((uint32_t)h[3] << 16));
        } else {
            // saturate, round to nearest even, four bytes in one store
            // (src/cpu/ref_io_helper.hpp store_float_value -> saturate_and_round)
            const float lo = ddt == dt_s8 ? -128.f : 0.f, hi = ddt == dt_s8 ? 127.f : 255.f;
            uint32_t w = 0;
#pragma unroll
            for (int i = 0; i < 4; i++)
                w |= ((uint32_t)round_sat(o[i], lo, hi) & 0xffu) << (8 * i);
            *(uint32_t *)((uint8_t *)p.dst + dof + idx) = w;
        }
    };
    if (in_regs) {
#pragma unroll
        for (int g = 0; g < MAXV; g++) {
            const int64_t q = lane + 64 * g;
            if (q < C4) {
                float o[4];
#pragma unroll
                for (int i = 0; i < 4; i++) o[i] = finish(v[g][i]);
                store4(q * 4, o);
            }
        }
    } else {
        for (int64_t q = lane; q < C4; q += 64) {
            float t[4], o[4];
            load4<SDT>(srow, q * 4, t);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float d = t[i] - mx;
                o[i] = finish(p.log_softmax ? d : exp_nonpos(d));
            }
            store4(q * 4, o);
        }
    }
    for (int64_t c = C4 * 4 + lane; c < C; c += 64) {
        const float d = load_float(SDT, srow, c) - mx;
        store_float(ddt, finish(p.log_softmax ? d : exp_nonpos(d)), p.dst, dof + c);
    }
}

// Any axis, any strides: one thread per (outer, inner) position walks the
// axis three times (src/cpu/ref_softmax.cpp:196-312: division by the sum).
__global__ void __launch_bounds__(256)
softmax_generic_kernel(const softmax_params_t p) {
    const int64_t row = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (row >= p.rows) return;
    int64_t so, dof;
    row_offsets(p, row, so, dof);
    float mx = -3.402823466e+38f;
    for (int64_t c = 0; c < p.channels; c++)
        mx = fmaxf(mx, load_float(p.src_dt, p.src, so + c * p.src_cstr));
    float sum = 0.f;
    for (int64_t c = 0; c < p.channels; c++)
        sum += expf(load_float(p.src_dt, p.src, so + c * p.src_cstr) - mx);
    const float denom = p.log_softmax ? logf(sum) : sum;
    const float ss = p.src_scale ? load_float(p.src_scale_dt, p.src_scale, 0) : 1.f;
    const float ds = p.dst_scale
            ? 1.f / load_float(p.dst_scale_dt, p.dst_scale, 0)
            : 1.f;
    for (int64_t c = 0; c < p.channels; c++) {
        float d = load_float(p.src_dt, p.src, so + c * p.src_cstr) - mx;
        if (p.log_softmax)
            d -= denom;
        else
            d = expf(d) / denom;
        d *= ss;
        d *= ds;
        store_float(p.dst_dt, d, p.dst, dof + c * p.dst_cstr);
    }
}

bool float_or_int8(int dt) {
    return dt == dt_f32 || dt == dt_bf16 || dt == dt_f16 || dt == dt_s8
            || dt == dt_u8;
}

size_t dt_bytes(int dt) {
    return dt == dt_f32 ? 4 : (dt == dt_bf16 || dt == dt_f16) ? 2 : 1;
}

bool supported(const qmm_softmax_desc_t &d) {
    if (d.src.ndims < 1 || d.src.ndims > QMM_MAX_NDIMS) return false;
    if (d.dst.ndims != d.src.ndims) return false;
    for (int i = 0; i < d.src.ndims; i++)
        if (d.src.dims[i] != d.dst.dims[i] || d.src.dims[i] < 0) return false;
    if (d.axis < 0 || d.axis >= d.src.ndims) return false;
    if (!float_or_int8(d.src.dt) || !float_or_int8(d.dst.dt)) return false;
    if (d.alg != alg_softmax_accurate && d.alg != alg_softmax_log) return false;
    for (const qmm_quant_t *q : {&d.src_scale, &d.dst_scale})
        if (q->set
                && (q->mask != 0
                        || (q->dt != dt_f32 && q->dt != dt_f16
                                && q->dt != dt_bf16)))
            return false;
    return true;
}

// the row kernel's conditions (ref_softmax.hpp: dense implementation when the
// axis is the innermost one and src and dst share one dense layout)
bool rows_path(const qmm_softmax_desc_t &d) {
    const int nd = d.src.ndims;
    if (d.src.strides[d.axis] != 1 || d.dst.strides[d.axis] != 1) return false;
    const int64_t C = d.src.dims[d.axis];
    // same layout, no gaps: sorting the other dims by stride must give a dense
    // nest over rows of C elements, identically in src and dst
    int order[QMM_MAX_NDIMS], n = 0;
    for (int i = 0; i < nd; i++)
        if (i != d.axis) order[n++] = i;
    for (int i = 0; i < n; i++)
        for (int j = i + 1; j < n; j++)
            if (d.src.strides[order[j]] < d.src.strides[order[i]]) {
                const int t = order[i];
                order[i] = order[j];
                order[j] = t;
            }
    int64_t expect = C;
    for (int i = 0; i < n; i++) {
        const int k = order[i];
        if (d.src.dims[k] == 1) continue;
        if (d.src.strides[k] != expect || d.dst.strides[k] != expect)
            return false;
        expect *= d.src.dims[k];
    }
    // vector accesses: rows start on 16-byte (f32), 8-byte (16-bit) or 4-byte
    // (8-bit) boundaries when C is a multiple of 4; other C use scalar tails
    // only if every row start stays aligned, i.e. a single row
    if (C % 4 != 0) {
        int64_t rows = 1;
        for (int i = 0; i < nd; i++)
            if (i != d.axis) rows *= d.src.dims[i];
        if (rows != 1) return false;
    }
    return true;
}

} // namespace
} // namespace qmm

using namespace qmm;

extern "C" {

int qmm_softmax_supports(const qmm_softmax_desc_t *desc) {
    if (!desc) return QMM_INVALID_ARGUMENTS;
    return supported(*desc) ? QMM_OK : QMM_UNIMPLEMENTED;
}

const char *qmm_softmax_impl_name(const qmm_softmax_desc_t *desc) {
    if (!desc || !supported(*desc)) return "";
    return rows_path(*desc) ? "hip:gfx950:softmax_rows" : "hip:gfx950:softmax_generic";
}

int qmm_softmax_launch(const qmm_softmax_desc_t *desc,
        const qmm_softmax_args_t *args, void *hip_stream) {
    if (!desc || !args) return QMM_INVALID_ARGUMENTS;
    if (!supported(*desc)) return QMM_UNIMPLEMENTED;
    const qmm_softmax_desc_t &d = *desc;
    if (!args->src || !args->dst) return QMM_INVALID_ARGUMENTS;
    if ((d.src_scale.set && !args->src_scale)
            || (d.dst_scale.set && !args->dst_scale))
        return QMM_INVALID_ARGUMENTS;
    softmax_params_t p;
    ::memset(&p, 0, sizeof(p));
    p.src = args->src;
    p.dst = args->dst;
    p.src_scale = d.src_scale.set ? args->src_scale : nullptr;
    p.dst_scale = d.dst_scale.set ? args->dst_scale : nullptr;
    p.src_dt = d.src.dt;
    p.dst_dt = d.dst.dt;
    p.src_scale_dt = d.src_scale.dt;
    p.dst_scale_dt = d.dst_scale.dt;
    p.log_softmax = d.alg == alg_softmax_log;
    p.recip = d.src.dt == d.dst.dt;
    p.channels = d.src.dims[d.axis];
    p.src_cstr = d.src.strides[d.axis];
    p.dst_cstr = d.dst.strides[d.axis];
    p.rows = 1;
    for (int i = 0; i < d.src.ndims; i++) {
        if (i == d.axis) continue;
        p.odims[p.nouter] = d.src.dims[i];
        p.src_ostr[p.nouter] = d.src.strides[i];
        p.dst_ostr[p.nouter] = d.dst.strides[i];
        p.nouter++;
        p.rows *= d.src.dims[i];
    }
    if (p.rows == 0 || p.channels == 0) return QMM_OK;
    hipStream_t stream = (hipStream_t)hip_stream;
    const bool rows = rows_path(d)
            && ((uintptr_t)args->src % (4 * dt_bytes(d.src.dt)) == 0)
            && ((uintptr_t)args->dst % (4 * dt_bytes(d.dst.dt)) == 0);
    if (rows) {
        const unsigned grid = (unsigned)((p.rows + 3) / 4);
        switch (d.src.dt) {
            case dt_f32:
                hipLaunchKernelGGL(softmax_rows_kernel<dt_f32>, dim3(grid),
                        dim3(256), 0, stream, p);
                break;
            case dt_bf16:
                hipLaunchKernelGGL(softmax_rows_kernel<dt_bf16>, dim3(grid),
                        dim3(256), 0, stream, p);
                break;
            case dt_f16:
                hipLaunchKernelGGL(softmax_rows_kernel<dt_f16>, dim3(grid),
                        dim3(256), 0, stream, p);
                break;
            case dt_s8:
                hipLaunchKernelGGL(softmax_rows_kernel<dt_s8>, dim3(grid),
                        dim3(256), 0, stream, p);
                break;
            default:
                hipLaunchKernelGGL(softmax_rows_kernel<dt_u8>, dim3(grid),
                        dim3(256), 0, stream, p);
                break;
        }
    } else {
        hipLaunchKernelGGL(softmax_generic_kernel,
                dim3((unsigned)((p.rows + 255) / 256)), dim3(256), 0, stream, p);
    }
    return hipGetLastError() == hipSuccess ? QMM_OK : QMM_RUNTIME_ERROR;
}

} // extern "C"
