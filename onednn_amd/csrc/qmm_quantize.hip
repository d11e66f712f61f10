// hip:gfx950:quantize -- the reorder as a quantizer (f32 / bf16 / f16 ->
// s8 / u8 / s4 / u4 / f8 / 16-bit / f32 with scales and zero points,
// src/cpu/reorder/simple_reorder.hpp:2500-2640) for the case that matters at
// run time: both tensors row-major with the same dim order, i.e. an
// element-wise pass. It is a stream: a thread converts 8 neighbouring
// elements of a row (32 or 16 bytes in, 4 to 32 bytes out) for 8 rows in turn,
// so that per-column scales are fetched and inverted once. The arithmetic is the reference's, in its order:
//     d = src_scale * (in - src_zp);  d = d * (1 / dst_scale) + dst_zp;
// followed by the saturating / rounding store of the dst type. Everything else
// (transposing reorders, scales over leading dims of tensors with more than
// two dims) stays with the per-element kernel in qmm_generic.hip.
#include "qmm_device.hpp"
#include "qmm_plan.hpp"

namespace qmm {

// scales / zero points as a function of (row, col): element
// (row / gr) * sr + (col / gc) * sc of the buffer
QMM_D int64_t qr_off(const quant_rows_q_t &q, int64_t row, int64_t col) {
    return (row / q.gr) * q.sr + (col / q.gc) * q.sc;
}

// Rows per thread: 8 where an operand depends on the column only (it is
// fetched, and a dst scale inverted, once for all of them), else 1 (more
// threads in flight).
constexpr int QR_ROWS = 8;

QMM_D void qr_fetch_scale(const quant_rows_q_t &q, int64_t row, int64_t col,
        bool one, bool invert, float (&out)[8]) {
    if (one) {
        float v = load_float(q.dt, q.ptr, qr_off(q, row, col));
        if (invert) v = 1.f / v;
#pragma unroll
        for (int i = 0; i < 8; i++)
            out[i] = v;
    } else if (q.dt == dt_f32 && q.gc == 1) {
        // eight neighbouring f32 entries: two vector loads (the entry index is
        // a multiple of 8 and the buffer is 16-byte aligned, host-checked)
        const float4 *s = (const float4 *)((const float *)q.ptr
                + qr_off(q, row, col));
        const float4 a = s[0], b = s[1];
        const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
        for (int i = 0; i < 8; i++)
            out[i] = invert ? 1.f / v[i] : v[i];
    } else {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const float v = load_float(q.dt, q.ptr, qr_off(q, row, col + i));
            out[i] = invert ? 1.f / v : v;
        }
    }
}

template <int RPT>
__global__ void __launch_bounds__(256)
quantize_rows_kernel(const quant_rows_params_t p) {
    const int64_t c8 = p.cols / 8;
    constexpr int rpt = RPT;
    const int64_t row_blocks = (p.rows + rpt - 1) / rpt;
    const int64_t total = row_blocks * c8;
    const bool f32_in = p.src_dt == dt_f32;
    // a buffer that does not change within 8 columns is read once per row
    const bool ss_one = !p.src_scale.ptr || p.src_scale.sc == 0
            || p.src_scale.gc % 8 == 0;
    const bool ds_one = !p.dst_scale.ptr || p.dst_scale.sc == 0
            || p.dst_scale.gc % 8 == 0;
    const bool sz_one
            = !p.src_zp.ptr || p.src_zp.sc == 0 || p.src_zp.gc % 8 == 0;
    // ... and one that does not depend on the row, once per thread
    const bool ss_col = p.src_scale.ptr && p.src_scale.sr == 0;
    const bool ds_col = p.dst_scale.ptr && p.dst_scale.sr == 0;
    const bool sz_col = p.src_zp.ptr && p.src_zp.sr == 0;
    const float dst_zp = p.dst_zp ? (float)p.dst_zp[0] : 0.f;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total;
            t += (int64_t)gridDim.x * blockDim.x) {
        const int64_t row0 = (t / c8) * rpt, col = (t % c8) * 8;
        float ss[8], ds[8], szf[8];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            ss[i] = 1.f;
            ds[i] = 1.f;
            szf[i] = 0.f;
        }
        if (ss_col) qr_fetch_scale(p.src_scale, 0, col, ss_one, false, ss);
        if (ds_col) qr_fetch_scale(p.dst_scale, 0, col, ds_one, true, ds);
        if (sz_col) qr_fetch_scale(p.src_zp, 0, col, sz_one, false, szf);
        const int nrows = (int)min((int64_t)rpt, p.rows - row0);
#pragma unroll(RPT > 1 ? 2 : 1)
        for (int rr = 0; rr < nrows; rr++) {
            const int64_t row = row0 + rr;
            float in[8];
            if (f32_in) {
                typedef float v4fl __attribute__((ext_vector_type(4)));
                const v4fl *s = (const v4fl *)((const float *)p.src
                        + row * p.src_pitch + col);
                const v4fl a = __builtin_nontemporal_load(s);
                const v4fl b = __builtin_nontemporal_load(s + 1);
                in[0] = a[0], in[1] = a[1], in[2] = a[2], in[3] = a[3];
                in[4] = b[0], in[5] = b[1], in[6] = b[2], in[7] = b[3];
            } else {
                const uint4 v = *(const uint4 *)((const uint16_t *)p.src
                        + row * p.src_pitch + col);
                const uint32_t w[4] = {v.x, v.y, v.z, v.w};
                if (p.src_dt == dt_f16) {
#pragma unroll
                    for (int i = 0; i < 8; i++)
                        in[i] = (float)__builtin_bit_cast(_Float16,
                                (uint16_t)(w[i / 2] >> (16 * (i % 2))));
                } else {
#pragma unroll
                    for (int i = 0; i < 8; i++)
                        in[i] = u2f(i % 2 ? (w[i / 2] & 0xFFFF0000u)
                                          : (w[i / 2] << 16));
                }
            }
            if (p.src_scale.ptr && !ss_col)
                qr_fetch_scale(p.src_scale, row, col, ss_one, false, ss);
            if (p.dst_scale.ptr && !ds_col)
                qr_fetch_scale(p.dst_scale, row, col, ds_one, true, ds);
            if (p.src_zp.ptr && !sz_col)
                qr_fetch_scale(p.src_zp, row, col, sz_one, false, szf);
            float d[8];
            if (p.src_zp.ptr) {
#pragma unroll
                for (int i = 0; i < 8; i++) // the zero point is an integer
                    in[i] -= (float)(int)szf[i];
            } else {
#pragma unroll
                for (int i = 0; i < 8; i++)
                    in[i] -= 0.f; // the reference subtracts its default 0 too
            }
#pragma unroll
            for (int i = 0; i < 8; i++)
                d[i] = ss[i] * in[i] * ds[i] + dst_zp;
            const int64_t o = row * p.dst_pitch + col;
            const int ddt = p.dst_dt;
            if (ddt == dt_s8 || ddt == dt_u8) {
                const float lo = ddt == dt_s8 ? -128.f : 0.f;
                const float hi = ddt == dt_s8 ? 127.f : 255.f;
                uint32_t w[2] = {0, 0};
#pragma unroll
                for (int i = 0; i < 8; i++)
                    w[i / 4] |= (uint32_t)(round_sat(d[i], lo, hi) & 0xff)
                            << (8 * (i % 4));
                *(uint2 *)((uint8_t *)p.dst + o) = make_uint2(w[0], w[1]);
            } else if (ddt == dt_s4 || ddt == dt_u4) {
                const float lo = ddt == dt_s4 ? -8.f : 0.f;
                const float hi = ddt == dt_s4 ? 7.f : 15.f;
                uint32_t w = 0;
#pragma unroll
                for (int i = 0; i < 8; i++)
                    w |= (uint32_t)(round_sat(d[i], lo, hi) & 0xf) << (4 * i);
                *(uint32_t *)((uint8_t *)p.dst + (o >> 1)) = w;
            } else if (ddt == dt_bf16 || ddt == dt_f16) {
                uint32_t w[4];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const uint16_t a = ddt == dt_bf16 ? f32_to_bf16(d[2 * i])
                                                      : f32_to_f16(d[2 * i]);
                    const uint16_t b = ddt == dt_bf16
                            ? f32_to_bf16(d[2 * i + 1])
                            : f32_to_f16(d[2 * i + 1]);
                    w[i] = (uint32_t)a | ((uint32_t)b << 16);
                }
                *(uint4 *)((uint16_t *)p.dst + o)
                        = make_uint4(w[0], w[1], w[2], w[3]);
            } else if (ddt == dt_f32) {
                float4 *q = (float4 *)((float *)p.dst + o);
                q[0] = make_float4(d[0], d[1], d[2], d[3]);
                q[1] = make_float4(d[4], d[5], d[6], d[7]);
            } else {
#pragma unroll
                for (int i = 0; i < 8; i++)
                    store_float(ddt, d[i], p.dst, o + i);
            }
        }
    }
}

void launch_quantize_rows(const quant_rows_params_t &p0, hipStream_t stream) {
    quant_rows_params_t p = p0;
    const bool col_only = (p.src_scale.ptr && p.src_scale.sr == 0
                                  && p.src_scale.sc != 0)
            || (p.dst_scale.ptr && p.dst_scale.sr == 0 && p.dst_scale.sc != 0);
    p.rows_per_thread = col_only ? QR_ROWS : 1;
    const int64_t total = ((p.rows + p.rows_per_thread - 1) / p.rows_per_thread)
            * (p.cols / 8);
    if (total <= 0) return;
    int64_t blocks = (total + 255) / 256;
    if (blocks > 262144) blocks = 262144;
    if (col_only)
        hipLaunchKernelGGL(quantize_rows_kernel<QR_ROWS>, dim3((unsigned)blocks),
                dim3(256), 0, stream, p);
    else
        hipLaunchKernelGGL(quantize_rows_kernel<1>, dim3((unsigned)blocks),
                dim3(256), 0, stream, p);
}

} // namespace qmm
