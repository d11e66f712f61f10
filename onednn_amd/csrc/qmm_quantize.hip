// hip:gfx950:quantize -- the reorder as a quantizer (f32 / bf16 / f16 ->
// s8 / u8 / s4 / u4 / f8 / 16-bit / f32 with scales and zero points,
// src/cpu/reorder/simple_reorder.hpp:2500-2640) for the case that matters at
// run time: both tensors row-major with the same dim order, i.e. an
// element-wise pass. It is a stream: a thread converts 8 neighbouring
// elements of a row (32 or 16 bytes in, 4 to 32 bytes out) for 8 rows in turn,
// so that per-column scales are fetched and inverted once. The arithmetic is the reference's, in its order:
//     d = src_scale * (in - src_zp);  d = d * (1 / dst_scale) + dst_zp;
// followed by the saturating / rounding store of the dst type. 2-D tensors
// whose sides disagree on the dim order go through quantize_transpose_kernel
// (a tile through LDS); everything else (scales over leading dims of tensors
// with more than two dims, permutations of more dims) stays with the
// per-element kernel in qmm_generic.hip.
#include "qmm_device.hpp"
#include "qmm_plan.hpp"

namespace qmm {

// scales / zero points as a function of (row, col): element
// (row / gr) * sr + (col / gc) * sc of the buffer
// (rows and columns are below 2^31, host-checked: 32-bit divisions, and none
// where the group is 1 or the stride 0)
QMM_D int64_t qr_off(const quant_rows_q_t &q, int64_t row, int64_t col) {
    const uint32_t r = (uint32_t)row, c = (uint32_t)col;
    const uint32_t rg = q.gr == 1 || q.sr == 0 ? r : r / (uint32_t)q.gr;
    const uint32_t cg = q.gc == 1 || q.sc == 0 ? c : c / (uint32_t)q.gc;
    return (int64_t)rg * q.sr + (int64_t)cg * q.sc;
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
    // A workgroup covers 256 >> tpr_log2 row blocks (of RPT rows) with
    // 1 << tpr_log2 threads each, for one group of 1 << tpr_log2 chunks of 8
    // columns; neighbouring workgroups are neighbours along a row. One 32-bit
    // division per workgroup in the index arithmetic.
    const uint32_t c8 = (uint32_t)(p.cols / 8);
    constexpr int rpt = RPT;
    const uint32_t tpr = 1u << p.tpr_log2;
    const uint32_t rw = blockIdx.x / (uint32_t)p.col_groups;
    const uint32_t cg = blockIdx.x - rw * (uint32_t)p.col_groups;
    const int64_t row0 = ((int64_t)rw * (256u >> p.tpr_log2)
                                 + (threadIdx.x >> p.tpr_log2))
            * rpt;
    if (row0 >= p.rows) return;
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
    const uint32_t cb = cg * tpr + (threadIdx.x & (tpr - 1));
    if (cb < c8) {
        const int64_t col = (int64_t)cb * 8;
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
        constexpr int UN = RPT > 1 ? 2 : 1;
#pragma unroll UN
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

// The quantizer that runs every step (a linear layer's activations): f32 /
// bf16 / f16 rows -> s8 / u8 with nothing but one f32 dst scale for the tensor
// or per row, and a dst zero point. The arithmetic of the kernel above with
// its defaults taken out (1 * x and x - 0 are x): d = in * (1 / scale) + zp,
// each step rounded. A thread converts Q8_CHUNKS chunks of 8 columns,
// 1 << tpr_log2 chunks apart, all requested before the first is used; a
// workgroup covers 256 >> tpr_log2 rows of one group of Q8_CHUNKS << tpr_log2
// chunks.
constexpr int Q8_CHUNKS = 4;
template <int SRC, bool PER_ROW> // SRC: 0 f32, 1 bf16, 2 f16
__global__ void __launch_bounds__(256)
quantize8_kernel(const quant_rows_params_t p) {
    const uint32_t c8 = (uint32_t)(p.cols / 8);
    const uint32_t tpr = 1u << p.tpr_log2;
    const uint32_t rw = blockIdx.x / (uint32_t)p.col_groups;
    const uint32_t cg = blockIdx.x - rw * (uint32_t)p.col_groups;
    const int64_t row = (int64_t)rw * (256u >> p.tpr_log2)
            + (threadIdx.x >> p.tpr_log2);
    if (row >= p.rows) return;
    constexpr int U = Q8_CHUNKS;
    const uint32_t cb0 = cg * U * tpr + (threadIdx.x & (tpr - 1));
    if (cb0 >= c8) return;
    uint32_t cb[U]; // chunks past the row's end read the first again
#pragma unroll
    for (int u = 0; u < U; u++) cb[u] = cb0 + u * tpr < c8 ? cb0 + u * tpr : cb0;
    uint4 raw[U][2];
#pragma unroll
    for (int u = 0; u < U; u++) {
        if constexpr (SRC == 0) {
            const uint4 *s = (const uint4 *)((const float *)p.src
                    + row * p.src_pitch + (int64_t)cb[u] * 8);
            raw[u][0] = s[0];
            raw[u][1] = s[1];
        } else {
            raw[u][0] = *(const uint4 *)((const uint16_t *)p.src
                    + row * p.src_pitch + (int64_t)cb[u] * 8);
        }
    }
    float inv = 1.f;
    if (p.dst_scale.ptr)
        inv = 1.f / ((const float *)p.dst_scale.ptr)[PER_ROW ? row : 0];
    const float dst_zp = p.dst_zp ? (float)p.dst_zp[0] : 0.f;
    const bool sgn = p.dst_dt == dt_s8;
    const float lo = sgn ? -128.f : 0.f, hi = sgn ? 127.f : 255.f;
#pragma unroll
    for (int u = 0; u < U; u++) {
        if (u > 0 && cb0 + u * tpr >= c8) break;
        float in[8];
        if constexpr (SRC == 0) {
            const uint32_t w[8] = {raw[u][0].x, raw[u][0].y, raw[u][0].z,
                    raw[u][0].w, raw[u][1].x, raw[u][1].y, raw[u][1].z,
                    raw[u][1].w};
#pragma unroll
            for (int i = 0; i < 8; i++) in[i] = u2f(w[i]);
        } else {
            const uint32_t w[4]
                    = {raw[u][0].x, raw[u][0].y, raw[u][0].z, raw[u][0].w};
#pragma unroll
            for (int i = 0; i < 8; i++) {
                if constexpr (SRC == 2)
                    in[i] = (float)__builtin_bit_cast(_Float16,
                            (uint16_t)(w[i / 2] >> (16 * (i % 2))));
                else
                    in[i] = u2f(i % 2 ? (w[i / 2] & 0xFFFF0000u)
                                      : (w[i / 2] << 16));
            }
        }
        uint32_t o[2] = {0, 0};
#pragma unroll
        for (int i = 0; i < 8; i++)
            o[i / 4] |= (uint32_t)(round_sat(in[i] * inv + dst_zp, lo, hi) & 0xff)
                    << (8 * (i % 4));
        *(uint2 *)((uint8_t *)p.dst + row * p.dst_pitch + (int64_t)cb[u] * 8)
                = make_uint2(o[0], o[1]);
    }
}

// The same with one f32 dst scale per column (a layer's weights): a thread
// owns one chunk of 8 columns, inverts its 8 scales once and converts 8 rows,
// all of them requested before the first is used.
template <int SRC>
__global__ void __launch_bounds__(256)
quantize8_cols_kernel(const quant_rows_params_t p) {
    constexpr int R = QR_ROWS, V = SRC == 0 ? 2 : 1;
    const uint32_t c8 = (uint32_t)(p.cols / 8);
    const uint32_t tpr = 1u << p.tpr_log2;
    const uint32_t rw = blockIdx.x / (uint32_t)p.col_groups;
    const uint32_t cg = blockIdx.x - rw * (uint32_t)p.col_groups;
    const int64_t row0 = ((int64_t)rw * (256u >> p.tpr_log2)
                                 + (threadIdx.x >> p.tpr_log2))
            * R;
    const uint32_t cb = cg * tpr + (threadIdx.x & (tpr - 1));
    if (row0 >= p.rows || cb >= c8) return;
    const int64_t col = (int64_t)cb * 8;
    uint4 raw[R][V];
#pragma unroll
    for (int r = 0; r < R; r++) {
        // rows past the end read the last row again and are not stored
        const int64_t row = min(row0 + r, p.rows - 1);
        const uint4 *s = (const uint4 *)((const char *)p.src
                + (row * p.src_pitch + col) * (SRC == 0 ? 4 : 2));
#pragma unroll
        for (int v = 0; v < V; v++) raw[r][v] = s[v];
    }
    const float4 *sp = (const float4 *)((const float *)p.dst_scale.ptr + col);
    const float4 sa = sp[0], sb = sp[1];
    const float inv[8] = {1.f / sa.x, 1.f / sa.y, 1.f / sa.z, 1.f / sa.w,
            1.f / sb.x, 1.f / sb.y, 1.f / sb.z, 1.f / sb.w};
    const float dst_zp = p.dst_zp ? (float)p.dst_zp[0] : 0.f;
    const bool sgn = p.dst_dt == dt_s8;
    const float lo = sgn ? -128.f : 0.f, hi = sgn ? 127.f : 255.f;
#pragma unroll
    for (int r = 0; r < R; r++) {
        if (row0 + r >= p.rows) break;
        float in[8];
        if constexpr (SRC == 0) {
            const uint32_t w[8] = {raw[r][0].x, raw[r][0].y, raw[r][0].z,
                    raw[r][0].w, raw[r][V - 1].x, raw[r][V - 1].y,
                    raw[r][V - 1].z, raw[r][V - 1].w};
#pragma unroll
            for (int i = 0; i < 8; i++) in[i] = u2f(w[i]);
        } else {
            const uint32_t w[4]
                    = {raw[r][0].x, raw[r][0].y, raw[r][0].z, raw[r][0].w};
#pragma unroll
            for (int i = 0; i < 8; i++) {
                if constexpr (SRC == 2)
                    in[i] = (float)__builtin_bit_cast(_Float16,
                            (uint16_t)(w[i / 2] >> (16 * (i % 2))));
                else
                    in[i] = u2f(i % 2 ? (w[i / 2] & 0xFFFF0000u)
                                      : (w[i / 2] << 16));
            }
        }
        uint32_t o[2] = {0, 0};
#pragma unroll
        for (int i = 0; i < 8; i++)
            o[i / 4] |= (uint32_t)(round_sat(in[i] * inv[i] + dst_zp, lo, hi)
                                & 0xff)
                    << (8 * (i % 4));
        *(uint2 *)((uint8_t *)p.dst + (row0 + r) * p.dst_pitch + col)
                = make_uint2(o[0], o[1]);
    }
}

// The quantizer over a 2-D tensor that changes its dim order on the way (a
// row-major f32 / bf16 / f16 source into a column-major quantized tensor or the
// other way round: weights stored [N, K] quantized into [K, N], say). A
// workgroup owns a tile: it reads along the source's stride-1 dim into LDS
// (odd pitch: the transposed read-back is free of bank conflicts), then does
// the arithmetic of quantize_rows_kernel per element (scales and zero points
// addressed by the element's row and column, so every mask and group shape of
// the row kernel is taken) and stores along the destination's stride-1 dim,
// two neighbouring elements per thread (a 4-bit pair is one byte).
// QT_FAST x QT_SLOW: the tile's extent along the destination's stride-1 dim
// (128 elements: a whole 128-byte line of an 8-bit destination per row piece)
// and along the source's (64 elements: 256 bytes of an f32 source)
constexpr int QT_FAST = 128, QT_SLOW = 64;
__global__ void __launch_bounds__(256)
quantize_transpose_kernel(const quant_tr_params_t p) {
    __shared__ float tile[QT_SLOW][QT_FAST + 1]; // [slow][fast] of the destination
    const int tid = threadIdx.x;
    const bool dst_col_major = p.dst_sr == 1; // else stride 1 over columns
    // origin of the tile: blockIdx.x walks the SOURCE's stride-1 dim, so that
    // the workgroups in flight together read neighbouring pieces of the same
    // source lines' neighbourhood instead of pieces a whole (often power-of-two)
    // pitch apart, which all fall on the same memory channels
    const int64_t f0 = (int64_t)blockIdx.y * QT_FAST, s0 = (int64_t)blockIdx.x * QT_SLOW;
    const int64_t r0 = dst_col_major ? f0 : s0, c0 = dst_col_major ? s0 : f0;
    // the source values as f32, read along the source's stride-1 dim, which is
    // the destination's slow one
    // (every load of the thread is issued before the first value is used)
    constexpr int NL = QT_FAST * QT_SLOW / 256;
    const int ls = tid & (QT_SLOW - 1);
    // the element of the tile's first line the thread reads, and the step to
    // the next line: along the destination's stride-1 dim
    const int64_t line = dst_col_major ? p.src_sr : p.src_sc;
    const int64_t fmax = (dst_col_major ? p.rows : p.cols) - 1 - f0; // last valid line
    const int64_t base = dst_col_major
            ? r0 * p.src_sr + min(c0 + ls, p.cols - 1) * p.src_sc
            : min(r0 + ls, p.rows - 1) * p.src_sr + c0 * p.src_sc;
    uint32_t raw[NL];
    if (p.src_dt == dt_f32) {
#pragma unroll
        for (int i = 0; i < NL; i++) {
            const int64_t lf = min((int64_t)(tid / QT_SLOW + (256 / QT_SLOW) * i), fmax);
            raw[i] = ((const uint32_t *)p.src)[base + lf * line];
        }
    } else {
#pragma unroll
        for (int i = 0; i < NL; i++) {
            const int64_t lf = min((int64_t)(tid / QT_SLOW + (256 / QT_SLOW) * i), fmax);
            raw[i] = ((const uint16_t *)p.src)[base + lf * line];
        }
    }
#pragma unroll
    for (int i = 0; i < NL; i++) {
        const int lf = tid / QT_SLOW + (256 / QT_SLOW) * i;
        tile[ls][lf] = p.src_dt == dt_f32 ? u2f(raw[i])
                : p.src_dt == dt_f16
                ? (float)__builtin_bit_cast(_Float16, (uint16_t)raw[i])
                : u2f(raw[i] << 16);
    }
    __syncthreads();
    const int ddt = p.dst_dt;
    const bool nib = ddt == dt_s4 || ddt == dt_u4;
    const float dst_zp = p.dst_zp ? (float)p.dst_zp[0] : 0.f;
    // A thread's pair keeps its place along the destination's stride-1 dim
    // through all its 8 steps: what does not depend on the other dim (a scale
    // per column on the way into a row-major tensor, say) is fetched, and a
    // dst scale inverted, once.
    const int fast = (tid & (QT_FAST / 2 - 1)) * 2;
    const auto along = [&](const quant_rows_q_t &q) { // varies with the slow dim?
        return q.ptr && (dst_col_major ? q.sc != 0 : q.sr != 0);
    };
    const bool ss_var = along(p.src_scale), ds_var = along(p.dst_scale),
               sz_var = along(p.src_zp);
    const auto fetch = [&](int64_t r, int64_t c, bool second, float (&ss)[2],
                               float (&ds)[2], float (&sz)[2], bool want_var) {
#pragma unroll
        for (int e = 0; e < 2; e++) {
            const int64_t re = min(r + (dst_col_major && e && second ? 1 : 0), p.rows - 1);
            const int64_t ce = min(c + (!dst_col_major && e && second ? 1 : 0), p.cols - 1);
            if (p.src_scale.ptr && ss_var == want_var)
                ss[e] = load_float(p.src_scale.dt, p.src_scale.ptr,
                        qr_off(p.src_scale, re, ce));
            if (p.dst_scale.ptr && ds_var == want_var)
                ds[e] = 1.f
                        / load_float(p.dst_scale.dt, p.dst_scale.ptr,
                                qr_off(p.dst_scale, re, ce));
            // the zero point is an integer
            if (p.src_zp.ptr && sz_var == want_var)
                sz[e] = (float)(int)load_float(
                        p.src_zp.dt, p.src_zp.ptr, qr_off(p.src_zp, re, ce));
        }
    };
    float ss[2] = {1.f, 1.f}, ds[2] = {1.f, 1.f}, sz[2] = {0.f, 0.f};
    {
        const int64_t r = dst_col_major ? r0 + fast : r0, c = dst_col_major ? c0 : c0 + fast;
        fetch(r, c, true, ss, ds, sz, false);
    }
    constexpr int SLOW_STEP = 256 / (QT_FAST / 2);
#pragma unroll 4
    for (int i = 0; i < QT_SLOW / SLOW_STEP; i++) {
        const int slow = tid / (QT_FAST / 2) + SLOW_STEP * i;
        const int64_t r = r0 + (dst_col_major ? fast : slow);
        const int64_t c = c0 + (dst_col_major ? slow : fast);
        if (r >= p.rows || c >= p.cols) continue;
        // the pair's second element: the next row (column-major dst) or column
        const bool second = dst_col_major ? r + 1 < p.rows : c + 1 < p.cols;
        if (ss_var || ds_var || sz_var) fetch(r, c, second, ss, ds, sz, true);
        // (the reference subtracts its default zero point 0 too)
        const float d0 = ss[0] * (tile[slow][fast] - sz[0]) * ds[0] + dst_zp;
        const float d1 = second ? ss[1] * (tile[slow][fast + 1] - sz[1]) * ds[1] + dst_zp : 0.f;
        const int64_t o = r * p.dst_sr + c * p.dst_sc;
        if (nib) {
            // the host admits 4-bit destinations only where every pair starts
            // on a byte and is whole
            const float lo = ddt == dt_s4 ? -8.f : 0.f, hi = ddt == dt_s4 ? 7.f : 15.f;
            ((uint8_t *)p.dst)[o >> 1] = (uint8_t)((round_sat(d0, lo, hi) & 0xf)
                    | ((round_sat(d1, lo, hi) & 0xf) << 4));
        } else if ((ddt == dt_s8 || ddt == dt_u8) && second) {
            const float lo = ddt == dt_s8 ? -128.f : 0.f, hi = ddt == dt_s8 ? 127.f : 255.f;
            // one two-byte store at any address
            typedef uint16_t u16_any __attribute__((aligned(1)));
            *(u16_any *)((uint8_t *)p.dst + o) = (uint16_t)((round_sat(d0, lo, hi) & 0xff)
                    | ((round_sat(d1, lo, hi) & 0xff) << 8));
        } else {
            store_float(ddt, d0, p.dst, o);
            if (second) store_float(ddt, d1, p.dst, o + 1);
        }
    }
}

void launch_quantize_transpose(const quant_tr_params_t &p, hipStream_t stream) {
    if (p.rows <= 0 || p.cols <= 0) return;
    const bool dst_col_major = p.dst_sr == 1;
    const int64_t fast = dst_col_major ? p.rows : p.cols, slow = dst_col_major ? p.cols : p.rows;
    const dim3 grid((unsigned)((slow + QT_SLOW - 1) / QT_SLOW),
            (unsigned)((fast + QT_FAST - 1) / QT_FAST));
    hipLaunchKernelGGL(quantize_transpose_kernel, grid, dim3(256), 0, stream, p);
}

// whether the 8-bit kernels cover the plan; how the dst scale runs (0: one
// or none, 1: per row, 2: per column)
static bool quantize8_takes(const quant_rows_params_t &p, int &mode) {
    if (p.dst_dt != dt_s8 && p.dst_dt != dt_u8) return false;
    if (p.src_scale.ptr || p.src_zp.ptr) return false;
    mode = 0;
    const quant_rows_q_t &q = p.dst_scale;
    if (!q.ptr) return true;
    if (q.dt != dt_f32) return false;
    if (q.sr == 0 && q.sc == 0) return true;
    if (q.sc == 0 && q.sr == 1 && q.gr == 1) mode = 1;
    if (q.sr == 0 && q.sc == 1 && q.gc == 1) mode = 2;
    return mode != 0;
}

void launch_quantize_rows(const quant_rows_params_t &p0, hipStream_t stream) {
    quant_rows_params_t p = p0;
    int mode = 0;
    if (quantize8_takes(p, mode)) {
        const int64_t c8 = p.cols / 8, c16 = (c8 + Q8_CHUNKS - 1) / Q8_CHUNKS;
        if (p.rows <= 0 || c8 <= 0) return;
        if (mode == 2) {
            p.tpr_log2 = 0;
            while (p.tpr_log2 < 8 && (int64_t(1) << p.tpr_log2) < c8)
                p.tpr_log2++;
            const int64_t tpr = int64_t(1) << p.tpr_log2;
            const int64_t rows_wg = (256 >> p.tpr_log2) * QR_ROWS;
            p.col_groups = (int32_t)((c8 + tpr - 1) / tpr);
            const dim3 grid((unsigned)(((p.rows + rows_wg - 1) / rows_wg)
                    * p.col_groups));
            auto go = [&](auto kern) {
                hipLaunchKernelGGL(kern, grid, dim3(256), 0, stream, p);
            };
            if (p.src_dt == dt_f32)
                go(quantize8_cols_kernel<0>);
            else if (p.src_dt == dt_bf16)
                go(quantize8_cols_kernel<1>);
            else
                go(quantize8_cols_kernel<2>);
            return;
        }
        const bool per_row = mode == 1;
        p.tpr_log2 = 0;
        while (p.tpr_log2 < 8 && (int64_t(1) << p.tpr_log2) < c16)
            p.tpr_log2++;
        const int64_t per_wg = 256 >> p.tpr_log2, span = int64_t(Q8_CHUNKS) << p.tpr_log2;
        p.col_groups = (int32_t)((c8 + span - 1) / span);
        // below 2^31: the plan bounds rows * cols
        const dim3 grid((unsigned)(((p.rows + per_wg - 1) / per_wg) * p.col_groups));
        auto go = [&](auto kern) {
            hipLaunchKernelGGL(kern, grid, dim3(256), 0, stream, p);
        };
        switch ((p.src_dt == dt_f32 ? 0 : p.src_dt == dt_bf16 ? 2 : 4)
                | (per_row ? 1 : 0)) {
            case 0: go(quantize8_kernel<0, false>); break;
            case 1: go(quantize8_kernel<0, true>); break;
            case 2: go(quantize8_kernel<1, false>); break;
            case 3: go(quantize8_kernel<1, true>); break;
            case 4: go(quantize8_kernel<2, false>); break;
            default: go(quantize8_kernel<2, true>); break;
        }
        return;
    }
    const bool col_only = (p.src_scale.ptr && p.src_scale.sr == 0
                                  && p.src_scale.sc != 0)
            || (p.dst_scale.ptr && p.dst_scale.sr == 0 && p.dst_scale.sc != 0);
    p.rows_per_thread = col_only ? QR_ROWS : 1;
    const int64_t row_blocks
            = (p.rows + p.rows_per_thread - 1) / p.rows_per_thread;
    const int64_t c8 = p.cols / 8;
    if (row_blocks <= 0 || c8 <= 0) return;
    // threads per row block: the power of two at or above the chunks of a row,
    // 256 at most
    p.tpr_log2 = 0;
    while (p.tpr_log2 < 8 && (int64_t(1) << p.tpr_log2) < c8)
        p.tpr_log2++;
    const int64_t per_wg = 256 >> p.tpr_log2;
    const int64_t tpr = int64_t(1) << p.tpr_log2;
    p.col_groups = (int32_t)((c8 + tpr - 1) / tpr);
    // below 2^31: the plan bounds rows * cols
    const dim3 grid(
            (unsigned)(((row_blocks + per_wg - 1) / per_wg) * p.col_groups));
    if (col_only)
        hipLaunchKernelGGL(quantize_rows_kernel<QR_ROWS>, grid, dim3(256), 0,
                stream, p);
    else
        hipLaunchKernelGGL(
                quantize_rows_kernel<1>, grid, dim3(256), 0, stream, p);
}

} // namespace qmm
