// Host side of the thin C ABI (include/qmm_hip.h): implementation selection,
// plan creation and kernel launches. Pure host code apart from the HIP runtime
// calls; it never computes a result itself.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstring>
#include <atomic>
#include <mutex>
#include <string>

#include "qmm_device.hpp"
#include "qmm_hip.h"
#include "qmm_plan.hpp"

namespace qmm {
void launch_matmul_generic(const generic_params_t *dev_params,
        const generic_params_t &host_params, const qmm_matmul_args_t &args,
        hipStream_t stream);
void launch_reorder_generic(const generic_reorder_params_t &params,
        const qmm_reorder_args_t &args, hipStream_t stream);
bool gemm_b8_uses_tile256(const gemm_params_t &p, bool f8, int variant);
bool gemm_b8x_two_per_cu(const gemm_params_t &p, bool f8);
void launch_flip_u8(const void *src, void *dst, int64_t batch, int64_t M,
        int64_t K, int64_t lda, int64_t a_sb, hipStream_t stream);
void launch_gemm_b8(const gemm_params_t &p, bool f8, int variant,
        hipStream_t stream);
bool launch_gemv_w4(const gemv_params_t &p, hipStream_t stream);
void launch_quantize_rows(const quant_rows_params_t &p, hipStream_t stream);
void launch_quantize_transpose(const quant_tr_params_t &p, hipStream_t stream);
void launch_w4a8_prep(const w4a8_prep_t &p, hipStream_t stream);
void launch_gemv_b8(const gemm_params_t &p, hipStream_t stream);
void launch_gemm_f16(const gemm16_params_t &p, hipStream_t stream);
void launch_rowsum_b8(const void *src, int32_t *dst, int64_t batch, int64_t M,
        int64_t K, int64_t lda, int64_t a_sb, bool a_is_u8, const void *src_zp,
        int src_zp_dt, hipStream_t stream);
void launch_gemm_f16w8(const gemm_params_t &p, int splits, float *part,
        hipStream_t stream);
int gemm_f16w8_splits(int64_t M, int64_t N, int64_t K);
void launch_gemm_w4a8(const w4a8_params_t &p, int variant, hipStream_t stream);
void launch_gemm_w4a8_small(const w4a8_small_t &p, bool has_zp,
        hipStream_t stream);
bool gemm_w4a8_small_takes(const w4a8_prep_t &q);
void launch_gemm_w4a8_tiny(const w4a8_small_t &p, bool has_zp, int nwv,
        hipStream_t stream);
int gemm_w4a8_tiny_max_groups(bool half);
bool gemm_w4a8_mid_takes(int M, int group_k);
int gemm_w4a8_mid_gpc(int M, int group_k);
int gemm_w4a8_mid_wave_bytes(int M, int group_k, bool src_zp);
void launch_gemm_w4a8_mid(const w4a8_small_t &p, bool has_zp, int nwv,
        hipStream_t stream);
void launch_pack_w4k(const void *src, void *dst, int dt, int64_t batch,
        int64_t K, int64_t N, int64_t sb, int64_t sk, int64_t sn,
        hipStream_t stream);
void launch_unpack_w4k(const void *src, void *dst, int dt, int64_t batch,
        int64_t K, int64_t N, int64_t sb, int64_t sk, int64_t sn,
        hipStream_t stream);
void launch_pack_b8(const void *src, void *dst, int dt, int64_t batch,
        int64_t K, int64_t N, int64_t sb, int64_t sk, int64_t sn,
        bool with_colsum, hipStream_t stream);
void launch_unpack_b8(const void *src, void *dst, int dt, int64_t batch,
        int64_t K, int64_t N, int64_t sb, int64_t sk, int64_t sn,
        hipStream_t stream);
void launch_pack_w4(const void *src, void *dst, int dt, int64_t batch,
        int64_t K, int64_t N, int64_t sb, int64_t sk, int64_t sn,
        hipStream_t stream);
void launch_pack_w8(const void *src, void *dst, int dt, int64_t batch,
        int64_t K, int64_t N, int64_t sb, int64_t sk, int64_t sn,
        hipStream_t stream);
void launch_unpack_w8(const void *src, void *dst, int dt, int64_t batch,
        int64_t K, int64_t N, int64_t sb, int64_t sk, int64_t sn,
        hipStream_t stream);
void launch_unpack_w4(const void *src, void *dst, int dt, int64_t batch,
        int64_t K, int64_t N, int64_t sb, int64_t sk, int64_t sn,
        hipStream_t stream);
} // namespace qmm

using namespace qmm;

namespace {

thread_local std::string g_last_error;

int fail(int code, const char *msg) {
    g_last_error = msg;
    return code;
}
int hip_fail(hipError_t e, const char *what) {
    g_last_error = std::string(what) + ": " + hipGetErrorString(e);
    return QMM_RUNTIME_ERROR;
}

bool is_int8(int dt) { return dt == dt_s8 || dt == dt_u8; }
bool is_int4(int dt) { return dt == dt_s4 || dt == dt_u4; }
bool is_wei_int(int dt) { return is_int8(dt) || is_int4(dt); }
bool one_of(int v, std::initializer_list<int> l) {
    for (int x : l)
        if (v == x) return true;
    return false;
}

int dims_mask(const int64_t *d1, const int64_t *d2, int nd) {
    int mask = 0;
    for (int d = 0; d < nd; d++)
        if (d1[d] == d2[d]) mask |= 1 << d;
    return mask;
}

// geometry of a scales / zero-points buffer over tensor dims `tdims`
void quant_geom(generic_quant_t &q, const qmm_quant_t &a, int nd,
        const int64_t *tdims, int64_t g0, int64_t g1) {
    std::memset(&q, 0, sizeof(q));
    q.g0 = g0 > 0 ? g0 : 1;
    q.g1 = g1 > 0 ? g1 : 1;
    q.nelems = 1;
    if (!a.set) return;
    int64_t dims[QMM_MAX_NDIMS];
    for (int d = 0; d < nd; d++)
        dims[d] = (a.mask & (1 << d)) ? tdims[d] : 1;
    if (nd >= 2) {
        dims[nd - 1] /= q.g1;
        dims[nd - 2] /= q.g0;
    }
    int64_t s = 1;
    for (int d = nd - 1; d >= 0; d--) {
        q.strides[d] = (a.mask & (1 << d)) ? s : 0;
        s *= dims[d] > 0 ? dims[d] : 1;
    }
    q.nelems = s;
    q.indexed = s > 1;
}

int64_t group_or(const qmm_quant_t &a, int which, int64_t dflt) {
    if (!a.set || !a.has_groups) return dflt;
    const int64_t g = which == 0 ? a.g0 : a.g1;
    return g > 0 ? g : dflt;
}

void prelu_strides(int64_t *strides, const qmm_tensor_t &dst, int mask) {
    // prelu weights: f32, dims = masked dst dims, layout a/ab/acb/acdb/acdeb
    // (src/cpu/primitive_attr_postops.cpp:196-225)
    static const int perm[6][5] = {{0}, {0}, {0, 1}, {0, 2, 1}, {0, 2, 3, 1},
            {0, 2, 3, 4, 1}};
    const int nd = dst.ndims;
    int64_t s = 1;
    for (int i = nd - 1; i >= 0; i--) {
        const int d = nd <= 5 ? perm[nd][i] : i;
        const int64_t dim = (mask & (1 << d)) ? dst.dims[d] : 0;
        strides[d] = s;
        s *= dim > 0 ? dim : 1;
    }
}

void build_generic(generic_params_t &P, const qmm_matmul_desc_t &D) {
    std::memset(&P, 0, sizeof(P));
    P.desc = D;
    const int nd = D.dst.ndims;
    P.M = D.dst.dims[nd - 2];
    P.N = D.dst.dims[nd - 1];
    P.K = D.src.dims[nd - 1];
    P.batch = 1;
    for (int d = 0; d < nd - 2; d++)
        P.batch *= D.dst.dims[d];
    P.src_mask = dims_mask(D.dst.dims, D.src.dims, nd);
    P.wei_mask = dims_mask(D.dst.dims, D.wei.dims, nd);
    P.bia_mask = D.bias.ndims ? dims_mask(D.dst.dims, D.bias.dims, nd) : 0;
    P.int_path = is_int8(D.src.dt);
    P.decompress = !P.int_path && is_wei_int(D.wei.dt) && D.apply_to_int;
    P.sum_dt = D.dst.dt;
    for (int i = 0; i < D.npo; i++) {
        if (D.po[i].kind == pk_sum && !P.has_sum) {
            P.has_sum = 1;
            if (D.po[i].dt != dt_undef) P.sum_dt = D.po[i].dt;
        }
        if (D.po[i].kind == pk_prelu)
            prelu_strides(P.desc.po[i].src1.strides, D.dst, D.po[i].mask);
    }
    P.dst_zp_mult = D.zps[QMM_DST].set && D.zps[QMM_DST].mask > 0;
    const qmm_quant_t &ss = D.scales[QMM_SRC], &ws = D.scales[QMM_WEI];
    const qmm_quant_t &sz = D.zps[QMM_SRC], &wz = D.zps[QMM_WEI];
    quant_geom(P.q_src_scale, ss, nd, D.src.dims, 1, group_or(ss, 1, 1));
    quant_geom(P.q_src_zp, sz, nd, D.src.dims, 1, group_or(sz, 1, 1));
    quant_geom(P.q_wei_scale, ws, nd, D.wei.dims, group_or(ws, 0, 1),
            group_or(ws, 1, 1));
    quant_geom(P.q_wei_zp, wz, nd, D.wei.dims, group_or(wz, 0, 1),
            group_or(wz, 1, 1));
    // K groups of the integer path: the smallest group over the four entries.
    // An entry without explicit groups varies per k if its mask covers K
    // (group of 1) and otherwise spans all of K.
    int64_t ng = 1;
    if (P.K > 0) {
        const int64_t K = P.K;
        const int src_kbit = 1 << (nd - 1), wei_kbit = 1 << (nd - 2);
        auto kgroup = [&](const qmm_quant_t &a, int which, int kbit) {
            if (!a.set) return K;
            if (a.has_groups) return group_or(a, which, K);
            return (a.mask & kbit) ? (int64_t)1 : K;
        };
        int64_t t;
        t = K / kgroup(sz, 1, src_kbit);
        if (t > ng) ng = t;
        t = K / kgroup(wz, 0, wei_kbit);
        if (t > ng) ng = t;
        t = K / kgroup(ss, 1, src_kbit);
        if (t > ng) ng = t;
        t = K / kgroup(ws, 0, wei_kbit);
        if (t > ng) ng = t;
    }
    P.ngroups_k = ng;
    P.group_k = P.K > 0 ? P.K / ng : 0;
    P.wei_scale_stride_n = (ws.set && (ws.mask & (1 << (nd - 1)))) ? 1 : 0;
}

// Fold the batch dims of `t` (dims relative to dst's) into one linear stride.
// Returns false if no single stride describes it.
bool fold_batch(const qmm_tensor_t &t, const qmm_tensor_t &dst, int64_t &sb) {
    const int nd = dst.ndims;
    sb = 0;
    if (nd <= 2) return true;
    // effective stride per batch dim (0 where broadcast)
    int64_t es[QMM_MAX_NDIMS];
    for (int d = 0; d < nd - 2; d++)
        es[d] = (t.dims[d] == dst.dims[d] && dst.dims[d] > 1) ? t.strides[d] : 0;
    // innermost non-unit batch dim sets the stride, outer ones must nest
    int64_t expect = -1;
    for (int d = nd - 3; d >= 0; d--) {
        if (dst.dims[d] == 1) continue;
        if (expect < 0) {
            sb = es[d];
            expect = es[d] * dst.dims[d];
        } else {
            if (es[d] != expect) return false;
            expect *= dst.dims[d];
        }
    }
    return true;
}

bool fold_tensor(ep_tensor_t &e, const qmm_tensor_t &t,
        const qmm_tensor_t &dst, const void *ptr) {
    const int nd = dst.ndims;
    e.ptr = ptr;
    e.dt = t.dt;
    e.sm = t.dims[nd - 2] == dst.dims[nd - 2] ? t.strides[nd - 2] : 0;
    e.sn = t.dims[nd - 1] == dst.dims[nd - 1] ? t.strides[nd - 1] : 0;
    return fold_batch(t, dst, e.sb);
}

// a quant buffer seen as a (b, m, n) tensor over the dst coordinates;
// `is_src`: dims are (.., M, K) else (.., K, N). Only single-K-group buffers.
bool fold_quant(ep_tensor_t &e, const generic_quant_t &q, const qmm_quant_t &a,
        const qmm_tensor_t &t, const qmm_tensor_t &dst, bool is_src,
        const void *ptr) {
    const int nd = dst.ndims;
    e.ptr = ptr;
    e.dt = a.dt;
    e.sb = e.sm = e.sn = 0;
    if (!q.indexed) return true;
    if (is_src) {
        e.sm = q.strides[nd - 2];
    } else {
        if (q.g1 != 1) return false;
        e.sn = q.strides[nd - 1];
    }
    qmm_tensor_t qt = t;
    for (int d = 0; d < nd; d++)
        qt.strides[d] = q.strides[d];
    for (int d = 0; d < nd - 2; d++)
        if (!(a.mask & (1 << d))) qt.dims[d] = 1; // broadcast
    return fold_batch(qt, dst, e.sb);
}

// Build the compact epilogue; false if the problem does not fit it.
bool build_epilogue(epilogue_t &ep, const generic_params_t &P,
        const qmm_matmul_args_t *A, bool scales_in_kernel = false) {
    const qmm_matmul_desc_t &D = P.desc;
    const int nd = D.dst.ndims;
    std::memset(&ep, 0, sizeof(ep));
    const qmm_matmul_args_t zero_args = {};
    if (!A) A = &zero_args;
    if (!fold_tensor(ep.dst, D.dst, D.dst, A->dst)) return false;
    if (D.bias.ndims) {
        if (!fold_tensor(ep.bias, D.bias, D.dst, A->bias)) return false;
        if (!A->bias) ep.bias.ptr = (const void *)1; // shape check only
    }
    const qmm_quant_t &ss = D.scales[QMM_SRC], &ws = D.scales[QMM_WEI];
    if (ss.set && !scales_in_kernel) {
        if (P.q_src_scale.g1 != P.K && (ss.mask & (1 << (nd - 1))))
            return false; // K-grouped src scales
        if (!fold_quant(ep.src_scale, P.q_src_scale, ss, D.src, D.dst, true,
                    A->scales[QMM_SRC]))
            return false;
        if (!A->scales[QMM_SRC]) ep.src_scale.ptr = (const void *)1;
    }
    if (ws.set && !P.decompress && !scales_in_kernel) {
        if ((ws.mask & (1 << (nd - 2))) && P.q_wei_scale.g0 != P.K)
            return false; // K-grouped weights scales
        if (!fold_quant(ep.wei_scale, P.q_wei_scale, ws, D.wei, D.dst, false,
                    A->scales[QMM_WEI]))
            return false;
        if (!A->scales[QMM_WEI]) ep.wei_scale.ptr = (const void *)1;
    }
    if (D.scales[QMM_DST].set) {
        if (D.scales[QMM_DST].mask != 0) return false;
        ep.dst_scale = A->scales[QMM_DST] ? A->scales[QMM_DST] : (const void *)1;
        ep.dst_scale_dt = D.scales[QMM_DST].dt;
    }
    if (D.zps[QMM_DST].set) {
        if (D.zps[QMM_DST].dt != dt_s32) return false;
        ep.dst_zp = A->zps[QMM_DST] ? (const int32_t *)A->zps[QMM_DST]
                                    : (const int32_t *)1;
        ep.dst_zp_sn = P.dst_zp_mult;
    }
    if (D.npo > EP_MAX_PO) return false;
    ep.npo = D.npo;
    for (int i = 0; i < D.npo; i++) {
        const qmm_postop_t &e = P.desc.po[i];
        ep_postop_t &o = ep.po[i];
        o.kind = e.kind;
        o.alg = e.alg;
        o.alpha = e.alpha;
        o.beta = e.beta;
        o.scale = e.scale;
        o.zero_point = e.zero_point;
        if (e.kind == pk_binary) {
            if (!fold_tensor(o.t, e.src1, D.dst, A->po_arg[i])) return false;
        } else if (e.kind == pk_prelu) {
            qmm_tensor_t w = D.dst;
            w.dt = dt_f32;
            for (int d = 0; d < nd; d++) {
                // -1 never equals a dst dim: masked-out dims broadcast
                w.dims[d] = (e.mask & (1 << d)) ? D.dst.dims[d] : -1;
                w.strides[d] = e.src1.strides[d];
            }
            if (!fold_tensor(o.t, w, D.dst, A->po_arg[i])) return false;
        } else if (e.kind == pk_sum) {
            o.t.dt = P.sum_dt;
        } else if (e.kind != pk_eltwise) {
            return false;
        }
    }
    // straight-line shapes (see EP_FAST_* in qmm_device.hpp)
    ep.fast = EP_FAST_NONE;
    ep.fast_ext = 0;
    // (scales of any type: every kernel converts them to f32 as it loads them)
    const bool dst_base = ep.dst.dt == dt_bf16 || ep.dst.dt == dt_f32;
    const bool dst_more = one_of(ep.dst.dt, {dt_f16, dt_s8, dt_u8});
    const bool bias_ok = !ep.bias.ptr || ep.bias.sm == 0; // per column
    if (bias_ok && ep.dst.sn == 1 && (dst_base || dst_more)
            && ep.npo <= 1) {
        if (ep.npo == 0) {
            ep.fast = EP_FAST_PLAIN;
        } else {
            const ep_postop_t &o = ep.po[0];
            if (o.kind == pk_eltwise && o.scale == 1.f && o.alg == alg_relu)
                ep.fast = EP_FAST_RELU;
            else if (o.kind == pk_eltwise && o.scale == 1.f
                    && o.alg == alg_swish)
                ep.fast = EP_FAST_SWISH;
            else if (o.kind == pk_binary && o.alg == alg_bin_add
                    && o.t.dt == dt_f32 && o.t.sn == 1)
                ep.fast = EP_FAST_ADD;
            else if (o.kind == pk_sum && o.zero_point == 0
                    && o.t.dt == ep.dst.dt
                    && one_of(ep.dst.dt, {dt_f32, dt_bf16, dt_f16}))
                ep.fast = EP_FAST_SUM;
            else if (o.kind == pk_eltwise && o.alg == alg_gelu_erf)
                ep.fast = EP_FAST_GELU_ERF;
            else if (o.kind == pk_eltwise && o.alg == alg_gelu_tanh)
                ep.fast = EP_FAST_GELU_TANH;
            else if (o.kind == pk_binary
                    && (o.alg == alg_bin_add || o.alg == alg_bin_mul)
                    && o.t.sn == 1 && o.t.dt == dt_f32)
                ep.fast = EP_FAST_BIN32;
            else if (o.kind == pk_binary
                    && (o.alg == alg_bin_add || o.alg == alg_bin_mul)
                    && o.t.sn == 1 && one_of(o.t.dt, {dt_f16, dt_bf16}))
                ep.fast = EP_FAST_BIN16;
        }
        if (ep.fast != EP_FAST_NONE)
            ep.fast_ext = ep.bias.ptr || ep.dst_scale || ep.dst_zp || dst_more
                    || ep.fast > EP_FAST_SUM;
    }
    return true;
}

// ---------------------------------------------------------------------------
bool plain_wei_strides(const qmm_matmul_desc_t &D, int64_t &sb, int64_t &sk,
        int64_t &sn) {
    const int nd = D.wei.ndims;
    sk = D.wei.strides[nd - 2];
    sn = D.wei.strides[nd - 1];
    return fold_batch(D.wei, D.dst, sb);
}

int64_t wei_batch(const qmm_matmul_desc_t &D) {
    int64_t b = 1;
    for (int d = 0; d < D.wei.ndims - 2; d++)
        b *= D.wei.dims[d];
    return b;
}

int supports_gemm_b8(const qmm_matmul_desc_t &D, const generic_params_t &P) {
    const int nd = D.dst.ndims;
    const bool i8 = is_int8(D.src.dt) && is_int8(D.wei.dt);
    const bool f8 = D.src.dt == dt_f8_e4m3 && D.wei.dt == dt_f8_e4m3;
    if (!i8 && !f8) return QMM_UNIMPLEMENTED;
    if (i8 && !one_of(D.dst.dt, {dt_f32, dt_bf16, dt_f16, dt_s32, dt_s8, dt_u8}))
        return QMM_UNIMPLEMENTED;
    if (f8 && !one_of(D.dst.dt, {dt_f32, dt_bf16, dt_f16, dt_f8_e4m3, dt_f8_e5m2}))
        return QMM_UNIMPLEMENTED;
    if (P.M == 0 || P.N == 0 || P.K == 0) return QMM_UNIMPLEMENTED;
    if (P.M > INT32_MAX || P.N > INT32_MAX || P.K > INT32_MAX
            || P.batch > 65535)
        return QMM_UNIMPLEMENTED;
    if (!one_of(D.wei_layout, {QMM_LAYOUT_PLAIN, QMM_LAYOUT_MFMA_B8}))
        return QMM_UNIMPLEMENTED;
    // weights batch dims: all present or all broadcast
    const int64_t wb = wei_batch(D);
    if (wb != 1 && wb != P.batch) return QMM_UNIMPLEMENTED;
    if (D.wei_layout == QMM_LAYOUT_PLAIN) {
        int64_t sb, sk, sn;
        if (!plain_wei_strides(D, sb, sk, sn)) return QMM_UNIMPLEMENTED;
    }
    // source rows K-contiguous, 16-byte granular
    if (D.src.strides[nd - 1] != 1 || P.K % 16 != 0
            || D.src.strides[nd - 2] % 16 != 0)
        return QMM_UNIMPLEMENTED;
    int64_t a_sb;
    if (!fold_batch(D.src, D.dst, a_sb) || a_sb % 16 != 0)
        return QMM_UNIMPLEMENTED;
    if (D.zps[QMM_WEI].set) {
        // one zero point for the tensor or per column (no groups): applied
        // through the source's row sums in the general kernel's epilogue
        const qmm_quant_t &wz = D.zps[QMM_WEI];
        if (!i8 || (wz.mask & ~(1 << (nd - 1))) || wz.has_groups)
            return QMM_UNIMPLEMENTED;
        if (!one_of(wz.dt, {dt_s32, dt_s8, dt_u8})) return QMM_UNIMPLEMENTED;
    }
    if (D.zps[QMM_SRC].set) {
        if (!i8 || D.zps[QMM_SRC].mask != 0) return QMM_UNIMPLEMENTED;
        if (!one_of(D.zps[QMM_SRC].dt, {dt_s32, dt_s8, dt_u8}))
            return QMM_UNIMPLEMENTED;
    }
    if (f8 && D.scales[QMM_SRC].set && D.scales[QMM_SRC].mask != 0)
        return QMM_UNIMPLEMENTED;
    if (f8 && D.scales[QMM_WEI].set
            && (D.scales[QMM_WEI].mask & ~(1 << (nd - 1))))
        return QMM_UNIMPLEMENTED;
    if (f8 && D.zps[QMM_DST].set) return QMM_UNIMPLEMENTED;
    epilogue_t ep;
    if (!build_epilogue(ep, P, nullptr)) return QMM_UNIMPLEMENTED;
    return QMM_OK;
}

// K extent of one entry of a scales / zero-points buffer: the group size if it
// has K groups, 1 if it varies per k without groups, K if it does not vary
int64_t k_extent(const qmm_quant_t &a, int which, int kbit, int64_t K) {
    if (!a.set) return K;
    if (a.has_groups) return group_or(a, which, K);
    return (a.mask & kbit) ? (int64_t)1 : K;
}

// mfma_w4a8 with source zero points or a u8 source: the tiled kernel's third
// mode (weights column sums per group from a pre-pass), at every M
bool w4a8_src_zp_mode(const qmm_matmul_desc_t &D) {
    return D.zps[QMM_SRC].set || D.src.dt == dt_u8;
}

int supports_gemm_w4a8(const qmm_matmul_desc_t &D, const generic_params_t &P) {
    const int nd = D.dst.ndims;
    if (nd != 2) return QMM_UNIMPLEMENTED;
    if ((D.src.dt != dt_s8 && D.src.dt != dt_u8) || !is_int4(D.wei.dt))
        return QMM_UNIMPLEMENTED;
    if (!one_of(D.dst.dt, {dt_f32, dt_bf16, dt_f16, dt_s32, dt_s8, dt_u8}))
        return QMM_UNIMPLEMENTED;
    if (P.M == 0 || P.N == 0 || P.K == 0) return QMM_UNIMPLEMENTED;
    if (P.M > (1 << 30) || P.N > (1 << 30) || P.K > 131072)
        return QMM_UNIMPLEMENTED;
    if (!one_of(D.wei_layout, {QMM_LAYOUT_PLAIN, QMM_LAYOUT_MFMA_W4K64}))
        return QMM_UNIMPLEMENTED;
    if (D.src.strides[1] != 1 || D.src.strides[0] % 16 != 0)
        return QMM_UNIMPLEMENTED;
    // whole 64-k tiles per group, every buffer's K extent a whole number of
    // groups
    // (or groups of 32 k, two per tile: the tiled kernel at every M)
    const int64_t gk = P.group_k;
    if (P.K % 64 != 0 || (gk % 64 != 0 && gk != 32) || gk > 32768)
        return QMM_UNIMPLEMENTED;
    if (gk == 32 && w4a8_src_zp_mode(D)) return QMM_UNIMPLEMENTED;
    const qmm_quant_t &ss = D.scales[QMM_SRC], &ws = D.scales[QMM_WEI];
    const qmm_quant_t &wz = D.zps[QMM_WEI], &sz = D.zps[QMM_SRC];
    if (k_extent(ss, 1, 2, P.K) % gk || k_extent(ws, 0, 1, P.K) % gk
            || k_extent(wz, 0, 1, P.K) % gk || k_extent(sz, 1, 2, P.K) % gk)
        return QMM_UNIMPLEMENTED;
    // Source zero points, or a u8 source (read as s8 = u8 - 128 with the zero
    // point moved along): the group's s32 sum is 16 * sum (s - z_s)(w - z_w),
    // |s - z_s| <= 383 with 8-bit source zero points, so the bound of the
    // weights zero-point comment below tightens to gk <= 8192 (4-bit or no
    // weights zero points) / 1024 (8-bit ones); s32 source zero points have
    // no bound and stay with the generic implementation.
    const bool src_zp_mode = w4a8_src_zp_mode(D);
    if (sz.set && !one_of(sz.dt, {dt_s8, dt_u8})) return QMM_UNIMPLEMENTED;
    if (src_zp_mode
            && gk > (wz.set && one_of(wz.dt, {dt_s8, dt_u8}) ? 1024 : 8192))
        return QMM_UNIMPLEMENTED;
    if (ss.set && !one_of(ss.dt, {dt_f32, dt_f16, dt_bf16}))
        return QMM_UNIMPLEMENTED;
    if (ws.set) {
        if (!one_of(ws.dt, {dt_f32, dt_f16, dt_bf16})) return QMM_UNIMPLEMENTED;
        if (P.q_wei_scale.g1 != 1) return QMM_UNIMPLEMENTED; // N groups
    }
    if (wz.set) {
        // The kernels keep 16 * sum s * (w - z) of a group in s32 (the weights
        // enter the MFMA as 16 w') and apply the zero point through the
        // group's source row sum with a 24-bit multiply. That sum is bounded by
        // 16 * 128 * max|w - z| * gk: within s32 for 4-bit zero points at every
        // group size taken here (|w - z| <= 23, gk <= 32768), for 8-bit ones
        // (|w - z| <= 255) up to gk = 3968; s32 zero points have no bound.
        // The rest goes to the generic implementation.
        if (!one_of(wz.dt, {dt_s8, dt_u8, dt_s4, dt_u4}))
            return QMM_UNIMPLEMENTED;
        if (one_of(wz.dt, {dt_s8, dt_u8}) && gk > 3968) return QMM_UNIMPLEMENTED;
        if (P.q_wei_zp.g1 != 1) return QMM_UNIMPLEMENTED;
    }
    epilogue_t ep;
    if (!build_epilogue(ep, P, nullptr, true)) return QMM_UNIMPLEMENTED;
    return QMM_OK;
}

// scratchpad of mfma_w4a8 behind the packed weights: the per-group arrays
struct w4a8_scratch_t {
    int64_t Mpad, Npad, ng;
    bool has_zp, src_zp;
    size_t ss_off, rs_off, sw_off, zw_off, zs_off, c2_off, total;
};
w4a8_scratch_t w4a8_scratch(const qmm_matmul_desc_t &D,
        const generic_params_t &P) {
    w4a8_scratch_t s;
    s.Mpad = round_up(P.M, 256) + 256;
    s.Npad = round_up(P.N, 256) + 256;
    s.ng = P.ngroups_k;
    s.src_zp = w4a8_src_zp_mode(D);
    s.has_zp = D.zps[QMM_WEI].set || D.wei.dt == dt_u4 || s.src_zp;
    const size_t rows = (size_t)s.ng * s.Mpad * 4, cols = (size_t)s.ng * s.Npad * 4;
    s.ss_off = 0;
    s.sw_off = rows;
    s.rs_off = rows + cols;
    s.zw_off = s.rs_off + (s.has_zp ? rows : 0);
    s.zs_off = s.zw_off + (s.has_zp ? cols : 0);
    s.c2_off = s.zs_off + (s.src_zp ? rows : 0);
    s.total = s.c2_off + (s.src_zp ? cols : 0);
    return s;
}

// rows <= 64: how the split-K streaming kernel cuts K
struct w4a8_small_plan_t {
    bool use;
    int splits, gps, ldp;
    size_t part_bytes;
};
w4a8_small_plan_t w4a8_small_plan(const generic_params_t &P, int variant) {
    w4a8_small_plan_t s;
    std::memset(&s, 0, sizeof(s));
    // whole 64-k tiles per group, or groups of 32 k
    const bool half = P.group_k == 32;
    s.use = P.M <= W4A8_SMALL_MAX_M && variant == 0 && (P.group_k >= 64 || half);
    if (!s.use) return s;
    const int64_t ng = P.ngroups_k, tpg = P.group_k / 64;
    const int64_t nblk = (P.N + 127) / 128;
    // as many workgroups as the chip holds at once (2 per CU, 1 for 64 rows),
    // but no more slices than keep the partial results (written and read once
    // each) small next to the weights
    const int64_t slots = P.M > 32 ? 256 : 512;
    int64_t want = slots / nblk;
    const int64_t cap = P.K / (16 * P.M) > 2 ? P.K / (16 * P.M) : 2;
    if (want > cap) want = cap;
    if (want < 1) want = 1;
    if (want > ng) want = ng;
    int64_t gps = (ng + want - 1) / want;
    if (half) gps = (gps + 1) / 2 * 2; // whole tiles per slice
    // a slice of at most one chunk of 16 tiles where the groups allow it
    const int64_t one_chunk = half ? 32 : (16 / tpg > 1 ? 16 / tpg : 1);
    if (gps > one_chunk) gps = one_chunk;
    const int64_t max_gps = (half ? 2 : 1) * W4A8_SMALL_MAX_GPS;
    if (gps > max_gps) gps = max_gps;
    s.gps = (int)gps;
    s.splits = (int)((ng + gps - 1) / gps);
    s.ldp = (int)round_up(P.N, 4);
    s.part_bytes = (size_t)s.splits * P.M * s.ldp * 4;
    return s;
}

// f16 activations x u8 / s8 weights whose scales and zero points do not vary
// along K, at 256 rows and more (below that the decode implementation's
// kernels, which work on blocks of 64 rows, waste less of a tile): the weights
// in QMM_LAYOUT_MFMA_B8, converted to f16 in registers
int supports_gemm_f16w8(const qmm_matmul_desc_t &D, const generic_params_t &P) {
    if (D.dst.ndims != 2) return QMM_UNIMPLEMENTED;
    if (D.src.dt != dt_f16 || !is_int8(D.wei.dt) || !D.apply_to_int)
        return QMM_UNIMPLEMENTED;
    if (!one_of(D.dst.dt, {dt_f16, dt_f32})) return QMM_UNIMPLEMENTED;
    if (P.M < 256 || P.N == 0 || P.K < 5 * 32 || P.K % 32 != 0)
        return QMM_UNIMPLEMENTED;
    if (P.M > INT32_MAX || P.N > INT32_MAX || P.K > INT32_MAX)
        return QMM_UNIMPLEMENTED;
    if (!one_of(D.wei_layout, {QMM_LAYOUT_PLAIN, QMM_LAYOUT_MFMA_B8}))
        return QMM_UNIMPLEMENTED;
    if (D.src.strides[1] != 1 || D.src.strides[0] % 8 != 0)
        return QMM_UNIMPLEMENTED;
    // 32-bit offsets inside a block tile of the source / a column block of the
    // packed weights
    if (256 * 2 * D.src.strides[0] + 64 >= ((int64_t)1 << 32)
            || 8 * b8_geom(1, P.K, P.N).kb32 * 1024 >= ((int64_t)1 << 32))
        return QMM_UNIMPLEMENTED;
    if (D.zps[QMM_SRC].set || D.zps[QMM_DST].set) return QMM_UNIMPLEMENTED;
    if (D.scales[QMM_SRC].set && D.scales[QMM_SRC].mask != 0)
        return QMM_UNIMPLEMENTED;
    const qmm_quant_t &ws = D.scales[QMM_WEI], &wz = D.zps[QMM_WEI];
    if (ws.set) {
        if (!one_of(ws.dt, {dt_f32, dt_f16, dt_bf16})) return QMM_UNIMPLEMENTED;
        if ((ws.mask & ~2) || P.q_wei_scale.g1 != 1) return QMM_UNIMPLEMENTED;
    }
    if (wz.set) {
        // byte-sized zero points: 1152 - offset + zero point is then an integer
        // that f16 holds exactly
        if (!one_of(wz.dt, {dt_s8, dt_u8})) return QMM_UNIMPLEMENTED;
        if ((wz.mask & ~2) || P.q_wei_zp.g1 != 1) return QMM_UNIMPLEMENTED;
    }
    epilogue_t ep;
    if (!build_epilogue(ep, P, nullptr)) return QMM_UNIMPLEMENTED;
    return QMM_OK;
}

int supports_gemv_w4(const qmm_matmul_desc_t &D, const generic_params_t &P) {
    const int nd = D.dst.ndims;
    if (nd != 2) return QMM_UNIMPLEMENTED;
    const bool w8 = is_int8(D.wei.dt);
    if (!one_of(D.src.dt, {dt_bf16, dt_f16}) || !(is_int4(D.wei.dt) || w8)
            || !D.apply_to_int)
        return QMM_UNIMPLEMENTED;
    if (D.src.dt == dt_bf16 && !one_of(D.dst.dt, {dt_bf16, dt_f32}))
        return QMM_UNIMPLEMENTED;
    if (D.src.dt == dt_f16 && !one_of(D.dst.dt, {dt_f16, dt_f32}))
        return QMM_UNIMPLEMENTED;
    if (P.M == 0 || P.N == 0 || P.K == 0) return QMM_UNIMPLEMENTED;
    if (P.M > INT32_MAX || P.N > INT32_MAX || P.K > INT32_MAX)
        return QMM_UNIMPLEMENTED;
    if (!one_of(D.wei_layout,
                {QMM_LAYOUT_PLAIN, w8 ? QMM_LAYOUT_MFMA_W8 : QMM_LAYOUT_MFMA_W4}))
        return QMM_UNIMPLEMENTED;
    if (D.src.strides[1] != 1 || P.K % 8 != 0 || D.src.strides[0] % 8 != 0)
        return QMM_UNIMPLEMENTED;
    if (w8) {
        // 8-bit weights run in the kernel's all-unconditional-loads variant
        // only: 16-bit scales, byte-sized zero points, K groups of 128 << s
        // (or one group over all of K); the rest is the generic kernel's
        const qmm_quant_t &s8 = D.scales[QMM_WEI], &z8 = D.zps[QMM_WEI];
        if (!s8.set || !one_of(s8.dt, {dt_f16, dt_bf16})) return QMM_UNIMPLEMENTED;
        if (z8.set && !one_of(z8.dt, {dt_s8, dt_u8, dt_s4, dt_u4}))
            return QMM_UNIMPLEMENTED;
        auto pow2_of_128 = [&](int64_t g) {
            if (g >= round_up(P.K, 128)) return true;
            if (g % 128) return false;
            const int64_t q = g / 128;
            return (q & (q - 1)) == 0;
        };
        if ((s8.mask & 1) && !pow2_of_128(P.q_wei_scale.g0)) return QMM_UNIMPLEMENTED;
        if (z8.set && (z8.mask & 1) && !pow2_of_128(P.q_wei_zp.g0))
            return QMM_UNIMPLEMENTED;
        if (D.src.strides[0] >= ((int64_t)1 << 31) || P.M >= (1 << 23))
            return QMM_UNIMPLEMENTED;
    }
    if (D.zps[QMM_SRC].set || D.zps[QMM_DST].set) return QMM_UNIMPLEMENTED;
    if (D.scales[QMM_SRC].set && D.scales[QMM_SRC].mask != 0)
        return QMM_UNIMPLEMENTED;
    const qmm_quant_t &ws = D.scales[QMM_WEI], &wz = D.zps[QMM_WEI];
    if (ws.set) {
        if (!one_of(ws.dt, {dt_f32, dt_f16, dt_bf16})) return QMM_UNIMPLEMENTED;
        if (P.q_wei_scale.g1 != 1) return QMM_UNIMPLEMENTED; // N groups
        if ((ws.mask & 1) && (P.q_wei_scale.g0 % 32 != 0))
            return QMM_UNIMPLEMENTED;
        if ((ws.mask & 1) && P.K % P.q_wei_scale.g0 != 0)
            return QMM_UNIMPLEMENTED;
    }
    if (wz.set) {
        if (!one_of(wz.dt, {dt_s32, dt_s8, dt_u8, dt_s4, dt_u4}))
            return QMM_UNIMPLEMENTED;
        if (P.q_wei_zp.g1 != 1) return QMM_UNIMPLEMENTED;
        if ((wz.mask & 1) && (P.q_wei_zp.g0 % 32 != 0)) return QMM_UNIMPLEMENTED;
        if ((wz.mask & 1) && P.K % P.q_wei_zp.g0 != 0) return QMM_UNIMPLEMENTED;
    }
    epilogue_t ep;
    if (!build_epilogue(ep, P, nullptr)) return QMM_UNIMPLEMENTED;
    return QMM_OK;
}

// plain 16-bit matmul: no quantization attributes, source rows K-contiguous,
// weights and dst rows N-contiguous, batch dims that fold into one stride
int supports_gemm_f16(const qmm_matmul_desc_t &D, const generic_params_t &P) {
    const int nd = D.dst.ndims;
    if (!one_of(D.src.dt, {dt_f16, dt_bf16}) || D.wei.dt != D.src.dt)
        return QMM_UNIMPLEMENTED;
    if (D.dst.dt != D.src.dt && D.dst.dt != dt_f32) return QMM_UNIMPLEMENTED;
    if (D.wei_layout != QMM_LAYOUT_PLAIN) return QMM_UNIMPLEMENTED;
    for (int i = 0; i < 3; i++)
        if (D.scales[i].set || D.zps[i].set) return QMM_UNIMPLEMENTED;
    if (P.M == 0 || P.N == 0 || P.K == 0) return QMM_UNIMPLEMENTED;
    if (P.M > INT32_MAX || P.N > INT32_MAX || P.K > INT32_MAX
            || P.batch > 65535 || (P.M + 63) / 64 > 65535)
        return QMM_UNIMPLEMENTED;
    if (D.src.strides[nd - 1] != 1 || D.wei.strides[nd - 1] != 1
            || D.dst.strides[nd - 1] != 1)
        return QMM_UNIMPLEMENTED;
    int64_t sb;
    if (!fold_batch(D.src, D.dst, sb) || !fold_batch(D.wei, D.dst, sb))
        return QMM_UNIMPLEMENTED;
    epilogue_t ep;
    if (!build_epilogue(ep, P, nullptr)) return QMM_UNIMPLEMENTED;
    return QMM_OK;
}

int supports_generic(const qmm_matmul_desc_t &D, const generic_params_t &P) {
    if (D.wei_layout != QMM_LAYOUT_PLAIN) return QMM_UNIMPLEMENTED;
    const int s = D.src.dt, w = D.wei.dt, d = D.dst.dt;
    if (is_int8(s)) {
        // src/cpu/matmul/ref_matmul_int8.hpp:43-129
        if (!is_wei_int(w)) return QMM_UNIMPLEMENTED;
        if (!one_of(d, {dt_f32, dt_bf16, dt_f16, dt_s32, dt_s8, dt_u8}))
            return QMM_UNIMPLEMENTED;
    } else {
        // src/cpu/matmul/ref_matmul.hpp:44-157
        if (!one_of(s, {dt_f32, dt_bf16, dt_f16, dt_f8_e5m2, dt_f8_e4m3}))
            return QMM_UNIMPLEMENTED;
        if (!one_of(w, {dt_f32, dt_bf16, dt_f16, dt_f8_e5m2, dt_f8_e4m3, dt_u8,
                    dt_s8, dt_u4, dt_s4}))
            return QMM_UNIMPLEMENTED;
        if (!one_of(d, {dt_f32, dt_bf16, dt_f16, dt_f8_e5m2, dt_f8_e4m3}))
            return QMM_UNIMPLEMENTED;
        if (!(s == w || one_of(w, {dt_bf16, dt_f16, dt_u8, dt_s8, dt_u4, dt_s4})))
            return QMM_UNIMPLEMENTED;
        if (is_int8(w) && !D.apply_to_int) return QMM_UNIMPLEMENTED;
        if (s == dt_f32 && d != dt_f32) return QMM_UNIMPLEMENTED;
        if (s == dt_bf16 && !one_of(d, {dt_f32, dt_bf16})) return QMM_UNIMPLEMENTED;
        if (s == dt_f16 && !one_of(d, {dt_f32, dt_f16})) return QMM_UNIMPLEMENTED;
        if (D.zps[QMM_SRC].set || D.zps[QMM_DST].set) return QMM_UNIMPLEMENTED;
        if (D.scales[QMM_SRC].set && D.scales[QMM_SRC].mask != 0)
            return QMM_UNIMPLEMENTED;
        if (D.scales[QMM_WEI].set && !P.decompress
                && (D.scales[QMM_WEI].mask & ~(1 << (D.dst.ndims - 1))))
            return QMM_UNIMPLEMENTED;
    }
    if (D.scales[QMM_DST].set
            && ((D.scales[QMM_DST].mask & ~(3 << (D.dst.ndims - 2)))
                    || (D.scales[QMM_DST].has_groups
                            && (D.scales[QMM_DST].g0 != 1
                                    || D.scales[QMM_DST].g1 != 1))))
        return QMM_UNIMPLEMENTED;
    if (D.zps[QMM_DST].set && D.zps[QMM_DST].dt != dt_s32)
        return QMM_UNIMPLEMENTED;
    return QMM_OK;
}

const char *impl_names[impl_count] = {"hip:gfx950:mfma_b8",
        "hip:gfx950:mfma_w4a8", "hip:gfx950:mfma_f16w8", "hip:gfx950:decode_w4",
        "hip:gfx950:mfma_f16", "hip:gfx950:generic"};

// A kernel-selection override from the environment: an integer in [lo, hi],
// else the default.
int env_variant(const char *name, int lo, int hi, int dflt) {
    const char *v = std::getenv(name);
    if (!v || !*v) return dflt;
    char *end = nullptr;
    const long x = std::strtol(v, &end, 10);
    if (end == v || *end || x < lo || x > hi) return dflt;
    return (int)x;
}

} // namespace

extern "C" {

const char *qmm_last_error(void) {
    return g_last_error.c_str();
}

int qmm_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) return 0;
    return n;
}

int qmm_matmul_impl_count(void) {
    return impl_count;
}
const char *qmm_matmul_impl_name(int impl) {
    return impl >= 0 && impl < impl_count ? impl_names[impl] : "";
}

int qmm_matmul_impl_supports(int impl, const qmm_matmul_desc_t *desc) {
    if (!desc || desc->dst.ndims < 2 || desc->dst.ndims > QMM_MAX_NDIMS)
        return QMM_INVALID_ARGUMENTS;
    generic_params_t P;
    build_generic(P, *desc);
    switch (impl) {
        case impl_gemm_b8: return supports_gemm_b8(*desc, P);
        case impl_gemm_w4a8: return supports_gemm_w4a8(*desc, P);
        case impl_gemm_f16w8: return supports_gemm_f16w8(*desc, P);
        case impl_gemv_w4: return supports_gemv_w4(*desc, P);
        case impl_gemm_f16: return supports_gemm_f16(*desc, P);
        case impl_generic: return supports_generic(*desc, P);
        default: return QMM_INVALID_ARGUMENTS;
    }
}

size_t qmm_packed_size(int layout, int dt, int64_t batch, int64_t K, int64_t N) {
    (void)dt;
    if (layout == QMM_LAYOUT_MFMA_B8)
        return (size_t)b8_geom(batch, K, N).total_bytes;
    if (layout == QMM_LAYOUT_MFMA_W4)
        return (size_t)w4_geom(batch, K, N).total_bytes;
    if (layout == QMM_LAYOUT_MFMA_W4K64)
        return (size_t)w4k_geom(batch, K, N).total_bytes;
    if (layout == QMM_LAYOUT_MFMA_W8)
        return (size_t)w4_geom(batch, K, N).total_bytes * 2;
    return 0;
}

int qmm_matmul_impl_preferred_wei_layout(
        int impl, const qmm_matmul_desc_t *desc) {
    if (!desc) return QMM_LAYOUT_PLAIN;
    qmm_matmul_desc_t d = *desc;
    // strides of an undecided weights tensor are not meaningful yet
    for (int layout : {QMM_LAYOUT_MFMA_B8, QMM_LAYOUT_MFMA_W4K64,
                 QMM_LAYOUT_MFMA_W4, QMM_LAYOUT_MFMA_W8}) {
        d.wei_layout = layout;
        if (qmm_matmul_impl_supports(impl, &d) == QMM_OK) return layout;
    }
    return QMM_LAYOUT_PLAIN;
}

int qmm_matmul_preferred_wei_layout(const qmm_matmul_desc_t *desc) {
    for (int impl = 0; impl < impl_generic; impl++) {
        const int layout = qmm_matmul_impl_preferred_wei_layout(impl, desc);
        if (layout != QMM_LAYOUT_PLAIN) return layout;
    }
    return QMM_LAYOUT_PLAIN;
}

// Large u8-source problems go through the 256 x 256 kernel after a pre-pass
// that rewrites the source as s8: room for that copy, behind the packed weights.
// mfma_b8 with weights zero points or u8 weights: the source's row sums (s32
// per batch and row) live in the scratchpad behind the packed weights
static bool b8_needs_rowsum(const qmm_matmul_desc_t &D) {
    return is_int8(D.src.dt) && (D.wei.dt == dt_u8 || D.zps[QMM_WEI].set);
}
static size_t b8_rowsum_bytes(const qmm_matmul_desc_t &D) {
    if (!b8_needs_rowsum(D)) return 0;
    const int nd = D.dst.ndims;
    int64_t rows = D.dst.dims[nd - 2];
    for (int d = 0; d < nd - 2; d++)
        rows *= D.dst.dims[d];
    return (size_t)rows * 4;
}

static size_t u8_copy_bytes(const qmm_matmul_desc_t *desc) {
    const int nd = desc->dst.ndims;
    if (desc->src.dt != dt_u8) return 0;
    if (b8_needs_rowsum(*desc)) return 0; // never the 256 x 256 kernels
    const int64_t M = desc->dst.dims[nd - 2], N = desc->dst.dims[nd - 1];
    const int64_t K = desc->src.dims[nd - 1];
    int64_t batch = 1;
    for (int d = 0; d < nd - 2; d++)
        batch *= desc->dst.dims[d];
    if (K % 64 != 0 || K <= 256) return 0;
    if (((M + 255) / 256) * ((N + 255) / 256) * batch < 192) return 0;
    return (size_t)(batch * M * K);
}

static size_t round256(size_t v) {
    return (v + 255) / 256 * 256;
}

// mfma_f16w8 with its K range cut into slices: the slices' f32 sums
static size_t f16w8_part_bytes(const qmm_matmul_desc_t &D) {
    const int64_t M = D.dst.dims[0], N = D.dst.dims[1], K = D.src.dims[1];
    const int splits = gemm_f16w8_splits(M, N, K);
    return splits > 1 ? (size_t)splits * M * round_up(N, 4) * 4 : 0;
}

size_t qmm_matmul_scratch_size(int impl, const qmm_matmul_desc_t *desc) {
    const int nd = desc->wei.ndims;
    const int64_t K = desc->wei.dims[nd - 2], N = desc->wei.dims[nd - 1];
    if (impl == impl_gemm_b8) {
        const size_t packed = desc->wei_layout == QMM_LAYOUT_PLAIN
                ? qmm_packed_size(QMM_LAYOUT_MFMA_B8, desc->wei.dt,
                        wei_batch(*desc), K, N)
                : 0;
        const size_t copy = u8_copy_bytes(desc) + b8_rowsum_bytes(*desc);
        return copy ? round256(packed) + copy : packed;
    }
    if (impl == impl_gemm_w4a8) {
        generic_params_t P;
        build_generic(P, *desc);
        const size_t packed = desc->wei_layout == QMM_LAYOUT_PLAIN
                ? round256(qmm_packed_size(
                        QMM_LAYOUT_MFMA_W4K64, desc->wei.dt, 1, K, N))
                : 0;
        const w4a8_small_plan_t sm = w4a8_small_plan(P, 0);
        const size_t big = w4a8_scratch(*desc, P).total;
        // the tile-configuration override of the tuning hook bypasses the
        // small-row kernel, so leave room for either
        return packed + (sm.use && sm.part_bytes > big ? sm.part_bytes : big);
    }
    if (impl == impl_gemm_f16w8 && desc->wei_layout != QMM_LAYOUT_PLAIN)
        return f16w8_part_bytes(*desc);
    if (desc->wei_layout != QMM_LAYOUT_PLAIN) return 0;
    if (impl == impl_gemm_f16w8)
        return round256(qmm_packed_size(QMM_LAYOUT_MFMA_B8, desc->wei.dt, 1, K, N))
                + f16w8_part_bytes(*desc);
    if (impl == impl_gemv_w4)
        return qmm_packed_size(is_int8(desc->wei.dt) ? QMM_LAYOUT_MFMA_W8
                                                     : QMM_LAYOUT_MFMA_W4,
                desc->wei.dt, 1, K, N);
    return 0;
}

static void *static_scratch_ptr(hipStream_t stream);

int qmm_matmul_plan_create(
        qmm_plan_t **plan, int impl, const qmm_matmul_desc_t *desc) {
    if (!plan || !desc) return QMM_INVALID_ARGUMENTS;
    const int st = qmm_matmul_impl_supports(impl, desc);
    if (st != QMM_OK) return st;
    qmm_plan *p = new (std::nothrow) qmm_plan();
    if (!p) return QMM_OUT_OF_MEMORY;
    p->impl = impl;
    p->desc = *desc;
    p->dev = nullptr;
    build_generic(p->host, *desc);
    p->scratch_bytes = qmm_matmul_scratch_size(impl, desc);
    p->gemm_variant = env_variant("QMM_GEMM_VARIANT", 0, 6, 0);
    p->w4a8_variant = env_variant("QMM_W4A8_VARIANT", 0, 5, 0);
    p->b8x_variant = env_variant("QMM_B8X_VARIANT", 0, 5, 1);
    p->measure = env_variant("QMM_MEASURE", 0, 3, 0);
    // resolve the static scratch's address on the current device now, so that
    // qmm_matmul_launch_static_scratch() finds it ready (a plan used on another
    // device resolves it at its first launch there)
    if (p->scratch_bytes && p->scratch_bytes <= (size_t)QMM_STATIC_SCRATCH_BYTES)
        (void)static_scratch_ptr(nullptr);
    // the generic kernel reads its (large) descriptor from device memory; the
    // tiled kernels fall back to it for operands they cannot address (pointers
    // that are not 16-byte aligned), so every plan over plain weights keeps one
    if (desc->wei_layout == QMM_LAYOUT_PLAIN
            && supports_generic(*desc, p->host) == QMM_OK) {
        hipError_t e = hipMalloc((void **)&p->dev, sizeof(generic_params_t));
        if (e != hipSuccess) {
            delete p;
            return hip_fail(e, "hipMalloc(plan)");
        }
        e = hipMemcpy(p->dev, &p->host, sizeof(generic_params_t),
                hipMemcpyHostToDevice);
        if (e != hipSuccess) {
            (void)hipFree(p->dev);
            delete p;
            return hip_fail(e, "hipMemcpy(plan)");
        }
    }
    *plan = p;
    return QMM_OK;
}

void qmm_matmul_plan_destroy(qmm_plan_t *plan) {
    if (!plan) return;
    if (plan->dev) (void)hipFree(plan->dev);
    delete plan;
}

static bool aligned16(const void *p) {
    return ((uintptr_t)p & 15) == 0;
}

// ---- scratch for callers that cannot allocate ------------------------------
// One array per GPU, resident from the moment the library's code is loaded on
// that GPU until the process ends. Host code never uses the array's name as an
// address: that name is a host-side stand-in, the device address is asked for
// once per device (with that device current) and kept.
static __device__ __align__(256) unsigned char scratch[QMM_STATIC_SCRATCH_BYTES];

// `stream`: the device is the stream's when it names one (a launch may target
// a device that is not the calling thread's current one), else the current one.
static void *static_scratch_ptr(hipStream_t stream) {
    constexpr int MAX_DEV = 64;
    static std::mutex mu;
    static void *ptr[MAX_DEV] = {};
    int dev = -1;
    if (!stream || hipStreamGetDevice(stream, &dev) != hipSuccess) {
        if (hipGetDevice(&dev) != hipSuccess) dev = -1;
    }
    if (dev < 0 || dev >= MAX_DEV) {
        g_last_error = "no HIP device for the static scratch";
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(mu);
    if (!ptr[dev]) {
        // the symbol's address is per device: ask with that device current
        int cur = -1;
        (void)hipGetDevice(&cur);
        if (cur != dev && hipSetDevice(dev) != hipSuccess) {
            g_last_error = "hipSetDevice for the static scratch failed";
            return nullptr;
        }
        void *q = nullptr;
        const hipError_t e = hipGetSymbolAddress(&q, HIP_SYMBOL(scratch));
        if (cur != dev && cur >= 0) (void)hipSetDevice(cur);
        if (e != hipSuccess || !q) {
            g_last_error = std::string("hipGetSymbolAddress(scratch): ")
                    + hipGetErrorString(e);
            return nullptr;
        }
        ptr[dev] = q;
    }
    return ptr[dev];
}

int qmm_matmul_launch_static_scratch(const qmm_plan_t *plan,
        const qmm_matmul_args_t *args, void *hip_stream) {
    if (!plan || !args) return QMM_INVALID_ARGUMENTS;
    if (plan->scratch_bytes > (size_t)QMM_STATIC_SCRATCH_BYTES)
        return fail(QMM_INVALID_ARGUMENTS,
                "the problem needs more scratch than the static buffer holds "
                "(QMM_STATIC_SCRATCH_BYTES)");
    qmm_matmul_args_t a = *args;
    a.scratch = nullptr;
    if (plan->scratch_bytes) {
        a.scratch = static_scratch_ptr((hipStream_t)hip_stream);
        if (!a.scratch) return QMM_RUNTIME_ERROR;
    }
    return qmm_matmul_launch(plan, &a, hip_stream);
}

int qmm_matmul_launch(const qmm_plan_t *plan, const qmm_matmul_args_t *args,
        void *hip_stream) {
    if (!plan || !args) return QMM_INVALID_ARGUMENTS;
    hipStream_t stream = (hipStream_t)hip_stream;
    const qmm_matmul_desc_t &D = plan->desc;
    const generic_params_t &P = plan->host;
    const int nd = D.dst.ndims;
    if (P.M == 0 || P.N == 0 || P.batch == 0) return QMM_OK;
    if (!args->src || !args->wei || !args->dst)
        return fail(QMM_INVALID_ARGUMENTS, "null src/weights/dst pointer");
    for (int i = 0; i < 3; i++) {
        if (D.scales[i].set && !args->scales[i])
            return fail(QMM_INVALID_ARGUMENTS, "scales buffer is missing");
        if (D.zps[i].set && !args->zps[i])
            return fail(QMM_INVALID_ARGUMENTS, "zero points buffer is missing");
    }
    for (int i = 0; i < D.npo; i++)
        if ((D.po[i].kind == pk_binary || D.po[i].kind == pk_prelu)
                && !args->po_arg[i])
            return fail(QMM_INVALID_ARGUMENTS, "post-op argument is missing");
    if (D.bias.ndims && !args->bias)
        return fail(QMM_INVALID_ARGUMENTS, "bias pointer is missing");
    if (plan->scratch_bytes && !args->scratch)
        return fail(QMM_INVALID_ARGUMENTS, "scratch buffer is missing");

    const int gemm_variant = plan->gemm_variant;
    // 4: as 0, but 5 .. 64 rows take the split-K kernel and its reduction; 5: as
    // 0, but they take the one-launch kernel wherever it applies
    const bool w4a8_no_mid = plan->w4a8_variant == 4, w4a8_all_mid = plan->w4a8_variant == 5;
    const int w4a8_variant = plan->w4a8_variant >= 4 ? 0 : plan->w4a8_variant;
    int impl = plan->impl;
    if (impl != impl_generic && impl != impl_gemm_f16 && !aligned16(args->src)) {
        if (!plan->dev)
            return fail(QMM_INVALID_ARGUMENTS,
                    "source pointer must be 16-byte aligned");
        impl = impl_generic;
    }

    if (impl == impl_generic) {
        if (!plan->dev) return fail(QMM_RUNTIME_ERROR, "plan has no device copy");
        launch_matmul_generic(plan->dev, P, *args, stream);
    } else if (impl == impl_gemm_b8) {
        const bool f8 = D.src.dt == dt_f8_e4m3;
        gemm_params_t g;
        std::memset(&g, 0, sizeof(g));
        if (!build_epilogue(g.ep, P, args))
            return fail(QMM_RUNTIME_ERROR, "epilogue does not fold");
        g.A = (const uint8_t *)args->src;
        g.lda = D.src.strides[nd - 2];
        g.switches = (plan->b8x_variant == 0 ? GEMM_MFMA32 : 0)
                | (plan->b8x_variant == 2 ? GEMM_TWO_PER_CU : 0)
                | (plan->b8x_variant >= 3 ? GEMM_ONE_PER_CU : 0)
                | (plan->b8x_variant == 4 ? GEMM_NOT_PERSISTENT : 0)
                | (plan->b8x_variant == 5 ? GEMM_NO_STAGGER : 0)
                | (plan->measure & 1 ? GEMM_SKIP_EPILOGUE : 0)
                | (plan->measure & 2 ? GEMM_STAMPS : 0);
        fold_batch(D.src, D.dst, g.a_sb);
        const int64_t wb = wei_batch(D);
        const b8_geom_t geom = b8_geom(wb, P.K, P.N);
        const uint8_t *packed = (const uint8_t *)args->wei;
        if (D.wei_layout == QMM_LAYOUT_PLAIN) {
            int64_t sb, sk, sn;
            plain_wei_strides(D, sb, sk, sn);
            if (wb == 1) sb = 0;
            launch_pack_b8(args->wei, args->scratch, D.wei.dt, wb, P.K, P.N, sb,
                    sk, sn, !f8, stream);
            packed = (const uint8_t *)args->scratch;
        }
        g.B = packed;
        g.b_sb = wb == 1 ? 0 : geom.batch_bytes;
        g.colsum = f8 ? nullptr : (const int32_t *)(packed + geom.colsum_off);
        g.colsum_sb = wb == 1 ? 0 : geom.Npad;
        g.src_zp = D.zps[QMM_SRC].set ? args->zps[QMM_SRC] : nullptr;
        g.src_zp_dt = D.zps[QMM_SRC].dt;
        g.a_is_u8 = D.src.dt == dt_u8;
        g.M = (int32_t)P.M;
        g.N = (int32_t)P.N;
        g.K = (int32_t)P.K;
        g.batch = (int32_t)P.batch;
        g.kb32 = (int32_t)geom.kb32;
        g.nb32 = (int32_t)geom.nb32;
        // at most 64 rows of one matrix: the streaming kernel (it forms the
        // row sums a weights zero point needs itself)
        if (!f8 && P.M <= 64 && P.batch == 1 && gemm_variant == 0) {
            if (b8_needs_rowsum(D)) {
                const qmm_quant_t &wz = D.zps[QMM_WEI];
                g.wei_zp = wz.set ? args->zps[QMM_WEI] : nullptr;
                g.wei_zp_dt = wz.dt;
                g.wei_zp_sn = wz.set && (wz.mask & (1 << (nd - 1))) ? 1 : 0;
                g.w_off = D.wei.dt == dt_u8 ? 128 : 0;
            }
            launch_gemv_b8(g, stream);
            const hipError_t e = hipGetLastError();
            if (e != hipSuccess) return hip_fail(e, "kernel launch");
            return QMM_OK;
        }
        if (b8_needs_rowsum(D)) {
            const qmm_quant_t &wz = D.zps[QMM_WEI];
            int32_t *rs = (int32_t *)((uint8_t *)args->scratch
                    + (D.wei_layout == QMM_LAYOUT_PLAIN
                                    ? round256(geom.total_bytes)
                                    : 0));
            launch_rowsum_b8(g.A, rs, P.batch, P.M, P.K, g.lda, g.a_sb,
                    D.src.dt == dt_u8, g.src_zp, g.src_zp_dt, stream);
            g.rowsum = rs;
            g.wei_zp = wz.set ? args->zps[QMM_WEI] : nullptr;
            g.wei_zp_dt = wz.dt;
            g.wei_zp_sn = wz.set && (wz.mask & (1 << (nd - 1))) ? 1 : 0;
            g.w_off = D.wei.dt == dt_u8 ? 128 : 0;
        }
        g.M = (int32_t)P.M;
        g.N = (int32_t)P.N;
        g.K = (int32_t)P.K;
        g.batch = (int32_t)P.batch;
        g.kb32 = (int32_t)geom.kb32;
        g.nb32 = (int32_t)geom.nb32;
        // a u8 source is rewritten as s8 by a pre-pass only for the kernels that
        // cannot read it as it is (the 256 x 256 ones with more than 4 k-steps)
        if (g.a_is_u8 && u8_copy_bytes(&D) && args->scratch
                && !gemm_b8x_two_per_cu(g, f8)) {
            gemm_params_t h = g;
            uint8_t *copy = (uint8_t *)args->scratch
                    + (D.wei_layout == QMM_LAYOUT_PLAIN
                                    ? round256(geom.total_bytes)
                                    : 0);
            h.A = copy;
            h.lda = P.K;
            h.a_sb = P.M * P.K;
            h.a_preflipped = 1;
            if (gemm_b8_uses_tile256(h, f8, gemm_variant)) {
                launch_flip_u8(g.A, copy, P.batch, P.M, P.K, g.lda, g.a_sb,
                        stream);
                g = h;
            }
        }
        launch_gemm_b8(g, f8, gemm_variant, stream);
    } else if (impl == impl_gemm_w4a8) {
        w4a8_params_t g;
        std::memset(&g, 0, sizeof(g));
        if (!build_epilogue(g.ep, P, args, true))
            return fail(QMM_RUNTIME_ERROR, "epilogue does not fold");
        const w4k_geom_t geom = w4k_geom(1, P.K, P.N);
        const uint8_t *packed = (const uint8_t *)args->wei;
        uint8_t *arrays = (uint8_t *)args->scratch;
        if (D.wei_layout == QMM_LAYOUT_PLAIN) {
            launch_pack_w4k(args->wei, args->scratch, D.wei.dt, 1, P.K, P.N, 0,
                    D.wei.strides[0], D.wei.strides[1], stream);
            packed = (const uint8_t *)args->scratch;
            arrays += round256(geom.total_bytes);
        }
        const w4a8_scratch_t sc = w4a8_scratch(D, P);
        const qmm_quant_t &ss = D.scales[QMM_SRC], &ws = D.scales[QMM_WEI];
        const qmm_quant_t &wz = D.zps[QMM_WEI];
        w4a8_prep_t q;
        std::memset(&q, 0, sizeof(q));
        q.A = (const uint8_t *)args->src;
        q.lda = D.src.strides[0];
        q.ss = ss.set ? args->scales[QMM_SRC] : nullptr;
        q.sw = ws.set ? args->scales[QMM_WEI] : nullptr;
        q.zw = wz.set ? args->zps[QMM_WEI] : nullptr;
        q.ss_dt = ss.dt;
        q.sw_dt = ws.dt;
        q.zw_dt = wz.dt;
        q.w_off = D.wei.dt == dt_u4 ? 8 : 0;
        q.ss_sm = P.q_src_scale.strides[0];
        q.ss_sk = P.q_src_scale.strides[1];
        q.sw_sk = P.q_wei_scale.strides[0];
        q.sw_sn = P.q_wei_scale.strides[1];
        q.zw_sk = P.q_wei_zp.strides[0];
        q.zw_sn = P.q_wei_zp.strides[1];
        q.ss_g = (int32_t)k_extent(ss, 1, 2, P.K);
        q.sw_g = (int32_t)k_extent(ws, 0, 1, P.K);
        q.zw_g = (int32_t)k_extent(wz, 0, 1, P.K);
        q.M = (int32_t)P.M;
        q.N = (int32_t)P.N;
        q.K = (int32_t)P.K;
        q.gk = (int32_t)P.group_k;
        q.ng = (int32_t)sc.ng;
        q.Mpad = (int32_t)sc.Mpad;
        q.Npad = (int32_t)sc.Npad;
        q.ssT = (float *)(arrays + sc.ss_off);
        q.swT = (float *)(arrays + sc.sw_off);
        q.rsT = sc.has_zp ? (int32_t *)(arrays + sc.rs_off) : nullptr;
        q.zwT = sc.has_zp ? (int32_t *)(arrays + sc.zw_off) : nullptr;
        if (sc.src_zp) {
            const qmm_quant_t &sz = D.zps[QMM_SRC];
            q.zs = sz.set ? args->zps[QMM_SRC] : nullptr;
            q.zs_dt = sz.dt;
            q.zs_sm = P.q_src_zp.strides[0];
            q.zs_sk = P.q_src_zp.strides[1];
            q.zs_g = (int32_t)k_extent(sz, 1, 2, P.K);
            q.a_flip = D.src.dt == dt_u8 ? 0x80808080u : 0u;
            q.kt64 = (int32_t)geom.kt64;
            q.B = packed;
            q.zsT = (int32_t *)(arrays + sc.zs_off);
            q.c2T = (int32_t *)(arrays + sc.c2_off);
        }
        const w4a8_small_plan_t sm = w4a8_small_plan(P, w4a8_variant);
        // the single-token kernel where the split-K kernel is not used
        const bool tiny_only = !sm.use && w4a8_variant == 0 && P.M <= 4
                && (sc.src_zp || q.gk == 32);
        if ((sm.use || tiny_only) && gemm_w4a8_small_takes(q)) {
            w4a8_small_t h;
            std::memset(&h, 0, sizeof(h));
            h.q = q;
            h.B = packed;
            h.tpg = q.gk / 64;
            h.kt64 = (int32_t)geom.kt64;
            h.nb32 = (int32_t)geom.nb32;
            if (P.M <= 4) {
                // single-token decode: the waves of a workgroup cut K between
                // them, at most 16 groups (32 of 32 k) and preferably 16 tiles
                // per wave
                const bool half = q.gk == 32;
                const int64_t maxg = gemm_w4a8_tiny_max_groups(half);
                auto per_wave = [&](int n) {
                    int64_t g = (q.ng + n - 1) / n;
                    return half ? (g + 1) / 2 * 2 : g; // whole tiles per wave
                };
                auto tiles = [&](int64_t g) { return half ? g / 2 : g * h.tpg; };
                int nwv = 4;
                int64_t gpw = per_wave(4);
                if (tiles(gpw) > 16 || gpw > maxg) {
                    nwv = 8;
                    gpw = per_wave(8);
                }
                if (gpw <= maxg) {
                    h.gps = (int32_t)gpw;
                    h.ep = g.ep;
                    launch_gemm_w4a8_tiny(h, sc.has_zp, nwv, stream);
                    const hipError_t e = hipGetLastError();
                    if (e != hipSuccess) return hip_fail(e, "kernel launch");
                    return QMM_OK;
                }
            }
            // 5 .. 64 rows over at least 256 column blocks (one per CU and more:
            // measured on 4096 x 14336 weights, with / without zero points, source
            // scales per 32 k, a u8 source: 19.0 / 16.0 / 31.9 / 22.4 us against
            // 24.9 / 24.5 / 41.8 / 30.4 us for the split-K kernel and its reduction;
            // 48 rows 27.8 against 40.2; on 14336 x 4096 weights, 128 blocks, 27.6
            // against 26.6): one launch, the waves of a workgroup cut K between them
            if (!tiny_only && !w4a8_no_mid && gemm_w4a8_mid_takes((int)P.M, q.gk)
                    && ((P.N + 31) / 32 >= 256 || w4a8_all_mid)) {
                // (8 waves while there are fewer 32-column blocks than CUs)
                // eight waves where two such workgroups fit a CU's LDS or there
                // are fewer 32-column blocks than CUs anyway
                const int wb = gemm_w4a8_mid_wave_bytes((int)P.M, q.gk, sc.src_zp);
                const int nwv = (P.N + 31) / 32 < 256 && 8 * wb <= 160 * 1024 ? 8 : 4;
                h.splits = gemm_w4a8_mid_gpc((int)P.M, q.gk);
                int64_t gpw = (q.ng + nwv - 1) / nwv;
                if (q.gk == 32) gpw = (gpw + 1) / 2 * 2; // whole tiles per wave
                h.gps = (int32_t)gpw;
                h.ep = g.ep;
                launch_gemm_w4a8_mid(h, sc.has_zp, nwv, stream);
                const hipError_t e = hipGetLastError();
                if (e != hipSuccess) return hip_fail(e, "kernel launch");
                return QMM_OK;
            }
            if (!tiny_only) { // else (too many groups per wave): the tiled kernel
                h.gps = sm.gps;
                h.splits = sm.splits;
                h.ldp = sm.ldp;
                h.part = (float *)arrays;
                h.ep = g.ep;
                launch_gemm_w4a8_small(h, sc.has_zp, stream);
                const hipError_t e = hipGetLastError();
                if (e != hipSuccess) return hip_fail(e, "kernel launch");
                return QMM_OK;
            }
        }
        launch_w4a8_prep(q, stream);
        g.A = q.A;
        g.lda = q.lda;
        g.B = packed;
        g.ssT = q.ssT;
        g.rsT = q.rsT;
        g.swT = q.swT;
        g.zwT = q.zwT;
        g.zsT = q.zsT;
        g.c2T = q.c2T;
        g.a_flip = q.a_flip;
        g.M = q.M;
        g.N = q.N;
        g.K = q.K;
        g.Mpad = q.Mpad;
        g.Npad = q.Npad;
        g.kt64 = (int32_t)geom.kt64;
        g.nb32 = (int32_t)geom.nb32;
        g.tpg = q.gk / 64;
        g.ng = q.ng;
        launch_gemm_w4a8(g, w4a8_variant, stream);
    } else if (impl == impl_gemm_f16) {
        gemm16_params_t g;
        std::memset(&g, 0, sizeof(g));
        if (!build_epilogue(g.ep, P, args))
            return fail(QMM_RUNTIME_ERROR, "epilogue does not fold");
        g.A = (const uint16_t *)args->src;
        g.B = (const uint16_t *)args->wei;
        g.lda = D.src.strides[nd - 2];
        g.ldb = D.wei.strides[nd - 2];
        fold_batch(D.src, D.dst, g.a_sb);
        fold_batch(D.wei, D.dst, g.b_sb);
        g.M = (int32_t)P.M;
        g.N = (int32_t)P.N;
        g.K = (int32_t)P.K;
        g.batch = (int32_t)P.batch;
        g.bf = D.src.dt == dt_bf16;
        // the widest aligned load every row start of the operand allows
        auto granule = [](int64_t ld, int64_t sb, const void *ptr) {
            for (int g = 8; g > 1; g >>= 1)
                if (ld % g == 0 && sb % g == 0 && (uintptr_t)ptr % (2 * g) == 0)
                    return g;
            return 1;
        };
        g.a_vec = granule(g.lda, g.a_sb, args->src);
        g.b_vec = granule(g.ldb, g.b_sb, args->wei);
        g.tile = gemm_variant >= 1 && gemm_variant <= 3 ? gemm_variant : 0;
        launch_gemm_f16(g, stream);
    } else if (impl == impl_gemm_f16w8) {
        gemm_params_t g;
        std::memset(&g, 0, sizeof(g));
        if (!build_epilogue(g.ep, P, args))
            return fail(QMM_RUNTIME_ERROR, "epilogue does not fold");
        // the weights scales (left out of the epilogue for decompression
        // problems, whose other kernels apply them to the weights): one per
        // column or one in all, a factor of the f32 sum
        const qmm_quant_t &ws = D.scales[QMM_WEI], &wz = D.zps[QMM_WEI];
        if (ws.set
                && !fold_quant(g.ep.wei_scale, P.q_wei_scale, ws, D.wei, D.dst,
                        false, args->scales[QMM_WEI]))
            return fail(QMM_RUNTIME_ERROR, "weights scales do not fold");
        const b8_geom_t geom = b8_geom(1, P.K, P.N);
        const uint8_t *packed = (const uint8_t *)args->wei;
        if (D.wei_layout == QMM_LAYOUT_PLAIN) {
            launch_pack_b8(args->wei, args->scratch, D.wei.dt, 1, P.K, P.N, 0,
                    D.wei.strides[0], D.wei.strides[1], false, stream);
            packed = (const uint8_t *)args->scratch;
        }
        g.A = (const uint8_t *)args->src;
        g.lda = 2 * D.src.strides[0];
        g.B = packed;
        g.switches = (plan->b8x_variant == 4 ? GEMM_NOT_PERSISTENT : 0)
                | (plan->b8x_variant == 5 ? GEMM_NO_STAGGER : 0);
        g.wei_zp = wz.set ? args->zps[QMM_WEI] : nullptr;
        g.wei_zp_dt = wz.dt;
        g.wei_zp_sn = wz.set && (wz.mask & 2) ? 1 : 0;
        g.w_off = D.wei.dt == dt_u8 ? 128 : 0;
        g.M = (int32_t)P.M;
        g.N = (int32_t)P.N;
        g.K = (int32_t)P.K;
        g.batch = 1;
        g.kb32 = (int32_t)geom.kb32;
        g.nb32 = (int32_t)geom.nb32;
        // gemm_variant 1: never cut K into slices
        const int splits
                = gemm_variant == 1 ? 1 : gemm_f16w8_splits(P.M, P.N, P.K);
        float *part = (float *)((uint8_t *)args->scratch
                + (D.wei_layout == QMM_LAYOUT_PLAIN
                                ? round256(geom.total_bytes)
                                : 0));
        launch_gemm_f16w8(g, splits, part, stream);
    } else if (impl == impl_gemv_w4) {
        gemv_params_t g;
        std::memset(&g, 0, sizeof(g));
        if (!build_epilogue(g.ep, P, args))
            return fail(QMM_RUNTIME_ERROR, "epilogue does not fold");
        const w4_geom_t geom = w4_geom(1, P.K, P.N);
        const uint8_t *packed = (const uint8_t *)args->wei;
        g.w8 = is_int8(D.wei.dt);
        if (D.wei_layout == QMM_LAYOUT_PLAIN) {
            if (g.w8)
                launch_pack_w8(args->wei, args->scratch, D.wei.dt, 1, P.K, P.N,
                        0, D.wei.strides[0], D.wei.strides[1], stream);
            else
                launch_pack_w4(args->wei, args->scratch, D.wei.dt, 1, P.K, P.N,
                        0, D.wei.strides[0], D.wei.strides[1], stream);
            packed = (const uint8_t *)args->scratch;
        }
        g.A = (const uint16_t *)args->src;
        g.lda = D.src.strides[0];
        g.B = packed;
        const qmm_quant_t &ws = D.scales[QMM_WEI], &wz = D.zps[QMM_WEI];
        const int Kpad = (int)geom.Kpad;
        g.scales = ws.set ? args->scales[QMM_WEI] : nullptr;
        g.scale_dt = ws.dt;
        g.gs = (ws.set && (ws.mask & 1)) ? (int)P.q_wei_scale.g0 : Kpad;
        g.scale_per_n = ws.set && (ws.mask & 2);
        g.zps = wz.set ? args->zps[QMM_WEI] : nullptr;
        g.zp_dt = wz.dt;
        g.gz = (wz.set && (wz.mask & 1)) ? (int)P.q_wei_zp.g0 : 0;
        g.zp_per_n = wz.set && (wz.mask & 2);
        g.M = (int32_t)P.M;
        g.N = (int32_t)P.N;
        g.K = (int32_t)P.K;
        g.kg128 = (int32_t)geom.kg128;
        g.nb16 = (int32_t)geom.nb16;
        g.wei_signed = D.wei.dt == dt_s4 || D.wei.dt == dt_s8;
        g.act_f16 = D.src.dt == dt_f16;
        g.m0 = 0;
        if (!launch_gemv_w4(g, stream))
            return fail(QMM_RUNTIME_ERROR,
                    "decode_w4: no kernel takes this problem (8-bit weights "
                    "outside the forms the implementation admits)");
    } else {
        return fail(QMM_INVALID_ARGUMENTS, "unknown implementation");
    }
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return hip_fail(e, "kernel launch");
    return QMM_OK;
}

// ---------------------------------------------------------------------------
static bool is_plain_copy_dt(int a, int b) {
    return a == b;
}

int qmm_reorder_supports(const qmm_reorder_desc_t *d) {
    if (!d) return QMM_INVALID_ARGUMENTS;
    const int nd = d->src.ndims;
    if (nd != d->dst.ndims || nd < 1 || nd > QMM_MAX_NDIMS)
        return QMM_INVALID_ARGUMENTS;
    const bool quant = d->src_scale.set || d->dst_scale.set || d->src_zp.set
            || d->dst_zp.set;
    if (d->src_layout == QMM_LAYOUT_PLAIN && d->dst_layout == QMM_LAYOUT_PLAIN) {
        const int s = d->src.dt, t = d->dst.dt;
        if (!one_of(s, {dt_f32, dt_bf16, dt_f16, dt_f8_e4m3, dt_f8_e5m2, dt_s32,
                    dt_s8, dt_u8, dt_s4, dt_u4}))
            return QMM_UNIMPLEMENTED;
        if (!one_of(t, {dt_f32, dt_bf16, dt_f16, dt_f8_e4m3, dt_f8_e5m2, dt_s32,
                    dt_s8, dt_u8, dt_s4, dt_u4}))
            return QMM_UNIMPLEMENTED;
        if (is_int4(t)) {
            // the pair owner scheme needs a stride-1 dim of even extent
            bool ok = false;
            for (int i = 0; i < nd; i++)
                if (d->dst.strides[i] == 1 && d->dst.dims[i] % 2 == 0) ok = true;
            if (!ok) return QMM_UNIMPLEMENTED;
        }
        if (d->dst_zp.set && d->dst_zp.mask != 0) return QMM_UNIMPLEMENTED;
        return QMM_OK;
    }
    // packing / unpacking: same data type, no quantization, >= 2 dims
    if (quant || nd < 2 || !is_plain_copy_dt(d->src.dt, d->dst.dt))
        return QMM_UNIMPLEMENTED;
    const int packed
            = d->src_layout == QMM_LAYOUT_PLAIN ? d->dst_layout : d->src_layout;
    if (d->src_layout != QMM_LAYOUT_PLAIN && d->dst_layout != QMM_LAYOUT_PLAIN)
        return QMM_UNIMPLEMENTED;
    const qmm_tensor_t &pl
            = d->src_layout == QMM_LAYOUT_PLAIN ? d->src : d->dst;
    // batch dims of the plain side must nest densely
    qmm_tensor_t shape = pl;
    int64_t sb;
    if (!fold_batch(pl, shape, sb)) return QMM_UNIMPLEMENTED;
    if (packed == QMM_LAYOUT_MFMA_B8) {
        if (!one_of(pl.dt, {dt_s8, dt_u8, dt_f8_e4m3, dt_f8_e5m2}))
            return QMM_UNIMPLEMENTED;
        return QMM_OK;
    }
    if (packed == QMM_LAYOUT_MFMA_W8)
        return is_int8(pl.dt) ? QMM_OK : QMM_UNIMPLEMENTED;
    if (packed == QMM_LAYOUT_MFMA_W4 || packed == QMM_LAYOUT_MFMA_W4K64) {
        if (!is_int4(pl.dt)) return QMM_UNIMPLEMENTED;
        if (d->dst_layout == QMM_LAYOUT_PLAIN) {
            // unpack writes byte pairs along the stride-1 dim
            const bool n_inner = pl.strides[nd - 1] == 1
                    && pl.dims[nd - 1] % 2 == 0;
            const bool k_inner = pl.strides[nd - 2] == 1
                    && pl.dims[nd - 2] % 2 == 0;
            if (!n_inner && !k_inner) return QMM_UNIMPLEMENTED;
        }
        return QMM_OK;
    }
    return QMM_UNIMPLEMENTED;
}

// Row-wise quantizing pass (qmm_quantize.hip): both tensors plain, row-major
// in the same dim order with stride 1 along the last dim, rows of a multiple
// of 8 elements that start on the vector boundaries the kernel uses, a
// floating-point source; scales / zero points over rows and columns of a 2-D
// tensor (with or without groups), over the last dim only otherwise.
static int elem_bits(int dt) {
    switch (dt) {
        case dt_f32:
        case dt_s32: return 32;
        case dt_bf16:
        case dt_f16: return 16;
        case dt_s4:
        case dt_u4: return 4;
        default: return 8;
    }
}
static bool rows_quant(quant_rows_q_t &q, const qmm_quant_t &a, int nd,
        const int64_t *dims) {
    std::memset(&q, 0, sizeof(q));
    q.gr = q.gc = 1;
    q.dt = a.dt;
    if (!a.set) return true;
    const int last = 1 << (nd - 1), prev = nd >= 2 ? 1 << (nd - 2) : 0;
    if (a.mask & ~(last | (nd == 2 ? prev : 0))) return false;
    const int64_t g0 = a.has_groups && a.g0 > 0 ? a.g0 : 1;
    const int64_t g1 = a.has_groups && a.g1 > 0 ? a.g1 : 1;
    const int64_t C = dims[nd - 1];
    if (nd >= 2 && (dims[nd - 2] % g0 || C % g1)) return false;
    if (nd == 1 && a.has_groups) return false;
    q.gr = g0;
    q.gc = g1;
    q.sc = (a.mask & last) ? 1 : 0;
    q.sr = (a.mask & prev) && nd == 2 ? ((a.mask & last) ? C / g1 : 1) : 0;
    q.ptr = (const void *)1; // set at launch
    return true;
}
static bool reorder_rows_plan(const qmm_reorder_desc_t *d,
        quant_rows_params_t &p) {
    std::memset(&p, 0, sizeof(p));
    const int nd = d->src.ndims;
    if (d->src_layout != QMM_LAYOUT_PLAIN || d->dst_layout != QMM_LAYOUT_PLAIN)
        return false;
    if (!one_of(d->src.dt, {dt_f32, dt_bf16, dt_f16})) return false;
    if (!one_of(d->dst.dt, {dt_f32, dt_bf16, dt_f16, dt_s8, dt_u8, dt_s4,
                dt_u4, dt_f8_e4m3, dt_f8_e5m2}))
        return false;
    const int64_t C = d->src.dims[nd - 1];
    if (C % 8 != 0 || d->src.strides[nd - 1] != 1 || d->dst.strides[nd - 1] != 1)
        return false;
    int64_t rows = 1;
    for (int i = 0; i < nd - 1; i++)
        rows *= d->src.dims[i];
    // leading dims nest densely over the row pitch, identically on both sides
    const int64_t sp = nd >= 2 ? d->src.strides[nd - 2] : C;
    const int64_t dp = nd >= 2 ? d->dst.strides[nd - 2] : C;
    if (sp < C || dp < C) return false;
    // 32-bit index arithmetic, and a grid of at most 2^31 workgroups of 128
    // or more 8-column chunks
    if (rows >= (int64_t(1) << 31) || C >= (int64_t(1) << 31)
            || rows * C >= (int64_t(1) << 40))
        return false;
    for (int i = nd - 3; i >= 0; i--) {
        if (d->src.strides[i] != d->src.strides[i + 1] * d->src.dims[i + 1]
                || d->dst.strides[i]
                        != d->dst.strides[i + 1] * d->dst.dims[i + 1])
            return false;
    }
    // 8 elements are one or two 16-byte loads and one 4..32-byte store
    if ((sp * elem_bits(d->src.dt)) % 128 != 0) return false;
    const int out_bits = 8 * elem_bits(d->dst.dt);
    if ((dp * elem_bits(d->dst.dt)) % (out_bits > 128 ? 128 : out_bits) != 0)
        return false;
    if (!rows_quant(p.src_scale, d->src_scale, nd, d->src.dims)
            || !rows_quant(p.dst_scale, d->dst_scale, nd, d->src.dims)
            || !rows_quant(p.src_zp, d->src_zp, nd, d->src.dims))
        return false;
    if (d->dst_zp.set && d->dst_zp.mask != 0) return false;
    p.rows = rows;
    p.cols = C;
    p.src_pitch = sp;
    p.dst_pitch = dp;
    p.src_dt = d->src.dt;
    p.dst_dt = d->dst.dt;
    return true;
}

// The transposing quantizer (quantize_transpose_kernel): 2-D, a floating-point
// source, one side with stride 1 over rows and the other over columns, the
// quantization attributes of the row-wise pass; a 4-bit destination only where
// its pairs along the stride-1 dim are whole and start on a byte.
static bool reorder_transpose_plan(const qmm_reorder_desc_t *d,
        quant_tr_params_t &p) {
    std::memset(&p, 0, sizeof(p));
    if (d->src_layout != QMM_LAYOUT_PLAIN || d->dst_layout != QMM_LAYOUT_PLAIN
            || d->src.ndims != 2)
        return false;
    if (!one_of(d->src.dt, {dt_f32, dt_bf16, dt_f16})) return false;
    if (!one_of(d->dst.dt, {dt_f32, dt_bf16, dt_f16, dt_s8, dt_u8, dt_s4,
                dt_u4, dt_f8_e4m3, dt_f8_e5m2}))
        return false;
    const int64_t R = d->src.dims[0], C = d->src.dims[1];
    if (R < 2 || C < 2 || R >= (int64_t(1) << 31) || C >= (int64_t(1) << 31))
        return false;
    const int64_t *ss = d->src.strides, *ds = d->dst.strides;
    const bool src_cm = ss[0] == 1 && ss[1] >= R, src_rm = ss[1] == 1 && ss[0] >= C;
    const bool dst_cm = ds[0] == 1 && ds[1] >= R, dst_rm = ds[1] == 1 && ds[0] >= C;
    if (!((src_cm && !src_rm && dst_rm && !dst_cm)
                || (src_rm && !src_cm && dst_cm && !dst_rm)))
        return false;
    if (d->dst.dt == dt_s4 || d->dst.dt == dt_u4) {
        const int64_t pitch = dst_cm ? ds[1] : ds[0], run = dst_cm ? R : C;
        if (pitch % 2 || run % 2) return false;
    }
    // tiles along the destination's stride-1 dim are the grid's y
    if ((dst_cm ? R : C) > (int64_t)65535 * 128) return false;
    if (!rows_quant(p.src_scale, d->src_scale, 2, d->src.dims)
            || !rows_quant(p.dst_scale, d->dst_scale, 2, d->src.dims)
            || !rows_quant(p.src_zp, d->src_zp, 2, d->src.dims))
        return false;
    if (d->dst_zp.set && d->dst_zp.mask != 0) return false;
    p.rows = R;
    p.cols = C;
    p.src_sr = ss[0], p.src_sc = ss[1];
    p.dst_sr = ds[0], p.dst_sc = ds[1];
    p.src_dt = d->src.dt;
    p.dst_dt = d->dst.dt;
    return true;
}

const char *qmm_reorder_impl_name(const qmm_reorder_desc_t *d) {
    if (!d) return "";
    if (d->src_layout != QMM_LAYOUT_PLAIN || d->dst_layout != QMM_LAYOUT_PLAIN)
        return "hip:gfx950:prepack";
    quant_rows_params_t p;
    quant_tr_params_t t;
    return reorder_rows_plan(d, p)       ? "hip:gfx950:quantize"
            : reorder_transpose_plan(d, t) ? "hip:gfx950:quantize_transpose"
                                           : "hip:gfx950:reorder";
}

int qmm_reorder_launch(const qmm_reorder_desc_t *d,
        const qmm_reorder_args_t *args, void *hip_stream) {
    const int st = qmm_reorder_supports(d);
    if (st != QMM_OK) return st;
    if (!args || !args->src || !args->dst)
        return fail(QMM_INVALID_ARGUMENTS, "null reorder pointer");
    hipStream_t stream = (hipStream_t)hip_stream;
    const int nd = d->src.ndims;
    int64_t nelems = 1;
    for (int i = 0; i < nd; i++)
        nelems *= d->src.dims[i];
    if (nelems == 0) return QMM_OK;

    quant_rows_params_t qr;
    // tensors and scale buffers on the vector boundaries the kernel assumes
    const bool vec_ok = (((uintptr_t)args->src | (uintptr_t)args->dst
                                 | (uintptr_t)args->src_scale
                                 | (uintptr_t)args->dst_scale)
                                & 15)
            == 0;
    if (vec_ok && reorder_rows_plan(d, qr)) {
        if ((d->src_scale.set && !args->src_scale)
                || (d->dst_scale.set && !args->dst_scale)
                || (d->src_zp.set && !args->src_zp)
                || (d->dst_zp.set && !args->dst_zp))
            return fail(QMM_INVALID_ARGUMENTS, "reorder attribute buffer missing");
        qr.src = args->src;
        qr.dst = args->dst;
        qr.src_scale.ptr = d->src_scale.set ? args->src_scale : nullptr;
        qr.dst_scale.ptr = d->dst_scale.set ? args->dst_scale : nullptr;
        qr.src_zp.ptr = d->src_zp.set ? args->src_zp : nullptr;
        qr.dst_zp = d->dst_zp.set ? (const int32_t *)args->dst_zp : nullptr;
        launch_quantize_rows(qr, stream);
    } else if (quant_tr_params_t qt; reorder_transpose_plan(d, qt)) {
        if ((d->src_scale.set && !args->src_scale)
                || (d->dst_scale.set && !args->dst_scale)
                || (d->src_zp.set && !args->src_zp)
                || (d->dst_zp.set && !args->dst_zp))
            return fail(QMM_INVALID_ARGUMENTS, "reorder attribute buffer missing");
        qt.src = args->src;
        qt.dst = args->dst;
        qt.src_scale.ptr = d->src_scale.set ? args->src_scale : nullptr;
        qt.dst_scale.ptr = d->dst_scale.set ? args->dst_scale : nullptr;
        qt.src_zp.ptr = d->src_zp.set ? args->src_zp : nullptr;
        qt.dst_zp = d->dst_zp.set ? (const int32_t *)args->dst_zp : nullptr;
        launch_quantize_transpose(qt, stream);
    } else if (d->src_layout == QMM_LAYOUT_PLAIN
            && d->dst_layout == QMM_LAYOUT_PLAIN) {
        generic_reorder_params_t P;
        std::memset(&P, 0, sizeof(P));
        P.desc = *d;
        P.nelems = nelems;
        for (int i = 0; i < nd; i++)
            if (d->dst.strides[i] == 1 && d->dst.dims[i] % 2 == 0) P.pair_dim = i;
        quant_geom(P.q_src_scale, d->src_scale, nd, d->src.dims,
                group_or(d->src_scale, 0, 1), group_or(d->src_scale, 1, 1));
        quant_geom(P.q_dst_scale, d->dst_scale, nd, d->src.dims, 1, 1);
        quant_geom(P.q_src_zp, d->src_zp, nd, d->src.dims,
                group_or(d->src_zp, 0, 1), group_or(d->src_zp, 1, 1));
        if ((d->src_scale.set && !args->src_scale)
                || (d->dst_scale.set && !args->dst_scale)
                || (d->src_zp.set && !args->src_zp)
                || (d->dst_zp.set && !args->dst_zp))
            return fail(QMM_INVALID_ARGUMENTS, "reorder attribute buffer missing");
        launch_reorder_generic(P, *args, stream);
    } else {
        const bool packing = d->src_layout == QMM_LAYOUT_PLAIN;
        const qmm_tensor_t &pl = packing ? d->src : d->dst;
        const int packed = packing ? d->dst_layout : d->src_layout;
        const int64_t K = pl.dims[nd - 2], N = pl.dims[nd - 1];
        int64_t batch = 1;
        for (int i = 0; i < nd - 2; i++)
            batch *= pl.dims[i];
        int64_t sb = 0;
        qmm_tensor_t shape = pl;
        fold_batch(pl, shape, sb);
        const int64_t sk = pl.strides[nd - 2], sn = pl.strides[nd - 1];
        if (packed == QMM_LAYOUT_MFMA_B8) {
            if (packing)
                launch_pack_b8(args->src, args->dst, pl.dt, batch, K, N, sb, sk,
                        sn, pl.dt == dt_s8 || pl.dt == dt_u8, stream);
            else
                launch_unpack_b8(args->src, args->dst, pl.dt, batch, K, N, sb,
                        sk, sn, stream);
        } else if (packed == QMM_LAYOUT_MFMA_W8) {
            if (packing)
                launch_pack_w8(args->src, args->dst, pl.dt, batch, K, N, sb, sk,
                        sn, stream);
            else
                launch_unpack_w8(args->src, args->dst, pl.dt, batch, K, N, sb,
                        sk, sn, stream);
        } else if (packed == QMM_LAYOUT_MFMA_W4K64) {
            if (packing)
                launch_pack_w4k(args->src, args->dst, pl.dt, batch, K, N, sb, sk,
                        sn, stream);
            else
                launch_unpack_w4k(args->src, args->dst, pl.dt, batch, K, N, sb,
                        sk, sn, stream);
        } else {
            if (packing)
                launch_pack_w4(args->src, args->dst, pl.dt, batch, K, N, sb, sk,
                        sn, stream);
            else
                launch_unpack_w4(args->src, args->dst, pl.dt, batch, K, N, sb,
                        sk, sn, stream);
        }
    }
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return hip_fail(e, "reorder launch");
    return QMM_OK;
}

} // extern "C"
