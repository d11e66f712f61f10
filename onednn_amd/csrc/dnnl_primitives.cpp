// matmul and reorder primitive descriptors, the implementation-list walk,
// primitive creation and execution of the dnnl C API subset. Host-only: it
// validates exactly what the reference validates before dispatch, translates
// the descriptors into the POD form of include/qmm_hip.h and enqueues one
// launch on the stream.
//
// Rule sources in the reference:
//   shapes / broadcast      src/common/matmul.cpp:284-409  (invalid_arguments)
//   attribute legality      src/common/matmul.cpp:40-278   (unimplemented)
//   scales per impl         src/common/matmul_pd.hpp:186-244
//   zero points per impl    src/cpu/matmul/ref_matmul_int8.hpp:86-128,
//                           src/cpu/matmul/ref_matmul.hpp:131-152
//   sum consistency         src/common/primitive_attr.cpp:289-329
//   execute arguments       src/common/primitive_exec_types.cpp:27-92
//   reorder checks          src/common/reorder.cpp:66-160
#include <hip/hip_runtime_api.h>

#include <chrono>
#include <cstdio>
#include <new>

#include "dnnl_objects.hpp"
#include "sdpa_internal.h"

using namespace host;

int dnnl_amd_verbose_level();

namespace {

const dnnl_memory_desc g_zero_md;

bool is_int8(dnnl_data_type_t dt) { return dt == dnnl_s8 || dt == dnnl_u8; }
bool is_int4(dnnl_data_type_t dt) { return dt == dnnl_s4 || dt == dnnl_u4; }
bool is_f8(dnnl_data_type_t dt) {
    return dt == dnnl_f8_e5m2 || dt == dnnl_f8_e4m3;
}
bool is_f4(dnnl_data_type_t dt) {
    return dt == dnnl_f4_e2m1 || dt == dnnl_f4_e3m0;
}
bool is_integral(dnnl_data_type_t dt) {
    return dt == dnnl_s32 || is_int8(dt) || is_int4(dt);
}
bool implies(bool a, bool b) { return !a || b; }

// ---- shape checks: src/common/matmul.cpp:284-409 ----------------------------
dnnl_status_t matmul_shape_check(const dnnl_memory_desc *src,
        const dnnl_memory_desc *wei, const dnnl_memory_desc *bias,
        const dnnl_memory_desc *dst) {
    if (!src || !wei || !dst) return dnnl_invalid_arguments;
    const bool with_bias = bias && bias->ndims != 0;
    const int nd = dst->ndims;
    if (nd < 2 || nd > DNNL_MAX_NDIMS) return dnnl_invalid_arguments;
    if (src->ndims != nd || wei->ndims != nd) return dnnl_invalid_arguments;
    if (with_bias && bias->ndims != nd) return dnnl_invalid_arguments;
    const int m = nd - 2, n = nd - 1;
    if (dst->dims[m] != src->dims[m]) return dnnl_invalid_arguments;
    if (dst->dims[n] != wei->dims[n]) return dnnl_invalid_arguments;
    if (src->dims[n] != wei->dims[m]) return dnnl_invalid_arguments;
    if (with_bias) {
        if (bias->dims[n] != 1 && bias->dims[n] != dst->dims[n])
            return dnnl_invalid_arguments;
        if (bias->dims[m] != 1 && bias->dims[m] != dst->dims[m])
            return dnnl_invalid_arguments;
    }
    if ((is_int4(wei->data_type) || is_f4(wei->data_type))
            && wei->dims[n] % 2 != 0)
        return dnnl_invalid_arguments;
    if ((is_int4(src->data_type) || is_f4(src->data_type))
            && src->dims[n] % 2 != 0)
        return dnnl_invalid_arguments;
    for (int d = 0; d < nd - 2; d++) {
        const int64_t s = src->dims[d], w = wei->dims[d], o = dst->dims[d];
        const int64_t b = with_bias ? bias->dims[d] : 0;
        const int64_t R = DNNL_RUNTIME_DIM_VAL;
        if (s == R || w == R || o == R || b == R) {
            if (!(s == R && w == R && o == R)) return dnnl_invalid_arguments;
        } else {
            if (!(s == w && w == o) && !(s == 1 || w == 1))
                return dnnl_invalid_arguments;
            if (s == 1 && o != w) return dnnl_invalid_arguments;
            if (w == 1 && o != s) return dnnl_invalid_arguments;
            if (with_bias && b != 1 && b != o) return dnnl_invalid_arguments;
        }
    }
    // default accumulation type must exist
    // (src/common/type_helpers.hpp:444-478)
    const dnnl_data_type_t sd = src->data_type, wd = wei->data_type,
                           dd = dst->data_type;
    bool acc_ok = false;
    if (sd == dnnl_f32 && wd == dnnl_f32) acc_ok = true;
    if (sd == dnnl_f64 && wd == dnnl_f64) acc_ok = true;
    if (is_int8(sd) && (is_int8(wd) || is_int4(wd))) acc_ok = true;
    if ((sd == dnnl_bf16 || sd == dnnl_f32) && (is_int8(wd) || is_int4(wd)))
        acc_ok = true;
    for (dnnl_data_type_t t : {sd, wd, dd})
        if (t == dnnl_f16 || t == dnnl_bf16 || is_f8(t) || is_f4(t))
            acc_ok = true;
    return acc_ok ? dnnl_success : dnnl_invalid_arguments;
}

// ---- attribute legality: src/common/matmul.cpp:40-278 -----------------------
dnnl_status_t matmul_attr_check(const dnnl_memory_desc &src,
        const dnnl_memory_desc &wei, const dnnl_memory_desc &dst,
        const dnnl_engine *engine, const dnnl_primitive_attr &attr) {
    const dnnl_data_type_t src_dt = src.data_type, wei_dt = wei.data_type,
                           dst_dt = dst.data_type;
    const bool src_is_int8 = is_int8(src_dt), src_is_fp8 = is_f8(src_dt);
    const bool wei_is_int = is_int8(wei_dt) || is_int4(wei_dt);
    const bool wei_is_fp8 = is_f8(wei_dt);
    const dnnl_status_t U = dnnl_unimplemented;

    // Dropout and stochastic rounding pass the reference's common check
    // (src/common/matmul.cpp:52-79) and are computed by its ref_matmul only
    // (src/cpu/matmul/ref_matmul.cpp:186,214-228); no implementation here.
    if (!attr.dropout_desc.is_zero() || !attr.rounding.empty()) return U;

    // Which attribute kinds may be non-default at all (the skip mask of
    // src/common/matmul.cpp:52-79; the "groups" and "data type" mask bits
    // include the plain zero-points / scales bit).
    const bool zp_allowed
            = src_is_int8 || src_is_fp8 || wei_is_int || wei_is_fp8;
    if (!zp_allowed && !attr.has_default_zps()) return U;
    if (!(wei_is_int || wei_is_fp8)) {
        for (auto &kv : attr.zero_points)
            if (!kv.second.is_default()
                    && ((kv.second.dt != dnnl_s32
                                && kv.second.dt != dnnl_data_type_undef)
                            || kv.second.has_groups()))
                return U;
        for (auto &kv : attr.scales)
            if (kv.second.has_groups()) return U;
    }

    const int nds = src.ndims, ndw = wei.ndims;
    const int src_qmask_M = 1 << (nds - 2), src_qmask_K = 1 << (nds - 1);
    const int wei_qmask_K = 1 << (ndw - 2), wei_qmask_N = 1 << (ndw - 1);
    const int dst_qmask_M = src_qmask_K, dst_qmask_N = wei_qmask_N;

    if (!attr.has_default_scales()) {
        int64_t src_gk = 1;
        const quant_entry_t &ss = attr.scale(DNNL_ARG_SRC);
        if (!ss.is_default()) {
            const int mask = ss.mask;
            if (mask != 0 && mask != src_qmask_K
                    && mask != src_qmask_M + src_qmask_K)
                return U;
            if (ss.has_groups() && (mask & src_qmask_K)) src_gk = ss.group(1);
            if (src_gk > 1 && src_gk % 32 != 0) return U;
        }
        int64_t wei_gk = 1, wei_gn = 1;
        const quant_entry_t &ws = attr.scale(DNNL_ARG_WEIGHTS);
        if (!ws.is_default()) {
            if (ws.has_groups()) {
                if (ws.mask & wei_qmask_K) wei_gk = ws.group(0);
                if (ws.mask & wei_qmask_N) wei_gn = ws.group(1);
            }
            if (wei_gn > 1 && !attr.fpmath_apply_to_int) return U;
            if (wei_gk > 1 && wei_gk % 32 != 0) return U;
            if (wei_gn > 1 && wei_gn % 32 != 0) return U;
        }
        const quant_entry_t &ds = attr.scale(DNNL_ARG_DST);
        if (!ds.is_default()) {
            const int mask = ds.mask;
            if (engine->kind == dnnl_gpu) {
                if (mask != 0 && mask != dst_qmask_N && mask != dst_qmask_M
                        && mask != dst_qmask_N + dst_qmask_M)
                    return U;
            } else if (mask != 0)
                return U;
        }
        const bool divisible = implies(src_gk > 1 && wei_gk > 1,
                src_gk % wei_gk == 0 || wei_gk % src_gk == 0);
        if (!implies(src_gk > 1, (src_is_int8 || src_is_fp8) && divisible))
            return U;
    }

    if (!attr.has_default_zps()) {
        int64_t src_gk = 1;
        const quant_entry_t &sz = attr.zp(DNNL_ARG_SRC);
        if (!sz.is_default()) {
            const int mask = sz.mask;
            if (mask != 0 && mask != src_qmask_K
                    && mask != src_qmask_M + src_qmask_K)
                return U;
            if (sz.has_groups() && (mask & src_qmask_K)) src_gk = sz.group(1);
            if (src_gk > 1 && src_gk % 32 != 0) return U;
        }
        int64_t wei_gk = 1, wei_gn = 1;
        const quant_entry_t &wz = attr.zp(DNNL_ARG_WEIGHTS);
        if (!wz.is_default()) {
            if (wz.has_groups()) {
                if (wz.mask & wei_qmask_K) wei_gk = wz.group(0);
                if (wz.mask & wei_qmask_N) wei_gn = wz.group(1);
            }
            if (wei_gn > 1 && !attr.fpmath_apply_to_int) return U;
            if (wei_gk > 1 && wei_gk % 32 != 0) return U;
            if (wei_gn > 1 && wei_gn % 32 != 0) return U;
            if (is_int4(wz.dt)) {
                if ((wz.mask & wei_qmask_K) && wei.dims[ndw - 2] % 2 != 0)
                    return U;
                if ((wz.mask & wei_qmask_N) && wei.dims[ndw - 1] % 2 != 0)
                    return U;
            }
        }
        const quant_entry_t &dz = attr.zp(DNNL_ARG_DST);
        if (!dz.is_default()) {
            if (!(dz.mask == 0 || (dst.ndims == 2 && dz.mask == 2))) return U;
        }
        const bool divisible = implies(src_gk > 1 && wei_gk > 1,
                src_gk % wei_gk == 0 || wei_gk % src_gk == 0);
        if (!implies(src_gk > 1, src_is_int8 && divisible)) return U;
    }

    const dnnl_post_ops &po = attr.post_ops;
    if (!po.entries.empty()) {
        for (auto &e : po.entries)
            if (e.kind != dnnl_binary && e.kind != dnnl_eltwise
                    && e.kind != dnnl_prelu && e.kind != dnnl_sum)
                return U;
        // check_sum_consistency(dst_dt, src_is_int8, diverse sum dt allowed)
        const int si = po.find(dnnl_sum);
        if (si >= 0) {
            const dnnl_data_type_t sum_dt = po.entries[si].sum_dt;
            if (sum_dt != dnnl_data_type_undef && dst_dt != dnnl_data_type_undef
                    && dnnl_data_type_size(dst_dt) != dnnl_data_type_size(sum_dt))
                return U;
        }
        for (auto &e : po.entries) {
            if (e.kind != dnnl_sum) continue;
            const dnnl_data_type_t sdt
                    = e.sum_dt != dnnl_data_type_undef ? e.sum_dt : dst_dt;
            if (!src_is_int8 && e.sum_zero_point != 0) return U;
            if (e.sum_zero_point != 0 && sdt != dnnl_s8 && sdt != dnnl_u8
                    && sdt != dnnl_s32)
                return U;
        }
        for (auto &e : po.entries)
            if (e.kind == dnnl_binary && e.user_src1_desc.ndims != dst.ndims)
                return dnnl_invalid_arguments;
    }
    return dnnl_success;
}

// ---- per-implementation attribute rules -------------------------------------
// matmul_pd_t::attr_scales_ok (src/common/matmul_pd.hpp:186-244) plus the zero
// point rules of the two reference implementations.
bool impl_attr_ok(const pd_impl_t &pd) {
    const dnnl_primitive_attr &attr = pd.attr;
    const int nd = pd.dst.ndims;
    const int64_t M = pd.dst.dims[nd - 2], N = pd.dst.dims[nd - 1],
                  K = pd.src.dims[nd - 1];
    const int qM = 1 << (nd - 2), qK_src = 1 << (nd - 1);
    const int qK_wei = 1 << (nd - 2), qN = 1 << (nd - 1);
    for (auto &kv : attr.scales) {
        if (kv.second.is_default()) continue;
        const quant_entry_t &s = kv.second;
        if (kv.first == DNNL_ARG_WEIGHTS) {
            const int64_t g0 = s.group(0), g1 = s.group(1);
            if (s.has_groups()) {
                if (!(g0 == 1 || g1 == 1)) return false;
                // as written in the reference: the K check uses the second
                // group and the N check the first
                if (g0 > 1 && g1 > 0 && K % g1 != 0) return false;
                if (g1 > 1 && g0 > 0 && N % g0 != 0) return false;
                if (g0 <= 0 || g1 <= 0) return false;
                if (g0 > 1 && K % g0 != 0) return false;
                if (g1 > 1 && N % g1 != 0) return false;
            }
            const bool wei_int = is_int8(pd.wei.data_type)
                    || is_int4(pd.wei.data_type);
            const bool decomp_or_dynquant = wei_int
                    && implies(!is_integral(pd.src.data_type),
                            attr.fpmath_apply_to_int);
            if ((s.mask & qK_wei) && !decomp_or_dynquant) return false;
        } else if (kv.first == DNNL_ARG_SRC) {
            if (s.mask != 0 && s.mask != qK_src && s.mask != qM + qK_src)
                return false;
            if ((s.mask & qK_src) && !s.has_groups()) return false;
            if (s.has_groups()) {
                if (s.group(0) == 0 || s.group(1) <= 0) return false;
                if (K % s.group(1) != 0) return false;
                if (s.group(0) != 1) return false;
            }
        } else if (kv.first == DNNL_ARG_DST) {
            if (s.mask != 0 && s.mask != qN && s.mask != qM + qN) return false;
            if (s.has_groups()) {
                if (s.group(1) != 1 || s.group(0) <= 0 || M % s.group(0) != 0)
                    return false;
            }
        } else
            return false;
    }
    const bool int_src = is_int8(pd.src.data_type);
    const quant_entry_t &sz = attr.zp(DNNL_ARG_SRC), &wz = attr.zp(DNNL_ARG_WEIGHTS),
                        &dz = attr.zp(DNNL_ARG_DST);
    if (!sz.is_default()) {
        if (!int_src) return false;
        if (sz.mask != 0 && sz.mask != qK_src && sz.mask != qM + qK_src)
            return false;
        if (sz.has_groups()) {
            if (sz.group(0) != 1) return false;
            const int64_t gK = sz.group(1);
            if (gK <= 0 || (gK > 1 && K % gK != 0)) return false;
        }
    }
    if (!wz.is_default() && wz.has_groups()) {
        const int64_t gK = wz.group(0), gN = wz.group(1);
        if (gK <= 0 || gN <= 0) return false;
        if (gK > 1 && K % gK != 0) return false;
        if (gN > 1 && N % gN != 0) return false;
        if (!(gK == 1 || gN == 1)) return false;
    }
    if (!dz.is_default()) {
        if (!int_src) return false;
        if (dz.mask != 0 && dz.mask != qN) return false;
    }
    // sum consistency at implementation level
    // (check_sum_consistency(dst_dt, is_int8), diverse dts not allowed)
    const dnnl_post_ops &po = attr.post_ops;
    int si = po.find(dnnl_sum);
    if (si >= 0) {
        const dnnl_data_type_t first = po.entries[si].sum_dt;
        while ((si = po.find(dnnl_sum, si + 1)) >= 0)
            if (po.entries[si].sum_dt != first) return false;
    }
    return true;
}

void fill_quant(qmm_quant_t &q, const quant_entry_t &e, dnnl_data_type_t dflt) {
    std::memset(&q, 0, sizeof(q));
    q.g0 = q.g1 = 1;
    if (e.is_default()) return;
    q.set = 1;
    q.mask = e.mask;
    q.dt = e.dt != dnnl_data_type_undef ? e.dt : dflt;
    q.has_groups = e.has_groups();
    if (e.has_groups()) {
        q.g0 = e.group(0) > 0 ? e.group(0) : 1;
        q.g1 = e.group(1) > 0 ? e.group(1) : 1;
    }
}

bool collapse_broadcast_batch(qmm_matmul_desc_t &D);

// Build the kernel-level description from resolved descriptors.
void fill_mm_desc(pd_impl_t &pd) {
    qmm_matmul_desc_t &D = pd.mm;
    std::memset(&D, 0, sizeof(D));
    md_to_tensor(D.src, pd.src);
    md_to_tensor(D.wei, pd.wei);
    md_to_tensor(D.dst, pd.dst);
    if (pd.bias.ndims) md_to_tensor(D.bias, pd.bias);
    D.wei_layout = pd.wei.is_packed() ? pd.wei.packed_layout : QMM_LAYOUT_PLAIN;
    D.apply_to_int = pd.attr.fpmath_apply_to_int;
    const int args[3] = {DNNL_ARG_SRC, DNNL_ARG_WEIGHTS, DNNL_ARG_DST};
    for (int i = 0; i < 3; i++) {
        fill_quant(D.scales[i], pd.attr.scale(args[i]), dnnl_f32);
        fill_quant(D.zps[i], pd.attr.zp(args[i]), dnnl_s32);
    }
    D.npo = (int)pd.attr.post_ops.entries.size();
    for (int i = 0; i < D.npo; i++) {
        const post_op_entry_t &e = pd.attr.post_ops.entries[i];
        qmm_postop_t &o = D.po[i];
        o.kind = e.kind;
        switch (e.kind) {
            case dnnl_sum:
                o.scale = e.sum_scale;
                o.zero_point = e.sum_zero_point;
                o.dt = e.sum_dt;
                break;
            case dnnl_eltwise:
                o.alg = e.alg;
                o.alpha = e.alpha;
                o.beta = e.beta;
                o.scale = e.eltwise_scale;
                break;
            case dnnl_binary:
                o.alg = e.alg;
                md_to_tensor(o.src1, e.src1_desc);
                break;
            case dnnl_prelu: o.mask = e.prelu_mask; break;
            default: break;
        }
    }
    collapse_broadcast_batch(D);
}

// Weights that are one matrix for every batch entry ([1, .., 1, K, N]) under a
// source and a destination whose batch dims nest densely over their rows: the
// problem IS the 2-D product [batch x M, K] x [K, N], and as that it reaches the
// kernels that take two dims only (weights decompression, int8 x int4, f16 x
// 8-bit weights). Every tensor and attribute must read the same under the new
// shape: operands of bias / binary post-ops and scales / zero points either do
// not depend on (batch, M) at all or cover all of them densely; a prelu mask
// names the last dim only. Returns false and leaves D alone otherwise.
bool collapse_broadcast_batch(qmm_matmul_desc_t &D) {
    const int nd = D.dst.ndims;
    if (nd < 3) return false;
    const int nb = nd - 2;
    for (int d = 0; d < nb; d++)
        if (D.wei.dims[d] != 1) return false;
    // (batch .., M) as one row index with the M pitch
    auto rows_nest = [&](const qmm_tensor_t &t) {
        for (int d = 0; d < nb; d++)
            if (t.dims[d] != 1
                    && t.strides[d] != t.strides[d + 1] * t.dims[d + 1])
                return false;
        return true;
    };
    // an operand of dst's rank: 0 = no dependence on (batch, M), 1 = all of
    // them as in dst and nesting, -1 = anything else
    auto rows_kind = [&](const qmm_tensor_t &t) {
        if (t.ndims != nd) return -1;
        bool none = true, all = true;
        for (int d = 0; d <= nb; d++) {
            none = none && t.dims[d] == 1;
            all = all && t.dims[d] == D.dst.dims[d];
        }
        if (none) return 0;
        return all && rows_nest(t) ? 1 : -1;
    };
    if (!rows_nest(D.src) || !rows_nest(D.dst)) return false;
    int bias_kind = 0;
    if (D.bias.ndims && (bias_kind = rows_kind(D.bias)) < 0) return false;
    int po_kind[QMM_MAX_POST_OPS] = {};
    for (int i = 0; i < D.npo; i++) {
        if (D.po[i].kind == dnnl_binary
                && (po_kind[i] = rows_kind(D.po[i].src1)) < 0)
            return false;
        if (D.po[i].kind == dnnl_prelu && (D.po[i].mask & ~(1 << (nd - 1))))
            return false;
    }
    const int row_bits = (1 << (nb + 1)) - 1; // batch dims and M
    // scales / zero points: of the source and the destination over (batch, M)
    // all or none, without a group over M; of the weights whatever their batch
    // bits say (those dims are 1)
    int new_mask[2][3];
    for (int z = 0; z < 2; z++)
        for (int a = 0; a < 3; a++) {
            const qmm_quant_t &q = z ? D.zps[a] : D.scales[a];
            new_mask[z][a] = 0;
            if (!q.set) continue;
            if (a == QMM_WEI) {
                new_mask[z][a] = (q.mask >> nb) & 3;
                continue;
            }
            const int rb = q.mask & row_bits;
            if (rb != 0 && rb != row_bits) return false;
            if (rb && q.has_groups && q.g0 != 1) return false;
            new_mask[z][a] = (rb ? 1 : 0) | ((q.mask >> (nd - 1)) & 1 ? 2 : 0);
        }
    int64_t rows = 1;
    for (int d = 0; d <= nb; d++)
        rows *= D.dst.dims[d];
    auto to2d = [&](qmm_tensor_t &t, bool over_rows) {
        const int64_t d0 = over_rows ? rows : t.dims[nd - 2];
        const int64_t s0 = t.strides[nd - 2], d1 = t.dims[nd - 1],
                      s1 = t.strides[nd - 1];
        t.ndims = 2;
        t.dims[0] = d0, t.dims[1] = d1;
        t.strides[0] = s0, t.strides[1] = s1;
        for (int d = 2; d < QMM_MAX_NDIMS; d++)
            t.dims[d] = t.strides[d] = 0;
    };
    to2d(D.src, true);
    to2d(D.dst, true);
    to2d(D.wei, false);
    if (D.bias.ndims) to2d(D.bias, bias_kind == 1);
    for (int i = 0; i < D.npo; i++) {
        if (D.po[i].kind == dnnl_binary) to2d(D.po[i].src1, po_kind[i] == 1);
        if (D.po[i].kind == dnnl_prelu) D.po[i].mask = D.po[i].mask ? 2 : 0;
    }
    for (int z = 0; z < 2; z++)
        for (int a = 0; a < 3; a++) {
            qmm_quant_t &q = z ? D.zps[a] : D.scales[a];
            if (q.set) q.mask = new_mask[z][a];
        }
    return true;
}

int64_t batch_of(const dnnl_memory_desc &md) {
    int64_t b = 1;
    for (int d = 0; d < md.ndims - 2; d++)
        b *= md.dims[d];
    return b;
}

// Try implementation `impl` on the user's descriptors; resolves format any.
dnnl_status_t try_matmul_impl(pd_impl_t &pd, int impl) {
    pd.src = pd.user_src;
    pd.wei = pd.user_wei;
    pd.bias = pd.user_bias;
    pd.dst = pd.user_dst;
    for (dnnl_memory_desc *md : {&pd.src, &pd.bias, &pd.dst}) {
        if (md->is_any()) {
            if (md->has_runtime_dims()) return dnnl_unimplemented;
            dnnl_memory_desc r;
            md_init_plain(r, md->ndims, md->dims, md->data_type, nullptr);
            *md = r;
        }
    }
    if (pd.src.has_runtime_dims() || pd.wei.has_runtime_dims()
            || pd.dst.has_runtime_dims())
        return dnnl_unimplemented;
    for (const dnnl_memory_desc *md : {&pd.src, &pd.bias, &pd.dst})
        if (md->ndims && !md->is_plain()) return dnnl_unimplemented;
    const bool wei_any = pd.wei.is_any();
    if (wei_any) {
        dnnl_memory_desc r;
        md_init_plain(r, pd.wei.ndims, pd.wei.dims, pd.wei.data_type, nullptr);
        pd.wei = r;
    } else if (!pd.wei.is_plain() && !pd.wei.is_packed())
        return dnnl_unimplemented;

    // binary post-op operands given as format any take dst's layout, 1-D ones
    // stay plain (src/common/primitive_attr.cpp:267-287)
    for (auto &e : pd.attr.post_ops.entries) {
        if (e.kind != dnnl_binary) continue;
        e.src1_desc = e.user_src1_desc;
        if (e.src1_desc.is_any()) {
            dnnl_memory_desc r;
            int non_unit = 0;
            for (int d = 0; d < e.src1_desc.ndims; d++)
                non_unit += e.src1_desc.dims[d] != 1;
            bool same = true;
            for (int d = 0; d < pd.dst.ndims; d++)
                same = same && e.src1_desc.dims[d] == pd.dst.dims[d];
            if (non_unit <= 1 || !same)
                md_init_plain(r, e.src1_desc.ndims, e.src1_desc.dims,
                        e.src1_desc.data_type, nullptr);
            else
                md_init_plain(r, e.src1_desc.ndims, e.src1_desc.dims,
                        e.src1_desc.data_type, pd.dst.strides);
            e.src1_desc = r;
        } else if (!e.src1_desc.is_plain())
            return dnnl_unimplemented;
    }
    if (!impl_attr_ok(pd)) return dnnl_unimplemented;

    fill_mm_desc(pd);
    if (wei_any) {
        // the implementation names its preferred weights layout
        qmm_matmul_desc_t probe = pd.mm;
        const int want = qmm_matmul_impl_preferred_wei_layout(impl, &probe);
        probe.wei_layout = want;
        if (want != QMM_LAYOUT_PLAIN
                && qmm_matmul_impl_supports(impl, &probe) == QMM_OK) {
            const int nd = pd.wei.ndims;
            pd.wei.format_kind = dnnl_format_kind_opaque;
            pd.wei.packed_layout = want;
            pd.wei.packed_bytes = qmm_packed_size(want, pd.wei.data_type,
                    batch_of(pd.wei), pd.wei.dims[nd - 2], pd.wei.dims[nd - 1]);
            fill_mm_desc(pd);
        }
    }
    const int st = qmm_matmul_impl_supports(impl, &pd.mm);
    if (st != QMM_OK) return from_qmm(st);
    pd.impl = impl;
    pd.impl_name = qmm_matmul_impl_name(impl);
    pd.scratch_bytes = qmm_matmul_scratch_size(impl, &pd.mm);
    pd.scratchpad = dnnl_memory_desc();
    if (pd.scratch_bytes
            && pd.attr.scratchpad_mode == dnnl_scratchpad_mode_user) {
        dnnl_dims_t dims = {(int64_t)pd.scratch_bytes};
        md_init_plain(pd.scratchpad, 1, dims, dnnl_u8, nullptr);
    }
    return dnnl_success;
}

dnnl_status_t walk_matmul_impls(pd_impl_t &pd, int first) {
    for (int impl = first; impl < qmm_matmul_impl_count(); impl++) {
        const dnnl_status_t st = try_matmul_impl(pd, impl);
        if (st == dnnl_success) return st;
        if (st != dnnl_unimplemented) return st;
    }
    return first == 0 ? dnnl_unimplemented : dnnl_last_impl_reached;
}

const dnnl_primitive_kind_t kind_sdpa = DNNL_PRIMITIVE_KIND_SDPA;

int n_inputs(const pd_impl_t &pd) {
    if (pd.kind == dnnl_reorder || pd.kind == dnnl_softmax) return 1;
    if (pd.kind == kind_sdpa)
        return 3 + (pd.sdpa_mask.ndims != 0) + (pd.sd.scale_dt != 0);
    int n = 2 + (pd.bias.ndims != 0);
    for (auto &e : pd.attr.post_ops.entries)
        n += e.kind == dnnl_binary || e.kind == dnnl_prelu;
    return n;
}

enum class usage_t { unused, input, output };

usage_t arg_usage(const pd_impl_t &pd, int arg) {
    if (pd.kind == dnnl_matmul) {
        if (arg == DNNL_ARG_SRC || arg == DNNL_ARG_WEIGHTS) return usage_t::input;
        if (arg == DNNL_ARG_BIAS)
            return pd.bias.ndims ? usage_t::input : usage_t::unused;
        if (arg == DNNL_ARG_DST) return usage_t::output;
    } else if (pd.kind == dnnl_softmax) {
        if (arg == DNNL_ARG_SRC) return usage_t::input;
        if (arg == DNNL_ARG_DST) return usage_t::output;
    } else if (pd.kind == kind_sdpa) {
        // src/gpu/intel/ocl/micro_sdpa.cpp:674-690
        if (arg == DNNL_ARG_QUERIES || arg == DNNL_ARG_KEYS
                || arg == DNNL_ARG_VALUES)
            return usage_t::input;
        if (arg == DNNL_ARG_DST) return usage_t::output;
        if (arg == DNNL_ARG_SCALE)
            return pd.sd.scale_dt ? usage_t::input : usage_t::unused;
        if (arg == DNNL_ARG_ATTN_MASK)
            return pd.sdpa_mask.ndims ? usage_t::input : usage_t::unused;
        const struct {
            int arg;
            int set;
        } q[4] = {{DNNL_ARG_ATTR_SCALES | DNNL_ARG_KEYS, pd.sd.k_scale.set},
                {DNNL_ARG_ATTR_ZERO_POINTS | DNNL_ARG_KEYS, pd.sd.k_zp.set},
                {DNNL_ARG_ATTR_SCALES | DNNL_ARG_VALUES, pd.sd.v_scale.set},
                {DNNL_ARG_ATTR_ZERO_POINTS | DNNL_ARG_VALUES, pd.sd.v_zp.set}};
        for (auto &e : q)
            if (arg == e.arg) return e.set ? usage_t::input : usage_t::unused;
        if (arg == DNNL_ARG_SCRATCHPAD)
            return pd.scratchpad.ndims ? usage_t::output : usage_t::unused;
        return usage_t::unused;
    } else {
        if (arg == DNNL_ARG_FROM) return usage_t::input;
        if (arg == DNNL_ARG_TO) return usage_t::output;
    }
    if (arg & DNNL_ARG_ATTR_ZERO_POINTS)
        return pd.attr.zp(arg & ~DNNL_ARG_ATTR_ZERO_POINTS).is_default()
                ? usage_t::unused
                : usage_t::input;
    if (arg & DNNL_ARG_ATTR_SCALES)
        return pd.attr.scale(arg & ~DNNL_ARG_ATTR_SCALES).is_default()
                ? usage_t::unused
                : usage_t::input;
    if (arg == DNNL_ARG_SCRATCHPAD)
        return pd.scratchpad.ndims ? usage_t::output : usage_t::unused;
    const auto &po = pd.attr.post_ops.entries;
    for (int i = 0; i < (int)po.size(); i++) {
        if (po[i].kind == dnnl_binary
                && arg == (DNNL_ARG_ATTR_MULTIPLE_POST_OP(i) | DNNL_ARG_SRC_1))
            return usage_t::input;
        if (po[i].kind == dnnl_prelu
                && arg == (DNNL_ARG_ATTR_MULTIPLE_POST_OP(i) | DNNL_ARG_WEIGHTS))
            return usage_t::input;
    }
    return usage_t::unused;
}

const char *dt_name(int dt) {
    switch (dt) {
        case dnnl_f16: return "f16";
        case dnnl_bf16: return "bf16";
        case dnnl_f32: return "f32";
        case dnnl_s32: return "s32";
        case dnnl_s8: return "s8";
        case dnnl_u8: return "u8";
        case dnnl_f8_e5m2: return "f8_e5m2";
        case dnnl_f8_e4m3: return "f8_e4m3";
        case dnnl_s4: return "s4";
        case dnnl_u4: return "u4";
        default: return "undef";
    }
}

std::string dims_str(const dnnl_memory_desc &md) {
    std::string s;
    for (int d = 0; d < md.ndims; d++)
        s += (d ? "x" : "") + std::to_string(md.dims[d]);
    return s;
}

// inner product: the weights descriptor the user sees after an implementation
// resolved format any -- the matmul's packed layout under the inner product's
// dims, or the plain tensor that is the matmul's row-major [K, OC] (IC-major
// for the inner product: stride 1 along OC)
void ip_refresh_weights_md(pd_impl_t &pd) {
    if (!pd.ip) return;
    const dnnl_memory_desc &user = pd.ip_wei_user;
    if (pd.wei.is_packed()) {
        dnnl_memory_desc r = pd.wei;
        r.ndims = user.ndims;
        for (int d = 0; d < user.ndims; d++)
            r.dims[d] = user.dims[d];
        r.packed_transposed = true;
        pd.ip_wei = r;
    } else if (user.is_any()) {
        dnnl_dims_t strides;
        const int nd = user.ndims;
        strides[0] = 1;
        strides[nd - 1] = user.dims[0];
        for (int d = nd - 2; d >= 1; d--)
            strides[d] = strides[d + 1] * user.dims[d + 1];
        md_init_plain(pd.ip_wei, nd, user.dims, user.data_type, strides);
    } else {
        pd.ip_wei = user;
    }
}

// ---- runtime dims -----------------------------------------------------------
// The descriptors of the memory objects passed to execute stand in for the
// primitive descriptor's wherever that holds DNNL_RUNTIME_DIM_VAL (as
// ctx.memory_mdw does in the reference, src/common/primitive_exec_types.cpp);
// the concrete problem then goes through the ordinary implementation list.
// Each primitive remembers the last few shapes it has run.
constexpr size_t RT_CACHE_ENTRIES = 16;

bool rt_md_matches(const dnnl_memory_desc &want, const dnnl_memory_desc &got) {
    if (got.ndims != want.ndims || got.data_type != want.data_type) return false;
    // prepacked weights (all dims known): the very descriptor the primitive
    // descriptor reports
    if (!want.is_plain()) return md_equal(want, got);
    if (!got.is_plain() || got.has_runtime_dims()) return false;
    for (int d = 0; d < want.ndims; d++) {
        if (want.dims[d] != DNNL_RUNTIME_DIM_VAL && want.dims[d] != got.dims[d])
            return false;
        if (want.strides[d] != DNNL_RUNTIME_DIM_VAL
                && want.strides[d] != got.strides[d])
            return false;
    }
    return true;
}

dnnl_status_t resolve_runtime_matmul(dnnl_primitive *prim,
        const std::map<int, dnnl_memory_t> &args,
        std::shared_ptr<rt_entry_t> &out) {
    const pd_impl_t &pd = *prim->pd;
    auto md_of = [&](int arg) -> const dnnl_memory_desc * {
        auto it = args.find(arg);
        return it == args.end() ? nullptr : &it->second->md;
    };
    const dnnl_memory_desc *src = md_of(DNNL_ARG_SRC), *wei = md_of(DNNL_ARG_WEIGHTS),
                           *dst = md_of(DNNL_ARG_DST), *bias = md_of(DNNL_ARG_BIAS);
    if (!src || !wei || !dst) return dnnl_invalid_arguments;
    const bool with_bias = pd.bias.ndims != 0;
    if (with_bias && !bias) return dnnl_invalid_arguments;
    if (!rt_md_matches(pd.src, *src) || !rt_md_matches(pd.wei, *wei)
            || !rt_md_matches(pd.dst, *dst)
            || (with_bias && !rt_md_matches(pd.bias, *bias)))
        return dnnl_invalid_arguments;
    if (src->has_zero_dim() || wei->has_zero_dim() || dst->has_zero_dim()) {
        out.reset();
        return matmul_shape_check(src, wei, with_bias ? bias : nullptr, dst);
    }

    std::lock_guard<std::mutex> lock(prim->rt_mutex);
    for (auto &e : prim->rt)
        if (md_equal(e->src, *src) && md_equal(e->wei, *wei)
                && md_equal(e->dst, *dst)
                && (!with_bias || md_equal(e->bias, *bias))) {
            e->stamp = ++prim->rt_clock;
            out = e;
            return dnnl_success;
        }

    dnnl_status_t st
            = matmul_shape_check(src, wei, with_bias ? bias : nullptr, dst);
    if (st != dnnl_success) return st;
    st = matmul_attr_check(*src, *wei, *dst, pd.engine, pd.attr);
    if (st != dnnl_success) return st;
    auto e = std::make_shared<rt_entry_t>();
    e->src = *src;
    e->wei = *wei;
    e->dst = *dst;
    if (with_bias) e->bias = *bias;
    e->pd = std::make_shared<pd_impl_t>(pd);
    pd_impl_t &c = *e->pd;
    c.runtime = false;
    c.user_src = *src;
    c.user_wei = *wei;
    c.user_dst = *dst;
    c.user_bias = with_bias ? *bias : dnnl_memory_desc();
    // the scratchpad of a shape is not known to the user beforehand
    c.attr.scratchpad_mode = dnnl_scratchpad_mode_library;
    st = walk_matmul_impls(c, 0);
    if (st != dnnl_success) return st;
    const int qs = qmm_matmul_plan_create(&e->plan, c.impl, &c.mm);
    if (qs != QMM_OK) return from_qmm(qs);
    if (c.scratch_bytes && hipMalloc(&e->scratch, c.scratch_bytes) != hipSuccess)
        return dnnl_out_of_memory;
    e->stamp = ++prim->rt_clock;
    if (prim->rt.size() >= RT_CACHE_ENTRIES) {
        size_t oldest = 0;
        for (size_t i = 1; i < prim->rt.size(); i++)
            if (prim->rt[i]->stamp < prim->rt[oldest]->stamp) oldest = i;
        prim->rt.erase(prim->rt.begin() + oldest);
    }
    prim->rt.push_back(e);
    out = e;
    return dnnl_success;
}

} // namespace

scratch_guard_t::~scratch_guard_t() {
    if (event) (void)hipEventDestroy((hipEvent_t)event);
}

namespace {
// Holds the guard's mutex from before the launch until the event behind it is
// recorded. A stream under capture is left alone (an event recorded outside the
// capture cannot be waited for inside it): whoever captures orders the launches.
struct scratch_order_t {
    scratch_guard_t *g = nullptr;
    hipStream_t stream = nullptr;
    bool active = false;
    scratch_order_t(scratch_guard_t *guard, void *hip_stream) {
        if (!guard) return;
        stream = (hipStream_t)hip_stream;
        hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
        if (stream && hipStreamIsCapturing(stream, &cs) == hipSuccess
                && cs != hipStreamCaptureStatusNone)
            return;
        g = guard;
        g->mu.lock();
        active = true;
        if (g->used && g->last_stream != hip_stream && g->event)
            (void)hipStreamWaitEvent(stream, (hipEvent_t)g->event, 0);
    }
    ~scratch_order_t() {
        if (!active) return;
        if (!g->event) {
            hipEvent_t e = nullptr;
            if (hipEventCreateWithFlags(&e, hipEventDisableTiming) == hipSuccess)
                g->event = e;
        }
        if (g->event) (void)hipEventRecord((hipEvent_t)g->event, stream);
        g->last_stream = (void *)stream;
        g->used = true;
        g->mu.unlock();
    }
};
} // namespace

// An evicted or destroyed shape: hipFree waits for the kernels that still use
// the scratchpad.
rt_entry_t::~rt_entry_t() {
    if (plan) qmm_matmul_plan_destroy(plan);
    if (scratch) (void)hipFree(scratch);
}

extern "C" {

// ======================= matmul primitive descriptor =======================
dnnl_status_t dnnl_matmul_primitive_desc_create(dnnl_primitive_desc_t *out,
        dnnl_engine_t engine, const_dnnl_memory_desc_t src_desc,
        const_dnnl_memory_desc_t weights_desc,
        const_dnnl_memory_desc_t bias_desc, const_dnnl_memory_desc_t dst_desc,
        const_dnnl_primitive_attr_t attr) {
    if (!out || !engine) return dnnl_invalid_arguments;
    dnnl_status_t st
            = matmul_shape_check(src_desc, weights_desc, bias_desc, dst_desc);
    if (st != dnnl_success) return st;
    static const dnnl_primitive_attr default_attr;
    const dnnl_primitive_attr &a = attr ? *attr : default_attr;
    st = matmul_attr_check(*src_desc, *weights_desc, *dst_desc, engine, a);
    if (st != dnnl_success) return st;

    auto pd = std::make_shared<pd_impl_t>();
    pd->kind = dnnl_matmul;
    pd->engine = engine;
    pd->attr = a; // attributes are copied into the descriptor
    pd->user_src = *src_desc;
    pd->user_wei = *weights_desc;
    if (bias_desc) pd->user_bias = *bias_desc;
    pd->user_dst = *dst_desc;
    if (engine->kind != dnnl_gpu) return dnnl_unimplemented; // empty list
    bool runtime = false;
    for (const dnnl_memory_desc *md :
            {&pd->user_src, &pd->user_wei, &pd->user_bias, &pd->user_dst})
        runtime = runtime || (md->ndims && md->has_runtime_dims());
    if (runtime) {
        // format any cannot be resolved on a descriptor that has runtime dims
        // itself (src/common/matmul_pd.hpp:266-277); everything that depends
        // on the dims is decided per shape at execution
        for (const dnnl_memory_desc *md :
                {&pd->user_src, &pd->user_bias, &pd->user_dst})
            if (md->ndims && !md->is_plain()) return dnnl_unimplemented;
        pd->runtime = true;
        pd->src = pd->user_src;
        pd->wei = pd->user_wei;
        pd->bias = pd->user_bias;
        pd->dst = pd->user_dst;
        if (!pd->user_wei.is_plain()) {
            // Weights whose own dims are all known may still be `any` or
            // prepacked (the usual case: a linear layer with a run-time batch,
            // examples/tutorials/matmul/inference_int8_matmul.cpp:104-125).
            // The packed layout depends on K, N, the types and the attributes
            // only: it is resolved here on a stand-in problem in which every
            // runtime dim has a nominal value.
            if (pd->user_wei.has_runtime_dims()) return dnnl_unimplemented;
            if (!pd->user_wei.is_any() && !pd->user_wei.is_packed())
                return dnnl_unimplemented;
            pd_impl_t nominal = *pd;
            nominal.runtime = false;
            for (dnnl_memory_desc *md :
                    {&nominal.user_src, &nominal.user_bias, &nominal.user_dst}) {
                if (!md->ndims || !md->has_runtime_dims()) continue;
                bool rt_strides = false;
                for (int d = 0; d < md->ndims; d++) {
                    if (md->dims[d] == DNNL_RUNTIME_DIM_VAL)
                        md->dims[d] = d < md->ndims - 2 ? 4 : 256;
                    rt_strides = rt_strides
                            || md->strides[d] == DNNL_RUNTIME_DIM_VAL;
                }
                if (rt_strides) {
                    dnnl_memory_desc r;
                    md_init_plain(r, md->ndims, md->dims, md->data_type, nullptr);
                    *md = r;
                }
            }
            st = walk_matmul_impls(nominal, 0);
            if (st != dnnl_success) return st;
            pd->wei = nominal.wei;
        }
        for (auto &e : pd->attr.post_ops.entries)
            if (e.kind == dnnl_binary) {
                if (!e.user_src1_desc.is_plain()) return dnnl_unimplemented;
                e.src1_desc = e.user_src1_desc;
            }
        pd->impl_name = "hip:gfx950:runtime_dims";
    } else {
        st = walk_matmul_impls(*pd, 0);
        if (st != dnnl_success) return st;
    }
    dnnl_primitive_desc *h = new (std::nothrow) dnnl_primitive_desc {pd};
    if (!h) return dnnl_out_of_memory;
    *out = h;
    return dnnl_success;
}

// ======================= inner product (forward) ===========================
// src/common/inner_product.cpp:33-110 for the shape rules. The primitive is
// the matmul [MB, K] x [K, OC] with K = IC * spatial: a source whose trailing
// dims nest densely is that matrix as it lies in memory, and OC-major weights
// [OC, IC, spatial...] are the K x OC matrix with strides (1, pitch) -- no
// data moves. The descriptors the user sees (queries, format any) keep the
// inner product's dims; opaque weights are marked as transposed so that the
// prepacking reorder reads the user's [OC, IC, ...] tensor the same way.
static bool trailing_dims_nest(const dnnl_memory_desc &md) {
    if (!md.is_plain() || md.strides[md.ndims - 1] != 1) return false;
    for (int d = md.ndims - 2; d >= 1; d--)
        if (md.strides[d] != md.strides[d + 1] * md.dims[d + 1]) return false;
    return true;
}

dnnl_status_t dnnl_inner_product_forward_primitive_desc_create(
        dnnl_primitive_desc_t *out, dnnl_engine_t engine,
        dnnl_prop_kind_t prop_kind, const_dnnl_memory_desc_t src_desc,
        const_dnnl_memory_desc_t weights_desc,
        const_dnnl_memory_desc_t bias_desc, const_dnnl_memory_desc_t dst_desc,
        const_dnnl_primitive_attr_t attr) {
    if (!out || !engine || !src_desc || !weights_desc || !dst_desc)
        return dnnl_invalid_arguments;
    if (prop_kind != dnnl_forward_training && prop_kind != dnnl_forward_inference)
        return dnnl_invalid_arguments;
    if (bias_desc && bias_desc->ndims == 0) bias_desc = nullptr;
    const int nd = src_desc->ndims;
    if (nd < 2 || nd > 5 || weights_desc->ndims != nd || dst_desc->ndims != 2)
        return dnnl_invalid_arguments;
    if (src_desc->has_runtime_dims() || weights_desc->has_runtime_dims()
            || dst_desc->has_runtime_dims())
        return dnnl_unimplemented;
    const int64_t MB = src_desc->dims[0], OC = weights_desc->dims[0];
    int64_t K = 1;
    for (int d = 1; d < nd; d++) {
        if (src_desc->dims[d] != weights_desc->dims[d])
            return dnnl_invalid_arguments;
        K *= src_desc->dims[d];
    }
    if (dst_desc->dims[0] != MB || dst_desc->dims[1] != OC)
        return dnnl_invalid_arguments;
    if (bias_desc && (bias_desc->ndims != 1 || bias_desc->dims[0] != OC))
        return dnnl_invalid_arguments;
    if (engine->kind != dnnl_gpu) return dnnl_unimplemented;

    // the user-visible descriptors, format any resolved to row-major
    auto pd = std::make_shared<pd_impl_t>();
    pd->ip = true;
    pd->ip_src = *src_desc;
    pd->ip_wei = pd->ip_wei_user = *weights_desc;
    pd->ip_dst = *dst_desc;
    if (bias_desc) pd->ip_bias = *bias_desc;
    for (dnnl_memory_desc *md : {&pd->ip_src, &pd->ip_dst, &pd->ip_bias}) {
        if (md->ndims && md->is_any()) {
            dnnl_memory_desc r;
            md_init_plain(r, md->ndims, md->dims, md->data_type, nullptr);
            *md = r;
        }
    }
    if (!trailing_dims_nest(pd->ip_src) || !pd->ip_dst.is_plain()
            || (pd->ip_bias.ndims && !pd->ip_bias.is_plain()))
        return dnnl_unimplemented;

    // the matmul view
    dnnl_memory_desc m_src, m_wei, m_bias;
    {
        const dnnl_dims_t dims = {MB, K}, strides = {pd->ip_src.strides[0], 1};
        md_init_plain(m_src, 2, dims, pd->ip_src.data_type, strides);
    }
    const dnnl_dims_t wdims = {K, OC};
    if (pd->ip_wei.is_any()) {
        md_init_plain(m_wei, 2, wdims, pd->ip_wei.data_type, nullptr);
        m_wei.format_kind = dnnl_format_kind_any;
    } else if (pd->ip_wei.is_packed()) {
        if (!pd->ip_wei.packed_transposed) return dnnl_unimplemented;
        m_wei = pd->ip_wei;
        m_wei.ndims = 2;
        m_wei.dims[0] = K;
        m_wei.dims[1] = OC;
        m_wei.packed_transposed = false;
    } else if (trailing_dims_nest(pd->ip_wei)) { // OC-major
        const dnnl_dims_t strides = {1, pd->ip_wei.strides[0]};
        md_init_plain(m_wei, 2, wdims, pd->ip_wei.data_type, strides);
    } else if (nd == 2 && pd->ip_wei.is_plain() && pd->ip_wei.strides[0] == 1) {
        const dnnl_dims_t strides = {pd->ip_wei.strides[1], 1}; // IC-major
        md_init_plain(m_wei, 2, wdims, pd->ip_wei.data_type, strides);
    } else {
        return dnnl_unimplemented;
    }
    if (pd->ip_bias.ndims) {
        const dnnl_dims_t dims = {1, OC}, strides = {OC * pd->ip_bias.strides[0],
                                                  pd->ip_bias.strides[0]};
        md_init_plain(m_bias, 2, dims, pd->ip_bias.data_type, strides);
    }

    // attributes: the weights' OC dim is dim 0 here and dim 1 of the matmul
    static const dnnl_primitive_attr default_attr;
    dnnl_primitive_attr a = attr ? *attr : default_attr;
    {
        auto it = a.scales.find(DNNL_ARG_WEIGHTS);
        if (it != a.scales.end() && !it->second.is_default()) {
            if (it->second.mask == 1)
                it->second.mask = 2;
            else if (it->second.mask != 0 || it->second.group_ndims != 0)
                return dnnl_unimplemented;
        }
        if (!a.zp(DNNL_ARG_SRC).is_default() || !a.zp(DNNL_ARG_WEIGHTS).is_default()
                || !a.zp(DNNL_ARG_DST).is_default())
            return dnnl_unimplemented; // src/common/inner_product.cpp:99-103
    }
    dnnl_status_t st = matmul_shape_check(
            &m_src, &m_wei, pd->ip_bias.ndims ? &m_bias : nullptr, &pd->ip_dst);
    if (st != dnnl_success) return st;
    st = matmul_attr_check(m_src, m_wei, pd->ip_dst, engine, a);
    if (st != dnnl_success) return st;

    pd->kind = dnnl_matmul;
    pd->engine = engine;
    pd->attr = a;
    pd->user_src = m_src;
    pd->user_wei = m_wei;
    if (pd->ip_bias.ndims) pd->user_bias = m_bias;
    pd->user_dst = pd->ip_dst;
    st = walk_matmul_impls(*pd, 0);
    if (st != dnnl_success) return st;
    ip_refresh_weights_md(*pd);
    dnnl_primitive_desc *h = new (std::nothrow) dnnl_primitive_desc {pd};
    if (!h) return dnnl_out_of_memory;
    *out = h;
    return dnnl_success;
}

dnnl_status_t dnnl_primitive_desc_next_impl(dnnl_primitive_desc_t pd) {
    if (!pd || !pd->p) return dnnl_invalid_arguments;
    if (pd->p->kind != dnnl_matmul || pd->p->runtime)
        return dnnl_last_impl_reached;
    auto next = std::make_shared<pd_impl_t>(*pd->p);
    const dnnl_status_t st = walk_matmul_impls(*next, pd->p->impl + 1);
    if (st != dnnl_success) return dnnl_last_impl_reached;
    ip_refresh_weights_md(*next);
    pd->p = next;
    return dnnl_success;
}

dnnl_status_t dnnl_primitive_desc_clone(
        dnnl_primitive_desc_t *out, const_dnnl_primitive_desc_t existing) {
    if (!out || !existing) return dnnl_invalid_arguments;
    *out = new (std::nothrow) dnnl_primitive_desc {existing->p};
    return *out ? dnnl_success : dnnl_out_of_memory;
}

dnnl_status_t dnnl_primitive_desc_get_attr(
        const_dnnl_primitive_desc_t pd, const_dnnl_primitive_attr_t *attr) {
    if (!pd || !attr) return dnnl_invalid_arguments;
    *attr = &pd->p->attr;
    return dnnl_success;
}

dnnl_status_t dnnl_primitive_desc_destroy(dnnl_primitive_desc_t pd) {
    delete pd;
    return dnnl_success;
}

const_dnnl_memory_desc_t dnnl_primitive_desc_query_md(
        const_dnnl_primitive_desc_t pd, dnnl_query_t what, int index) {
    if (!pd) return nullptr;
    const pd_impl_t &p = *pd->p;
    // an inner product shows its own descriptors, not the matmul view
    const dnnl_memory_desc &q_src = p.ip ? p.ip_src : p.src;
    const dnnl_memory_desc &q_wei = p.ip ? p.ip_wei : p.wei;
    const dnnl_memory_desc &q_bias = p.ip ? p.ip_bias : p.bias;
    const dnnl_memory_desc &q_dst = p.ip ? p.ip_dst : p.dst;
    switch (what) {
        case dnnl_query_src_md: return index == 0 ? &q_src : &g_zero_md;
        case dnnl_query_weights_md:
            if (p.kind != dnnl_matmul) return &g_zero_md;
            return index == 0 ? &q_wei : index == 1 ? &q_bias : &g_zero_md;
        case dnnl_query_dst_md: return index == 0 ? &q_dst : &g_zero_md;
        case dnnl_query_scratchpad_md:
            return index == 0 ? &p.scratchpad : &g_zero_md;
        case dnnl_query_diff_src_md:
        case dnnl_query_diff_weights_md:
        case dnnl_query_diff_dst_md:
        case dnnl_query_workspace_md: return &g_zero_md;
        case dnnl_query_exec_arg_md: {
            if (p.kind == dnnl_matmul) {
                if (index == DNNL_ARG_SRC) return &q_src;
                if (index == DNNL_ARG_WEIGHTS) return &q_wei;
                if (index == DNNL_ARG_BIAS) return &q_bias;
                if (index == DNNL_ARG_DST) return &q_dst;
            } else if (p.kind == dnnl_softmax) {
                if (index == DNNL_ARG_SRC) return &p.src;
                if (index == DNNL_ARG_DST) return &p.dst;
            } else if (p.kind == kind_sdpa) {
                if (index == DNNL_ARG_QUERIES) return &p.src;
                if (index == DNNL_ARG_KEYS) return &p.sdpa_k;
                if (index == DNNL_ARG_VALUES) return &p.sdpa_v;
                if (index == DNNL_ARG_ATTN_MASK) return &p.sdpa_mask;
                if (index == DNNL_ARG_DST) return &p.dst;
                return &g_zero_md;
            } else {
                if (index == DNNL_ARG_FROM) return &p.src;
                if (index == DNNL_ARG_TO) return &p.dst;
            }
            if (index == DNNL_ARG_SCRATCHPAD) return &p.scratchpad;
            const auto &po = p.attr.post_ops.entries;
            for (int i = 0; i < (int)po.size(); i++)
                if (po[i].kind == dnnl_binary
                        && index
                                == (DNNL_ARG_ATTR_MULTIPLE_POST_OP(i)
                                        | DNNL_ARG_SRC_1))
                    return &po[i].src1_desc;
            return &g_zero_md;
        }
        default: return nullptr;
    }
}

dnnl_status_t dnnl_primitive_desc_query(const_dnnl_primitive_desc_t pd,
        dnnl_query_t what, int index, void *result) {
    if (!pd || !result) return dnnl_invalid_arguments;
    const pd_impl_t &p = *pd->p;
    switch (what) {
        case dnnl_query_engine: *(dnnl_engine_t *)result = p.engine; break;
        case dnnl_query_scratchpad_engine:
        case dnnl_query_reorder_src_engine:
        case dnnl_query_reorder_dst_engine:
            *(dnnl_engine_t *)result = p.engine;
            break;
        case dnnl_query_primitive_kind:
            *(dnnl_primitive_kind_t *)result = p.ip ? dnnl_inner_product : p.kind;
            break;
        case dnnl_query_num_of_inputs_s32: *(int *)result = n_inputs(p); break;
        case dnnl_query_num_of_outputs_s32: *(int *)result = 1; break;
        case dnnl_query_impl_info_str:
            *(const char **)result = p.impl_name.c_str();
            break;
        case dnnl_query_memory_consumption_s64:
            *(int64_t *)result
                    = p.attr.scratchpad_mode == dnnl_scratchpad_mode_library
                    ? (int64_t)p.scratch_bytes
                    : 0;
            break;
        case dnnl_query_prop_kind:
            *(dnnl_prop_kind_t *)result = p.prop_kind;
            break;
        case dnnl_query_alg_kind:
            if (p.kind != dnnl_softmax) return dnnl_unimplemented;
            *(dnnl_alg_kind_t *)result = (dnnl_alg_kind_t)p.sm.alg;
            break;
        case dnnl_query_axis_s32:
            if (p.kind != dnnl_softmax) return dnnl_unimplemented;
            *(int *)result = p.sm.axis;
            break;
        case dnnl_query_time_estimate_f64: *(double *)result = 0; break;
        default: {
            if ((what & dnnl_query_some_md) || what == dnnl_query_exec_arg_md) {
                const_dnnl_memory_desc_t md
                        = dnnl_primitive_desc_query_md(pd, what, index);
                if (!md) return dnnl_unimplemented;
                *(const_dnnl_memory_desc_t *)result = md;
                break;
            }
            return dnnl_unimplemented;
        }
    }
    return dnnl_success;
}

int dnnl_primitive_desc_query_s32(
        const_dnnl_primitive_desc_t pd, dnnl_query_t what, int index) {
    int v = 0;
    if (what == dnnl_query_num_of_inputs_s32
            || what == dnnl_query_num_of_outputs_s32)
        dnnl_primitive_desc_query(pd, what, index, &v);
    return v;
}

// ======================= reorder primitive descriptor =======================
dnnl_status_t dnnl_reorder_primitive_desc_create(dnnl_primitive_desc_t *out,
        const_dnnl_memory_desc_t src_md, dnnl_engine_t src_engine,
        const_dnnl_memory_desc_t dst_md, dnnl_engine_t dst_engine,
        const_dnnl_primitive_attr_t attr) {
    if (!out || !src_md || !src_engine || !dst_md || !dst_engine)
        return dnnl_invalid_arguments;
    if (src_md->is_any() || dst_md->is_any()) return dnnl_invalid_arguments;
    if (src_engine->kind != dst_engine->kind
            && src_engine->kind != dnnl_cpu && dst_engine->kind != dnnl_cpu)
        return dnnl_invalid_arguments;
    // consistent dims
    if (src_md->ndims != dst_md->ndims) return dnnl_invalid_arguments;
    for (int d = 0; d < src_md->ndims; d++)
        if (src_md->dims[d] != dst_md->dims[d]) return dnnl_invalid_arguments;
    static const dnnl_primitive_attr default_attr;
    const dnnl_primitive_attr &a = attr ? *attr : default_attr;
    if (!is_integral(src_md->data_type) && !a.zp(DNNL_ARG_SRC).is_default())
        return dnnl_invalid_arguments;
    if (!is_integral(dst_md->data_type) && !a.zp(DNNL_ARG_DST).is_default())
        return dnnl_invalid_arguments;
    if (!a.has_default_scales()) {
        for (auto &kv : a.scales)
            if (!kv.second.is_default() && kv.first != DNNL_ARG_SRC
                    && kv.first != DNNL_ARG_DST)
                return dnnl_unimplemented;
        const quant_entry_t &ss = a.scale(DNNL_ARG_SRC);
        if (is_int4(src_md->data_type) && !ss.is_default() && ss.mask <= 0)
            return dnnl_invalid_arguments;
        if (ss.has_groups()) {
            const int nd = src_md->ndims;
            if (nd < 2) return dnnl_invalid_arguments;
            if (ss.group(0) > 1 && src_md->dims[nd - 2] % ss.group(0) != 0)
                return dnnl_invalid_arguments;
            if (ss.group(1) > 1 && src_md->dims[nd - 1] % ss.group(1) != 0)
                return dnnl_invalid_arguments;
            if (!((ss.mask & (1 << (nd - 1))) && (ss.mask & (1 << (nd - 2)))))
                return dnnl_invalid_arguments;
        }
        if (a.scale(DNNL_ARG_DST).has_groups()) return dnnl_invalid_arguments;
    }
    if (src_engine != dst_engine || src_engine->kind != dnnl_gpu)
        return dnnl_unimplemented;
    if (src_md->has_runtime_dims()) return dnnl_unimplemented;
    if (!a.post_ops.entries.empty()) return dnnl_unimplemented;

    auto pd = std::make_shared<pd_impl_t>();
    pd->kind = dnnl_reorder;
    pd->engine = src_engine;
    pd->attr = a;
    pd->user_src = pd->src = *src_md;
    pd->user_dst = pd->dst = *dst_md;
    qmm_reorder_desc_t &R = pd->ro;
    std::memset(&R, 0, sizeof(R));
    md_to_tensor(R.src, *src_md);
    md_to_tensor(R.dst, *dst_md);
    R.src_layout = src_md->is_packed() ? src_md->packed_layout : QMM_LAYOUT_PLAIN;
    R.dst_layout = dst_md->is_packed() ? dst_md->packed_layout : QMM_LAYOUT_PLAIN;
    if (!(src_md->is_plain() || src_md->is_packed())
            || !(dst_md->is_plain() || dst_md->is_packed()))
        return dnnl_unimplemented;
    // Packed weights of an inner product carry dims [OC, IC, spatial...] over
    // the image of the matmul weights [K, OC]: hand the kernels that matrix.
    // The plain side's dims 1.. must nest (then K has one stride).
    const dnnl_memory_desc *tp = src_md->is_packed() && src_md->packed_transposed
            ? src_md
            : (dst_md->is_packed() && dst_md->packed_transposed ? dst_md
                                                                : nullptr);
    if (tp) {
        const dnnl_memory_desc *pl = tp == src_md ? dst_md : src_md;
        const int nd = pl->ndims;
        if (!pl->is_plain() || nd < 2) return dnnl_unimplemented;
        int64_t K = 1;
        for (int d = 1; d < nd; d++)
            K *= pl->dims[d];
        for (int d = nd - 2; d >= 1; d--)
            if (pl->strides[d] != pl->strides[d + 1] * pl->dims[d + 1])
                return dnnl_unimplemented;
        for (qmm_tensor_t *t : {&R.src, &R.dst}) {
            t->ndims = 2;
            t->dims[0] = K;
            t->dims[1] = pl->dims[0];
            t->strides[0] = pl->strides[nd - 1];
            t->strides[1] = pl->strides[0];
        }
    }
    fill_quant(R.src_scale, a.scale(DNNL_ARG_SRC), dnnl_f32);
    fill_quant(R.dst_scale, a.scale(DNNL_ARG_DST), dnnl_f32);
    fill_quant(R.src_zp, a.zp(DNNL_ARG_SRC), dnnl_s32);
    fill_quant(R.dst_zp, a.zp(DNNL_ARG_DST), dnnl_s32);
    const int st = qmm_reorder_supports(&R);
    if (st != QMM_OK) return from_qmm(st);
    pd->impl = 0;
    pd->impl_name = qmm_reorder_impl_name(&R);
    dnnl_primitive_desc *h = new (std::nothrow) dnnl_primitive_desc {pd};
    if (!h) return dnnl_out_of_memory;
    *out = h;
    return dnnl_success;
}

// ======================= softmax primitive descriptor ========================
// src/common/softmax.cpp:42-182 (descriptor and attribute checks),
// src/cpu/ref_softmax.hpp:44-70 (what the reference implementation takes)
dnnl_status_t dnnl_softmax_forward_primitive_desc_create(
        dnnl_primitive_desc_t *out, dnnl_engine_t engine,
        dnnl_prop_kind_t prop_kind, dnnl_alg_kind_t alg_kind,
        const_dnnl_memory_desc_t src_md, const_dnnl_memory_desc_t dst_md,
        int softmax_axis, const_dnnl_primitive_attr_t attr) {
    if (!out || !engine || !src_md || !dst_md) return dnnl_invalid_arguments;
    if (prop_kind != dnnl_forward_training && prop_kind != dnnl_forward_inference)
        return dnnl_invalid_arguments;
    if (alg_kind != dnnl_softmax_accurate && alg_kind != dnnl_softmax_log)
        return dnnl_invalid_arguments;
    if (softmax_axis < 0 || softmax_axis >= dst_md->ndims)
        return dnnl_invalid_arguments;
    if (src_md->is_any()) return dnnl_invalid_arguments;
    if (src_md->has_runtime_dims() || dst_md->has_runtime_dims())
        return dnnl_unimplemented;
    if (src_md->ndims != dst_md->ndims) return dnnl_invalid_arguments;
    for (int d = 0; d < src_md->ndims; d++)
        if (src_md->dims[d] != dst_md->dims[d]) return dnnl_invalid_arguments;
    if (engine->kind != dnnl_gpu) return dnnl_unimplemented;
    if (!src_md->is_plain() || !(dst_md->is_plain() || dst_md->is_any()))
        return dnnl_unimplemented;

    static const dnnl_primitive_attr default_attr;
    const dnnl_primitive_attr &a = attr ? *attr : default_attr;
    // attributes: post-ops in general and, for int8 src or dst, scales
    // (softmax.cpp:96-140); no post-op is implemented here
    if (!a.post_ops.entries.empty()) return dnnl_unimplemented;
    if (!a.has_default_zps()) return dnnl_unimplemented;
    if (!a.dropout_desc.is_zero() || !a.rounding.empty()) return dnnl_unimplemented;
    const bool int8 = is_int8(src_md->data_type) || is_int8(dst_md->data_type);
    if (!a.has_default_scales()) {
        if (!int8) return dnnl_unimplemented;
        for (auto &kv : a.scales) {
            if (kv.second.is_default()) continue;
            if (kv.first != DNNL_ARG_SRC && kv.first != DNNL_ARG_DST)
                return dnnl_unimplemented;
            if (kv.second.mask != 0 || kv.second.has_groups())
                return dnnl_unimplemented;
        }
    }
    // the reference keeps the exponentials in f32 unless the accumulation
    // mode is relaxed (ref_softmax.hpp:80-92); only the f32 form exists here
    if (a.acc_mode != dnnl_accumulation_mode_strict
            && src_md->data_type == dst_md->data_type
            && src_md->data_type != dnnl_f32 && !is_int8(dst_md->data_type))
        return dnnl_unimplemented;

    auto pd = std::make_shared<pd_impl_t>();
    pd->kind = dnnl_softmax;
    pd->engine = engine;
    pd->attr = a;
    pd->prop_kind = prop_kind;
    pd->user_src = pd->src = *src_md;
    pd->user_dst = *dst_md;
    pd->dst = *dst_md;
    if (dst_md->is_any()) {
        // softmax_pd.hpp set_default_formats: dst takes the layout of src
        if (!md_init_plain(pd->dst, src_md->ndims, src_md->dims,
                    dst_md->data_type, src_md->strides))
            return dnnl_invalid_arguments;
    }
    qmm_softmax_desc_t &S = pd->sm;
    std::memset(&S, 0, sizeof(S));
    md_to_tensor(S.src, pd->src);
    md_to_tensor(S.dst, pd->dst);
    S.axis = softmax_axis;
    S.alg = (int32_t)alg_kind;
    fill_quant(S.src_scale, a.scale(DNNL_ARG_SRC), dnnl_f32);
    fill_quant(S.dst_scale, a.scale(DNNL_ARG_DST), dnnl_f32);
    if (qmm_softmax_supports(&S) != QMM_OK) return dnnl_unimplemented;
    pd->impl = 0;
    pd->impl_name = qmm_softmax_impl_name(&S);
    dnnl_primitive_desc *h = new (std::nothrow) dnnl_primitive_desc();
    if (!h) return dnnl_out_of_memory;
    h->p = pd;
    *out = h;
    return dnnl_success;
}

// ======================= sdpa primitive descriptor ===========================
// src/common/sdpa_test_iface.cpp:27-44, sdpa_utils.hpp:51-180
dnnl_status_t sdpa_primitive_desc_create(dnnl_primitive_desc_t *out,
        dnnl_engine_t engine, const_dnnl_memory_desc_t q_md,
        const_dnnl_memory_desc_t k_md, const_dnnl_memory_desc_t v_md,
        const_dnnl_memory_desc_t dst_md, const_dnnl_memory_desc_t mask_md,
        dnnl_data_type_t scale_dt, bool invert_scale, dnnl_dim_t kv_head_number,
        bool causal_mask, const_dnnl_primitive_attr_t attr,
        const_dnnl_primitive_attr_t kq_attr,
        const_dnnl_primitive_attr_t vs_attr) {
    if (!out || !engine || !q_md || !k_md || !v_md || !dst_md)
        return dnnl_invalid_arguments;
    // sdpa_attr_check: scales f16 / f32, zero points u4 / s4 / u8 / s8 / s32,
    // nothing else on the primitive's own attributes
    for (const_dnnl_primitive_attr_t a : {kq_attr, vs_attr}) {
        if (!a) continue;
        const quant_entry_t &sc = a->scale(DNNL_ARG_WEIGHTS);
        const quant_entry_t &zp = a->zp(DNNL_ARG_WEIGHTS);
        if (!sc.is_default() && sc.dt != dnnl_f16 && sc.dt != dnnl_f32)
            return dnnl_invalid_arguments;
        if (!zp.is_default() && zp.dt != dnnl_s4 && zp.dt != dnnl_u4
                && zp.dt != dnnl_u8 && zp.dt != dnnl_s8 && zp.dt != dnnl_s32)
            return dnnl_invalid_arguments;
    }
    if (attr
            && (!attr->has_default_scales() || !attr->has_default_zps()
                    || !attr->post_ops.entries.empty()
                    || attr->fpmath_mode != dnnl_fpmath_mode_strict
                    || !attr->dropout_desc.is_zero() || !attr->rounding.empty()))
        return dnnl_unimplemented;
    // create_sdpa_pd: shapes
    const int nd = dst_md->ndims;
    if (q_md->ndims != nd || k_md->ndims != nd || v_md->ndims != nd || nd < 2)
        return dnnl_invalid_arguments;
    const int r = nd - 2, c = nd - 1;
    if (q_md->dims[c] != k_md->dims[r] || k_md->dims[c] != v_md->dims[r]
            || dst_md->dims[r] != q_md->dims[r] || dst_md->dims[c] != v_md->dims[c])
        return dnnl_invalid_arguments;
    if (engine->kind != dnnl_gpu) return dnnl_unimplemented;
    for (const_dnnl_memory_desc_t md : {q_md, k_md, v_md, dst_md})
        if (!md->is_plain() || md->has_runtime_dims()) return dnnl_unimplemented;
    if (mask_md && (!mask_md->is_plain() || mask_md->has_runtime_dims()))
        return dnnl_unimplemented;

    auto pd = std::make_shared<pd_impl_t>();
    pd->kind = kind_sdpa;
    pd->engine = engine;
    if (attr) pd->attr = *attr;
    pd->user_src = pd->src = *q_md;
    pd->sdpa_k = *k_md;
    pd->sdpa_v = *v_md;
    pd->user_dst = pd->dst = *dst_md;
    if (mask_md) pd->sdpa_mask = *mask_md;
    qmm_sdpa_desc_t &S = pd->sd;
    std::memset(&S, 0, sizeof(S));
    md_to_tensor(S.q, pd->src);
    md_to_tensor(S.k, pd->sdpa_k);
    md_to_tensor(S.v, pd->sdpa_v);
    md_to_tensor(S.dst, pd->dst);
    if (mask_md) md_to_tensor(S.mask, pd->sdpa_mask);
    S.scale_dt = scale_dt;
    S.invert_scale = invert_scale;
    S.causal = causal_mask;
    S.kv_head_number = kv_head_number;
    static const quant_entry_t none;
    fill_quant(S.k_scale, kq_attr ? kq_attr->scale(DNNL_ARG_WEIGHTS) : none, dnnl_f32);
    fill_quant(S.k_zp, kq_attr ? kq_attr->zp(DNNL_ARG_WEIGHTS) : none, dnnl_s32);
    fill_quant(S.v_scale, vs_attr ? vs_attr->scale(DNNL_ARG_WEIGHTS) : none, dnnl_f32);
    fill_quant(S.v_zp, vs_attr ? vs_attr->zp(DNNL_ARG_WEIGHTS) : none, dnnl_s32);
    if (qmm_sdpa_supports(&S) != QMM_OK) return dnnl_unimplemented;
    pd->impl = 0;
    pd->impl_name = qmm_sdpa_impl_name(&S);
    pd->scratch_bytes = qmm_sdpa_scratch_size(&S);
    if (pd->scratch_bytes
            && pd->attr.scratchpad_mode == dnnl_scratchpad_mode_user) {
        dnnl_dims_t dims = {(int64_t)pd->scratch_bytes};
        md_init_plain(pd->scratchpad, 1, dims, dnnl_u8, nullptr);
    }
    dnnl_primitive_desc *h = new (std::nothrow) dnnl_primitive_desc();
    if (!h) return dnnl_out_of_memory;
    h->p = pd;
    *out = h;
    return dnnl_success;
}

// ======================= primitives ========================================
dnnl_status_t dnnl_primitive_create(
        dnnl_primitive_t *primitive, const_dnnl_primitive_desc_t pd) {
    if (!primitive || !pd || !pd->p) return dnnl_invalid_arguments;
    dnnl_primitive *p = new (std::nothrow) dnnl_primitive();
    if (!p) return dnnl_out_of_memory;
    p->pd = pd->p;
    p->pd_handle.p = pd->p;
    if (p->pd->kind == dnnl_matmul && !p->pd->runtime) {
        const dnnl_engine *eng = p->pd->engine;
        if (eng->device < 0 || hipSetDevice(eng->device) != hipSuccess) {
            delete p;
            return dnnl_runtime_error;
        }
        const int st = qmm_matmul_plan_create(&p->plan, p->pd->impl, &p->pd->mm);
        if (st != QMM_OK) {
            delete p;
            return from_qmm(st);
        }
        if (p->pd->scratch_bytes
                && p->pd->attr.scratchpad_mode == dnnl_scratchpad_mode_library) {
            if (hipMalloc(&p->lib_scratch, p->pd->scratch_bytes) != hipSuccess) {
                qmm_matmul_plan_destroy(p->plan);
                delete p;
                return dnnl_out_of_memory;
            }
        }
    }
    if (p->pd->kind == kind_sdpa && p->pd->scratch_bytes
            && p->pd->attr.scratchpad_mode == dnnl_scratchpad_mode_library) {
        const dnnl_engine *eng = p->pd->engine;
        if (eng->device < 0 || hipSetDevice(eng->device) != hipSuccess
                || hipMalloc(&p->lib_scratch, p->pd->scratch_bytes)
                        != hipSuccess) {
            delete p;
            return eng->device < 0 ? dnnl_runtime_error : dnnl_out_of_memory;
        }
    }
    *primitive = p;
    return dnnl_success;
}

dnnl_status_t dnnl_primitive_get_primitive_desc(
        const_dnnl_primitive_t primitive, const_dnnl_primitive_desc_t *pd) {
    if (!primitive || !pd) return dnnl_invalid_arguments;
    *pd = &primitive->pd_handle;
    return dnnl_success;
}

dnnl_status_t dnnl_primitive_destroy(dnnl_primitive_t primitive) {
    if (!primitive) return dnnl_success;
    if (primitive->plan) qmm_matmul_plan_destroy(primitive->plan);
    if (primitive->lib_scratch) (void)hipFree(primitive->lib_scratch);
    delete primitive;
    return dnnl_success;
}

dnnl_status_t dnnl_primitive_execute(const_dnnl_primitive_t primitive,
        dnnl_stream_t stream, int nargs, const dnnl_exec_arg_t *c_args) {
    if (!primitive || !stream) return dnnl_invalid_arguments;
    if (nargs > 0 && !c_args) return dnnl_invalid_arguments;
    const pd_impl_t &upd = *primitive->pd;
    if (stream->engine != upd.engine) return dnnl_invalid_arguments;

    std::map<int, dnnl_memory_t> args;
    int n_in = 0, extra_in = 0, n_out = 0, extra_out = 0;
    for (int i = 0; i < nargs; i++) {
        const int arg = c_args[i].arg;
        dnnl_memory_t mem = c_args[i].memory;
        if (!mem) continue; // dummy arguments are allowed
        if (args.count(arg)) return dnnl_invalid_arguments;
        switch (arg_usage(upd, arg)) {
            case usage_t::input:
                args[arg] = mem;
                n_in++;
                extra_in += (arg & DNNL_ARG_ATTR_ZERO_POINTS)
                        || (arg & DNNL_ARG_ATTR_SCALES);
                break;
            case usage_t::output:
                args[arg] = mem;
                n_out++;
                extra_out += arg == DNNL_ARG_SCRATCHPAD;
                break;
            case usage_t::unused: break;
        }
    }
    if (n_in != n_inputs(upd) + extra_in) return dnnl_invalid_arguments;
    if (n_out != 1 + extra_out) return dnnl_invalid_arguments;

    auto handle = [&](int arg) -> void * {
        auto it = args.find(arg);
        return it == args.end() ? nullptr : it->second->handle;
    };
    if (upd.engine->device < 0
            || hipSetDevice(upd.engine->device) != hipSuccess)
        return dnnl_runtime_error;

    // a runtime-dims matmul becomes a concrete one here, per shape
    const pd_impl_t *concrete = &upd;
    qmm_plan_t *plan = primitive->plan;
    void *lib_scratch = primitive->lib_scratch;
    scratch_guard_t *guard = &primitive->guard;
    std::shared_ptr<rt_entry_t> rt_hold;
    if (upd.kind == dnnl_matmul && upd.runtime) {
        const dnnl_status_t rs = resolve_runtime_matmul(
                const_cast<dnnl_primitive *>(primitive), args, rt_hold);
        if (rs != dnnl_success) return rs;
        if (!rt_hold) return dnnl_success; // a zero dim: nothing to compute
        concrete = rt_hold->pd.get();
        plan = rt_hold->plan;
        lib_scratch = rt_hold->scratch;
        guard = &rt_hold->guard;
    }
    const pd_impl_t &pd = *concrete;

    const int verbose = dnnl_amd_verbose_level();
    std::chrono::steady_clock::time_point t0;
    if (verbose >= 1) {
        (void)hipStreamSynchronize((hipStream_t)stream->hip_stream);
        t0 = std::chrono::steady_clock::now();
    }

    int st = QMM_OK;
    if (pd.kind == dnnl_matmul) {
        // zero-dim problems succeed without touching memory
        // (src/cpu/matmul/ref_matmul_int8.cpp:64-66)
        if (pd.src.has_zero_dim() || pd.wei.has_zero_dim()
                || pd.dst.has_zero_dim())
            return dnnl_success;
        qmm_matmul_args_t A;
        std::memset(&A, 0, sizeof(A));
        A.src = handle(DNNL_ARG_SRC);
        A.wei = handle(DNNL_ARG_WEIGHTS);
        A.bias = handle(DNNL_ARG_BIAS);
        A.dst = handle(DNNL_ARG_DST);
        const int qa[3] = {DNNL_ARG_SRC, DNNL_ARG_WEIGHTS, DNNL_ARG_DST};
        for (int i = 0; i < 3; i++) {
            A.scales[i] = handle(DNNL_ARG_ATTR_SCALES | qa[i]);
            A.zps[i] = handle(DNNL_ARG_ATTR_ZERO_POINTS | qa[i]);
            // a scales / zero-points memory was promised by the attributes
            // (src/cpu/cpu_primitive.hpp:41-44)
            if (pd.mm.scales[i].set && !A.scales[i]) return dnnl_invalid_arguments;
            if (pd.mm.zps[i].set && !A.zps[i]) return dnnl_invalid_arguments;
        }
        const auto &po = pd.attr.post_ops.entries;
        for (int i = 0; i < (int)po.size(); i++) {
            if (po[i].kind == dnnl_binary)
                A.po_arg[i] = handle(
                        DNNL_ARG_ATTR_MULTIPLE_POST_OP(i) | DNNL_ARG_SRC_1);
            else if (po[i].kind == dnnl_prelu)
                A.po_arg[i] = handle(
                        DNNL_ARG_ATTR_MULTIPLE_POST_OP(i) | DNNL_ARG_WEIGHTS);
        }
        A.scratch = pd.scratchpad.ndims ? handle(DNNL_ARG_SCRATCHPAD)
                                        : lib_scratch;
        scratch_order_t order(
                A.scratch && A.scratch == lib_scratch ? guard : nullptr,
                stream->hip_stream);
        st = qmm_matmul_launch(plan, &A, stream->hip_stream);
    } else if (pd.kind == kind_sdpa) {
        if (pd.dst.has_zero_dim()) return dnnl_success;
        qmm_sdpa_args_t A;
        std::memset(&A, 0, sizeof(A));
        A.q = handle(DNNL_ARG_QUERIES);
        A.k = handle(DNNL_ARG_KEYS);
        A.v = handle(DNNL_ARG_VALUES);
        A.dst = handle(DNNL_ARG_DST);
        A.mask = handle(DNNL_ARG_ATTN_MASK);
        A.scale = handle(DNNL_ARG_SCALE);
        A.k_scale = handle(DNNL_ARG_ATTR_SCALES | DNNL_ARG_KEYS);
        A.k_zp = handle(DNNL_ARG_ATTR_ZERO_POINTS | DNNL_ARG_KEYS);
        A.v_scale = handle(DNNL_ARG_ATTR_SCALES | DNNL_ARG_VALUES);
        A.v_zp = handle(DNNL_ARG_ATTR_ZERO_POINTS | DNNL_ARG_VALUES);
        A.scratch = pd.scratchpad.ndims ? handle(DNNL_ARG_SCRATCHPAD)
                                        : lib_scratch;
        scratch_order_t order(
                A.scratch && A.scratch == lib_scratch ? guard : nullptr,
                stream->hip_stream);
        st = qmm_sdpa_launch(&pd.sd, &A, stream->hip_stream);
    } else if (pd.kind == dnnl_softmax) {
        if (pd.src.has_zero_dim()) return dnnl_success;
        qmm_softmax_args_t A;
        std::memset(&A, 0, sizeof(A));
        A.src = handle(DNNL_ARG_SRC);
        A.dst = handle(DNNL_ARG_DST);
        A.src_scale = handle(DNNL_ARG_ATTR_SCALES | DNNL_ARG_SRC);
        A.dst_scale = handle(DNNL_ARG_ATTR_SCALES | DNNL_ARG_DST);
        st = qmm_softmax_launch(&pd.sm, &A, stream->hip_stream);
    } else {
        if (pd.src.has_zero_dim()) return dnnl_success;
        qmm_reorder_args_t A;
        std::memset(&A, 0, sizeof(A));
        A.src = handle(DNNL_ARG_FROM);
        A.dst = handle(DNNL_ARG_TO);
        A.src_scale = handle(DNNL_ARG_ATTR_SCALES | DNNL_ARG_SRC);
        A.dst_scale = handle(DNNL_ARG_ATTR_SCALES | DNNL_ARG_DST);
        A.src_zp = handle(DNNL_ARG_ATTR_ZERO_POINTS | DNNL_ARG_SRC);
        A.dst_zp = handle(DNNL_ARG_ATTR_ZERO_POINTS | DNNL_ARG_DST);
        st = qmm_reorder_launch(&pd.ro, &A, stream->hip_stream);
    }
    if (st != QMM_OK) {
        if (verbose >= 1)
            std::fprintf(stderr, "onednn_verbose,v1,primitive,error,gpu,%s,%s\n",
                    pd.impl_name.c_str(), qmm_last_error());
        return from_qmm(st);
    }
    if (verbose >= 1) {
        (void)hipStreamSynchronize((hipStream_t)stream->hip_stream);
        const double ms = std::chrono::duration<double, std::milli>(
                std::chrono::steady_clock::now() - t0)
                                  .count();
        if (pd.kind == kind_sdpa)
            std::printf("onednn_verbose,v1,primitive,exec,gpu,sdpa,%s,undef,"
                        "q:%s k:%s dst:%s,,,%s:%s,%g\n",
                    pd.impl_name.c_str(), dt_name(pd.src.data_type),
                    dt_name(pd.sdpa_k.data_type), dt_name(pd.dst.data_type),
                    dims_str(pd.src).c_str(), dims_str(pd.sdpa_k).c_str(), ms);
        else if (pd.kind == dnnl_softmax)
            std::printf("onednn_verbose,v1,primitive,exec,gpu,softmax,%s,"
                        "forward_inference,src:%s dst:%s,,axis:%d,%s,%g\n",
                    pd.impl_name.c_str(), dt_name(pd.src.data_type),
                    dt_name(pd.dst.data_type), pd.sm.axis,
                    dims_str(pd.src).c_str(), ms);
        else if (pd.kind == dnnl_matmul)
            std::printf("onednn_verbose,v1,primitive,exec,gpu,matmul,%s,"
                        "undef,src:%s wei:%s dst:%s,,,%s:%s,%g\n",
                    pd.impl_name.c_str(), dt_name(pd.src.data_type),
                    dt_name(pd.wei.data_type), dt_name(pd.dst.data_type),
                    dims_str(pd.src).c_str(), dims_str(pd.wei).c_str(), ms);
        else
            std::printf("onednn_verbose,v1,primitive,exec,gpu,reorder,%s,"
                        "undef,src:%s dst:%s,,,%s,%g\n",
                    pd.impl_name.c_str(), dt_name(pd.src.data_type),
                    dt_name(pd.dst.data_type), dims_str(pd.src).c_str(), ms);
        std::fflush(stdout);
    }
    return dnnl_success;
}

} // extern "C"
