// hip:gfx950:generic -- the catch-all matmul implementation.
//
// One thread per destination element, looping over K exactly like the
// reference's scalar kernels, so every combination of the path's attributes
// (any strides up to 12 dims, batch broadcast, grouped scales / zero points on
// either operand, all post-ops, every dst type) has a GPU implementation whose
// result follows the reference operation for operation:
//   integer sources     src/cpu/matmul/ref_matmul_int8.cpp:154-261
//   float/fp8/decompress src/cpu/matmul/ref_matmul.cpp:130-233
// The integer path accumulates in s32 over each K group; an entry without
// explicit groups spans all of K.
//
// It is the last entry of the implementation list; the MFMA kernels in front
// of it take the shapes that matter for throughput.
#include "qmm_device.hpp"
#include "qmm_plan.hpp"

namespace qmm {

QMM_D int64_t tensor_off(const qmm_tensor_t &t, const int64_t *idx) {
    int64_t o = 0;
    for (int d = 0; d < t.ndims; d++)
        o += idx[d] * t.strides[d];
    return o;
}

QMM_D int64_t quant_off(const generic_quant_t &q, const int64_t *idx, int nd) {
    if (!q.indexed) return 0;
    int64_t o = 0;
    for (int d = 0; d < nd; d++) {
        int64_t i = idx[d];
        if (d == nd - 1) i /= q.g1;
        if (d == nd - 2) i /= q.g0;
        o += i * q.strides[d]; // stride 0 on masked-out dims
    }
    return o;
}

QMM_D float generic_post_ops(const generic_params_t &P,
        const qmm_matmul_args_t &A, float res, float dst_val,
        const int64_t *didx) {
    const qmm_matmul_desc_t &D = P.desc;
    const int nd = D.dst.ndims;
    for (int i = 0; i < D.npo; i++) {
        const qmm_postop_t &e = D.po[i];
        if (e.kind == pk_sum) {
            res += e.scale * (dst_val - (float)e.zero_point);
        } else if (e.kind == pk_eltwise) {
            res = eltwise_fwd(e.alg, res, e.alpha, e.beta) * e.scale;
        } else if (e.kind == pk_binary) {
            // broadcast where the operand's dim differs from dst's
            // (src/cpu/primitive_attr_postops.cpp:238-246)
            int64_t o = 0;
            for (int d = 0; d < nd; d++)
                if (e.src1.dims[d] == D.dst.dims[d])
                    o += didx[d] * e.src1.strides[d];
            res = binary_op(e.alg, res, load_float(e.src1.dt, A.po_arg[i], o));
        } else if (e.kind == pk_prelu) {
            if (res >= 0) continue;
            int64_t o = 0;
            for (int d = 0; d < nd; d++)
                if (e.mask & (1 << d)) o += didx[d] * e.src1.strides[d];
            res = ((const float *)A.po_arg[i])[o] * res;
        }
    }
    return res;
}

__global__ void __launch_bounds__(256)
matmul_generic_kernel(const generic_params_t *__restrict__ Pp,
        qmm_matmul_args_t A) {
    const generic_params_t &P = *Pp;
    const qmm_matmul_desc_t &D = P.desc;
    const int nd = D.dst.ndims;
    const int64_t total = P.batch * P.M * P.N;
    for (int64_t l = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; l < total;
            l += (int64_t)gridDim.x * blockDim.x) {
        int64_t didx[QMM_MAX_NDIMS], sidx[QMM_MAX_NDIMS], widx[QMM_MAX_NDIMS];
        {
            int64_t r = l;
            for (int d = nd - 1; d >= 0; d--) {
                didx[d] = r % D.dst.dims[d];
                r /= D.dst.dims[d];
            }
        }
        for (int d = 0; d < nd; d++) {
            sidx[d] = (P.src_mask >> d) & 1 ? didx[d] : 0;
            widx[d] = (P.wei_mask >> d) & 1 ? didx[d] : 0;
        }
        const int64_t m = didx[nd - 2], n = didx[nd - 1];
        sidx[nd - 2] = m;
        widx[nd - 1] = n;

        float d = 0.f;
        if (P.int_path) {
            for (int64_t g = 0; g < P.ngroups_k; g++) {
                int32_t acc = 0;
                for (int64_t k = g * P.group_k; k < (g + 1) * P.group_k; k++) {
                    sidx[nd - 1] = k;
                    widx[nd - 2] = k;
                    int s = load_int(D.src.dt, A.src, tensor_off(D.src, sidx));
                    int w = load_int(D.wei.dt, A.wei, tensor_off(D.wei, widx));
                    if (D.zps[QMM_SRC].set)
                        s -= load_int(D.zps[QMM_SRC].dt, A.zps[QMM_SRC],
                                quant_off(P.q_src_zp, sidx, nd));
                    if (D.zps[QMM_WEI].set)
                        w -= load_int(D.zps[QMM_WEI].dt, A.zps[QMM_WEI],
                                quant_off(P.q_wei_zp, widx, nd));
                    acc = (int32_t)((uint32_t)acc + (uint32_t)(s * w));
                }
                float acc_f = (float)acc;
                if (D.scales[QMM_SRC].set)
                    acc_f *= load_float(D.scales[QMM_SRC].dt, A.scales[QMM_SRC],
                            quant_off(P.q_src_scale, sidx, nd));
                if (D.scales[QMM_WEI].set)
                    acc_f *= load_float(D.scales[QMM_WEI].dt, A.scales[QMM_WEI],
                            quant_off(P.q_wei_scale, widx, nd));
                d += acc_f;
            }
        } else {
            float acc = 0.f;
            for (int64_t k = 0; k < P.K; k++) {
                sidx[nd - 1] = k;
                widx[nd - 2] = k;
                const float s = load_float(
                        D.src.dt, A.src, tensor_off(D.src, sidx));
                float w = load_float(D.wei.dt, A.wei, tensor_off(D.wei, widx));
                if (P.decompress) {
                    if (D.zps[QMM_WEI].set)
                        w -= (float)load_int(D.zps[QMM_WEI].dt, A.zps[QMM_WEI],
                                quant_off(P.q_wei_zp, widx, nd));
                    if (D.scales[QMM_WEI].set)
                        w *= load_float(D.scales[QMM_WEI].dt,
                                A.scales[QMM_WEI],
                                quant_off(P.q_wei_scale, widx, nd));
                }
                acc += s * w;
            }
            d = acc;
            if (D.scales[QMM_SRC].set)
                d *= load_float(D.scales[QMM_SRC].dt, A.scales[QMM_SRC], 0);
            if (D.scales[QMM_WEI].set && !P.decompress)
                d *= load_float(D.scales[QMM_WEI].dt, A.scales[QMM_WEI],
                        P.q_wei_scale.indexed ? P.wei_scale_stride_n * n : 0);
        }
        if (D.bias.ndims) {
            int64_t o = 0;
            for (int dd = 0; dd < nd; dd++)
                if ((P.bia_mask >> dd) & 1) o += didx[dd] * D.bias.strides[dd];
            d += load_float(D.bias.dt, A.bias, o);
        }
        const int64_t dst_off = tensor_off(D.dst, didx);
        if (D.npo) {
            const float dst_val = P.has_sum
                    ? load_float(P.sum_dt, A.dst, dst_off)
                    : 0.f;
            d = generic_post_ops(P, A, d, dst_val, didx);
        }
        if (D.scales[QMM_DST].set) {
            // one value: times its reciprocal (src/cpu/matmul/ref_matmul.cpp:
            // 208); masked over M and / or N (GPU engines only,
            // src/common/matmul.cpp:150-154): divided by the element's entry
            // of a dense [M or 1][N or 1] buffer
            // (src/gpu/intel/ocl/ref_matmul.cl:239-245)
            const int mask = D.scales[QMM_DST].mask;
            if (mask == 0) {
                d *= 1.f
                        / load_float(D.scales[QMM_DST].dt, A.scales[QMM_DST], 0);
            } else {
                const bool per_m = (mask >> (nd - 2)) & 1;
                const bool per_n = (mask >> (nd - 1)) & 1;
                const int64_t i = (per_m ? didx[nd - 2] * (per_n ? P.N : 1) : 0)
                        + (per_n ? n : 0);
                d /= load_float(D.scales[QMM_DST].dt, A.scales[QMM_DST], i);
            }
        }
        if (D.zps[QMM_DST].set)
            d += (float)((const int32_t *)A.zps[QMM_DST])[P.dst_zp_mult * n];
        store_float(D.dst.dt, d, A.dst, dst_off);
    }
}

// ---------------------------------------------------------------------------
// Generic reorder between plain strided tensors with optional scales and zero
// points: dst = sat_round(src_scale * (src - src_zp) / dst_scale + dst_zp)
// (src/cpu/reorder/simple_reorder.hpp:2500-2640). One thread per destination
// BYTE so that two 4-bit results sharing a byte are written by one thread.
__global__ void __launch_bounds__(256)
reorder_generic_kernel(const generic_reorder_params_t P, qmm_reorder_args_t A) {
    const qmm_reorder_desc_t &D = P.desc;
    const int nd = D.src.ndims;
    const bool dst4 = D.dst.dt == dt_s4 || D.dst.dt == dt_u4;
    // 4-bit destinations: a thread owns a pair of neighbours along the
    // innermost (stride 1) destination dim `pd`, which has an even extent
    const int64_t pairs = dst4 ? P.nelems / 2 : P.nelems;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < pairs;
            t += (int64_t)gridDim.x * blockDim.x) {
        uint8_t packed = 0;
        const int cnt = dst4 ? 2 : 1;
        int64_t o_first = 0;
        for (int h = 0; h < cnt; h++) {
            // logical index: iterate dims with `pd` fastest for 4-bit dst
            int64_t idx[QMM_MAX_NDIMS];
            int64_t r = dst4 ? t * 2 + h : t;
            if (dst4) {
                idx[P.pair_dim] = r % D.dst.dims[P.pair_dim];
                r /= D.dst.dims[P.pair_dim];
            }
            for (int d = nd - 1; d >= 0; d--) {
                if (dst4 && d == P.pair_dim) continue;
                idx[d] = r % D.dst.dims[d];
                r /= D.dst.dims[d];
            }
            float src_scale = 1.f, dst_scale = 1.f;
            if (D.src_scale.set)
                src_scale = load_float(D.src_scale.dt, A.src_scale,
                        quant_off(P.q_src_scale, idx, nd));
            if (D.dst_scale.set)
                dst_scale = 1.f
                        / load_float(D.dst_scale.dt, A.dst_scale,
                                quant_off(P.q_dst_scale, idx, nd));
            int src_zp = 0;
            if (D.src_zp.set)
                src_zp = (int)load_float(D.src_zp.dt, A.src_zp,
                        quant_off(P.q_src_zp, idx, nd));
            const float dst_zp
                    = D.dst_zp.set ? (float)((const int32_t *)A.dst_zp)[0] : 0.f;
            const float in
                    = load_float(D.src.dt, A.src, tensor_off(D.src, idx));
            float d = src_scale * (in - (float)src_zp);
            d = d * dst_scale + dst_zp;
            const int64_t o = tensor_off(D.dst, idx);
            if (!dst4) {
                store_float(D.dst.dt, d, A.dst, o);
            } else {
                int v = D.dst.dt == dt_u4 ? round_sat(d, 0.f, 15.f)
                                          : round_sat(d, -8.f, 7.f);
                if (h == 0) o_first = o;
                packed |= (uint8_t)((v & 0xf) << (4 * (int)(o & 1)));
            }
        }
        if (dst4) ((uint8_t *)A.dst)[o_first >> 1] = packed;
    }
}

void launch_matmul_generic(const generic_params_t *dev_params,
        const generic_params_t &host_params, const qmm_matmul_args_t &args,
        hipStream_t stream) {
    const int64_t total = host_params.batch * host_params.M * host_params.N;
    if (total == 0) return;
    int64_t blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(matmul_generic_kernel, dim3((unsigned)blocks), dim3(256),
            0, stream, dev_params, args);
}

void launch_reorder_generic(const generic_reorder_params_t &params,
        const qmm_reorder_args_t &args, hipStream_t stream) {
    if (params.nelems == 0) return;
    int64_t blocks = (params.nelems + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(reorder_generic_kernel, dim3((unsigned)blocks),
            dim3(256), 0, stream, params, args);
}

} // namespace qmm
