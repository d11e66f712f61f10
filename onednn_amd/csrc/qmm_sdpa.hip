// hip:gfx950:sdpa_f16 -- scaled dot-product attention in one kernel:
//   dst = softmax(scale * Q x K + mask) x V
// (the reference's internal sdpa primitive: src/common/sdpa_types.hpp:38-80,
// semantics src/gpu/intel/ocl/ref_sdpa.cl:21-78; its test's gold path is the
// matmul -> softmax -> matmul chain, tests/gtests/internals/test_sdpa.cpp:893-
// 1043). Q, K, V, dst are f16 or bf16 (the kernels' BF flag; the text below
// says f16 for both); K and V may instead be an s8 / u8 cache with one scale
// (and zero point) per key, dequantized to the queries' type as the chain's
// reorder does: f16(scale * (x - zero_point)), in f32 arithmetic for bf16
// queries and for f32 scales / s32 zero points.
//
// The scores never leave the CU. A workgroup owns 128 queries of one head (four
// waves of 32) and walks the keys 32 at a time:
//   * the K tile and the V tile [32 keys][D] are staged in LDS once per
//     workgroup (requested one tile ahead, so a step does not wait for memory);
//   * S^T = K x Q^T on v_mfma_f32_16x16x32_f16 with the K rows as the first
//     operand: a lane then holds, for ONE query (lane % 16), eight of the 32
//     keys, so the row maximum and sum are per-lane values plus two cross-lane
//     steps, and the eight probabilities, packed to f16, ARE the second
//     operand of O^T += V^T x P^T -- no shuffle between the two products. The
//     32 keys enter that product in the order the lanes hold them (k index
//     8c + i <-> key 4c + i for i < 4, key 16 + 4c + i - 4 otherwise); V^T in
//     that order comes out of the row-major tile through the transposing LDS
//     read (ds_read_b64_tr_b16);
//   * online softmax in the base-2 domain: running maximum m and sum l per
//     query, the output accumulators rescaled by 2^(m_old - m_new).
// HBM traffic is Q, K, V in and dst out; the chain moves the f32 scores and
// the probabilities through HBM in between (34 x more bytes at 2048 keys).
#include <hip/hip_runtime.h>
#include <string.h>

#include <algorithm>
#include <atomic>

#include "qmm_device.hpp"
#include "qmm_hip.h"

namespace qmm {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

constexpr int SDPA_WAVES = 4;
constexpr int SDPA_QB = 2; // 16-query blocks per wave
constexpr int SDPA_QW = 16 * SDPA_QB; // queries per wave
constexpr int SDPA_QT = SDPA_QW * SDPA_WAVES; // queries per workgroup
constexpr int SDPA_KT = 32; // keys per tile
#ifndef SDPA_MIN_BLOCKS
#define SDPA_MIN_BLOCKS 2
#endif
typedef short v4s __attribute__((ext_vector_type(4)));
typedef __bf16 v8b __attribute__((ext_vector_type(8)));

// BF: the 16-bit type of Q, K, V and dst is bf16 (else f16). Operands travel
// as raw 16-byte vectors; only the MFMA and the conversions know the type.
template <bool BF>
QMM_D v4f mma16(const v8h &a, const v8h &b, const v4f &c) {
    if constexpr (BF)
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                __builtin_bit_cast(v8b, a), __builtin_bit_cast(v8b, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}
template <bool BF>
QMM_D _Float16 cvt16(float v) { // the bits of v in the 16-bit type, carried as _Float16
    if constexpr (BF)
        return __builtin_bit_cast(_Float16, (__bf16)v); // v_cvt_pk_bf16_f32
    else
        return (_Float16)v;
}

struct sdpa_strides_t {
    int64_t b0, b1, row; // two outer dims, then the row dim (elements)
};

struct sdpa_params_t {
    const uint16_t *Q;
    const void *K, *V;
    uint16_t *dst;
    const void *mask; // nullptr: none
    const void *scale; // nullptr: 1
    const void *k_scale, *k_zp, *v_scale, *v_zp; // per (kv batch, key)
    sdpa_strides_t q, k, v, o, m;
    int64_t m_col; // mask stride over keys (0 or 1)
    int32_t B0, B1; // outer dims of Q / dst
    int32_t kv_div0, kv_div1; // q batch index / div = kv batch index
    int64_t qz_b0, qz_b1; // scale / zero-point index = kb0 * qz_b0 + kb1 * qz_b1 + key
    int32_t Qn, S;
    int32_t scale_dt, mask_dt, invert_scale, causal;
    int32_t kv_dt; // the queries' type, or dt_s8 / dt_u8
    int32_t ks_dt, kz_dt, vs_dt, vz_dt;
    int32_t pair_halves; // the grid fits the chip at once: see the kernel
    // few queries (decode): the keys are cut into nsplit ranges of tps tiles
    int32_t nsplit, tps;
    int32_t fastq, bf; // f16 scales and 8-bit zero points: f16 dequantisation
    float *part; // [head][split][16 queries][D + 2]: O (unnormalised), m, l
};

// Lanes that differ only in their 16-lane row hold parts of one query. The two
// exchange steps (row r <-> r ^ 1, half <-> other half) as vector-ALU lane
// swaps: v_permlane16_swap returns (rows 0 0 2 2, rows 1 1 3 3) of its two
// inputs' rows, v_permlane32_swap (lower lower, upper upper) halves; with both
// inputs the same value the two results are the partners of a butterfly.
typedef unsigned v2u __attribute__((ext_vector_type(2)));
QMM_D float rows_max(float v) {
    unsigned u = f2u(v);
    const v2u a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    u = f2u(fmaxf(u2f(a.x), u2f(a.y)));
    const v2u b = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return fmaxf(u2f(b.x), u2f(b.y));
}
QMM_D float rows_sum(float v) {
    unsigned u = f2u(v);
    const v2u a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    u = f2u(u2f(a.x) + u2f(a.y));
    const v2u b = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return u2f(b.x) + u2f(b.y);
}

// the mask is f32 or one of the 16-bit types
QMM_D float ld_mask(int dt, const void *p, int64_t i) {
    if (dt == dt_f32) return ((const float *)p)[i];
    const uint16_t h = ((const uint16_t *)p)[i];
    return dt == dt_bf16 ? __uint_as_float((uint32_t)h << 16)
                         : (float)__builtin_bit_cast(_Float16, h);
}

// the cache's scales are f16 or f32, its zero points s8, u8 or s32
QMM_D float ld_scale(int dt, const void *p, int64_t i) {
    return dt == dt_f16 ? (float)((const _Float16 *)p)[i] : ((const float *)p)[i];
}
QMM_D float ld_zp(int dt, const void *p, int64_t i) {
    return dt == dt_s8  ? (float)((const int8_t *)p)[i]
            : dt == dt_u8 ? (float)((const uint8_t *)p)[i]
                          : (float)((const int32_t *)p)[i];
}

// Eight cache bytes -> eight f16 values scale * (x - zero_point), in f16
// arithmetic: byte b behind the exponent pattern 0x64 is the f16 number
// 1024 + b, (1024 + b) - (1024 + z) is exact (integers up to 2048 are f16
// numbers), and an f16 scale times that small integer has at most 20
// significant bits, so rounding the f16 product is the same single rounding as
// f16(f32 product): the values of the reference's dequantizing reorder, at 1.5
// instructions per element. `raw`: bytes with the sign bit already flipped for
// s8; zb: zero point (+ 128 for s8), within [0, 1023].
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
QMM_D uint4 dequant8_f16(uint32_t w0, uint32_t w1, float s1, float zb) {
    const h2 off = h2 {(_Float16)(1024.f + zb), (_Float16)(1024.f + zb)};
    const h2 sc = h2 {(_Float16)s1, (_Float16)s1};
    const uint32_t w[2] = {w0, w1};
    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const uint32_t m = __builtin_amdgcn_perm(
                0x64646464u, w[j >> 1], (j & 1) ? 0x04030402u : 0x04010400u);
        const h2 v = (__builtin_bit_cast(h2, m) - off) * sc;
        o[j] = __builtin_bit_cast(uint32_t, v);
    }
    return make_uint4(o[0], o[1], o[2], o[3]);
}

// QUANT: K / V are an 8-bit cache; MASKED: an explicit mask tensor is added
template <int DC, bool QUANT, bool MASKED, bool BF>
__global__ void __launch_bounds__(SDPA_WAVES * 64, SDPA_MIN_BLOCKS)
sdpa_f16_kernel(const sdpa_params_t p) {
    constexpr int D = 32 * DC;
    constexpr int DVB = D / 16;
    constexpr int K_PITCH = D * 2 + 16; // bytes
    __shared__ __attribute__((aligned(16))) uint8_t lds_k2[2][SDPA_KT * K_PITCH];
    // V rows 32 bytes further apart than K rows: eight consecutive rows then
    // start on eight different groups of 8 banks, which is what the 8-byte
    // transposing reads below touch per row
    constexpr int V_PITCH = D * 2 + 32;
    __shared__ __attribute__((aligned(16))) uint8_t lds_v2[2][SDPA_KT * V_PITCH];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, c = lane >> 4;
    const int b1 = blockIdx.x % p.B1, b0 = blockIdx.x / p.B1;
    const int kb0 = b0 / p.kv_div0, kb1 = b1 / p.kv_div1;
    // Under a causal mask the last query tiles walk the most keys. Workgroups
    // are dispatched heads first, query tiles from the last to the first, so
    // the long walks start early and the short ones fill the gaps. When the
    // whole grid is resident at once (two workgroups per CU) nothing is left
    // to fill gaps with: then the second half of the grid runs first to last
    // instead, so that workgroups half a grid apart, which share a CU, add up
    // to the same number of key tiles everywhere.
    int rank = blockIdx.y;
    const int nq = gridDim.y;
    if (p.pair_halves && rank >= nq / 2) rank = nq / 2 + (nq - 1 - rank);
    const int q_wg = (nq - 1 - rank) * SDPA_QT;
    const int q_wave = q_wg + wave * SDPA_QW;

    const uint16_t *Qb = p.Q + b0 * p.q.b0 + b1 * p.q.b1;
    const uint8_t *Kb8 = (const uint8_t *)p.K;
    const uint8_t *Vb8 = (const uint8_t *)p.V;
    const int64_t k_base = kb0 * p.k.b0 + kb1 * p.k.b1;
    const int64_t v_base = kb0 * p.v.b0 + kb1 * p.v.b1;
    const int64_t qz_base = kb0 * p.qz_b0 + kb1 * p.qz_b1; // scales / zps
    constexpr bool quant = QUANT;

    // ---- the wave's query fragments: lane (r, c) holds Q[q][32 dc + 8 c ..]
    v8h qf[SDPA_QB][DC];
#pragma unroll
    for (int qb = 0; qb < SDPA_QB; qb++) {
        const int q = min(q_wave + qb * 16 + r, p.Qn - 1);
#pragma unroll
        for (int dc = 0; dc < DC; dc++)
            qf[qb][dc] = *(const v8h *)(Qb + q * p.q.row + dc * 32 + c * 8);
    }
    float sc = 1.f;
    if (p.scale) {
        sc = load_float(p.scale_dt, p.scale, 0);
        if (p.invert_scale) sc = 1.f / sc;
    }
    constexpr float L2E = 1.44269504088896340736f;
    const float sc2 = sc * L2E;

    v4f oacc[SDPA_QB][DVB];
#pragma unroll
    for (int qb = 0; qb < SDPA_QB; qb++)
#pragma unroll
        for (int d = 0; d < DVB; d++) oacc[qb][d] = v4f {0.f, 0.f, 0.f, 0.f};
    float m_run[SDPA_QB], l_run[SDPA_QB];
#pragma unroll
    for (int qb = 0; qb < SDPA_QB; qb++) {
        m_run[qb] = -INFINITY;
        l_run[qb] = 0.f;
    }

    int n_tiles = (p.S + SDPA_KT - 1) / SDPA_KT;
    if (p.causal) {
        const int last_q = min(q_wg + SDPA_QT, p.Qn) - 1;
        n_tiles = min(n_tiles, last_q / SDPA_KT + 1);
    }
    const uint8_t *mask_b = nullptr;
    if (MASKED) {
        const size_t msz = p.mask_dt == dt_f32 ? 4 : 2;
        mask_b = (const uint8_t *)p.mask + (b0 * p.m.b0 + b1 * p.m.b1) * msz;
    }

    // ---- staging: a thread carries NS (key, 8-element chunk) pieces of a
    // tile from global memory to LDS. The pieces of tile kt + 1 are requested
    // before tile kt is multiplied and written to LDS after it, so a
    // workgroup's walk over the keys (up to S / 32 dependent steps) does not
    // pay a trip to memory per step.
    constexpr int PIECES = SDPA_KT * (D / 8);
    constexpr int NS = (PIECES + SDPA_WAVES * 64 - 1) / (SDPA_WAVES * 64);
    uint4 pk[NS], pv[NS]; // f16: 8 values each; 8-bit: x, y hold 8 values
    float pks[NS], pvs[NS], pkz[NS], pvz[NS];
    auto fetch = [&](int kt) {
#pragma unroll
        for (int n = 0; n < NS; n++) {
            const int i = min(tid + n * SDPA_WAVES * 64, PIECES - 1);
            const int kk = i / (D / 8), ch = i % (D / 8);
            const int key = min(kt * SDPA_KT + kk, p.S - 1); // clamped: zeroed below
            if (!quant) {
                pk[n] = *(const uint4 *)((const uint16_t *)Kb8 + k_base
                        + key * p.k.row + ch * 8);
                pv[n] = *(const uint4 *)((const uint16_t *)Vb8 + v_base
                        + key * p.v.row + ch * 8);
            } else {
                const uint2 kq = *(const uint2 *)(Kb8 + k_base + key * p.k.row
                        + ch * 8);
                const uint2 vq = *(const uint2 *)(Vb8 + v_base + key * p.v.row
                        + ch * 8);
                pk[n] = make_uint4(kq.x, kq.y, 0, 0);
                pv[n] = make_uint4(vq.x, vq.y, 0, 0);
                pks[n] = p.k_scale ? ld_scale(p.ks_dt, p.k_scale, qz_base + key)
                                   : 1.f;
                pvs[n] = p.v_scale ? ld_scale(p.vs_dt, p.v_scale, qz_base + key)
                                   : 1.f;
                pkz[n] = p.k_zp ? ld_zp(p.kz_dt, p.k_zp, qz_base + key) : 0.f;
                pvz[n] = p.v_zp ? ld_zp(p.vz_dt, p.v_zp, qz_base + key) : 0.f;
            }
        }
    };
    auto commit = [&](int kt) {
        uint8_t *lds_k = lds_k2[kt & 1], *lds_v = lds_v2[kt & 1];
#pragma unroll
        for (int n = 0; n < NS; n++) {
            const int i = tid + n * SDPA_WAVES * 64;
            if (i >= PIECES) break; // fewer pieces than threads
            const int kk = i / (D / 8), ch = i % (D / 8);
            uint4 kv = pk[n], vv = pv[n];
            if (quant) {
                // the cache's reorder: f16(scale * (x - zero_point))
                // s8 bytes are read as u8 after flipping the sign bit (x + 128),
                // and the 128 joins the zero point: (x + 128) - (zp + 128) is
                // the same exact difference, and unsigned bytes convert in one
                // instruction each
                const bool sgn = p.kv_dt == dt_s8;
                const uint32_t flip = sgn ? 0x80808080u : 0u;
                const float kzb = pkz[n] + (sgn ? 128.f : 0.f);
                const float vzb = pvz[n] + (sgn ? 128.f : 0.f);
                const uint32_t kw[2] = {pk[n].x ^ flip, pk[n].y ^ flip};
                const uint32_t vw[2] = {pv[n].x ^ flip, pv[n].y ^ flip};
                if (p.fastq) {
                    kv = dequant8_f16(kw[0], kw[1], pks[n], kzb);
                    vv = dequant8_f16(vw[0], vw[1], pvs[n], vzb);
                } else {
                uint32_t kh[8], vh[8];
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const float kf = (float)((kw[j >> 2] >> (8 * (j & 3))) & 0xff);
                    const float vf = (float)((vw[j >> 2] >> (8 * (j & 3))) & 0xff);
                    kh[j] = __builtin_bit_cast(
                            uint16_t, cvt16<BF>(pks[n] * (kf - kzb)));
                    vh[j] = __builtin_bit_cast(
                            uint16_t, cvt16<BF>(pvs[n] * (vf - vzb)));
                }
                kv = make_uint4(kh[0] | (kh[1] << 16), kh[2] | (kh[3] << 16),
                        kh[4] | (kh[5] << 16), kh[6] | (kh[7] << 16));
                vv = make_uint4(vh[0] | (vh[1] << 16), vh[2] | (vh[3] << 16),
                        vh[4] | (vh[5] << 16), vh[6] | (vh[7] << 16));
                }
            }
            if (kt * SDPA_KT + kk >= p.S) {
                // keys past the end: zero, so that probability 0 x V stays 0
                kv = make_uint4(0, 0, 0, 0);
                vv = make_uint4(0, 0, 0, 0);
            }
            *(uint4 *)(lds_k + kk * K_PITCH + ch * 16) = kv;
            *(uint4 *)(lds_v + kk * V_PITCH + ch * 16) = vv;
        }
    };

    // Two LDS buffers: while tile kt is multiplied out of one, tile kt + 1
    // (requested an iteration earlier) is written into the other between the
    // two products, and tile kt + 2 is requested. One barrier per tile.
    if (n_tiles > 0) {
        fetch(0);
        commit(0);
        if (n_tiles > 1) fetch(1);
    }
    __syncthreads();
    for (int kt = 0; kt < n_tiles; kt++) {
        const int key0 = kt * SDPA_KT;
        const uint8_t *lds_k = lds_k2[kt & 1], *lds_v = lds_v2[kt & 1];

        // ---- S^T = K x Q^T: st[qb][kb] register i = key 16 kb + 4 c + i
        v4f st[SDPA_QB][2];
#pragma unroll
        for (int qb = 0; qb < SDPA_QB; qb++)
#pragma unroll
            for (int kb = 0; kb < 2; kb++) st[qb][kb] = v4f {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int dc = 0; dc < DC; dc++) {
                const v8h a = *(const v8h *)(lds_k + (kb * 16 + r) * K_PITCH
                        + dc * 64 + c * 16);
#pragma unroll
                for (int qb = 0; qb < SDPA_QB; qb++)
                    st[qb][kb] = mma16<BF>(a, qf[qb][dc], st[qb][kb]);
            }

        // ---- scale, mask, online softmax (base 2), probabilities to f16.
        // Wave-uniform: does this tile need the per-key checks at all?
        const bool edge = key0 + SDPA_KT > p.S
                || (p.causal && key0 + SDPA_KT - 1 > q_wave);
        v8h pb[SDPA_QB];
        bool rescale = false;
        float alpha_q[SDPA_QB];
#pragma unroll
        for (int qb = 0; qb < SDPA_QB; qb++) {
            const int q = q_wave + qb * 16 + r;
            if (!MASKED && !edge && sc2 > 0.f) {
                // interior tile, nothing added to the scores: the maximum is
                // taken on the raw products and the scale rides in the
                // exponent's multiply-add (one instruction per score less)
                float mr = fmaxf(fmaxf(st[qb][0][0], st[qb][0][1]),
                        fmaxf(st[qb][0][2], st[qb][0][3]));
                mr = fmaxf(mr, fmaxf(fmaxf(st[qb][1][0], st[qb][1][1]),
                                       fmaxf(st[qb][1][2], st[qb][1][3])));
                const float m_new = fmaxf(m_run[qb], rows_max(mr) * sc2);
                const float alpha = __builtin_amdgcn_exp2f(m_run[qb] - m_new);
                rescale |= m_new != m_run[qb];
                alpha_q[qb] = alpha;
                m_run[qb] = m_new;
                float ls = 0.f;
                _Float16 ph[8];
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const float pv1 = __builtin_amdgcn_exp2f(
                            __builtin_fmaf(st[qb][i >> 2][i & 3], sc2, -m_new));
                    ls += pv1;
                    ph[i] = cvt16<BF>(pv1);
                }
                l_run[qb] = l_run[qb] * alpha + ls;
                pb[qb] = v8h {ph[0], ph[1], ph[2], ph[3], ph[4], ph[5], ph[6], ph[7]};
                continue;
            }
            float sv[8];
#pragma unroll
            for (int kb = 0; kb < 2; kb++)
#pragma unroll
                for (int i = 0; i < 4; i++)
                    sv[kb * 4 + i] = st[qb][kb][i] * sc2;
            if (MASKED) {
                // every load unconditional: positions past the ends re-read the
                // last row / key (they are overwritten or never stored)
                const int64_t mrow = (int64_t)min(q, p.Qn - 1) * p.m.row;
                float mv[8];
#pragma unroll
                for (int kb = 0; kb < 2; kb++)
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const int key = min(key0 + kb * 16 + 4 * c + i, p.S - 1);
                        const int64_t mo = mrow + key * p.m_col;
                        mv[kb * 4 + i] = ld_mask(p.mask_dt, mask_b, mo);
                    }
#pragma unroll
                for (int i = 0; i < 8; i++) sv[i] += L2E * mv[i];
            }
            if (edge) {
#pragma unroll
                for (int kb = 0; kb < 2; kb++)
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const int key = key0 + kb * 16 + 4 * c + i;
                        if (key >= p.S || (p.causal && key > q))
                            sv[kb * 4 + i] = -INFINITY;
                    }
            }
            float mt = sv[0];
#pragma unroll
            for (int i = 1; i < 8; i++) mt = fmaxf(mt, sv[i]);
            mt = rows_max(mt);
            const float m_new = fmaxf(m_run[qb], mt);
            // nothing but masked keys so far: keep everything at zero
            const float m_use = m_new == -INFINITY ? 0.f : m_new;
            const float alpha = __builtin_amdgcn_exp2f(m_run[qb] - m_use);
            rescale |= m_new != m_run[qb];
            alpha_q[qb] = alpha;
            m_run[qb] = m_new;
            float ls = 0.f;
            _Float16 ph[8];
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const float pv1 = __builtin_amdgcn_exp2f(sv[i] - m_use);
                ls += pv1;
                ph[i] = cvt16<BF>(pv1);
            }
            l_run[qb] = l_run[qb] * alpha + ls;
            pb[qb] = v8h {ph[0], ph[1], ph[2], ph[3], ph[4], ph[5], ph[6], ph[7]};
        }
        // the accumulators only move when some query's maximum did
        if (__builtin_amdgcn_ballot_w64(rescale)) {
#pragma unroll
            for (int qb = 0; qb < SDPA_QB; qb++)
#pragma unroll
                for (int d = 0; d < DVB; d++) oacc[qb][d] *= alpha_q[qb];
        }

        if (kt + 1 < n_tiles) {
            commit(kt + 1); // the other buffer: last read before the previous barrier
            if (kt + 2 < n_tiles) fetch(kt + 2);
        }

        // ---- O^T += V^T x P^T. The first operand is V^T [16 d][32 keys] from
        // the row-major tile: ds_read_b64_tr_b16 hands lane i of a 16-lane
        // group element (i & 3) of the 8-byte chunk that lane (i >> 2) + 4 t
        // of the group addressed, t = 0..3. With lane j addressing row
        // (key) 4 c + (j >> 2), columns d0 + 4 (j & 3) .. + 3, lane r receives
        // V[4 c + t][d0 + r]: its column of V for four keys. Two reads (keys
        // 4 c .. and 16 + 4 c ..) make the eight keys of its k slots.
#pragma unroll
        for (int d = 0; d < DVB; d++) {
            const uint8_t *va = lds_v + (4 * c + (r >> 2)) * V_PITCH
                    + (d * 16 + 4 * (r & 3)) * 2;
            const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (v4s __attribute__((address_space(3))) *)va);
            const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (v4s __attribute__((address_space(3))) *)(va + 16 * V_PITCH));
            typedef short v8s __attribute__((ext_vector_type(8)));
            const v8h a = __builtin_bit_cast(v8h,
                    v8s {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]});
#pragma unroll
            for (int qb = 0; qb < SDPA_QB; qb++)
                oacc[qb][d] = mma16<BF>(a, pb[qb], oacc[qb][d]);
        }
        __syncthreads();
    }

    // ---- normalise and store: register i of oacc[qb][d] is dst[q][16 d + 4 c + i]
    uint16_t *Ob = p.dst + b0 * p.o.b0 + b1 * p.o.b1;
#pragma unroll
    for (int qb = 0; qb < SDPA_QB; qb++) {
        const float l = rows_sum(l_run[qb]);
        const int q = q_wave + qb * 16 + r;
        if (q >= p.Qn) continue;
#pragma unroll
        for (int d = 0; d < DVB; d++) {
            uint16_t h[4];
#pragma unroll
            for (int i = 0; i < 4; i++)
                h[i] = __builtin_bit_cast(uint16_t, cvt16<BF>(oacc[qb][d][i] / l));
            *(uint2 *)(Ob + (int64_t)q * p.o.row + d * 16 + 4 * c) = make_uint2(
                    h[0] | ((uint32_t)h[1] << 16), h[2] | ((uint32_t)h[3] << 16));
        }
    }
}


// ---- few queries (at most 16 per head: the decode step) ----------------------
// One workgroup per (head, key range); its four waves take the range's key
// tiles in turn, each with its own running maximum, sum and accumulators and
// its own piece of LDS (the V tile it transposes): no barrier until the end,
// where wave 0 merges the four states. A launch is then heads x splits
// workgroups streaming K and V once, instead of one workgroup per head walking
// all keys. With more than one split the merged state goes to the scratchpad
// (unnormalised accumulators, maximum, sum per query) and sdpa_combine_kernel
// finishes.
template <int DC, bool QUANT, bool MASKED, bool BF>
__global__ void __launch_bounds__(SDPA_WAVES * 64)
sdpa_decode_kernel(const sdpa_params_t p) {
    constexpr int D = 32 * DC;
    constexpr int DVB = D / 16;
    constexpr int V_PITCH = D * 2 + 32;
    constexpr int ST = D + 2; // floats of one query's state
    __shared__ __attribute__((aligned(16))) uint8_t lds_v4[SDPA_WAVES][SDPA_KT * V_PITCH];
    __shared__ float lds_st[SDPA_WAVES][16 * ST];
    // a tile's 32 key scales and zero points of K and of V, per wave
    __shared__ float lds_q[SDPA_WAVES][4 * SDPA_KT];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, c = lane >> 4;
    const int head = blockIdx.x, split = blockIdx.y;
    const int b1 = head % p.B1, b0 = head / p.B1;
    const int kb0 = b0 / p.kv_div0, kb1 = b1 / p.kv_div1;
    const uint16_t *Qb = p.Q + b0 * p.q.b0 + b1 * p.q.b1;
    const uint8_t *Kb8 = (const uint8_t *)p.K, *Vb8 = (const uint8_t *)p.V;
    const int64_t k_base = kb0 * p.k.b0 + kb1 * p.k.b1;
    const int64_t v_base = kb0 * p.v.b0 + kb1 * p.v.b1;
    const int64_t qz_base = kb0 * p.qz_b0 + kb1 * p.qz_b1;
    uint8_t *lds_v = lds_v4[wave];

    const int q = r; // the single 16-query block; rows past Qn repeat the last
    v8h qf[DC];
#pragma unroll
    for (int dc = 0; dc < DC; dc++)
        qf[dc] = *(const v8h *)(Qb + (int64_t)min(q, p.Qn - 1) * p.q.row + dc * 32
                + c * 8);
    float sc = 1.f;
    if (p.scale) {
        sc = load_float(p.scale_dt, p.scale, 0);
        if (p.invert_scale) sc = 1.f / sc;
    }
    constexpr float L2E = 1.44269504088896340736f;
    const float sc2 = sc * L2E;
    const uint8_t *mask_b = nullptr;
    if (MASKED) {
        const size_t msz = p.mask_dt == dt_f32 ? 4 : 2;
        mask_b = (const uint8_t *)p.mask + (b0 * p.m.b0 + b1 * p.m.b1) * msz;
    }

    v4f oacc[DVB];
#pragma unroll
    for (int d = 0; d < DVB; d++) oacc[d] = v4f {0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;

    int n_tiles = (p.S + SDPA_KT - 1) / SDPA_KT;
    if (p.causal) n_tiles = min(n_tiles, (p.Qn - 1) / SDPA_KT + 1);
    const int t_begin = split * p.tps, t_end = min(n_tiles, t_begin + p.tps);

    // K fragments straight from memory in operand order (lane (r, c): key
    // 16 kb + r, 8 values at 32 dc + 8 c); V rows through the wave's LDS piece
    uint4 kr[2][DC], vr[D / 16];
    float qsz[2]; // lanes 0..31: K scale, zero point of key lane; 32..63: V's
    float *qz = lds_q[wave];
    auto fetch = [&](int kt) {
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
            const int key = min(kt * SDPA_KT + kb * 16 + r, p.S - 1);
#pragma unroll
            for (int dc = 0; dc < DC; dc++) {
                if (!QUANT) {
                    kr[kb][dc] = *(const uint4 *)((const uint16_t *)Kb8 + k_base
                            + key * p.k.row + dc * 32 + c * 8);
                } else {
                    const uint2 w = *(const uint2 *)(Kb8 + k_base + key * p.k.row
                            + dc * 32 + c * 8);
                    kr[kb][dc] = make_uint4(w.x, w.y, 0, 0);
                }
            }
        }
        if (QUANT) {
            // one scale and one zero point per lane: the tile's 32 keys, K's in
            // the lower half of the wave, V's in the upper
            const int key = min(kt * SDPA_KT + (lane & 31), p.S - 1);
            const bool up = lane >= 32;
            const void *sp = up ? p.v_scale : p.k_scale;
            const void *zp = up ? p.v_zp : p.k_zp;
            qsz[0] = sp ? ld_scale(up ? p.vs_dt : p.ks_dt, sp, qz_base + key) : 1.f;
            qsz[1] = zp ? ld_zp(up ? p.vz_dt : p.kz_dt, zp, qz_base + key) : 0.f;
        }
        // V: the tile's 8-element pieces in turn (piece i: key i / (D / 8), chunk
        // i % (D / 8)), lane l carries the pieces l, l + 64, ...
#pragma unroll
        for (int n = 0; n < D / 16; n++) {
            const int i = lane + 64 * n;
            const int kk = i / (D / 8), ch = i % (D / 8);
            const int key = min(kt * SDPA_KT + kk, p.S - 1);
            if (!QUANT) {
                vr[n] = *(const uint4 *)((const uint16_t *)Vb8 + v_base
                        + key * p.v.row + ch * 8);
            } else {
                const uint2 w = *(const uint2 *)(Vb8 + v_base + key * p.v.row
                        + ch * 8);
                vr[n] = make_uint4(w.x, w.y, 0, 0);
            }
        }
    };
    auto dequant8 = [&](const uint4 &raw, float s1, float z1) {
        const bool sgn = p.kv_dt == dt_s8;
        const uint32_t flip = sgn ? 0x80808080u : 0u;
        const float zb = z1 + (sgn ? 128.f : 0.f);
        const uint32_t w[2] = {raw.x ^ flip, raw.y ^ flip};
        if (p.fastq) return dequant8_f16(w[0], w[1], s1, zb);
        uint32_t h[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const float f = (float)((w[j >> 2] >> (8 * (j & 3))) & 0xff);
            h[j] = __builtin_bit_cast(uint16_t, cvt16<BF>(s1 * (f - zb)));
        }
        return make_uint4(h[0] | (h[1] << 16), h[2] | (h[3] << 16),
                h[4] | (h[5] << 16), h[6] | (h[7] << 16));
    };

    int kt = t_begin + wave;
    if (kt < t_end) fetch(kt);
    for (; kt < t_end; kt += SDPA_WAVES) {
        const int key0 = kt * SDPA_KT;
        // this tile's operands out of the request registers
        if (QUANT) {
            // [K scale | V scale | K zero point | V zero point] x 32 keys
            qz[lane] = qsz[0];
            qz[64 + lane] = qsz[1];
        }
        v8h ka[2][DC];
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int dc = 0; dc < DC; dc++) {
                uint4 w = QUANT ? dequant8(kr[kb][dc], qz[kb * 16 + r],
                                          qz[64 + kb * 16 + r])
                                : kr[kb][dc];
                if (key0 + kb * 16 + r >= p.S) w = make_uint4(0, 0, 0, 0);
                ka[kb][dc] = __builtin_bit_cast(v8h, w);
            }
#pragma unroll
        for (int n = 0; n < D / 16; n++) {
            const int i = lane + 64 * n;
            const int kk = i / (D / 8), ch = i % (D / 8);
            uint4 w = QUANT ? dequant8(vr[n], qz[32 + kk], qz[96 + kk]) : vr[n];
            if (key0 + kk >= p.S) w = make_uint4(0, 0, 0, 0);
            *(uint4 *)(lds_v + kk * V_PITCH + ch * 16) = w;
        }
        if (kt + SDPA_WAVES < t_end) fetch(kt + SDPA_WAVES);

        v4f st[2] = {v4f {0.f, 0.f, 0.f, 0.f}, v4f {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int dc = 0; dc < DC; dc++)
                st[kb] = mma16<BF>(ka[kb][dc], qf[dc], st[kb]);
        float sv[8];
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int i = 0; i < 4; i++) sv[kb * 4 + i] = st[kb][i] * sc2;
        if (MASKED) {
            const int64_t mrow = (int64_t)min(q, p.Qn - 1) * p.m.row;
#pragma unroll
            for (int kb = 0; kb < 2; kb++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int key = min(key0 + kb * 16 + 4 * c + i, p.S - 1);
                    const int64_t mo = mrow + key * p.m_col;
                    sv[kb * 4 + i] += L2E * ld_mask(p.mask_dt, mask_b, mo);
                }
        }
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int key = key0 + kb * 16 + 4 * c + i;
                if (key >= p.S || (p.causal && key > q)) sv[kb * 4 + i] = -INFINITY;
            }
        float mt = sv[0];
#pragma unroll
        for (int i = 1; i < 8; i++) mt = fmaxf(mt, sv[i]);
        mt = rows_max(mt);
        const float m_new = fmaxf(m_run, mt);
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);
        m_run = m_new;
        float ls = 0.f;
        _Float16 ph[8];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const float pv1 = __builtin_amdgcn_exp2f(sv[i] - m_use);
            ls += pv1;
            ph[i] = cvt16<BF>(pv1);
        }
        l_run = l_run * alpha + ls;
        const v8h pb = v8h {ph[0], ph[1], ph[2], ph[3], ph[4], ph[5], ph[6], ph[7]};
#pragma unroll
        for (int d = 0; d < DVB; d++) {
            oacc[d] *= alpha;
            const uint8_t *va = lds_v + (4 * c + (r >> 2)) * V_PITCH
                    + (d * 16 + 4 * (r & 3)) * 2;
            const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (v4s __attribute__((address_space(3))) *)va);
            const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (v4s __attribute__((address_space(3))) *)(va + 16 * V_PITCH));
            typedef short v8s __attribute__((ext_vector_type(8)));
            const v8h a = __builtin_bit_cast(v8h,
                    v8s {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]});
            oacc[d] = mma16<BF>(a, pb, oacc[d]);
        }
    }

    // ---- merge the four waves' states: query r, accumulator rows d = 16 dv + 4 c + i
    const float l_wave = rows_sum(l_run);
    float *mine = lds_st[wave] + r * ST;
#pragma unroll
    for (int d = 0; d < DVB; d++)
#pragma unroll
        for (int i = 0; i < 4; i++) mine[d * 16 + 4 * c + i] = oacc[d][i];
    if (c == 0) {
        mine[D] = m_run;
        mine[D + 1] = l_wave;
    }
    __syncthreads();
    if (wave != 0) return;
    float m_all = -INFINITY;
#pragma unroll
    for (int w = 0; w < SDPA_WAVES; w++) m_all = fmaxf(m_all, lds_st[w][r * ST + D]);
    const float m_use = m_all == -INFINITY ? 0.f : m_all;
    float l_all = 0.f, wgt[SDPA_WAVES];
#pragma unroll
    for (int w = 0; w < SDPA_WAVES; w++) {
        wgt[w] = __builtin_amdgcn_exp2f(lds_st[w][r * ST + D] - m_use);
        l_all += wgt[w] * lds_st[w][r * ST + D + 1];
    }
    if (q >= p.Qn) return;
    if (p.nsplit == 1) {
        uint16_t *Ob = p.dst + b0 * p.o.b0 + b1 * p.o.b1 + (int64_t)q * p.o.row;
#pragma unroll
        for (int d = 0; d < DVB; d++) {
            uint16_t h[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                float o = 0.f;
#pragma unroll
                for (int w = 0; w < SDPA_WAVES; w++)
                    o += wgt[w] * lds_st[w][r * ST + d * 16 + 4 * c + i];
                h[i] = __builtin_bit_cast(uint16_t, cvt16<BF>(o / l_all));
            }
            *(uint2 *)(Ob + d * 16 + 4 * c) = make_uint2(
                    h[0] | ((uint32_t)h[1] << 16), h[2] | ((uint32_t)h[3] << 16));
        }
    } else {
        float *out = p.part + (((int64_t)head * p.nsplit + split) * 16 + q) * ST;
#pragma unroll
        for (int d = 0; d < DVB; d++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                float o = 0.f;
#pragma unroll
                for (int w = 0; w < SDPA_WAVES; w++)
                    o += wgt[w] * lds_st[w][r * ST + d * 16 + 4 * c + i];
                out[d * 16 + 4 * c + i] = o;
            }
        if (c == 0) {
            out[D] = m_all;
            out[D + 1] = l_all;
        }
    }
}

// the splits' states of one (head, query) -> dst. The weights of the splits
// are formed once in LDS; a thread then owns one d (two of 256) and adds the splits'
// accumulators with independent loads.
constexpr int SDPA_MAX_SPLIT = 256;
__global__ void __launch_bounds__(128)
sdpa_combine_kernel(const sdpa_params_t p, const int D) {
    __shared__ float w_s[SDPA_MAX_SPLIT];
    __shared__ float red[2];
    const int head = blockIdx.x, q = blockIdx.y, t = threadIdx.x;
    const int b1 = head % p.B1, b0 = head / p.B1;
    const int ST = D + 2;
    const float *st = p.part + ((int64_t)head * p.nsplit * 16 + q) * ST;
    // every thread finds the maximum itself (at most 256 values from L2)
    float m_all = -INFINITY;
    for (int s1 = t; s1 < p.nsplit; s1 += 128)
        m_all = fmaxf(m_all, st[(int64_t)s1 * 16 * ST + D]);
#pragma unroll
    for (int o = 32; o; o >>= 1) m_all = fmaxf(m_all, __shfl_xor(m_all, o));
    if ((t & 63) == 0) red[t >> 6] = m_all;
    __syncthreads();
    m_all = fmaxf(red[0], red[1]);
    const float m_use = m_all == -INFINITY ? 0.f : m_all;
    float l_part = 0.f;
    for (int s1 = t; s1 < p.nsplit; s1 += 128) {
        const float *e = st + (int64_t)s1 * 16 * ST;
        const float w = __builtin_amdgcn_exp2f(e[D] - m_use);
        w_s[s1] = w;
        l_part += w * e[D + 1];
    }
#pragma unroll
    for (int o = 32; o; o >>= 1) l_part += __shfl_xor(l_part, o);
    __syncthreads(); // red[] has been read by everyone
    if ((t & 63) == 0) red[t >> 6] = l_part;
    __syncthreads();
    const float l_all = red[0] + red[1];
    for (int d = t; d < D; d += 128) { // head sizes up to 256: two per thread
        float o = 0.f;
#pragma unroll 8
        for (int s1 = 0; s1 < p.nsplit; s1++)
            o += w_s[s1] * st[(int64_t)s1 * 16 * ST + d];
        p.dst[b0 * p.o.b0 + b1 * p.o.b1 + (int64_t)q * p.o.row + d]
                = p.bf ? f32_to_bf16(o / l_all)
                       : __builtin_bit_cast(uint16_t, (_Float16)(o / l_all));
    }
}

// how a decode-sized problem is cut over the keys
struct sdpa_split_t {
    int nsplit, tps;
};
sdpa_split_t decode_split(int64_t heads, int64_t S, int64_t Qn, bool causal) {
    int64_t tiles = (S + SDPA_KT - 1) / SDPA_KT;
    if (causal) tiles = std::min<int64_t>(tiles, (Qn - 1) / SDPA_KT + 1);
    // enough workgroups to fill the chip twice, at least one tile per wave
    int64_t want = std::max<int64_t>(1, 512 / std::max<int64_t>(1, heads));
    int64_t tps = std::max<int64_t>(SDPA_WAVES, (tiles + want - 1) / want);
    tps = (tps + SDPA_WAVES - 1) / SDPA_WAVES * SDPA_WAVES;
    sdpa_split_t r;
    r.tps = (int)tps;
    r.nsplit = (int)std::max<int64_t>(1, (tiles + tps - 1) / tps);
    if (r.nsplit > SDPA_MAX_SPLIT) {
        tps = (tiles + SDPA_MAX_SPLIT - 1) / SDPA_MAX_SPLIT;
        tps = (tps + SDPA_WAVES - 1) / SDPA_WAVES * SDPA_WAVES;
        r.tps = (int)tps;
        r.nsplit = (int)((tiles + tps - 1) / tps);
    }
    return r;
}

// ---- host side ---------------------------------------------------------------
bool outer_strides(const qmm_tensor_t &t, sdpa_strides_t &s) {
    const int nd = t.ndims;
    if (nd < 2 || nd > 4) return false;
    s.row = t.strides[nd - 2];
    s.b1 = nd >= 3 ? t.strides[nd - 3] : 0;
    s.b0 = nd >= 4 ? t.strides[nd - 4] : 0;
    return true;
}

int64_t outer_dim(const qmm_tensor_t &t, int which) { // 0: outermost of two
    const int nd = t.ndims;
    if (which == 1) return nd >= 3 ? t.dims[nd - 3] : 1;
    return nd >= 4 ? t.dims[nd - 4] : 1;
}

bool quant_ok(const qmm_quant_t &q, bool scale) {
    if (!q.set) return true;
    if (scale) return q.dt == dt_f16 || q.dt == dt_f32;
    return q.dt == dt_s8 || q.dt == dt_u8 || q.dt == dt_s32;
}

bool supported(const qmm_sdpa_desc_t &d, sdpa_params_t *out) {
    const int nd = d.q.ndims;
    if (nd < 2 || nd > 4) return false;
    if (d.k.ndims != nd || d.v.ndims != nd || d.dst.ndims != nd) return false;
    if ((d.q.dt != dt_f16 && d.q.dt != dt_bf16) || d.dst.dt != d.q.dt) return false;
    if (d.k.dt != d.v.dt) return false;
    // K / V in the queries' type, or an 8-bit cache
    if (d.k.dt != d.q.dt && d.k.dt != dt_s8 && d.k.dt != dt_u8) return false;
    const int64_t Qn = d.q.dims[nd - 2], D = d.q.dims[nd - 1];
    const int64_t S = d.k.dims[nd - 1];
    if (d.k.dims[nd - 2] != D || d.v.dims[nd - 2] != S) return false;
    if (d.v.dims[nd - 1] != D) return false; // head size of V = head size of Q
    if (d.dst.dims[nd - 2] != Qn || d.dst.dims[nd - 1] != D) return false;
    // head sizes: 1, 2, 3, 4 or 8 chunks of 32
    if (D != 32 && D != 64 && D != 96 && D != 128 && D != 256) return false;
    if (Qn < 1 || S < 1 || Qn > (1 << 30) || S > (1 << 30)) return false;
    // innermost-contiguous rows: Q [q][d], K as the transposed view of a
    // [keys][d] cache, V [keys][d], dst [q][d]
    if (d.q.strides[nd - 1] != 1 || d.k.strides[nd - 2] != 1
            || d.v.strides[nd - 1] != 1 || d.dst.strides[nd - 1] != 1)
        return false;
    // 16-byte (f16) or 8-byte (8-bit) vector loads of 8 elements
    const int64_t al = 8;
    if (d.q.strides[nd - 2] % al || d.k.strides[nd - 1] % al
            || d.v.strides[nd - 2] % al || d.dst.strides[nd - 2] % 4)
        return false;
    sdpa_params_t p;
    ::memset(&p, 0, sizeof(p));
    p.B0 = (int32_t)outer_dim(d.q, 0);
    p.B1 = (int32_t)outer_dim(d.q, 1);
    if (outer_dim(d.dst, 0) != p.B0 || outer_dim(d.dst, 1) != p.B1) return false;
    // K / V batch dims: equal, or dividing the query's (grouped heads)
    const int64_t k0 = outer_dim(d.k, 0), k1 = outer_dim(d.k, 1);
    if (outer_dim(d.v, 0) != k0 || outer_dim(d.v, 1) != k1) return false;
    if (k0 < 1 || k1 < 1 || p.B0 % k0 || p.B1 % k1) return false;
    if (d.kv_head_number > 0 && nd >= 3 && d.kv_head_number != k1) return false;
    p.kv_div0 = (int32_t)(p.B0 / k0);
    p.kv_div1 = (int32_t)(p.B1 / k1);
    for (int i = 0; i < nd - 2; i++) {
        if (d.q.strides[i] % al || d.k.strides[i] % al || d.v.strides[i] % al
                || d.dst.strides[i] % 4)
            return false;
    }
    outer_strides(d.q, p.q);
    outer_strides(d.k, p.k);
    p.k.row = d.k.strides[nd - 1]; // one key to the next
    outer_strides(d.v, p.v);
    outer_strides(d.dst, p.o);
    if (d.mask.ndims) {
        if (d.mask.ndims != nd) return false;
        if (d.mask.dt != dt_f16 && d.mask.dt != dt_bf16 && d.mask.dt != dt_f32)
            return false;
        // each dim equal to the scores' or 1 (broadcast)
        const int64_t want[4] = {p.B0, p.B1, Qn, S};
        int64_t ms[4] = {0, 0, 0, 0};
        for (int i = 0; i < nd; i++) {
            const int64_t w = want[4 - nd + i];
            if (d.mask.dims[i] != w && d.mask.dims[i] != 1) return false;
            ms[4 - nd + i] = d.mask.dims[i] == 1 ? 0 : d.mask.strides[i];
        }
        p.m.b0 = ms[0];
        p.m.b1 = ms[1];
        p.m.row = ms[2];
        p.m_col = ms[3];
        p.mask_dt = d.mask.dt;
    }
    if (d.scale_dt != dt_undef && d.scale_dt != dt_f16 && d.scale_dt != dt_bf16
            && d.scale_dt != dt_f32)
        return false;
    // quantized cache: one scale / zero point per (batch, key), i.e. a mask
    // over the batch dims and the key dim with the head-size dim in one group
    const bool quant = d.k.dt != d.q.dt;
    for (const qmm_quant_t *q : {&d.k_scale, &d.k_zp, &d.v_scale, &d.v_zp})
        if (q->set && !quant) return false;
    if (!quant_ok(d.k_scale, true) || !quant_ok(d.v_scale, true)
            || !quant_ok(d.k_zp, false) || !quant_ok(d.v_zp, false))
        return false;
    if (quant) {
        // the last two dims both masked, the head-size dim in one group (K is
        // [.., D, S]: dim nd-2; V is [.., S, D]: dim nd-1); the batch dims
        // masked or not, alike in every entry
        const int last2 = 3 << (nd - 2);
        int batch_bits = -1;
        for (const qmm_quant_t *q : {&d.k_scale, &d.k_zp, &d.v_scale, &d.v_zp}) {
            if (!q->set) continue;
            if ((q->mask & last2) != last2 || (q->mask >> nd)) return false;
            const int bb = q->mask & ~last2;
            if (batch_bits >= 0 && bb != batch_bits) return false;
            batch_bits = bb;
        }
        for (const qmm_quant_t *q : {&d.k_scale, &d.k_zp})
            if (q->set && (q->g0 != D || q->g1 != 1)) return false;
        for (const qmm_quant_t *q : {&d.v_scale, &d.v_zp})
            if (q->set && (q->g0 != 1 || q->g1 != D)) return false;
        if (batch_bits < 0) batch_bits = 0;
        const bool m1 = nd >= 3 && ((batch_bits >> (nd - 3)) & 1);
        const bool m0 = nd >= 4 && ((batch_bits >> (nd - 4)) & 1);
        p.qz_b1 = m1 ? S : 0;
        p.qz_b0 = m0 ? (m1 ? k1 * S : S) : 0;
    }
    p.Qn = (int32_t)Qn;
    p.S = (int32_t)S;
    p.scale_dt = d.scale_dt;
    p.invert_scale = d.invert_scale;
    p.causal = d.causal;
    p.kv_dt = d.k.dt;
    p.bf = d.q.dt == dt_bf16;
    p.fastq = quant && d.q.dt == dt_f16
            && (!d.k_scale.set || d.k_scale.dt == dt_f16)
            && (!d.v_scale.set || d.v_scale.dt == dt_f16)
            && (!d.k_zp.set || d.k_zp.dt == dt_s8 || d.k_zp.dt == dt_u8)
            && (!d.v_zp.set || d.v_zp.dt == dt_s8 || d.v_zp.dt == dt_u8);
    p.ks_dt = d.k_scale.dt;
    p.kz_dt = d.k_zp.dt;
    p.vs_dt = d.v_scale.dt;
    p.vz_dt = d.v_zp.dt;
    if (out) *out = p;
    return true;
}

} // namespace
} // namespace qmm

using namespace qmm;

extern "C" {

int qmm_sdpa_supports(const qmm_sdpa_desc_t *desc) {
    if (!desc) return QMM_INVALID_ARGUMENTS;
    return supported(*desc, nullptr) ? QMM_OK : QMM_UNIMPLEMENTED;
}

const char *qmm_sdpa_impl_name(const qmm_sdpa_desc_t *desc) {
    if (!desc || !supported(*desc, nullptr)) return "";
    return desc->q.dt == dt_bf16 ? "hip:gfx950:sdpa_bf16" : "hip:gfx950:sdpa_f16";
}

size_t qmm_sdpa_scratch_size(const qmm_sdpa_desc_t *desc) {
    sdpa_params_t p;
    if (!desc || !supported(*desc, &p) || p.Qn > 16) return 0;
    const sdpa_split_t sp
            = decode_split((int64_t)p.B0 * p.B1, p.S, p.Qn, p.causal != 0);
    if (sp.nsplit <= 1) return 0;
    const int64_t D = desc->q.dims[desc->q.ndims - 1];
    return (size_t)p.B0 * p.B1 * sp.nsplit * 16 * (D + 2) * sizeof(float);
}

int qmm_sdpa_launch(const qmm_sdpa_desc_t *desc, const qmm_sdpa_args_t *args,
        void *hip_stream) {
    if (!desc || !args) return QMM_INVALID_ARGUMENTS;
    sdpa_params_t p;
    if (!supported(*desc, &p)) return QMM_UNIMPLEMENTED;
    if (!args->q || !args->k || !args->v || !args->dst)
        return QMM_INVALID_ARGUMENTS;
    if ((desc->mask.ndims && !args->mask)
            || (desc->scale_dt != dt_undef && !args->scale)
            || (desc->k_scale.set && !args->k_scale)
            || (desc->k_zp.set && !args->k_zp)
            || (desc->v_scale.set && !args->v_scale)
            || (desc->v_zp.set && !args->v_zp))
        return QMM_INVALID_ARGUMENTS;
    for (const void *ptr : {args->q, args->k, args->v, (const void *)args->dst})
        if ((uintptr_t)ptr & 15) return QMM_INVALID_ARGUMENTS;
    p.Q = (const uint16_t *)args->q;
    p.K = args->k;
    p.V = args->v;
    p.dst = (uint16_t *)args->dst;
    p.mask = desc->mask.ndims ? args->mask : nullptr;
    p.scale = desc->scale_dt != dt_undef ? args->scale : nullptr;
    p.k_scale = desc->k_scale.set ? args->k_scale : nullptr;
    p.k_zp = desc->k_zp.set ? args->k_zp : nullptr;
    p.v_scale = desc->v_scale.set ? args->v_scale : nullptr;
    p.v_zp = desc->v_zp.set ? args->v_zp : nullptr;
    const int D = (int)desc->q.dims[desc->q.ndims - 1];
    const bool qn = p.kv_dt != desc->q.dt, mk = p.mask != nullptr;
    const bool bf = p.bf != 0;
    if (p.Qn <= 16) {
        const sdpa_split_t sp
                = decode_split((int64_t)p.B0 * p.B1, p.S, p.Qn, p.causal != 0);
        p.nsplit = sp.nsplit;
        p.tps = sp.tps;
        p.part = (float *)args->scratch;
        if (p.nsplit > 1 && !p.part) return QMM_INVALID_ARGUMENTS;
        const dim3 dgrid((unsigned)(p.B0 * p.B1), (unsigned)p.nsplit);
        auto god = [&](auto kern) {
            hipLaunchKernelGGL(kern, dgrid, dim3(SDPA_WAVES * 64), 0,
                    (hipStream_t)hip_stream, p);
        };
        // template arguments from the run-time choices
#define SDPA_PICK(KERN, GO, DCV) \
    switch ((qn ? 4 : 0) | (bf ? 2 : 0) | (mk ? 1 : 0)) { \
        case 0: GO(KERN<DCV, false, false, false>); break; \
        case 1: GO(KERN<DCV, false, true, false>); break; \
        case 2: GO(KERN<DCV, false, false, true>); break; \
        case 3: GO(KERN<DCV, false, true, true>); break; \
        case 4: GO(KERN<DCV, true, false, false>); break; \
        case 5: GO(KERN<DCV, true, true, false>); break; \
        case 6: GO(KERN<DCV, true, false, true>); break; \
        case 7: GO(KERN<DCV, true, true, true>); break; \
        default: return QMM_UNIMPLEMENTED; \
    }
        switch (D) {
            case 32: SDPA_PICK(sdpa_decode_kernel, god, 1) break;
            case 64: SDPA_PICK(sdpa_decode_kernel, god, 2) break;
            case 96: SDPA_PICK(sdpa_decode_kernel, god, 3) break;
            case 128: SDPA_PICK(sdpa_decode_kernel, god, 4) break;
            case 256: SDPA_PICK(sdpa_decode_kernel, god, 8) break;
            default: return QMM_UNIMPLEMENTED;
        }
        if (p.nsplit > 1)
            hipLaunchKernelGGL(sdpa_combine_kernel,
                    dim3((unsigned)(p.B0 * p.B1), (unsigned)p.Qn), dim3(128), 0,
                    (hipStream_t)hip_stream, p, D);
        return hipGetLastError() == hipSuccess ? QMM_OK : QMM_RUNTIME_ERROR;
    }
    const dim3 grid((unsigned)(p.B0 * p.B1),
            (unsigned)((p.Qn + SDPA_QT - 1) / SDPA_QT));
    if (grid.y > 65535) return QMM_UNIMPLEMENTED;
    // compute units of the device (asked once; every MI355X has the same)
    static std::atomic<int> cu_count {0};
    int cus = cu_count.load(std::memory_order_relaxed);
    if (cus == 0) {
        int dev = 0;
        cus = 256;
        if (hipGetDevice(&dev) == hipSuccess)
            (void)hipDeviceGetAttribute(
                    &cus, hipDeviceAttributeMultiprocessorCount, dev);
        cu_count.store(cus, std::memory_order_relaxed);
    }
    p.pair_halves = p.causal && grid.y % 2 == 0
            && (int64_t)grid.x * grid.y <= (int64_t)SDPA_MIN_BLOCKS * cus;
    auto go = [&](auto kern) {
        hipLaunchKernelGGL(kern, grid, dim3(SDPA_WAVES * 64), 0,
                (hipStream_t)hip_stream, p);
    };
    switch (D) {
        case 32: SDPA_PICK(sdpa_f16_kernel, go, 1) break;
        case 64: SDPA_PICK(sdpa_f16_kernel, go, 2) break;
        case 96: SDPA_PICK(sdpa_f16_kernel, go, 3) break;
        case 128: SDPA_PICK(sdpa_f16_kernel, go, 4) break;
        case 256: SDPA_PICK(sdpa_f16_kernel, go, 8) break;
        default: return QMM_UNIMPLEMENTED;
    }
#undef SDPA_PICK
    return hipGetLastError() == hipSuccess ? QMM_OK : QMM_RUNTIME_ERROR;
}

} // extern "C"
