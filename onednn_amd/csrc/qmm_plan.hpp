// Host/device parameter blocks of the kernels and the plan object behind
// qmm_matmul_plan_create(). Shared by the .hip kernels and the host dispatch.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>

#include "qmm_device.hpp"
#include "qmm_hip.h"

namespace qmm {

// Raises a kernel's dynamic LDS limit once per kernel; safe to call from
// several host threads that launch concurrently.
inline void ensure_dynamic_lds(const void *kern, int bytes) {
    static std::mutex mu;
    static const void *seen[1024]; // (far more than the library has kernels)
    static int n = 0;
    std::lock_guard<std::mutex> lock(mu);
    for (int i = 0; i < n; i++)
        if (seen[i] == kern) return;
    (void)hipFuncSetAttribute(
            kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (n < 1024) seen[n++] = kern;
}

// A scales / zero-points buffer as the generic kernels index it: dense
// row-major over the masked dims, last two dims divided by the groups
// (src/cpu/matmul/matmul_utils.hpp:156-196). strides[d] == 0 where the mask
// bit is clear.
struct generic_quant_t {
    int32_t indexed; // 0: single element at offset 0
    int32_t pad_;
    int64_t g0, g1;
    int64_t strides[QMM_MAX_NDIMS];
    int64_t nelems;
};

struct generic_params_t {
    qmm_matmul_desc_t desc;
    int64_t M, N, K, batch;
    int32_t src_mask, wei_mask, bia_mask; // dims equal to dst's
    int32_t int_path, decompress, has_sum, sum_dt, dst_zp_mult;
    int64_t ngroups_k, group_k;
    int64_t wei_scale_stride_n;
    generic_quant_t q_src_scale, q_wei_scale, q_src_zp, q_wei_zp;
};

struct generic_reorder_params_t {
    qmm_reorder_desc_t desc;
    int64_t nelems;
    int32_t pair_dim; // 4-bit dst: the stride-1 dim
    int32_t pad_;
    generic_quant_t q_src_scale, q_dst_scale, q_src_zp;
};

// ---- packed layouts -------------------------------------------------------
// QMM_LAYOUT_MFMA_B8: byte offset of element (k, n) inside one batch slice.
struct b8_geom_t {
    int64_t K, N, Kpad, Npad, kb32, nb32;
    int64_t batch_bytes; // data bytes per batch slice
    int64_t colsum_off; // byte offset of the s32 column sums (all batches)
    int64_t total_bytes;
};
QMM_HD int64_t round_up(int64_t a, int64_t b) { return (a + b - 1) / b * b; }
QMM_HD b8_geom_t b8_geom(int64_t batch, int64_t K, int64_t N) {
    b8_geom_t g;
    g.K = K;
    g.N = N;
    g.Kpad = round_up(K, 128);
    g.Npad = round_up(N, 32);
    g.kb32 = g.Kpad / 32;
    g.nb32 = g.Npad / 32;
    g.batch_bytes = g.Kpad * g.Npad;
    g.colsum_off = round_up(batch * g.batch_bytes, 256);
    g.total_bytes = g.colsum_off + batch * g.Npad * 4;
    return g;
}
QMM_HD int64_t b8_offset(const b8_geom_t &g, int64_t k, int64_t n) {
    const int64_t lane = 32 * ((k % 32) / 16) + (n % 32);
    return (((n / 32) * g.kb32 + k / 32) * 64 + lane) * 16 + (k % 16);
}

// QMM_LAYOUT_MFMA_W4: nibble index of element (k, n) inside one batch slice.
struct w4_geom_t {
    int64_t K, N, Kpad, Npad, kg128, nb16;
    int64_t batch_bytes, total_bytes;
};
QMM_HD w4_geom_t w4_geom(int64_t batch, int64_t K, int64_t N) {
    w4_geom_t g;
    g.K = K;
    g.N = N;
    g.Kpad = round_up(K, 128);
    g.Npad = round_up(N, 16);
    g.kg128 = g.Kpad / 128;
    g.nb16 = g.Npad / 16;
    g.batch_bytes = g.Kpad * g.Npad / 2;
    g.total_bytes = batch * g.batch_bytes;
    return g;
}
// One 16-column x 128-k tile is 1024 bytes = 64 lanes x 4 dwords. Lane
// 16*c + n%16 holds, in dword s, the eight values k = 128*g + 32*s + 8*c + j;
// value j sits in the nibble at bit 4*p with p = j/2 + 4*(j%2), so that
// (dword >> 4*i) & 0x000F000F yields the pair (j = 2i, j = 2i+1) in the low
// and high half-words.
QMM_HD int64_t w4_nibble_index(const w4_geom_t &g, int64_t k, int64_t n) {
    const int64_t tile = (n / 16) * g.kg128 + k / 128;
    const int64_t kk = k % 128;
    const int64_t s = kk / 32, c = (kk % 32) / 8, j = kk % 8;
    const int64_t lane = 16 * c + (n % 16);
    const int64_t p = j / 2 + 4 * (j % 2);
    return ((tile * 64 + lane) * 4 + s) * 8 + p;
}

// QMM_LAYOUT_MFMA_W4K64: nibble index of element (k, n) inside one batch slice.
struct w4k_geom_t {
    int64_t K, N, Kpad, Npad, kt64, nb32;
    int64_t batch_bytes, total_bytes;
};
QMM_HD w4k_geom_t w4k_geom(int64_t batch, int64_t K, int64_t N) {
    w4k_geom_t g;
    g.K = K;
    g.N = N;
    g.Kpad = round_up(K, 64);
    g.Npad = round_up(N, 32);
    g.kt64 = g.Kpad / 64;
    g.nb32 = g.Npad / 32;
    g.batch_bytes = g.Kpad * g.Npad / 2;
    g.total_bytes = batch * g.batch_bytes;
    return g;
}
QMM_HD int64_t w4k_nibble_index(const w4k_geom_t &g, int64_t k, int64_t n) {
    const int64_t tile = (n / 32) * g.kt64 + k / 64;
    const int64_t kk = k % 64;
    const int64_t i = kk / 32, h = (kk % 32) / 16, q = (kk % 16) / 8, j = kk % 8;
    const int64_t lane = 32 * h + (n % 32);
    const int64_t p = 2 * (j % 4) + j / 4;
    return ((tile * 64 + lane) * 4 + 2 * i + q) * 8 + p;
}

// ---- MFMA GEMM (int8 / fp8) -----------------------------------------------
enum {
    GEMM_MFMA32 = 1,
    GEMM_SKIP_EPILOGUE = 2,
    GEMM_STAMPS = 4,
    GEMM_TWO_PER_CU = 8,
    GEMM_ONE_PER_CU = 16,
    // the int8 256 x 256 kernel on 16 x 16 MFMAs: one workgroup per tile
    // instead of one per CU walking its tiles (a measurement switch)
    GEMM_NOT_PERSISTENT = 32,
    // the persistent int8 kernel with all its workgroups starting together
    // (a measurement switch)
    GEMM_NO_STAGGER = 64
};

struct gemm_params_t {
    const uint8_t *A; // src, rows K-contiguous
    int64_t lda, a_sb; // bytes
    const uint8_t *B; // QMM_LAYOUT_MFMA_B8
    int64_t b_sb; // bytes between batch slices (0: broadcast)
    const int32_t *colsum; // [batch][Npad] or nullptr
    int64_t colsum_sb; // elements
    const void *src_zp; // single value or nullptr
    int32_t src_zp_dt;
    int32_t a_is_u8;
    int32_t M, N, K, batch;
    int32_t kb32; // K blocks of 32 in the packed weights
    int32_t nb32;
    int32_t tiles_m, tiles_n;
    int32_t a_preflipped; // u8 source already rewritten as s8 (x ^ 0x80)
    // weights zero points / u8 weights (stored as s8 = u8 - 128): the zero
    // point of the stored weights is zp[n * wei_zp_sn] - w_off, applied through
    // rowsum (see rowsum_b8_kernel); nullptr rowsum: neither
    const void *wei_zp; // nullptr: 0
    int32_t wei_zp_dt, wei_zp_sn, w_off;
    // plan-level switches (qmm_hip.h, kernel-selection overrides and
    // QMM_MEASURE): GEMM_MFMA32 keeps the 256 x 256 loops on 32 x 32 MFMAs;
    // GEMM_SKIP_EPILOGUE ends the 256 x 256 kernels after the main loop (nothing
    // is stored); GEMM_STAMPS makes them record time stamps per block tile;
    // GEMM_TWO_PER_CU / GEMM_ONE_PER_CU force the int8 tiling (256 x 128 with two
    // workgroups per CU / 256 x 256 with one) that is otherwise chosen by shape
    int32_t switches;
    const int32_t *rowsum; // [batch][M]
    epilogue_t ep;
};

// ---- plain 16-bit batched matmul (qmm_gemm_f16.hip) ---------------------------
struct gemm16_params_t {
    const uint16_t *A, *B; // src rows K-contiguous, weights rows N-contiguous
    int64_t lda, a_sb, ldb, b_sb; // elements
    int32_t M, N, K, batch;
    int32_t bf; // bf16 (else f16)
    int32_t a_vec, b_vec; // elements per aligned load the rows allow: 8, 4, 2 or 1
    int32_t tile; // 0: by problem size; 1: 64 x 64 tiles; 2: 128 x 128 tiles; 3: the walking kernel
    epilogue_t ep;
};

// ---- decode kernel (4-bit / 8-bit weights, 16-bit activations) -------------
struct gemv_params_t {
    const uint16_t *A; // activations [M][K], bf16 or f16
    int64_t lda; // elements
    const uint8_t *B; // QMM_LAYOUT_MFMA_W4
    const void *scales; // [K/gs][N]
    const void *zps; // [K/gz][N] or single or nullptr
    int32_t scale_dt, zp_dt;
    int32_t gs, gz; // K group sizes (multiples of 32); gz == 0: single zp
    int32_t scale_per_n, zp_per_n; // 0: broadcast over n
    int32_t M, N, K;
    int32_t kg128, nb16;
    int32_t wei_signed; // s4 weights
    int32_t act_f16; // activations are f16 (else bf16)
    int32_t m0; // first row handled by this launch
    // fast variant: K groups are 128 << shift wide (host-checked); -1: single
    int32_t gs_shift, gz_shift;
    int32_t w8; // 8-bit weights, QMM_LAYOUT_MFMA_W8 (fast variant only)
    epilogue_t ep;
};

// ---- s8 activations x 4-bit weights, K-grouped scales on both sides ---------
// The scale / zero-point buffers are rewritten per launch into the scratchpad,
// transposed to [group][row or column], by w4a8_prep_kernel.
struct w4a8_params_t {
    const uint8_t *A; // s8 rows, K-contiguous
    int64_t lda; // bytes
    const uint8_t *B; // QMM_LAYOUT_MFMA_W4K64
    const float *ssT; // [ng][Mpad] source scales
    const int32_t *rsT; // [ng][Mpad] source row sums per group, or nullptr
    const float *swT; // [ng][Npad] weights scales / 16
    const int32_t *zwT; // [ng][Npad] -16 * (zero point - offset), or nullptr
    // source zero points / u8 source (both or neither): [ng][Mpad] the zero
    // point of the source taken as s8, [ng][Npad] -16 * (column sum of the
    // stored nibbles - group * (zero point - offset))
    const int32_t *zsT, *c2T;
    int32_t M, N, K;
    int32_t Mpad, Npad;
    int32_t kt64, nb32;
    int32_t tpg; // 64-k tiles per group; 0: groups of 32 k, two per tile
    int32_t ng;
    int32_t tiles_m, tiles_n;
    uint32_t a_flip; // 0x80808080 for a u8 source (read as s8 = u8 - 128)
    epilogue_t ep;
};

struct w4a8_prep_t {
    const uint8_t *A;
    int64_t lda;
    const void *ss, *sw, *zw; // nullptr: default value
    int32_t ss_dt, sw_dt, zw_dt;
    int32_t w_off; // 8 for u4 weights (stored as u - 8)
    int64_t ss_sm, ss_sk, sw_sk, sw_sn, zw_sk, zw_sn; // strides, elements
    int32_t ss_g, sw_g, zw_g; // K extent of one entry
    int32_t M, N, K, gk, ng, Mpad, Npad;
    float *ssT;
    int32_t *rsT;
    float *swT;
    int32_t *zwT;
    // source zero points / u8 source
    const void *zs; // nullptr: 0
    int32_t zs_dt, zs_g;
    int64_t zs_sm, zs_sk;
    uint32_t a_flip;
    int32_t kt64;
    const uint8_t *B; // packed weights (column sums)
    int32_t *zsT, *c2T; // nullptr unless the source has zero points or is u8
};

// Rows <= 64 (decode): the K range is cut into `splits` slices of `gps` groups,
// one workgroup per (64 columns, slice); slice results are summed in slice
// order by w4a8_reduce_kernel, which also runs the epilogue. No pre-pass: the
// workgroup converts the scales of its slice itself (fields of `q`; its
// transposed-array pointers are unused).
struct w4a8_small_t {
    w4a8_prep_t q;
    const uint8_t *B; // QMM_LAYOUT_MFMA_W4K64
    int32_t tpg, kt64, nb32;
    int32_t gps, splits;
    int32_t ldp; // row pitch of the partial results, floats
    float *part; // [splits][M][ldp]
    epilogue_t ep;
};
constexpr int W4A8_SMALL_MAX_GPS = 16; // groups per slice (LDS)
constexpr int W4A8_SMALL_MAX_M = 64;

// ---- reorder as a quantizer over rows (qmm_quantize.hip) --------------------
struct quant_rows_q_t {
    const void *ptr; // nullptr: default value
    int64_t sr, sc; // strides of the buffer over (row / gr, col / gc)
    int64_t gr, gc;
    int32_t dt;
    int32_t pad_;
};
struct quant_rows_params_t {
    const void *src;
    void *dst;
    int64_t rows, cols; // cols % 8 == 0
    int64_t src_pitch, dst_pitch; // elements
    int32_t src_dt, dst_dt;
    int32_t rows_per_thread, tpr_log2; // set by the launcher
    quant_rows_q_t src_scale, dst_scale, src_zp;
    const int32_t *dst_zp; // single value or nullptr
    int32_t col_groups, pad_; // set by the launcher
};

// ---- the same over a 2-D tensor whose two sides disagree on the dim order ----
struct quant_tr_params_t {
    const void *src;
    void *dst;
    int64_t rows, cols;
    // element strides over (row, col): on each side one of them is 1, and not
    // the same one on both
    int64_t src_sr, src_sc, dst_sr, dst_sc;
    int32_t src_dt, dst_dt;
    quant_rows_q_t src_scale, dst_scale, src_zp;
    const int32_t *dst_zp; // single value or nullptr
};

enum impl_id_t : int {
    impl_gemm_b8 = 0, // int8 / fp8 MFMA GEMM
    impl_gemm_w4a8 = 1, // s8 x int4 MFMA GEMM with K-grouped scales
    impl_gemm_f16w8 = 2, // f16 activations x 8-bit weights at many rows
    impl_gemv_w4 = 3, // decode: 4-bit / 8-bit weights, 16-bit activations
    impl_gemm_f16 = 4, // plain f16 / bf16 batched matmul
    impl_generic = 5,
    impl_count = 6
};

} // namespace qmm

struct qmm_plan {
    int impl;
    qmm::generic_params_t host; // generic parameters (always filled)
    qmm::generic_params_t *dev; // device copy, used by the generic kernel
    qmm_matmul_desc_t desc;
    size_t scratch_bytes;
    // kernel-selection overrides (qmm_hip.h: QMM_GEMM_VARIANT, QMM_W4A8_VARIANT,
    // QMM_B8X_VARIANT), read from the environment when the plan is created and
    // fixed for the plan's life
    int gemm_variant, w4a8_variant, b8x_variant;
    int measure; // QMM_MEASURE: 1 skip the 256 x 256 kernels' epilogue, 2 time stamps
};
