// hip:gfx950:mfma_b8, large-problem kernels: int8 (s8 x s8 -> s32) and fp8
// (e4m3 x e4m3 -> f32, further down) GEMM with a 256 x 256 x 64 block tile, four waves of 128 x 128 each (one per SIMD, the
// 256 accumulator registers of a wave hold its tile), and a hand-ordered main
// loop.
//
// Why this shape. With one wave per SIMD nothing hides a stalled instruction,
// so the loop is written as an explicit sequence: every v_mfma_i32_32x32x32_i8
// (32 cycles of matrix-core time) is followed by at most two cheap
// instructions, the LDS fragment reads for the next 16 MFMAs and the
// global -> LDS loads two tiles ahead are spread between the MFMAs, and the
// waits are counted (lgkmcnt / vmcnt) instead of full. Measured on MI355X
// (per-dispatch counters) a k-step still takes about 1.5 times its MFMA
// cycles: what the loop waits for is the L2 -> LDS operand stream, and the
// 256 x 256 tile is what minimises that stream per MFMA (32 KiB per 128 MFMAs
// and CU). gemm_b8y_kernel below is the same design on 16 x 16 x 64 MFMAs and
// is preferred where its K constraints hold.
//
// Pipeline (k-step = 64 k, two MFMA sub-steps of 32 k):
//   LDS ring of 4 stages x (A 256x64 + B 256x64 bytes). Loop iteration kt first
//   finishes tile kt-1 (its second sub-step) while requesting the A half of
//   tile kt+2, then starts tile kt (its first sub-step) while requesting the B
//   half of tile kt+2. One barrier per iteration, preceded by vmcnt(8): tile kt
//   has landed for every wave, and the stage tile kt+2 goes to (last read in
//   iteration kt-1, by fragments every wave has consumed since) is free.
//   Fragments are double buffered in registers and read one sub-step ahead.
//
// Semantics are those of qmm_gemm_b8.hip (same packed weights, same source
// zero-point compensation through the stored column sums, same epilogue
// arithmetic as src/cpu/matmul/ref_matmul_int8.cpp:195-259); only epilogues of
// the straight-line kinds (EP_FAST_*) are handled here, everything else stays
// with the general kernel.
#include <algorithm>
#include <cstring>
#include <type_traits>

#include "qmm_device.hpp"
#include "qmm_plan.hpp"

// rows of a staged tile in flight in the straight-line epilogue
#ifndef QMM_EP_UNR
#define QMM_EP_UNR 8
#endif

namespace qmm {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

// ---- measurement aid (QMM_MEASURE, qmm_hip.h) --------------------------------
// With GEMM_STAMPS the first lane of a workgroup records (core clock counter,
// constant 100 MHz counter) at four points of its block tile -- kernel entry,
// main loop entry, main loop exit, end of the epilogue -- into a device array
// that qmm_gemm_stamps_read() copies out; GEMM_SKIP_EPILOGUE ends the kernel
// after the main loop. Both are a scalar branch on a kernel argument in the
// normal path. Only the int8 256 x 256 kernel on 16 x 16 x 64 MFMAs (even
// k-step count) has them: the fp8 kernel and the 256 x 128 kernel have no
// registers to spare for the extra code.
[[maybe_unused]] constexpr int STAMP_TILES = 4096, STAMP_SLOTS = 8;
#if defined(QMM_B8X_PART) && (QMM_B8X_PART == 4 || QMM_B8X_PART == 5)
#define QX_HAVE_STAMPS 1
static __device__ unsigned long long g_gemm_stamps[STAMP_TILES * STAMP_SLOTS * 2];
// slots: 0 kernel entry, 1 main loop entry, 2 main loop exit, 3 end of the
// epilogue; inside the epilogue 4 / 6 after the first / second half of the tile
// is staged and 5 after the first half's rows are stored
#define QX_STAMP_IF(first, slot) \
    if ((p.switches & GEMM_STAMPS) && (first)) { \
        const unsigned t = (qx_stamp_id + gridDim.x * blockIdx.y) % STAMP_TILES; \
        g_gemm_stamps[(t * STAMP_SLOTS + (slot)) * 2] = clock64(); \
        g_gemm_stamps[(t * STAMP_SLOTS + (slot)) * 2 + 1] = wall_clock64(); \
    }
#define QX_STAMP(slot) QX_STAMP_IF(tid == 0, slot)
// keeps the accumulators alive without storing them
#define QX_SKIP_EPILOGUE(NI, NJ, NR) \
    if (p.switches & GEMM_SKIP_EPILOGUE) { \
        unsigned s = 0; \
        for (int i = 0; i < NI; i++) \
            for (int j = 0; j < NJ; j++) \
                for (int r = 0; r < NR; r++) \
                    s += __builtin_bit_cast(unsigned, acc[i][j][r]); \
        if (s == 0x12345678u) ((unsigned *)p.ep.dst.ptr)[tid] = s; \
        QX_STAMP(3) \
        return; \
    }
#endif

namespace b8x {

constexpr int BM = 256, BN = 256, BK = 64, NT = 256;
constexpr int STAGES = 4;
constexpr int A_BYTES = BM * BK, B_BYTES = BN * BK;
constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
constexpr uint32_t RING = STAGES * STAGE_BYTES; // 128 KiB, power of two
constexpr int STG_WAVE = 64 * 128 * 4; // epilogue staging of one wave (in the ring)
// The kernels on 16 x 16 MFMAs stage with a row pitch of 132 words: a lane
// group of 16 holds rows 4 apart, which a pitch of 128 would put on the same
// banks.
constexpr int STG_PITCH16 = 132;
constexpr int STG_WAVE16 = 64 * STG_PITCH16 * 4;
constexpr int SS_OFF = 4 * STG_WAVE16; // 256 per-row source scales (f32)
// what the epilogue of the kernels on 16 x 16 MFMAs needs per column of the
// block tile, staged before the main loop: weights scale (f32), source
// zero-point compensation (s32), per-column bias (f32), dst zero point (f32)
constexpr int WS_OFF = SS_OFF + 1024;
constexpr int CS_OFF = WS_OFF + 1024;
constexpr int BI_OFF = CS_OFF + 1024;
constexpr int ZP_OFF = BI_OFF + 1024;
// per row: the source row's sum with its zero-point term (s32), read where the
// weights have zero points
constexpr int RS_OFF = ZP_OFF + 1024;
constexpr int LDS_TOTAL = RS_OFF + 1024;

template <int N, typename F>
QMM_D void static_for(F &&f) {
    if constexpr (N > 0) {
        static_for<N - 1>(f);
        f(std::integral_constant<int, N - 1> {});
    }
}

// chunk swizzle of the row-major A tile (4 chunks of 16 bytes per row)
QMM_D int a_swz(int row, int q) {
    return q ^ ((row >> 2) & 3);
}
// the same for fragments of 16 rows x 4 chunks (lane = row % 16 + 16 * chunk):
// measured free of bank conflicts (SQ_LDS_BANK_CONFLICT), which the swizzle
// above is not for that access shape
QMM_D int a_swz16(int row, int q) {
    return q ^ ((row >> 1) & 3);
}

} // namespace b8x

// The main loop is assembled from these pieces. The memory instructions are
// inline assembly so that they stay exactly where they are written and carry
// no compiler-inserted waits; the MFMAs are builtins (the compiler knows their
// latency when it later reads the accumulators) pinned in place by scheduling
// barriers.
#define QX_SB() __builtin_amdgcn_sched_barrier(0)
#define QX_MF(i, j, cb) \
    { \
        QX_SB(); \
        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8( \
                fa[cb][i], fb[cb][j], acc[i][j], 0, 0, 0); \
        QX_SB(); \
    }
#define QX_DSR(dst, addr, off) \
    asm volatile("ds_read_b128 %0, %1 offset:%2" \
                 : "=v"(dst) \
                 : "v"(addr), "n"(off))
#define QX_WL(n) asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(n))
#define QX_WV(n) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(n) : "memory")
// LDS destination of a direct load = M0 + 16 * lane
#define QX_M0(sreg, imm) \
    asm volatile("s_add_u32 m0, %0, %1" ::"s"(sreg), "n"(imm) : "m0", "scc")
#define QX_DMA(voff, sbase) \
    asm volatile("global_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase) \
                 : "memory")
#define QX_RD_A(nb, va, i) QX_DSR(fa[nb][i], va, (i)*2048)
#define QX_RD_B(nb, vb, nki, j) QX_DSR(fb[nb][j], vb, ((j)*2 + (nki)) * 1024)

// 16 MFMAs on fragment buffer CB. The 8 fragments of the next sub-step are
// read into buffer NB in the order a0 b0 b1 b2 b3 a1 a2 a3 (the order the next
// sub-step's counted waits assume); D0..D3 are direct loads (or empty).
#define QX_SUB(CB, NB, NA, NBA, NKI, D0, D1, D2, D3) \
    QX_WL(3); \
    QX_MF(0, 0, CB); QX_RD_A(NB, NA, 0); \
    QX_MF(0, 1, CB); QX_RD_B(NB, NBA, NKI, 0); \
    QX_MF(0, 2, CB); QX_RD_B(NB, NBA, NKI, 1); \
    QX_MF(0, 3, CB); QX_RD_B(NB, NBA, NKI, 2); \
    QX_WL(6); \
    QX_MF(1, 0, CB); QX_RD_B(NB, NBA, NKI, 3); \
    D0; QX_MF(1, 1, CB); D1; QX_MF(1, 2, CB); D2; QX_MF(1, 3, CB); \
    QX_WL(6); \
    D3; QX_MF(2, 0, CB); \
    QX_MF(2, 1, CB); QX_MF(2, 2, CB); QX_RD_A(NB, NA, 1); QX_MF(2, 3, CB); \
    QX_WL(6); \
    QX_MF(3, 0, CB); QX_RD_A(NB, NA, 2); QX_MF(3, 1, CB); \
    QX_MF(3, 2, CB); QX_RD_A(NB, NA, 3); QX_MF(3, 3, CB);
// the four direct loads of one tile half (V: per-lane offsets, SB: base
// pointer, SD: LDS destination of the wave); each M0 write sits one MFMA before
// the load that uses it
#define QX_D0(V, SB, SD) QX_M0(SD, 0 * 4096)
#define QX_D1(V, SB, SD) \
    QX_DMA(V[0], SB); \
    QX_M0(SD, 1 * 4096)
#define QX_D2(V, SB, SD) \
    QX_DMA(V[1], SB); \
    QX_M0(SD, 2 * 4096)
#define QX_D3(V, SB, SD) \
    QX_DMA(V[2], SB); \
    QX_M0(SD, 3 * 4096)
#define QX_D4(V, SB, SD) QX_DMA(V[3], SB)
#define QX_SUB_D(CB, NB, NA, NBA, NKI, V, SB, SD) \
    QX_WL(3); \
    QX_MF(0, 0, CB); QX_RD_A(NB, NA, 0); \
    QX_MF(0, 1, CB); QX_RD_B(NB, NBA, NKI, 0); \
    QX_MF(0, 2, CB); QX_RD_B(NB, NBA, NKI, 1); \
    QX_MF(0, 3, CB); QX_RD_B(NB, NBA, NKI, 2); \
    QX_WL(6); \
    QX_MF(1, 0, CB); QX_RD_B(NB, NBA, NKI, 3); \
    QX_D0(V, SB, SD); QX_MF(1, 1, CB); QX_D1(V, SB, SD); QX_MF(1, 2, CB); \
    QX_D2(V, SB, SD); QX_MF(1, 3, CB); \
    QX_WL(6); \
    QX_D3(V, SB, SD); QX_MF(2, 0, CB); QX_D4(V, SB, SD); \
    QX_MF(2, 1, CB); QX_MF(2, 2, CB); QX_RD_A(NB, NA, 1); QX_MF(2, 3, CB); \
    QX_WL(6); \
    QX_MF(3, 0, CB); QX_RD_A(NB, NA, 2); QX_MF(3, 1, CB); \
    QX_MF(3, 2, CB); QX_RD_A(NB, NA, 3); QX_MF(3, 3, CB);
#define QX_SUB_LAST(CB) \
    QX_WL(0); \
    QX_MF(0, 0, CB); QX_MF(0, 1, CB); QX_MF(0, 2, CB); QX_MF(0, 3, CB); \
    QX_MF(1, 0, CB); QX_MF(1, 1, CB); QX_MF(1, 2, CB); QX_MF(1, 3, CB); \
    QX_MF(2, 0, CB); QX_MF(2, 1, CB); QX_MF(2, 2, CB); QX_MF(2, 3, CB); \
    QX_MF(3, 0, CB); QX_MF(3, 1, CB); QX_MF(3, 2, CB); QX_MF(3, 3, CB);

// epilogue_fast4 for a full group of four bf16 results: same arithmetic, the
// conversion done by v_cvt_pk_bf16_f32 (round to nearest even; the caller runs
// with f32 denormals flushed, which reproduces the reference's subnormal -> 0).
QMM_D void epilogue_fast4_bf16(const epilogue_t &ep, float (&d)[4], bool has_ss,
        float ss, bool has_ws, const float (&ws)[4], int64_t b, int64_t m,
        int64_t n) {
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
    uint16_t *q = (uint16_t *)ep.dst.ptr + dst_off;
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
        const float *y = (const float *)ep.po[0].t.ptr + b * ep.po[0].t.sb
                + m * ep.po[0].t.sm + n;
#pragma unroll
        for (int i = 0; i < 4; i++)
            d[i] += y[i];
    } else if (fast == EP_FAST_SUM) {
        const float sc = ep.po[0].scale;
#pragma unroll
        for (int i = 0; i < 4; i++)
            d[i] += sc * (bf16_to_f32(q[i]) - 0.f);
    }
    uint32_t h0, h1;
    asm("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(h0) : "v"(d[0]), "v"(d[1]));
    asm("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(h1) : "v"(d[2]), "v"(d[3]));
    if ((((uintptr_t)q) & 7) == 0) {
        *(uint2 *)q = make_uint2(h0, h1);
    } else {
        q[0] = (uint16_t)h0;
        q[1] = (uint16_t)(h0 >> 16);
        q[2] = (uint16_t)h1;
        q[3] = (uint16_t)(h1 >> 16);
    }
}

// Epilogue of 64 staged rows when the wave's 128 x 128 tile lies fully inside
// the matrix and the dst rows are vector-aligned: no per-lane conditions, so
// the rows pipeline. FAST is the recognised epilogue shape, DSTK the dst type,
// EXT whether bias / dst scale / dst zero point take part (epilogue_full4).
// Operands of the post-ops that read a second tensor are requested a batch of
// rows ahead of the stores: 16 rows in the kernels with the LEAN epilogue
// (BATCHED), 4 in the others, whose register allocation does not survive more
// (with 8 the compiler spills 2 KB per lane and moves scalar operands of the
// direct loads into vector registers).
// LPR: lanes that share a staged row (4 columns each): 32 for a wave tile of
// 128 columns (two rows per pass over the 64 staged rows), 16 for one of 64.
template <int FAST, int DSTK, bool EXT, bool F8, int PITCH, bool BATCHED,
        int LPR = 32>
QMM_D void ep_rows_full(const epilogue_t &ep, const int *stg_r,
        const float *ssl, int lane, const ep_cols_t &cols,
        const int (&cs4)[4], int64_t bz, int64_t m_first, int64_t en) {
    constexpr int RPI = 64 / LPR, NIT = 64 / RPI; // rows per pass, passes
    const int ecol = (lane & (LPR - 1)) * 4, lrow = lane / LPR;
    // rows in flight: fewer where a row is a long computation of its own
    constexpr int UNR = FAST == EP_FAST_GELU_ERF || FAST == EP_FAST_GELU_TANH
            ? 2
            : (FAST > EP_FAST_SUM || EXT ? 4 : QMM_EP_UNR);
    auto to_f32 = [&](const int4 &t, float (&d)[4]) {
        if constexpr (F8) { // f32 accumulators, staged as bits
            d[0] = u2f((uint32_t)t.x);
            d[1] = u2f((uint32_t)t.y);
            d[2] = u2f((uint32_t)t.z);
            d[3] = u2f((uint32_t)t.w);
        } else {
            d[0] = (float)(int32_t)((uint32_t)t.x + (uint32_t)cs4[0]);
            d[1] = (float)(int32_t)((uint32_t)t.y + (uint32_t)cs4[1]);
            d[2] = (float)(int32_t)((uint32_t)t.z + (uint32_t)cs4[2]);
            d[3] = (float)(int32_t)((uint32_t)t.w + (uint32_t)cs4[3]);
        }
    };
    if constexpr (ep_reads_operand<FAST>()) {
        // a batch of rows' operands requested before the first of their stores
        constexpr int BATCH = BATCHED ? 16 : 4;
#pragma unroll 1
        for (int it0 = 0; it0 < NIT; it0 += BATCH) {
            uint4 pre[BATCH];
#pragma unroll
            for (int k = 0; k < BATCH; k++)
                pre[k] = ep_operand_load<FAST, DSTK>(ep, cols, bz,
                        m_first + (it0 + k) * RPI + lrow, en);
#pragma unroll
            for (int k = 0; k < BATCH; k++) {
                const int row = (it0 + k) * RPI + lrow;
                const int4 t = *(const int4 *)&stg_r[row * PITCH + ecol];
                const float ss = ssl[row];
                float d[4];
                to_f32(t, d);
                epilogue_full4<FAST, DSTK, EXT, true>(
                        ep, cols, d, ss, bz, m_first + row, en, pre[k]);
            }
        }
        return;
    }
#pragma unroll UNR
    for (int it = 0; it < NIT; it++) {
        const int row = it * RPI + lrow;
        const int4 t = *(const int4 *)&stg_r[row * PITCH + ecol];
        const float ss = ssl[row];
        float d[4];
        to_f32(t, d);
        epilogue_full4<FAST, DSTK, EXT>(ep, cols, d, ss, bz, m_first + row, en);
    }
}

// Column operands of the epilogue of one block tile, and its per-row source
// scales, written to LDS by the first 256 threads before the main loop (the
// loads' latency passes under the prologue): absent ones as 1.0 / 0, columns
// past N likewise.
// TABS: where the six 1 KiB tables start (SS_OFF in the 256 x 256 kernels).
template <int TABS = b8x::SS_OFF>
QMM_D void tile_operands_stage(const gemm_params_t &p, uint8_t *lds, int tid,
        int m0, int n0, int bz) {
    using namespace b8x;
    const epilogue_t &ep = p.ep;
    float ss = 1.f, ws = 1.f, bi = 0.f, zp = 0.f;
    int cs = 0;
    if (ep.src_scale.ptr)
        ss = load_float(ep.src_scale.dt, ep.src_scale.ptr,
                bz * ep.src_scale.sb
                        + (int64_t)min(m0 + tid, p.M - 1) * ep.src_scale.sm);
    const int n = n0 + tid;
    if (n < p.N) {
        if (ep.wei_scale.ptr) ws = ep_load(ep.wei_scale, bz, 0, n);
        if (ep.bias.ptr && ep.bias.sm == 0) bi = ep_load(ep.bias, bz, 0, n);
        if (ep.dst_zp) zp = (float)ep.dst_zp[ep.dst_zp_sn * n];
        int comp = p.a_is_u8 ? 128 : 0;
        if (p.src_zp) comp -= load_int(p.src_zp_dt, p.src_zp, 0);
        if (comp != 0 && p.colsum)
            cs = comp * p.colsum[(int64_t)bz * p.colsum_sb + n];
    }
    ((float *)(lds + TABS))[tid] = ss;
    ((float *)(lds + TABS + (WS_OFF - SS_OFF)))[tid] = ws;
    ((int *)(lds + TABS + (CS_OFF - SS_OFF)))[tid] = cs;
    ((float *)(lds + TABS + (BI_OFF - SS_OFF)))[tid] = bi;
    ((float *)(lds + TABS + (ZP_OFF - SS_OFF)))[tid] = zp;
    if (p.rowsum)
        ((int *)(lds + TABS + (RS_OFF - SS_OFF)))[tid]
                = p.rowsum[(int64_t)bz * p.M + min(m0 + tid, p.M - 1)];
}

// Epilogue of one block tile, shared by the int8 and fp8 kernels.
// LEAN: only the shapes up to EP_FAST_SUM with a float dst run straight-line
// (fp8 and short-K launches; everything else they accept takes the row path)
// The accumulators are NFI x NFJ fragments per wave: 4 x 4 of 32 x 32, or
// 8 x NFJ of 16 x 16 (a wave tile of 128 x 16 NFJ).
// TABS: start of the operand tables (tile_operands_stage). NARROW: a wave tile
// of 64 columns whose staged rows are shared by 16 lanes (pitch 68 words, four
// rows per pass) -- the 256 x 128 kernel; otherwise a row takes 32 lanes and
// lanes past the wave tile's columns idle.
template <bool F8, bool LEAN, typename AccT, int NFI, int NFJ,
        int TABS = b8x::SS_OFF, bool NARROW = false>
QMM_D void tile_epilogue(const gemm_params_t &p, AccT (&acc)[NFI][NFJ],
        uint8_t *lds, uint32_t lds_base, int wave, int lane, int m0, int n0,
        int wm0, int wn0, int bz, [[maybe_unused]] unsigned qx_stamp_id = 0) {
    using namespace b8x;
    constexpr bool MI16 = NFI == 8;
    constexpr int WN = MI16 ? 16 * NFJ : 128; // columns of the wave tile
    constexpr int PITCH = NARROW ? WN + 4 : (MI16 ? STG_PITCH16 : 128);
    constexpr int STGW = NARROW ? 64 * PITCH * 4
                                : (MI16 ? STG_WAVE16 : STG_WAVE);
    constexpr int LPR = NARROW ? WN / 4 : 32; // lanes per staged row
    constexpr int RPI = 64 / LPR; // rows per pass
    static_assert(!NARROW || (MI16 && WN == 64), "narrow staging: 64 columns");
    constexpr int WS_T = TABS + (WS_OFF - SS_OFF), CS_T = TABS + (CS_OFF - SS_OFF),
                  BI_T = TABS + (BI_OFF - SS_OFF), ZP_T = TABS + (ZP_OFF - SS_OFF);
    // 32 x 32 fragments: accumulator register r of lane l is row
    // 8*(r/4) + 4*(l/32) + r%4, column l%32; written to LDS register by
    // register. 16 x 16 fragments are computed transposed (the kernels pass the
    // weights as the MFMA's first operand): register r of lane l is row l%16,
    // column 4*(l/16) + r, so a lane's four registers are neighbouring columns
    // of one row and go to LDS as one 16-byte write.
    // The wave tile goes through LDS in two halves of 64 rows (the ring is
    // free now, every wave takes a quarter of it), straight from the
    // accumulator registers, and comes back row-wise, 4 neighbouring columns
    // per lane, so that the arithmetic exists once per half and every store is
    // a dense vector. A wave reads back only what it wrote itself: LDS
    // executes a wave's instructions in order, no barrier is involved.
    const epilogue_t &ep = p.ep;
    // The row interpreter walks the post-op list with a run-time index: it
    // reads the parameter block where it lies (the kernel argument segment,
    // whose first and only argument is the gemm_params_t), so that the
    // by-value copy `p` stays in registers.
    const epilogue_t &epk
            = ((const gemm_params_t *)__builtin_amdgcn_kernarg_segment_ptr())->ep;
    const uint32_t stg_w = lds_base + wave * STGW
            + (MI16 ? (lane & 15) * PITCH + 4 * (lane >> 4)
                    : 4 * (lane >> 5) * 128 + (lane & 31))
                    * 4;
    const int *const stg_r = (const int *)lds + wave * (STGW / 4);
    const float *const ssl = (const float *)(lds + TABS) + wm0;
    const int ecol = (lane & (LPR - 1)) * 4;
    const bool lane_on = ecol < WN; // lanes past a 112-column wave tile idle
    const int en = n0 + wn0 + ecol;
    const int envalid = lane_on ? min(4, p.N - en) : 0;
    const bool has_ss = ep.src_scale.ptr != nullptr;
    const bool has_ws = ep.wei_scale.ptr != nullptr;
    const bool to_bf16 = ep.dst.dt == dt_bf16;
    const bool ext = ep.fast_ext != 0;
    const int dstk = ep.dst.dt == dt_f32 ? EP_DST_F32
            : ep.dst.dt == dt_bf16       ? EP_DST_BF16
            : ep.dst.dt == dt_f16        ? EP_DST_F16
                                         : EP_DST_Q8;
    // what depends on the lane's 4 columns only: weights scales, a per-column
    // bias, dst zero points, the zero-point compensation
    ep_cols_t cols;
    int cs4[4] = {0, 0, 0, 0};
    if constexpr (MI16) {
        // staged by tile_operands_stage()
        epilogue_cols_load(ep, cols, bz, en, 0);
        const int cw = lane_on ? wn0 + ecol : 0;
        const float4 w4 = *(const float4 *)(lds + WS_T + cw * 4);
        const int4 c4 = *(const int4 *)(lds + CS_T + cw * 4);
        const float4 b4 = *(const float4 *)(lds + BI_T + cw * 4);
        const float4 z4 = *(const float4 *)(lds + ZP_T + cw * 4);
        cols.ws[0] = w4.x, cols.ws[1] = w4.y, cols.ws[2] = w4.z, cols.ws[3] = w4.w;
        cols.bias[0] = b4.x, cols.bias[1] = b4.y, cols.bias[2] = b4.z, cols.bias[3] = b4.w;
        cols.zp[0] = z4.x, cols.zp[1] = z4.y, cols.zp[2] = z4.z, cols.zp[3] = z4.w;
        cs4[0] = c4.x, cs4[1] = c4.y, cs4[2] = c4.z, cs4[3] = c4.w;
    } else {
        epilogue_cols_load(ep, cols, bz, en, envalid > 0 ? envalid : 0);
        int comp = p.a_is_u8 ? 128 : 0;
        if (p.src_zp) comp -= load_int(p.src_zp_dt, p.src_zp, 0);
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (i < envalid && comp != 0 && p.colsum)
                cs4[i] = comp * p.colsum[(int64_t)bz * p.colsum_sb + en + i];
    }
    float ws4[4] = {cols.ws[0], cols.ws[1], cols.ws[2], cols.ws[3]};
    // bf16 results: the reference conversion maps f32 subnormals to +-0
    // (src/common/bfloat16.cpp:22-56). With single-precision denormals flushed
    // for the rest of the wave's life, the last multiply of the chain (or the
    // packed conversion's input stage) produces that zero and
    // v_cvt_pk_bf16_f32 does the round-to-nearest-even.
    if (to_bf16 && !ext && ep.fast != EP_FAST_NONE) epilogue_flush_denormals();
    // wave-uniform: whole wave tile inside the matrix, dst rows (and a binary
    // operand's rows) aligned for vector access
    // Weights zero points (and u8 weights, stored as s8 = u8 - 128): the s32
    // accumulator also loses z_w'[n] x rowsum[m], rowsum being the source row's
    // sum with its zero-point term, one s32 per row from a pre-pass
    // (rowsum_b8_kernel): sum (s - z_s)(w - z_w) = P + comp colsum[n]
    // - z_w'[n] (rowsum[m] + K comp). The staged sums are corrected in LDS by
    // the lanes that read them back, ahead of either row path.
    const bool has_wz = MI16 && !F8 && p.rowsum != nullptr;
    int zw4[4] = {0, 0, 0, 0};
    if (has_wz) {
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (i < envalid)
                zw4[i] = (p.wei_zp ? load_int(p.wei_zp_dt, p.wei_zp,
                                  (int64_t)(en + i) * p.wei_zp_sn)
                                   : 0)
                        - p.w_off;
    }
    const bool full = m0 + wm0 + 128 <= p.M && n0 + wn0 + WN <= p.N
            && ep.fast != EP_FAST_NONE && epilogue_full4_ok(ep)
            && (!LEAN || (ep.fast <= EP_FAST_SUM && dstk <= EP_DST_F16));
    static_for<2>([&](auto H) {
        constexpr int h = decltype(H)::value;
        if constexpr (MI16) {
#pragma unroll
            for (int i2 = 0; i2 < 4; i2++)
#pragma unroll
                for (int j = 0; j < NFJ; j++)
                    asm volatile("ds_write_b128 %0, %1 offset:%2" ::"v"(stg_w),
                                 "a"(acc[4 * h + i2][j]),
                                 "n"((i2 * 16 * PITCH + j * 16) * 4)
                                 : "memory");
        } else {
#pragma unroll
            for (int i2 = 0; i2 < 2; i2++)
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int r = 0; r < 16; r++)
                        asm volatile("ds_write_b32 %0, %1 offset:%2" ::"v"(stg_w),
                                     "a"(acc[2 * h + i2][j][r]),
                                     "n"(((i2 * 32 + 8 * (r / 4) + (r % 4)) * 128
                                                 + j * 32)
                                             * 4)
                                     : "memory");
        }
#ifdef QX_HAVE_STAMPS
        QX_STAMP_IF(wave == 0 && lane == 0, 4 + 2 * h)
#endif
        if (has_wz && lane_on) {
            // s32 arithmetic that wraps like the reference's int sums
            int *const stg_m = (int *)lds + wave * (STGW / 4);
            const int *const rsl
                    = (const int *)(lds + TABS + (RS_OFF - SS_OFF)) + wm0 + h * 64;
#pragma unroll 4
            for (int it = 0; it < 64 / RPI; it++) {
                const int row = it * RPI + lane / LPR;
                const uint32_t rs = (uint32_t)rsl[row];
                int4 t = *(const int4 *)&stg_m[row * PITCH + ecol];
                t.x = (int)((uint32_t)t.x - (uint32_t)zw4[0] * rs);
                t.y = (int)((uint32_t)t.y - (uint32_t)zw4[1] * rs);
                t.z = (int)((uint32_t)t.z - (uint32_t)zw4[2] * rs);
                t.w = (int)((uint32_t)t.w - (uint32_t)zw4[3] * rs);
                *(int4 *)&stg_m[row * PITCH + ecol] = t;
            }
        }
        if (full) {
            const int64_t m_first = m0 + wm0 + h * 64;
            const float *const ssh = ssl + h * 64;
#define QX_EP_ROWS(F, D, X) \
    do { \
        if (lane_on) \
            ep_rows_full<F, D, X, F8, PITCH, LEAN, LPR>( \
                    ep, stg_r, ssh, lane, cols, cs4, bz, m_first, en); \
    } while (0)
#define QX_EP_DST(F) \
    switch (dstk) { \
        case EP_DST_F32: \
            if (ext) QX_EP_ROWS(F, EP_DST_F32, true); \
            else if constexpr (F <= EP_FAST_SUM) QX_EP_ROWS(F, EP_DST_F32, false); \
            break; \
        case EP_DST_BF16: \
            if (ext) QX_EP_ROWS(F, EP_DST_BF16, true); \
            else if constexpr (F <= EP_FAST_SUM) QX_EP_ROWS(F, EP_DST_BF16, false); \
            break; \
        case EP_DST_F16: QX_EP_ROWS(F, EP_DST_F16, true); break; \
        default: \
            if constexpr (!LEAN && F != EP_FAST_SUM) \
                QX_EP_ROWS(F, EP_DST_Q8, true); \
            break; \
    }
#define QX_EP_CASE(F) \
    case F: \
        if constexpr (!LEAN || F <= EP_FAST_SUM) { QX_EP_DST(F) } \
        break;
            switch (ep.fast) {
                QX_EP_CASE(EP_FAST_PLAIN)
                QX_EP_CASE(EP_FAST_RELU)
                QX_EP_CASE(EP_FAST_SWISH)
                QX_EP_CASE(EP_FAST_ADD)
                QX_EP_CASE(EP_FAST_SUM)
                QX_EP_CASE(EP_FAST_GELU_ERF)
                QX_EP_CASE(EP_FAST_GELU_TANH)
                QX_EP_CASE(EP_FAST_BIN32)
                QX_EP_CASE(EP_FAST_BIN16)
                default: break;
            }
#undef QX_EP_ROWS
#undef QX_EP_DST
#undef QX_EP_CASE
        } else {
#pragma unroll 2
            for (int it = 0; it < 64 / RPI; it++) {
                const int row = it * RPI + lane / LPR;
                const int4 t = *(const int4 *)&stg_r[row * PITCH + ecol];
                const int lrow = h * 64 + row;
                const int m = m0 + wm0 + lrow;
                const float ss = ssl[lrow];
                if (m < p.M && envalid > 0) {
                    float v[4];
                    if constexpr (F8) {
                        v[0] = u2f((uint32_t)t.x);
                        v[1] = u2f((uint32_t)t.y);
                        v[2] = u2f((uint32_t)t.z);
                        v[3] = u2f((uint32_t)t.w);
                    } else {
                        v[0] = (float)(int32_t)((uint32_t)t.x + (uint32_t)cs4[0]);
                        v[1] = (float)(int32_t)((uint32_t)t.y + (uint32_t)cs4[1]);
                        v[2] = (float)(int32_t)((uint32_t)t.z + (uint32_t)cs4[2]);
                        v[3] = (float)(int32_t)((uint32_t)t.w + (uint32_t)cs4[3]);
                    }
                    if (ep.fast == EP_FAST_NONE || ext)
                        epilogue_rows4(
                                epk, cols, v, has_ss, ss, bz, m, en, envalid);
                    else if (to_bf16 && envalid == 4)
                        epilogue_fast4_bf16(
                                ep, v, has_ss, ss, has_ws, ws4, bz, m, en);
                    else
                        epilogue_fast4(ep, v, has_ss, ss, has_ws, ws4, bz, m,
                                en, envalid);
                }
            }
        }
#ifdef QX_HAVE_STAMPS
        if constexpr (h == 0) { QX_STAMP_IF(wave == 0 && lane == 0, 5) }
#endif
    });
}

// SHORTK: K of at most 4 k-steps (attention-score shapes): all of K fits the
// LDS ring, so every tile is requested at once and multiplied after a single
// wait; these problems are bound by the dst stream and share the epilogue.
// u8 sources (top bits flipped after the fragment read, +128 * colsum in the
// epilogue) are taken on that path only; the pipelined path takes them once a
// pre-pass has rewritten them as s8 (a_preflipped).
template <bool SHORTK>
__global__ void __launch_bounds__(b8x::NT, 1)
gemm_b8x_kernel(const gemm_params_t p) {
    using namespace b8x;
    typedef __attribute__((address_space(3))) uint8_t lds_u8;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm0 = (wave >> 1) * 128, wn0 = (wave & 1) * 128;

    // ---- XCD-aware tile order (see qmm_gemm_b8.hip) ----
    const int ntiles = p.tiles_m * p.tiles_n;
    int lt;
    {
        const int per = (ntiles + 7) / 8;
        const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
        lt = xcd * per + slot;
        if (slot >= per || lt >= ntiles) return;
    }
    constexpr int GROUP_M = 8;
    const int group = lt / (GROUP_M * p.tiles_n);
    const int first_m = group * GROUP_M;
    const int gsz = min(p.tiles_m - first_m, GROUP_M);
    const int tile_m = first_m + (lt % (GROUP_M * p.tiles_n)) % gsz;
    const int tile_n = (lt % (GROUP_M * p.tiles_n)) / gsz;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int bz = blockIdx.y;

    const int KT = p.K / BK; // host guarantees K % 64 == 0 and KT >= 4
    const uint32_t lds_base = __builtin_amdgcn_readfirstlane(
            (uint32_t)(uintptr_t)(lds_u8 *)lds);

    // Per-lane 32-bit offsets from the tile's base pointers. Chunk c = tid +
    // 256 j of the A tile is row c / 4, LDS chunk position c % 4, and holds
    // the row's chunk (c % 4) ^ swz(row): the swizzle is applied on the global
    // side because a direct load fills LDS in lane order. Rows past M and
    // column blocks past the packed N re-read the last valid ones.
    uint32_t a_vo[4], b_vo[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int c = tid + j * NT;
        const int row = c >> 2, cp = c & 3;
        const int gm = min(m0 + row, p.M - 1) - m0;
        a_vo[j] = (uint32_t)gm * (uint32_t)p.lda + a_swz(row, cp) * 16;
        const int nbl = c >> 7, rem = c & 127;
        const int nb = min(n0 / 32 + nbl, p.nb32 - 1) - n0 / 32;
        b_vo[j] = (uint32_t)nb * (uint32_t)p.kb32 * 1024u + rem * 16;
    }
    auto sgpr_ptr = [](const uint8_t *q) {
        const uint64_t v = (uint64_t)q;
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
        const uint32_t hi
                = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
        return (const uint8_t *)(((uint64_t)hi << 32) | lo);
    };
    // next tile half to request: global base and this wave's LDS slot
    const uint8_t *sa = sgpr_ptr(
            p.A + (int64_t)bz * p.a_sb + (int64_t)m0 * p.lda);
    const uint8_t *sb = sgpr_ptr(p.B + (int64_t)bz * p.b_sb
            + (int64_t)(n0 / 32) * p.kb32 * 1024);
    uint32_t dA = lds_base + wave * 1024;
    uint32_t dB = dA + A_BYTES;
#define QX_ADV_A() \
    { \
        sa += BK; \
        dA = ((dA - lds_base + STAGE_BYTES) & (RING - 1)) + lds_base; \
    }
#define QX_ADV_B() \
    { \
        sb += 2048; \
        dB = ((dB - lds_base + STAGE_BYTES) & (RING - 1)) + lds_base; \
    }
#define QX_FETCH(V, SB, SD) \
    { \
        QX_M0(SD, 0 * 4096); asm volatile("s_nop 0"); QX_DMA(V[0], SB); \
        QX_M0(SD, 1 * 4096); asm volatile("s_nop 0"); QX_DMA(V[1], SB); \
        QX_M0(SD, 2 * 4096); asm volatile("s_nop 0"); QX_DMA(V[2], SB); \
        QX_M0(SD, 3 * 4096); asm volatile("s_nop 0"); QX_DMA(V[3], SB); \
    }

    // fragment addresses inside stage 0
    const int arow = wm0 + (lane & 31);
    const uint32_t a_off0
            = lds_base + arow * BK + a_swz(arow, (lane >> 5)) * 16;
    const uint32_t a_off1
            = lds_base + arow * BK + a_swz(arow, 2 + (lane >> 5)) * 16;
    const uint32_t b_off = lds_base + A_BYTES + ((wn0 >> 5) * 128 + lane) * 16;

    v16i acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                acc[i][j][r] = 0;
    v4i fa[2][4], fb[2][4];

    // per-row source scales of the tile (1.0 when there are none)
    {
        float s = 1.f;
        if (p.ep.src_scale.ptr)
            s = load_float(p.ep.src_scale.dt, p.ep.src_scale.ptr,
                    bz * p.ep.src_scale.sb
                            + (int64_t)min(m0 + tid, p.M - 1) * p.ep.src_scale.sm);
        ((float *)(lds + SS_OFF))[tid] = s;
    }

    if constexpr (SHORTK) {
        for (int t = 0; t < KT; t++) {
            QX_FETCH(a_vo, sa, dA); QX_ADV_A();
            QX_FETCH(b_vo, sb, dB); QX_ADV_B();
        }
        QX_WV(0);
        __syncthreads();
        const uint32_t flip
                = p.a_is_u8 && !p.a_preflipped ? 0x80808080u : 0u;
        for (int t = 0; t < KT; t++) {
#pragma unroll
            for (int ki = 0; ki < 2; ki++) {
                const uint8_t *S = lds + t * STAGE_BYTES;
                const int arel = arow * BK + a_swz(arow, 2 * ki + (lane >> 5)) * 16;
                const int brel = A_BYTES + ((wn0 >> 5) * 128 + lane) * 16 + ki * 1024;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    v4i v = *(const v4i *)(S + arel + i * 2048);
                    v.x ^= flip;
                    v.y ^= flip;
                    v.z ^= flip;
                    v.w ^= flip;
                    fa[0][i] = v;
                }
#pragma unroll
                for (int j = 0; j < 4; j++)
                    fb[0][j] = *(const v4i *)(S + brel + j * 2048);
#pragma unroll
                for (int i = 0; i < 4; i++)
#pragma unroll
                    for (int j = 0; j < 4; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
                                fa[0][i], fb[0][j], acc[i][j], 0, 0, 0);
            }
        }
        __syncthreads();
    } else {
        // ---- prologue: tiles 0 and 1 and the A half of tile 2 ----
        QX_FETCH(a_vo, sa, dA); QX_ADV_A();
        QX_FETCH(b_vo, sb, dB); QX_ADV_B();
        QX_FETCH(a_vo, sa, dA); QX_ADV_A();
        QX_FETCH(b_vo, sb, dB); QX_ADV_B();
        QX_FETCH(a_vo, sa, dA); QX_ADV_A();
        QX_WV(12);
        __syncthreads();
        QX_RD_A(0, a_off0, 0);
        QX_RD_B(0, b_off, 0, 0);
        QX_RD_B(0, b_off, 0, 1);
        QX_RD_B(0, b_off, 0, 2);
        QX_RD_B(0, b_off, 0, 3);
        QX_RD_A(0, a_off0, 1);
        QX_RD_A(0, a_off0, 2);
        QX_RD_A(0, a_off0, 3);
        uint32_t st = 0; // ring offset of the tile whose first half was started
        {
            const uint32_t va1 = a_off1, vb = b_off;
            QX_SUB_D(0, 1, va1, vb, 1, b_vo, sb, dB) // B half of tile 2
            QX_ADV_B();
        }
        // k-step kt: second half of tile kt-1 (requesting the A half of tile
        // kt+2), then first half of tile kt (requesting the B half of tile kt+2)
        for (int kt = 1; kt <= KT - 3; kt++) {
            const uint32_t stn = (st + STAGE_BYTES) & (RING - 1);
            const uint32_t van = a_off0 + stn, vbn = b_off + stn,
                           va1 = a_off1 + stn;
            QX_WV(8); // tile kt has landed
            __builtin_amdgcn_s_barrier();
            QX_SUB_D(1, 0, van, vbn, 0, a_vo, sa, dA)
            QX_ADV_A();
            QX_SUB_D(0, 1, va1, vbn, 1, b_vo, sb, dB)
            QX_ADV_B();
            st = stn;
        }
#pragma unroll 1
        for (int kt = KT - 2; kt <= KT - 1; kt++) {
            const uint32_t stn = (st + STAGE_BYTES) & (RING - 1);
            const uint32_t van = a_off0 + stn, vbn = b_off + stn,
                           va1 = a_off1 + stn;
            QX_WV(0);
            __builtin_amdgcn_s_barrier();
            QX_SUB(1, 0, van, vbn, 0, , , , )
            QX_SUB(0, 1, va1, vbn, 1, , , , )
            st = stn;
        }
        QX_SUB_LAST(1)
        __syncthreads();
    }

    tile_epilogue<false, SHORTK>(
            p, acc, lds, lds_base, wave, lane, m0, n0, wm0, wn0, bz);
}


// ---- int8 on 16 x 16 x 64 MFMAs ---------------------------------------------
// Same block tile, LDS ring, direct loads and epilogue as gemm_b8x_kernel, but
// the wave's 128 x 128 tile is 8 x 8 fragments of v_mfma_i32_16x16x64_i8: one
// instruction contracts a whole 64-k tile (16 cycles), so each accumulator is
// read and written half as often per multiply-accumulate as with the
// 32 x 32 x 32 shape. On MI355X that is what the sustained clock responds to:
// a loop of nothing but MFMAs on random int8 data holds 3.9 POP/s with this
// shape and 2.9-3.2 POP/s with 32 x 32 x 32 (both 4.6-4.8 POP/s on zeros).
// An operand fragment is one 16-byte read: lane l holds row (column) l % 16,
// k 16 * (l / 16) .. + 15 -- chunk l / 16 of the row in the swizzled A tile, and
// for B the chunk of the packed tile that holds that column and k range.
// A k-step multiplies the fragments read during the previous k-step (64 MFMAs),
// reads the next tile's 16 fragments into the other register buffer and
// requests the tile two further on (8 direct loads), one barrier per k-step.
// The weights fragment is the MFMA's first operand: the accumulator comes out
// transposed (register r of lane l is row l % 16, column 4 * (l / 16) + r of
// the fragment), four neighbouring columns of one row per lane, which is what
// the epilogue stores.
#define QY_MF(i, j, cb) \
    { \
        QX_SB(); \
        acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8( \
                fb[cb][j], fa[cb][i], acc[i][j], 0, 0, 0); \
        QX_SB(); \
    }
#define QY_RA(nb, i) \
    { \
        fa[nb][i] = *(const v4i *)(ldsn + a_rel + (i)*1024); \
        QX_SB(); \
    }
#define QY_RB(nb, j) \
    { \
        fb[nb][j] = *(const v4i *)(ldsn + b_rel + ((j) >> 1) * 2048 + ((j)&1) * 256); \
        QX_SB(); \
    }
// row i of the fragment grid: 8 MFMAs, with up to four other instructions
// (X0..X3) after the 1st, 3rd, 5th and 7th
#define QY_ROW(i, CB, X0, X1, X2, X3) \
    QY_MF(i, 0, CB); X0; QY_MF(i, 1, CB); QY_MF(i, 2, CB); X1; \
    QY_MF(i, 3, CB); QY_MF(i, 4, CB); X2; QY_MF(i, 5, CB); \
    QY_MF(i, 6, CB); X3; QY_MF(i, 7, CB);
// the 16 fragment reads and the direct loads (with their M0 writes) are spread
// evenly over the 64 MFMAs: requests issued in a cluster run into the rate the
// L2 -> LDS path accepts them at
#define QY_STEP(CB, NB, DA0, DA1, DA2, DA3, DA4, DB0, DB1, DB2, DB3, DB4) \
    QY_ROW(0, CB, QY_RA(NB, 0), QY_RB(NB, 0), DA0, QY_RB(NB, 1)) \
    QY_ROW(1, CB, QY_RB(NB, 2), DA1, QY_RB(NB, 3), QY_RB(NB, 4)) \
    QY_ROW(2, CB, DA2, QY_RB(NB, 5), QY_RB(NB, 6), DA3) \
    QY_ROW(3, CB, QY_RB(NB, 7), QY_RA(NB, 1), DA4, QY_RA(NB, 2)) \
    QY_ROW(4, CB, QY_RA(NB, 3), DB0, QY_RA(NB, 4), QY_RA(NB, 5)) \
    QY_ROW(5, CB, DB1, QY_RA(NB, 6), QY_RA(NB, 7), DB2) \
    QY_ROW(6, CB, , , DB3, ) \
    QY_ROW(7, CB, , DB4, , )
#define QY_STEP_D(CB, NB) \
    QY_STEP(CB, NB, QX_D0(a_vo, sa, dA), QX_D1(a_vo, sa, dA), \
            QX_D2(a_vo, sa, dA), QX_D3(a_vo, sa, dA), QX_D4(a_vo, sa, dA), \
            QX_D0(b_vo, sb, dB), QX_D1(b_vo, sb, dB), QX_D2(b_vo, sb, dB), \
            QX_D3(b_vo, sb, dB), QX_D4(b_vo, sb, dB))
#define QY_STEP_ND(CB, NB) QY_STEP(CB, NB, , , , , , , , , , )
#define QY_LAST(CB) \
    QY_ROW(0, CB, , , , ) QY_ROW(1, CB, , , , ) QY_ROW(2, CB, , , , ) \
    QY_ROW(3, CB, , , , ) QY_ROW(4, CB, , , , ) QY_ROW(5, CB, , , , ) \
    QY_ROW(6, CB, , , , ) QY_ROW(7, CB, , , , )

// gemm_b8y_kernel puts its workgroups out of step on purpose: when an XCD's
// share is F >= 1 whole rounds and R more tiles, the workgroups without a tile
// in that last round start half a tile late (their CUs would idle at the end
// instead). The two groups then run their main loops and their epilogues half
// a tile apart for the whole launch: the power a CU does not draw while it
// converts and stores a tile is there for the main loops of the others, which
// run at a higher clock than when every CU multiplies at once. Returns whether
// the launch has such a late half; half_tile_ticks in ticks of the constant
// 100 MHz counter (a bounded wait: every wave leaves it).
QMM_D bool late_half_start(const gemm_params_t &p, int per, int W, int tid,
        unsigned long long half_tile_ticks) {
    const int F = per / W, R = per - F * W;
    const bool late_half = !(p.switches & GEMM_NO_STAGGER) && F >= 1 && R > 0
            && gridDim.y == 1;
    if (late_half && (int)(blockIdx.x >> 3) >= R) {
        if (tid == 0) {
            const unsigned long long t0 = wall_clock64();
            while (wall_clock64() - t0 < half_tile_ticks)
                __builtin_amdgcn_s_sleep(64);
        }
        __syncthreads();
    }
    return late_half;
}

#if defined(QMM_B8X_PART) && (QMM_B8X_PART == 4 || QMM_B8X_PART == 5)
// One block tile of gemm_b8y_kernel.
// ODD: an odd number of k-steps (the register buffers alternate per k-step, so
// the two parities end on different buffers; one instantiation each keeps the
// tail single and the accumulators out of scratch). A 224-column block tile
// (wave tiles of 128 x 112, four equal rounds of workgroups on a 4096 x 14336
// dst instead of three and a half) was measured at 0.6 % and is not kept.
template <bool ODD>
QMM_D void gemm_b8y_tile(const gemm_params_t &p, uint8_t *lds,
        const uint32_t lds_base, const int tid, const int lane, const int wave,
        const int m0, const int n0, const int bz,
        [[maybe_unused]] const unsigned qx_stamp_id) {
    using namespace b8x;
    constexpr int NFJ = 8;
    const int wm0 = (wave >> 1) * 128, wn0 = (wave & 1) * (16 * NFJ);

    const int KT = p.K / BK; // host guarantees K % 64 == 0, KT >= 5 and KT % 2 == ODD
    if constexpr (!ODD) { QX_STAMP(0) }

    uint32_t a_vo[4], b_vo[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int c = tid + j * NT;
        const int row = c >> 2, cp = c & 3;
        const int gm = min(m0 + row, p.M - 1) - m0;
        a_vo[j] = (uint32_t)gm * (uint32_t)p.lda + a_swz16(row, cp) * 16;
        const int nbl = c >> 7, rem = c & 127;
        const int nb = min(n0 / 32 + nbl, p.nb32 - 1) - n0 / 32;
        b_vo[j] = (uint32_t)nb * (uint32_t)p.kb32 * 1024u + rem * 16;
    }
    auto sgpr_ptr = [](const uint8_t *q) {
        const uint64_t v = (uint64_t)q;
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
        const uint32_t hi
                = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
        return (const uint8_t *)(((uint64_t)hi << 32) | lo);
    };
    const uint8_t *sa = sgpr_ptr(
            p.A + (int64_t)bz * p.a_sb + (int64_t)m0 * p.lda);
    const uint8_t *sb = sgpr_ptr(p.B + (int64_t)bz * p.b_sb
            + (int64_t)(n0 / 32) * p.kb32 * 1024);
    uint32_t dA = lds_base + wave * 1024;
    uint32_t dB = dA + A_BYTES;

    // fragment offsets inside a stage: lane group g = lane / 16 takes k chunk g
    const int g = lane >> 4;
    const int arow = wm0 + (lane & 15);
    const int a_rel = arow * BK + a_swz16(arow, g) * 16;
    const int b_rel = A_BYTES + (wn0 >> 5) * 2048 + (g >> 1) * 1024
            + ((g & 1) * 32 + (lane & 15)) * 16;

    v4i acc[8][NFJ];
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int j = 0; j < NFJ; j++)
#pragma unroll
            for (int r = 0; r < 4; r++)
                acc[i][j][r] = 0;
    v4i fa[2][8], fb[2][NFJ];

    tile_operands_stage(p, lds, tid, m0, n0, bz);

    // ---- prologue: tiles 0..3 requested (the whole ring); tile 0's
    // fragments read ----
    QX_FETCH(a_vo, sa, dA); QX_ADV_A();
    QX_FETCH(b_vo, sb, dB); QX_ADV_B();
    QX_FETCH(a_vo, sa, dA); QX_ADV_A();
    QX_FETCH(b_vo, sb, dB); QX_ADV_B();
    QX_FETCH(a_vo, sa, dA); QX_ADV_A();
    QX_FETCH(b_vo, sb, dB); QX_ADV_B();
    QX_FETCH(a_vo, sa, dA); QX_ADV_A();
    QX_FETCH(b_vo, sb, dB); QX_ADV_B();
    QX_WV(24);
    __syncthreads();
    uint32_t st = 0; // ring offset of the tile whose fragments are read next
    {
        const uint8_t *ldsn = lds;
        QX_SB();
        QY_RA(0, 0); QY_RB(0, 0); QY_RB(0, 1); QY_RB(0, 2); QY_RB(0, 3);
        QY_RB(0, 4); QY_RB(0, 5); QY_RB(0, 6); QY_RB(0, 7); QY_RA(0, 1);
        QY_RA(0, 2); QY_RA(0, 3); QY_RA(0, 4); QY_RA(0, 5); QY_RA(0, 6);
        QY_RA(0, 7);
    }
    // k-step kt: multiplies tile kt-1 (buffer (kt-1)&1), reads tile kt's
    // fragments, requests tile kt+3 into the stage tile kt-1 was read from
    // during the previous k-step
#define QY_KSTEP(WAITV, BODY) \
    { \
        st = (st + STAGE_BYTES) & (RING - 1); \
        const uint8_t *ldsn = lds + st; \
        QX_WV(WAITV); \
        __builtin_amdgcn_s_barrier(); \
        QX_SB(); \
        BODY \
    }
    if constexpr (!ODD) { QX_STAMP(1) }
    // requesting steps kt = 1 .. KT-4, in pairs; an odd KT leaves one more
    constexpr int PAIRED_END = ODD ? 6 : 5;
    for (int kt = 1; kt <= KT - PAIRED_END; kt += 2) {
        QY_KSTEP(16, QY_STEP_D(0, 1) QX_ADV_A(); QX_ADV_B();)
        QY_KSTEP(16, QY_STEP_D(1, 0) QX_ADV_A(); QX_ADV_B();)
    }
    if constexpr (ODD) {
        QY_KSTEP(16, QY_STEP_D(0, 1)) // kt = KT-4: requests tile KT-1
        QY_KSTEP(16, QY_STEP_ND(1, 0)) // kt = KT-3
        QY_KSTEP(8, QY_STEP_ND(0, 1)) // kt = KT-2
        QY_KSTEP(0, QY_STEP_ND(1, 0)) // kt = KT-1
        QY_LAST(0)
    } else {
        QY_KSTEP(16, QY_STEP_ND(0, 1)) // kt = KT-3
        QY_KSTEP(8, QY_STEP_ND(1, 0)) // kt = KT-2
        QY_KSTEP(0, QY_STEP_ND(0, 1)) // kt = KT-1
        QY_LAST(1)
    }
    __syncthreads();
    if constexpr (!ODD) {
        QX_STAMP(2)
        QX_SKIP_EPILOGUE(8, NFJ, 4)
    }

    tile_epilogue<false, false>(p, acc, lds, lds_base, wave, lane, m0, n0, wm0,
            wn0, bz, qx_stamp_id);
    if constexpr (!ODD) { QX_STAMP(3) }
}

// Persistent: the grid is 8 x W workgroups, W per XCD (one per CU: the LDS ring
// leaves no room for a second), and workgroup w of an XCD takes the tiles
// w, w + W, ... of the XCD's share in turn: a tile starts when its predecessor
// on the CU has stored its last row, without a trip through the dispatcher.
template <bool ODD>
__global__ void __launch_bounds__(b8x::NT, 1)
gemm_b8y_kernel(const gemm_params_t p) {
    using namespace b8x;
    typedef __attribute__((address_space(3))) uint8_t lds_u8;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t lds_base = __builtin_amdgcn_readfirstlane(
            (uint32_t)(uintptr_t)(lds_u8 *)lds);
    const int bz = blockIdx.y;

    const int ntiles = p.tiles_m * p.tiles_n;
    const int per = (ntiles + 7) / 8;
    const int xcd = blockIdx.x & 7, W = gridDim.x >> 3;
    // half of (prologue + epilogue ~ 12 us, 0.64 us a k-step). The two groups
    // no longer meet each other's operand slices in the L2, so where the split
    // is 16 : 16 each group takes a 4 x 4 block of tiles (4 + 4 operand panels)
    // out of a round's 8 x 4 instead of 8 x 2 (8 + 2).
    const bool square_groups
            = late_half_start(p, per, W, tid, 600 + (p.K / BK) * 32) && W == 32
            && per % 32 == 16;
    for (int slot = blockIdx.x >> 3, it = 0; slot < per; slot += W, it++) {
        constexpr int GROUP_M = 8;
        int lt = xcd * per + slot;
        if (square_groups && it * W + 32 <= per) {
            // a whole round: 32 consecutive tiles, 8 rows x 4 columns when they
            // start on a row-group boundary and lie in one full row group
            const int w = blockIdx.x >> 3, base = lt - w;
            const int o = base % (GROUP_M * p.tiles_n);
            const int rows_left
                    = p.tiles_m - base / (GROUP_M * p.tiles_n) * GROUP_M;
            if (o % GROUP_M == 0 && o + 32 <= GROUP_M * p.tiles_n
                    && rows_left >= GROUP_M)
                lt = base + ((w & 15) >> 2) * GROUP_M + (w >> 4) * 4 + (w & 3);
        }
        if (lt >= ntiles) break;
        const int group = lt / (GROUP_M * p.tiles_n);
        const int first_m = group * GROUP_M;
        const int gsz = min(p.tiles_m - first_m, GROUP_M);
        const int tile_m = first_m + (lt % (GROUP_M * p.tiles_n)) % gsz;
        const int tile_n = (lt % (GROUP_M * p.tiles_n)) / gsz;
        gemm_b8y_tile<ODD>(p, lds, lds_base, tid, lane, wave, tile_m * BM,
                tile_n * BN, bz, it * gridDim.x + blockIdx.x);
        // the staging area and the operand tables are the next tile's ring
        // and tables
        __syncthreads();
    }
}
#endif // int8, 16 x 16 x 64

// ---- int8, two workgroups per CU -----------------------------------------------
// The kernels above keep one wave per SIMD, so the matrix cores idle while a
// workgroup runs its prologue and its epilogue (a sixth of a launch on a
// 4096 x 4096 x 14336 problem with a swish epilogue). Here the block tile is
// 256 x 128 (four waves of 128 x 64: 8 x 4 fragments of v_mfma_i32_16x16x64_i8,
// 128 accumulator registers), a workgroup needs under 80 KiB of LDS and under
// 256 registers per lane, and two workgroups share a CU: while one stages,
// converts and stores its tile the other one's MFMAs have the matrix cores,
// and in the main loop the two waves of a SIMD fill each other's gaps. The
// price is operand traffic per MFMA: a k-step moves 24 KiB into LDS for 32 MFMAs
// per wave (32 KiB for 64 above) and reads 12 fragments for them (16 for 64).
// LDS ring of 3 stages x (A 256 x 64 + B 128 x 64 bytes); k-step kt multiplies
// the fragments of tile kt-1 (read during the previous k-step), reads tile
// kt's, and requests tile kt+2 into the stage tile kt-1 was read from; one
// vmcnt + barrier per k-step. The MFMAs are inline assembly with the
// accumulators constrained to the accumulator file (with the builtin and 128
// accumulators the register allocator shuttles them between the two files
// inside the loop), which wants ONE code path for all k-steps: the loop body
// is a pair of k-steps (the two fragment buffers), the pair count is
// ceil(k-steps / 2), a phantom last tile multiplies the zero padding of the
// packed weights (K is padded to 128 there) against a re-read of the last
// source tile, and request pointers stop advancing at the last tile.
#if defined(QMM_B8X_PART) && QMM_B8X_PART == 7
namespace b8w {
constexpr int BM = 256, BN = 128, BK = 64, NT = 256;
constexpr int STAGES = 3;
constexpr int A_BYTES = BM * BK, B_BYTES = BN * BK;
constexpr int STAGE_BYTES = A_BYTES + B_BYTES; // 24 KiB
constexpr int RING = STAGES * STAGE_BYTES; // 72 KiB
constexpr int STG_PITCH = 68, STG_WAVE = 64 * STG_PITCH * 4; // epilogue staging
static_assert(4 * STG_WAVE <= RING, "the staging reuses the ring");
constexpr int TABS = RING; // six 1 KiB operand tables (tile_operands_stage)
constexpr int LDS_TOTAL = TABS + 6 * 1024;
} // namespace b8w

#define QW_MF(i, j, cb) \
    { \
        QX_SB(); \
        asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" \
                     : "+a"(acc[i][j]) \
                     : "v"(fb[cb][j]), "v"(fa[cb][i])); \
        QX_SB(); \
    }
#define QW_RA(nb, i) \
    { \
        fa[nb][i] = *(const v4i *)(ldsn + a_rel + (i)*1024); \
        QX_SB(); \
    }
#define QW_RB(nb, j) \
    { \
        fb[nb][j] = *(const v4i *)(ldsn + b_rel + ((j) >> 1) * 2048 + ((j)&1) * 256); \
        QX_SB(); \
    }
// advance to the next 64-k tile, staying on the last one once it is reached
#define QW_ADV_A() \
    { \
        const int go = adv_a > 0; \
        sa += go ? BK : 0; \
        adv_a -= go; \
        dA = dA + STAGE_BYTES >= lds_base + RING ? dA + STAGE_BYTES - RING \
                                                 : dA + STAGE_BYTES; \
    }
#define QW_ADV_B() \
    { \
        const int go = adv_b > 0; \
        sb += go ? 2048 : 0; \
        adv_b -= go; \
        dB = dB + STAGE_BYTES >= lds_base + A_BYTES + RING \
                ? dB + STAGE_BYTES - RING \
                : dB + STAGE_BYTES; \
    }
// row i of the fragment grid: 4 MFMAs with one other instruction after each
// (u8 sources: a fragment's top bits are flipped in the k-step that reads it,
// a row of MFMAs after its read was issued and a whole k-step before its use:
// the MFMAs are inline assembly, so the compiler inserts no wait states between
// a vector instruction that writes an operand and the MFMA that reads it)
#define QW_FLIP(NB, i) \
    if constexpr (U8) { \
        fa[NB][i][0] ^= 0x80808080; \
        fa[NB][i][1] ^= 0x80808080; \
        fa[NB][i][2] ^= 0x80808080; \
        fa[NB][i][3] ^= 0x80808080; \
        QX_SB(); \
    }
#define QW_ROW(i, CB, X0, X1, X2, X3) \
    QW_MF(i, 0, CB); X0; QW_MF(i, 1, CB); X1; QW_MF(i, 2, CB); X2; \
    QW_MF(i, 3, CB); X3;
// the B loads are two per wave: M0, load, M0, load
#define QW_DB0() QX_M0(dB, 0 * 4096)
#define QW_DB1() \
    QX_DMA(b_vo[0], sb); \
    QX_M0(dB, 1 * 4096)
#define QW_DB2() QX_DMA(b_vo[1], sb)
// one k-step: 32 MFMAs on buffer CB; the next tile's 12 fragments into buffer
// NB and the 6 direct loads of the tile after next, one instruction per MFMA
#define QW_STEP(CB, NB) \
    QW_ROW(0, CB, QW_RA(NB, 0), QW_RB(NB, 0), QX_D0(a_vo, sa, dA), QW_RB(NB, 1)) \
    QW_ROW(1, CB, QW_RB(NB, 2), QX_D1(a_vo, sa, dA), QW_RB(NB, 3), QW_RA(NB, 1)) \
    QW_ROW(2, CB, QX_D2(a_vo, sa, dA), QW_RA(NB, 2), QW_RA(NB, 3), QX_D3(a_vo, sa, dA)) \
    QW_ROW(3, CB, QW_RA(NB, 4), QX_D4(a_vo, sa, dA), QW_RA(NB, 5), QW_DB0()) \
    QW_ROW(4, CB, QW_RA(NB, 6), QW_DB1(), QW_RA(NB, 7), QW_DB2()) \
    QW_ROW(5, CB, QW_FLIP(NB, 0), QW_FLIP(NB, 1), QW_FLIP(NB, 2), QW_FLIP(NB, 3)) \
    QW_ROW(6, CB, QW_FLIP(NB, 4), QW_FLIP(NB, 5), QW_FLIP(NB, 6), QW_FLIP(NB, 7)) \
    QW_ROW(7, CB, , , , )

// U8: the source is u8: its fragments are turned into s8 = u8 - 128 by
// flipping the top bit of every byte (the epilogue adds 128 x the weights'
// column sums back).
template <bool U8>
__global__ void __launch_bounds__(b8w::NT, 2)
gemm_b8w_kernel(const gemm_params_t p) {
    using namespace b8w;
    using b8x::a_swz16;
    typedef __attribute__((address_space(3))) uint8_t lds_u8;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm0 = (wave >> 1) * 128, wn0 = (wave & 1) * 64;

    const int ntiles = p.tiles_m * p.tiles_n;
    int lt;
    {
        const int per = (ntiles + 7) / 8;
        const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
        lt = xcd * per + slot;
        if (slot >= per || lt >= ntiles) return;
    }
    constexpr int GROUP_M = 8;
    const int group = lt / (GROUP_M * p.tiles_n);
    const int first_m = group * GROUP_M;
    const int gsz = min(p.tiles_m - first_m, GROUP_M);
    const int tile_m = first_m + (lt % (GROUP_M * p.tiles_n)) % gsz;
    const int tile_n = (lt % (GROUP_M * p.tiles_n)) / gsz;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int bz = blockIdx.y;

    const int KT = p.K / BK; // host guarantees K % 64 == 0 and KT >= 4
    const uint32_t lds_base = __builtin_amdgcn_readfirstlane(
            (uint32_t)(uintptr_t)(lds_u8 *)lds);

    uint32_t a_vo[4], b_vo[2];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int c = tid + j * NT;
        const int row = c >> 2, cp = c & 3;
        const int gm = min(m0 + row, p.M - 1) - m0;
        a_vo[j] = (uint32_t)gm * (uint32_t)p.lda + a_swz16(row, cp) * 16;
    }
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int c = tid + j * NT;
        const int nbl = c >> 7, rem = c & 127;
        const int nb = min(n0 / 32 + nbl, p.nb32 - 1) - n0 / 32;
        b_vo[j] = (uint32_t)nb * (uint32_t)p.kb32 * 1024u + rem * 16;
    }
    auto sgpr_ptr = [](const uint8_t *q) {
        const uint64_t v = (uint64_t)q;
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
        const uint32_t hi
                = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
        return (const uint8_t *)(((uint64_t)hi << 32) | lo);
    };
    const uint8_t *sa = sgpr_ptr(
            p.A + (int64_t)bz * p.a_sb + (int64_t)m0 * p.lda);
    const uint8_t *sb = sgpr_ptr(p.B + (int64_t)bz * p.b_sb
            + (int64_t)(n0 / 32) * p.kb32 * 1024);
    uint32_t dA = lds_base + wave * 1024;
    uint32_t dB = dA + A_BYTES;
    // tile advances left: the source stops at its last tile, the packed weights
    // at the last tile of their zero-padded K
    int adv_a = KT - 1, adv_b = p.kb32 / 2 - 1;

    const int g = lane >> 4;
    const int arow = wm0 + (lane & 15);
    const int a_rel = arow * BK + a_swz16(arow, g) * 16;
    const int b_rel = A_BYTES + (wn0 >> 5) * 2048 + (g >> 1) * 1024
            + ((g & 1) * 32 + (lane & 15)) * 16;

    v4i acc[8][4];
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int r = 0; r < 4; r++)
                acc[i][j][r] = 0;
    v4i fa[2][8], fb[2][4];

    tile_operands_stage<TABS>(p, lds, tid, m0, n0, bz);

    // ---- prologue: tiles 0..2 requested (the whole ring); tile 0's fragments
    // read ----
#define QW_FETCH_B() \
    { \
        QX_M0(dB, 0 * 4096); asm volatile("s_nop 0"); QX_DMA(b_vo[0], sb); \
        QX_M0(dB, 1 * 4096); asm volatile("s_nop 0"); QX_DMA(b_vo[1], sb); \
    }
    QX_FETCH(a_vo, sa, dA); QW_ADV_A();
    QW_FETCH_B(); QW_ADV_B();
    QX_FETCH(a_vo, sa, dA); QW_ADV_A();
    QW_FETCH_B(); QW_ADV_B();
    QX_FETCH(a_vo, sa, dA); QW_ADV_A();
    QW_FETCH_B(); QW_ADV_B();
    QX_WV(12);
    __syncthreads();
    uint32_t st = 0; // ring offset of the tile whose fragments are read next
    {
        const uint8_t *ldsn = lds;
        QX_SB();
        QW_RA(0, 0); QW_RB(0, 0); QW_RB(0, 1); QW_RB(0, 2); QW_RB(0, 3);
        QW_RA(0, 1); QW_RA(0, 2); QW_RA(0, 3); QW_RA(0, 4); QW_RA(0, 5);
        QW_RA(0, 6); QW_RA(0, 7);
        QW_FLIP(0, 0) QW_FLIP(0, 1) QW_FLIP(0, 2) QW_FLIP(0, 3)
        QW_FLIP(0, 4) QW_FLIP(0, 5) QW_FLIP(0, 6) QW_FLIP(0, 7)
    }
    // k-step: tile kt has landed for every wave (the 6 requests of tile kt+1
    // may still be in flight), and every wave has read what it needed from the
    // stage tile kt+2 goes to
#define QW_KSTEP(CB, NB) \
    { \
        st = st + STAGE_BYTES >= (uint32_t)RING ? 0u : st + STAGE_BYTES; \
        const uint8_t *ldsn = lds + st; \
        QX_WV(6); \
        __builtin_amdgcn_s_barrier(); \
        QX_SB(); \
        QW_STEP(CB, NB) \
        QW_ADV_A(); \
        QW_ADV_B(); \
    }
    const int pairs = (KT + 1) / 2;
    for (int it = 0; it < pairs; it++) {
        QW_KSTEP(0, 1)
        QW_KSTEP(1, 0)
    }
    // the last MFMAs are still writing, and the surplus requests must have
    // landed before the ring is reused as staging
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    QX_WV(0);
    __syncthreads();

    tile_epilogue<false, false, v4i, 8, 4, TABS, true>(
            p, acc, lds, lds_base, wave, lane, m0, n0, wm0, wn0, bz);
}

void launch_b8x_int8_two_per_cu(const gemm_params_t &p, hipStream_t stream) {
    using namespace b8w;
    gemm_params_t q = p;
    q.tiles_m = (p.M + BM - 1) / BM;
    q.tiles_n = (p.N + BN - 1) / BN;
    const int ntiles = q.tiles_m * q.tiles_n;
    const int grid_x = ((ntiles + 7) / 8) * 8;
    auto go = [&](auto kern) {
        ensure_dynamic_lds((const void *)kern, LDS_TOTAL);
        hipLaunchKernelGGL(kern, dim3(grid_x, p.batch), dim3(NT), LDS_TOTAL,
                stream, q);
    };
    if (p.a_is_u8 && !p.a_preflipped)
        go(gemm_b8w_kernel<true>);
    else
        go(gemm_b8w_kernel<false>);
}
#endif // int8, two workgroups per CU

// ---- fp8 (e4m3 x e4m3 -> f32) ----------------------------------------------
// Same tile, ring and epilogue. v_mfma_f32_32x32x64_f8f6f4 consumes a whole
// 64-k tile per instruction (64 cycles), so a k-step is one group of 16 MFMAs
// on the fragments read during the previous k-step; the 16 fragment reads of
// the next tile and the 8 direct loads three tiles further on are spread between
// them. The fragment reads are ordinary LDS loads here (the compiler counts
// their waits itself; it does not see the direct loads, so it adds no vmcnt);
// the scheduling barriers keep everything where it is written. An operand is
// the pair (k 0..31 fragment, k 32..63 fragment) of the int8 path, i.e. lane
// half h holds k 16h..16h+15 and 32+16h..32+16h+15 -- the same permutation on
// both operands.
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

#define QF_MF(i, j, cb) \
    { \
        QX_SB(); \
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4( \
                __builtin_shufflevector(fa[cb][0][i], fa[cb][1][i], 0, 1, 2, \
                        3, 4, 5, 6, 7), \
                __builtin_shufflevector(fb[cb][0][j], fb[cb][1][j], 0, 1, 2, \
                        3, 4, 5, 6, 7), \
                acc[i][j], 0, 0, 0, 0, 0, 0); \
        QX_SB(); \
    }
#define QF_RA(nb, h, i) \
    { \
        fa[nb][h][i] = *(const v4i *)(ldsn + (h ? a_rel1 : a_rel0) + (i)*2048); \
        QX_SB(); \
    }
#define QF_RB(nb, h, j) \
    { \
        fb[nb][h][j] = *(const v4i *)(ldsn + b_rel + ((j)*2 + (h)) * 1024); \
        QX_SB(); \
    }
// one k-step: 16 MFMAs on buffer CB, the next tile's fragments into buffer NB
// (order a0 b0 b1 b2 b3 a1 a2 a3, both halves each); D*: direct loads or empty
// one fragment read after every MFMA; the direct loads (with their M0 writes)
// spread evenly over the k-step
#define QF_STEP(CB, NB, DA0, DA1, DA2, DA3, DA4, DB0, DB1, DB2, DB3, DB4) \
    QF_MF(0, 0, CB); QF_RA(NB, 0, 0); \
    QF_MF(0, 1, CB); QF_RA(NB, 1, 0); DA0; \
    QF_MF(0, 2, CB); QF_RB(NB, 0, 0); DA1; \
    QF_MF(0, 3, CB); QF_RB(NB, 1, 0); \
    QF_MF(1, 0, CB); QF_RB(NB, 0, 1); DA2; \
    QF_MF(1, 1, CB); QF_RB(NB, 1, 1); DA3; \
    QF_MF(1, 2, CB); QF_RB(NB, 0, 2); \
    QF_MF(1, 3, CB); QF_RB(NB, 1, 2); DA4; \
    QF_MF(2, 0, CB); QF_RB(NB, 0, 3); DB0; \
    QF_MF(2, 1, CB); QF_RB(NB, 1, 3); \
    QF_MF(2, 2, CB); QF_RA(NB, 0, 1); DB1; \
    QF_MF(2, 3, CB); QF_RA(NB, 1, 1); DB2; \
    QF_MF(3, 0, CB); QF_RA(NB, 0, 2); \
    QF_MF(3, 1, CB); QF_RA(NB, 1, 2); DB3; \
    QF_MF(3, 2, CB); QF_RA(NB, 0, 3); DB4; \
    QF_MF(3, 3, CB); QF_RA(NB, 1, 3);
#define QF_STEP_D(CB, NB) \
    QF_STEP(CB, NB, QX_D0(a_vo, sa, dA), QX_D1(a_vo, sa, dA), \
            QX_D2(a_vo, sa, dA), QX_D3(a_vo, sa, dA), QX_D4(a_vo, sa, dA), \
            QX_D0(b_vo, sb, dB), QX_D1(b_vo, sb, dB), QX_D2(b_vo, sb, dB), \
            QX_D3(b_vo, sb, dB), QX_D4(b_vo, sb, dB))
#define QF_STEP_ND(CB, NB) QF_STEP(CB, NB, , , , , , , , , , )
#define QF_LAST(CB) \
    QF_MF(0, 0, CB); QF_MF(0, 1, CB); QF_MF(0, 2, CB); QF_MF(0, 3, CB); \
    QF_MF(1, 0, CB); QF_MF(1, 1, CB); QF_MF(1, 2, CB); QF_MF(1, 3, CB); \
    QF_MF(2, 0, CB); QF_MF(2, 1, CB); QF_MF(2, 2, CB); QF_MF(2, 3, CB); \
    QF_MF(3, 0, CB); QF_MF(3, 1, CB); QF_MF(3, 2, CB); QF_MF(3, 3, CB);

#if defined(QMM_B8X_PART) && QMM_B8X_PART == 3
__global__ void __launch_bounds__(b8x::NT, 1)
gemm_f8x_kernel(const gemm_params_t p) {
    using namespace b8x;
    typedef __attribute__((address_space(3))) uint8_t lds_u8;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm0 = (wave >> 1) * 128, wn0 = (wave & 1) * 128;

    const int ntiles = p.tiles_m * p.tiles_n;
    int lt;
    {
        const int per = (ntiles + 7) / 8;
        const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
        lt = xcd * per + slot;
        if (slot >= per || lt >= ntiles) return;
    }
    constexpr int GROUP_M = 8;
    const int group = lt / (GROUP_M * p.tiles_n);
    const int first_m = group * GROUP_M;
    const int gsz = min(p.tiles_m - first_m, GROUP_M);
    const int tile_m = first_m + (lt % (GROUP_M * p.tiles_n)) % gsz;
    const int tile_n = (lt % (GROUP_M * p.tiles_n)) / gsz;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int bz = blockIdx.y;

    const int KT = p.K / BK; // host guarantees K % 128 == 0 and KT >= 6
    const uint32_t lds_base = __builtin_amdgcn_readfirstlane(
            (uint32_t)(uintptr_t)(lds_u8 *)lds);

    uint32_t a_vo[4], b_vo[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int c = tid + j * NT;
        const int row = c >> 2, cp = c & 3;
        const int gm = min(m0 + row, p.M - 1) - m0;
        a_vo[j] = (uint32_t)gm * (uint32_t)p.lda + a_swz(row, cp) * 16;
        const int nbl = c >> 7, rem = c & 127;
        const int nb = min(n0 / 32 + nbl, p.nb32 - 1) - n0 / 32;
        b_vo[j] = (uint32_t)nb * (uint32_t)p.kb32 * 1024u + rem * 16;
    }
    auto sgpr_ptr = [](const uint8_t *q) {
        const uint64_t v = (uint64_t)q;
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
        const uint32_t hi
                = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
        return (const uint8_t *)(((uint64_t)hi << 32) | lo);
    };
    const uint8_t *sa = sgpr_ptr(
            p.A + (int64_t)bz * p.a_sb + (int64_t)m0 * p.lda);
    const uint8_t *sb = sgpr_ptr(p.B + (int64_t)bz * p.b_sb
            + (int64_t)(n0 / 32) * p.kb32 * 1024);
    uint32_t dA = lds_base + wave * 1024;
    uint32_t dB = dA + A_BYTES;

    // fragment offsets inside a stage
    const int arow = wm0 + (lane & 31);
    const int a_rel0 = arow * BK + a_swz(arow, (lane >> 5)) * 16;
    const int a_rel1 = arow * BK + a_swz(arow, 2 + (lane >> 5)) * 16;
    const int b_rel = A_BYTES + ((wn0 >> 5) * 128 + lane) * 16;

    v16f acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                acc[i][j][r] = 0.f;
    v4i fa[2][2][4], fb[2][2][4];

    {
        float s = 1.f;
        if (p.ep.src_scale.ptr)
            s = load_float(p.ep.src_scale.dt, p.ep.src_scale.ptr,
                    bz * p.ep.src_scale.sb
                            + (int64_t)min(m0 + tid, p.M - 1) * p.ep.src_scale.sm);
        ((float *)(lds + SS_OFF))[tid] = s;
    }

    // ---- prologue: tiles 0..3 requested (the whole ring); tile 0's
    // fragments read ----
    QX_FETCH(a_vo, sa, dA); QX_ADV_A();
    QX_FETCH(b_vo, sb, dB); QX_ADV_B();
    QX_FETCH(a_vo, sa, dA); QX_ADV_A();
    QX_FETCH(b_vo, sb, dB); QX_ADV_B();
    QX_FETCH(a_vo, sa, dA); QX_ADV_A();
    QX_FETCH(b_vo, sb, dB); QX_ADV_B();
    QX_FETCH(a_vo, sa, dA); QX_ADV_A();
    QX_FETCH(b_vo, sb, dB); QX_ADV_B();
    QX_WV(24);
    __syncthreads();
    uint32_t st = 0; // ring offset of the tile whose fragments are read next
    {
        const uint8_t *ldsn = lds;
        QX_SB();
        QF_RA(0, 0, 0); QF_RA(0, 1, 0);
        QF_RB(0, 0, 0); QF_RB(0, 1, 0); QF_RB(0, 0, 1); QF_RB(0, 1, 1);
        QF_RB(0, 0, 2); QF_RB(0, 1, 2); QF_RB(0, 0, 3); QF_RB(0, 1, 3);
        QF_RA(0, 0, 1); QF_RA(0, 1, 1); QF_RA(0, 0, 2); QF_RA(0, 1, 2);
        QF_RA(0, 0, 3); QF_RA(0, 1, 3);
    }
    // k-step kt: multiplies tile kt-1 (buffer (kt-1)&1), reads tile kt's
    // fragments, requests tile kt+3 into the stage tile kt-1 was read from
    // during the previous k-step
#define QF_KSTEP(WAITV, BODY) \
    { \
        st = (st + STAGE_BYTES) & (RING - 1); \
        const uint8_t *ldsn = lds + st; \
        QX_WV(WAITV); \
        __builtin_amdgcn_s_barrier(); \
        QX_SB(); \
        BODY \
    }
    for (int kt = 1; kt <= KT - 5; kt += 2) {
        QF_KSTEP(16, QF_STEP_D(0, 1) QX_ADV_A(); QX_ADV_B();)
        QF_KSTEP(16, QF_STEP_D(1, 0) QX_ADV_A(); QX_ADV_B();)
    }
    QF_KSTEP(16, QF_STEP_ND(0, 1)) // kt = KT-3
    QF_KSTEP(8, QF_STEP_ND(1, 0)) // kt = KT-2
    QF_KSTEP(0, QF_STEP_ND(0, 1)) // kt = KT-1
    QF_LAST(1)
    __syncthreads();

    tile_epilogue<true, true>(
            p, acc, lds, lds_base, wave, lane, m0, n0, wm0, wn0, bz);
}

#endif // fp8 kernel

// ---- fp8 on 16 x 16 x 128 MFMAs -------------------------------------------------
// v_mfma_f32_16x16x128_f8f6f4 contracts 128 k per instruction, i.e. two stages
// of the ring: a k-step is 128 k, 64 MFMAs of 32 cycles, and the ring holds two
// k-steps. Lane l of an operand holds row (column) l % 16 and 32 bytes of k:
// lane group g = l / 16 takes, from stage g / 2 of the pair, the 16-byte chunks
// g % 2 and g % 2 + 2 of the row -- two ds_read_b128 per fragment, measured free
// of bank conflicts with the 16-row swizzle; the B chunks of the packed tile that
// hold the same k are one 256-byte run per lane group.
// The fragments of a k-step are single-buffered (8 + 8 fragments of 8 registers)
// and the MFMAs walk the 8 x 8 fragment grid in growing squares, so that
// fragment n of either operand is first needed at MFMA n * n: fragments 4..7 are
// read during the first quarter of their own k-step, fragments 0..3 of the next
// k-step during the last quarter of this one, into a second register set; one
// memory instruction per MFMA slot throughout.
// Two barriers per k-step: after MFMA 17 every wave has read what it needs from
// this k-step's pair of stages, which then receives the k-step after next (16
// direct loads per wave); after MFMA 45 the next pair has landed for everyone
// and its first fragments are read.
// The 16 direct loads of a k-step are spread over MFMAs 9..62, about one in
// three (the second barrier's vmcnt counts the 12 issued before it): issued
// back to back (20 consecutive slots) they cost 18 % of the
// kernel's cycles, wherever in the k-step the cluster sat -- the L2 -> LDS path
// takes requests at a limited rate, and the stream has to be even.
// Measured (8192^3, MI355X): 2.50-2.59 PFLOP/s against 2.38-2.46 for the
// 32 x 32 x 64 loop in the same session, at 1.96-1.99 GHz against 1.5-1.7 GHz.
#define QZ_S(i, PS) ((i) < 4 ? (PS) : 0)
// The weights fragment is the first operand (transposed accumulator, see
// QY_MF). The MFMA is inline assembly with the accumulator constrained to an AGPR:
// with the builtin, the register allocator kept part of the accumulators in
// VGPRs on some paths and moved them at every loop seam (60 v_accvgpr_read per
// two k-steps, each waiting for its MFMA). Operand waits are still the
// compiler's (it sees the loads that feed the "v" operands); the accumulator of
// one MFMA is next touched 64 MFMAs later.
#define QZ_MF(i, j, PS) \
    { \
        QX_SB(); \
        asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %2, %1, %0" \
                     : "+a"(acc[i][j]) \
                     : "v"(__builtin_shufflevector(fal[QZ_S(i, PS)][i], \
                               fah[QZ_S(i, PS)][i], 0, 1, 2, 3, 4, 5, 6, 7)), \
                     "v"(__builtin_shufflevector(fbl[QZ_S(j, PS)][j], \
                             fbh[QZ_S(j, PS)][j], 0, 1, 2, 3, 4, 5, 6, 7))); \
        QX_SB(); \
    }
// one ds_read_b128 each: with 32-cycle MFMAs a single memory instruction
// between two MFMAs is hidden, two are not
#define QZ_RA_LO(S, i, base) \
    { \
        fal[S][i] = *(const v4i *)((base) + a_lo + (i)*1024); \
        QX_SB(); \
    }
#define QZ_RA_HI(S, i, base) \
    { \
        fah[S][i] = *(const v4i *)((base) + a_hi + (i)*1024); \
        QX_SB(); \
    }
#define QZ_RB_LO(S, j, base) \
    { \
        fbl[S][j] = *(const v4i *)((base) + b_lo + ((j) >> 1) * 2048 + ((j)&1) * 256); \
        QX_SB(); \
    }
#define QZ_RB_HI(S, j, base) \
    { \
        fbh[S][j] = *(const v4i *)((base) + b_lo + 1024 + ((j) >> 1) * 2048 + ((j)&1) * 256); \
        QX_SB(); \
    }
#define QZ_RA(S, i, base) QZ_RA_LO(S, i, base) QZ_RA_HI(S, i, base)
#define QZ_RB(S, j, base) QZ_RB_LO(S, j, base) QZ_RB_HI(S, j, base)
// DMA(x): x when this k-step requests the one after next, PRE(x): x when a
// next k-step exists; QZ_BAR_A / QZ_BAR_B as described above
#define QZ_STEP_BODY(PS, NS, DMA, PRE, QZ_BAR_A, QZ_BAR_B) \
    QZ_MF(0, 0, PS); QZ_RA_LO(0, 4, ldsc); QZ_RA_HI(0, 4, ldsc); \
    QZ_MF(0, 1, PS); QZ_RB_LO(0, 4, ldsc); QZ_RB_HI(0, 4, ldsc); \
    QZ_MF(1, 1, PS); QZ_RA_LO(0, 5, ldsc); QZ_RA_HI(0, 5, ldsc); \
    QZ_MF(1, 0, PS); QZ_RB_LO(0, 5, ldsc); QZ_RB_HI(0, 5, ldsc); \
    QZ_MF(0, 2, PS); QZ_RA_LO(0, 6, ldsc); QZ_RA_HI(0, 6, ldsc); \
    QZ_MF(1, 2, PS); QZ_RB_LO(0, 6, ldsc); QZ_RB_HI(0, 6, ldsc); \
    QZ_MF(2, 2, PS); QZ_RA_LO(0, 7, ldsc); QZ_RA_HI(0, 7, ldsc); \
    QZ_MF(2, 1, PS); QZ_RB_LO(0, 7, ldsc); QZ_RB_HI(0, 7, ldsc); \
    QZ_MF(2, 0, PS); QZ_BAR_A; \
    QZ_MF(0, 3, PS); DMA(QX_D0(a_vo, sa, dA)); \
    QZ_MF(1, 3, PS); \
    QZ_MF(2, 3, PS); \
    QZ_MF(3, 3, PS); DMA(QX_D1(a_vo, sa, dA)); \
    QZ_MF(3, 2, PS); \
    QZ_MF(3, 1, PS); \
    QZ_MF(3, 0, PS); DMA(QX_D2(a_vo, sa, dA)); \
    QZ_MF(0, 4, PS); \
    QZ_MF(1, 4, PS); DMA(QX_D3(a_vo, sa, dA)); \
    QZ_MF(2, 4, PS); \
    QZ_MF(3, 4, PS); \
    QZ_MF(4, 4, PS); DMA(QX_D4(a_vo, sa, dA)); DMA(QZ_ADV_A()); \
    QZ_MF(4, 3, PS); \
    QZ_MF(4, 2, PS); \
    QZ_MF(4, 1, PS); DMA(QX_D0(a_vo, sa, dA)); \
    QZ_MF(4, 0, PS); \
    QZ_MF(0, 5, PS); \
    QZ_MF(1, 5, PS); DMA(QX_D1(a_vo, sa, dA)); \
    QZ_MF(2, 5, PS); \
    QZ_MF(3, 5, PS); \
    QZ_MF(4, 5, PS); DMA(QX_D2(a_vo, sa, dA)); \
    QZ_MF(5, 5, PS); \
    QZ_MF(5, 4, PS); DMA(QX_D3(a_vo, sa, dA)); \
    QZ_MF(5, 3, PS); \
    QZ_MF(5, 2, PS); \
    QZ_MF(5, 1, PS); DMA(QX_D4(a_vo, sa, dA)); DMA(QZ_ADV_A()); \
    QZ_MF(5, 0, PS); \
    QZ_MF(0, 6, PS); \
    QZ_MF(1, 6, PS); DMA(QX_D0(b_vo, sb, dB)); \
    QZ_MF(2, 6, PS); \
    QZ_MF(3, 6, PS); \
    QZ_MF(4, 6, PS); DMA(QX_D1(b_vo, sb, dB)); \
    QZ_MF(5, 6, PS); \
    QZ_MF(6, 6, PS); \
    QZ_MF(6, 5, PS); DMA(QX_D2(b_vo, sb, dB)); \
    QZ_MF(6, 4, PS); \
    QZ_MF(6, 3, PS); DMA(QX_D3(b_vo, sb, dB)); \
    QZ_MF(6, 2, PS); \
    QZ_MF(6, 1, PS); \
    QZ_MF(6, 0, PS); DMA(QX_D4(b_vo, sb, dB)); DMA(QZ_ADV_B()); \
    QZ_MF(0, 7, PS); QZ_BAR_B; \
    QZ_MF(1, 7, PS); PRE(QZ_RA_LO(NS, 0, ldsn)); PRE(QZ_RA_HI(NS, 0, ldsn)); \
    QZ_MF(2, 7, PS); PRE(QZ_RB_LO(NS, 0, ldsn)); PRE(QZ_RB_HI(NS, 0, ldsn)); DMA(QX_D0(b_vo, sb, dB)); \
    QZ_MF(3, 7, PS); PRE(QZ_RA_LO(NS, 1, ldsn)); \
    QZ_MF(4, 7, PS); PRE(QZ_RA_HI(NS, 1, ldsn)); \
    QZ_MF(5, 7, PS); PRE(QZ_RB_LO(NS, 1, ldsn)); DMA(QX_D1(b_vo, sb, dB)); \
    QZ_MF(6, 7, PS); PRE(QZ_RB_HI(NS, 1, ldsn)); \
    QZ_MF(7, 7, PS); PRE(QZ_RA_LO(NS, 2, ldsn)); \
    QZ_MF(7, 6, PS); PRE(QZ_RA_HI(NS, 2, ldsn)); DMA(QX_D2(b_vo, sb, dB)); \
    QZ_MF(7, 5, PS); PRE(QZ_RB_LO(NS, 2, ldsn)); \
    QZ_MF(7, 4, PS); PRE(QZ_RB_HI(NS, 2, ldsn)); DMA(QX_D3(b_vo, sb, dB)); \
    QZ_MF(7, 3, PS); PRE(QZ_RA_LO(NS, 3, ldsn)); \
    QZ_MF(7, 2, PS); PRE(QZ_RA_HI(NS, 3, ldsn)); \
    QZ_MF(7, 1, PS); PRE(QZ_RB_LO(NS, 3, ldsn)); DMA(QX_D4(b_vo, sb, dB)); DMA(QZ_ADV_B()); \
    QZ_MF(7, 0, PS); PRE(QZ_RB_HI(NS, 3, ldsn));
// advance to the next 64-k tile, staying on the last one once it is reached
#define QZ_ADV_A() \
    { \
        const int go = adv_a > 0; \
        sa += go ? BK : 0; \
        adv_a -= go; \
        dA = ((dA - lds_base + STAGE_BYTES) & (RING - 1)) + lds_base; \
    }
#define QZ_ADV_B() \
    { \
        const int go = adv_b > 0; \
        sb += go ? 2048 : 0; \
        adv_b -= go; \
        dB = ((dB - lds_base + STAGE_BYTES) & (RING - 1)) + lds_base; \
    }
#define QZ_ON(x) x
#define QZ_OFF(x)
// every wave has issued its reads of this pair of stages: the requests that
// follow land hundreds of cycles later, LDS serves a wave's reads in order
#define QZ_BARRIER_A \
    { \
        __builtin_amdgcn_s_barrier(); \
        QX_SB(); \
    }
#define QZ_BARRIER_B(WAITV) \
    { \
        QX_WV(WAITV); \
        __builtin_amdgcn_s_barrier(); \
        QX_SB(); \
    }
#define QZ_NONE \
    { }

#if defined(QMM_B8X_PART) && QMM_B8X_PART == 6
__global__ void __launch_bounds__(b8x::NT, 1)
gemm_f8y_kernel(const gemm_params_t p) {
    using namespace b8x;
    typedef __attribute__((address_space(3))) uint8_t lds_u8;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm0 = (wave >> 1) * 128, wn0 = (wave & 1) * 128;
    const uint32_t lds_base = __builtin_amdgcn_readfirstlane(
            (uint32_t)(uintptr_t)(lds_u8 *)lds);
    const int bz = blockIdx.y;
    const int KS = p.K / 128; // host guarantees K % 256 == 0 and KS >= 4

    // persistent, as gemm_b8y_kernel: workgroup w of an XCD walks the tiles
    // w, w + W, ... of the XCD's share
    const int ntiles = p.tiles_m * p.tiles_n;
    const int per = (ntiles + 7) / 8;
    const int xcd = blockIdx.x & 7, W = gridDim.x >> 3;
    for (int slot = blockIdx.x >> 3; slot < per; slot += W) {
    const int lt = xcd * per + slot;
    if (lt >= ntiles) break;
    constexpr int GROUP_M = 8;
    const int group = lt / (GROUP_M * p.tiles_n);
    const int first_m = group * GROUP_M;
    const int gsz = min(p.tiles_m - first_m, GROUP_M);
    const int tile_m = first_m + (lt % (GROUP_M * p.tiles_n)) % gsz;
    const int tile_n = (lt % (GROUP_M * p.tiles_n)) / gsz;
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    uint32_t a_vo[4], b_vo[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int c = tid + j * NT;
        const int row = c >> 2, cp = c & 3;
        const int gm = min(m0 + row, p.M - 1) - m0;
        a_vo[j] = (uint32_t)gm * (uint32_t)p.lda + a_swz16(row, cp) * 16;
        const int nbl = c >> 7, rem = c & 127;
        const int nb = min(n0 / 32 + nbl, p.nb32 - 1) - n0 / 32;
        b_vo[j] = (uint32_t)nb * (uint32_t)p.kb32 * 1024u + rem * 16;
    }
    auto sgpr_ptr = [](const uint8_t *q) {
        const uint64_t v = (uint64_t)q;
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
        const uint32_t hi
                = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
        return (const uint8_t *)(((uint64_t)hi << 32) | lo);
    };
    const uint8_t *sa = sgpr_ptr(
            p.A + (int64_t)bz * p.a_sb + (int64_t)m0 * p.lda);
    const uint8_t *sb = sgpr_ptr(p.B + (int64_t)bz * p.b_sb
            + (int64_t)(n0 / 32) * p.kb32 * 1024);
    uint32_t dA = lds_base + wave * 1024;
    uint32_t dB = dA + A_BYTES;
    // tile advances left after the four of the prologue
    int adv_a = p.K / BK - 5, adv_b = p.K / BK - 5;

    // fragment offsets inside a pair of stages
    const int g = lane >> 4;
    const int arow = wm0 + (lane & 15);
    const int a_lo = (g >> 1) * STAGE_BYTES + arow * BK
            + a_swz16(arow, g & 1) * 16;
    const int a_hi = (g >> 1) * STAGE_BYTES + arow * BK
            + a_swz16(arow, (g & 1) + 2) * 16;
    const int b_lo = (g >> 1) * STAGE_BYTES + A_BYTES + (wn0 >> 5) * 2048
            + (g & 1) * 512 + (lane & 15) * 16;
    const uint8_t *const pair0 = lds, *const pair1 = lds + 2 * STAGE_BYTES;

    v4f acc[8][8];
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int j = 0; j < 8; j++)
#pragma unroll
            for (int r = 0; r < 4; r++)
                acc[i][j][r] = 0.f;
    // [set][fragment], low and high 16 bytes of each lane's 32; set 1 only for
    // fragments 0..3
    v4i fal[2][8], fah[2][8], fbl[2][8], fbh[2][8];

    tile_operands_stage(p, lds, tid, m0, n0, bz);

    // ---- prologue: k-steps 0 and 1 requested (the whole ring); the first
    // fragments of k-step 0 read ----
    QX_FETCH(a_vo, sa, dA); QX_ADV_A();
    QX_FETCH(b_vo, sb, dB); QX_ADV_B();
    QX_FETCH(a_vo, sa, dA); QX_ADV_A();
    QX_FETCH(b_vo, sb, dB); QX_ADV_B();
    QX_FETCH(a_vo, sa, dA); QX_ADV_A();
    QX_FETCH(b_vo, sb, dB); QX_ADV_B();
    QX_FETCH(a_vo, sa, dA); QX_ADV_A();
    QX_FETCH(b_vo, sb, dB); QX_ADV_B();
    QX_WV(16);
    __syncthreads();
    QX_SB();
    QZ_RA(0, 0, pair0); QZ_RB(0, 0, pair0); QZ_RA(0, 1, pair0);
    QZ_RB(0, 1, pair0); QZ_RA(0, 2, pair0); QZ_RB(0, 2, pair0);
    QZ_RA(0, 3, pair0); QZ_RB(0, 3, pair0);

    // k-step t works on pair t % 2 with fragment set t % 2 for fragments 0..2
#define QZ_STEP_FULL(PS, NS, CUR, NXT) \
    { \
        const uint8_t *const ldsc = CUR, *const ldsn = NXT; \
        QZ_STEP_BODY(PS, NS, QZ_ON, QZ_ON, QZ_BARRIER_A, QZ_BARRIER_B(12)) \
    }
    // One code path for every k-step, so that each accumulator keeps its
    // register from the first MFMA to the epilogue (at the seam between a loop
    // and separate tail copies the register allocator permutes them, and it
    // cannot know that the inline-assembly MFMAs are still writing): the last
    // two k-steps request again what the ring already holds -- the source
    // pointers stop advancing at the last tile -- into stages nobody reads any
    // more, and read "next" fragments that are never used.
    for (int t = 0; t < KS; t += 2) {
        QZ_STEP_FULL(0, 1, pair0, pair1)
        QZ_STEP_FULL(1, 0, pair1, pair0)
    }
    // the last MFMAs are still writing (16 passes), and the surplus requests
    // must have landed before the ring is reused as staging
    asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
    QX_WV(0);
    __syncthreads();

    tile_epilogue<true, true>(
            p, acc, lds, lds_base, wave, lane, m0, n0, wm0, wn0, bz);
    // the staging area and the operand tables are the next tile's ring and
    // tables
    __syncthreads();
    } // tiles of this workgroup
}
#endif // fp8, 16 x 16 x 128


template <typename K>
static void launch_b8x(K kern, const gemm_params_t &p, hipStream_t stream) {
    using namespace b8x;
    gemm_params_t q = p;
    q.tiles_m = (p.M + BM - 1) / BM;
    q.tiles_n = (p.N + BN - 1) / BN;
    const int ntiles = q.tiles_m * q.tiles_n;
    const int grid_x = ((ntiles + 7) / 8) * 8;
    ensure_dynamic_lds((const void *)kern, LDS_TOTAL);
    hipLaunchKernelGGL(kern, dim3(grid_x, p.batch), dim3(NT), LDS_TOTAL,
            stream, q);
}

// The persistent kernel: W workgroups per XCD, one per CU (fewer when an XCD's
// share of the tiles is smaller). GEMM_NOT_PERSISTENT: one workgroup per tile.
static int cus_per_xcd() {
    static int n = 0;
    if (!n) {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess
                || hipDeviceGetAttribute(
                           &cus, hipDeviceAttributeMultiprocessorCount, dev)
                        != hipSuccess
                || cus < 8)
            cus = 256;
        n = cus / 8;
    }
    return n;
}
template <typename K>
static void launch_b8y_persistent(
        K kern, const gemm_params_t &p, hipStream_t stream) {
    using namespace b8x;
    gemm_params_t q = p;
    q.tiles_m = (p.M + BM - 1) / BM;
    q.tiles_n = (p.N + BN - 1) / BN;
    const int per = (q.tiles_m * q.tiles_n + 7) / 8;
    const int W = (p.switches & GEMM_NOT_PERSISTENT)
            ? per
            : std::min(cus_per_xcd(), per);
    ensure_dynamic_lds((const void *)kern, LDS_TOTAL);
    hipLaunchKernelGGL(
            kern, dim3(8 * W, p.batch), dim3(NT), LDS_TOTAL, stream, q);
}

// One kernel per translation unit (QMM_B8X_PART), so that they build in
// parallel; the unit without the macro holds the dispatcher.
#if defined(QMM_B8X_PART)
#if QMM_B8X_PART == 1
void launch_b8x_int8(const gemm_params_t &p, hipStream_t stream) {
    launch_b8x(gemm_b8x_kernel<false>, p, stream);
}
#elif QMM_B8X_PART == 2
void launch_b8x_short_k(const gemm_params_t &p, hipStream_t stream) {
    launch_b8x(gemm_b8x_kernel<true>, p, stream);
}
#elif QMM_B8X_PART == 3
void launch_b8x_fp8(const gemm_params_t &p, hipStream_t stream) {
    launch_b8x(gemm_f8x_kernel, p, stream);
}
#elif QMM_B8X_PART == 4
void launch_b8x_int8_mi16(const gemm_params_t &p, hipStream_t stream) {
    launch_b8y_persistent(gemm_b8y_kernel<false>, p, stream);
}
int gemm_stamps_read_int8(void *host, size_t bytes) {
    // through pinned memory, as every other copy of the library to the host
    void *pinned = nullptr;
    if (hipHostMalloc(&pinned, bytes, hipHostMallocDefault) != hipSuccess)
        return 0;
    const bool ok = hipMemcpyFromSymbol(pinned, HIP_SYMBOL(g_gemm_stamps), bytes,
                            0, hipMemcpyDeviceToHost)
            == hipSuccess;
    if (ok) memcpy(host, pinned, bytes);
    (void)hipHostFree(pinned);
    return ok;
}
#elif QMM_B8X_PART == 5
void launch_b8x_int8_mi16_odd(const gemm_params_t &p, hipStream_t stream) {
    launch_b8y_persistent(gemm_b8y_kernel<true>, p, stream);
}
#elif QMM_B8X_PART == 6
void launch_b8x_fp8_mi16(const gemm_params_t &p, hipStream_t stream) {
    launch_b8y_persistent(gemm_f8y_kernel, p, stream);
}

#endif
#else
void launch_b8x_fp8_mi16(const gemm_params_t &p, hipStream_t stream);
void launch_b8x_int8_two_per_cu(const gemm_params_t &p, hipStream_t stream);
int gemm_stamps_read_int8(void *host, size_t bytes);
void launch_b8x_int8_mi16(const gemm_params_t &p, hipStream_t stream);
void launch_b8x_int8_mi16_odd(const gemm_params_t &p, hipStream_t stream);
void launch_b8x_int8(const gemm_params_t &p, hipStream_t stream);
void launch_b8x_short_k(const gemm_params_t &p, hipStream_t stream);
void launch_b8x_fp8(const gemm_params_t &p, hipStream_t stream);
bool gemm_b8x_two_per_cu(const gemm_params_t &p, bool f8);

// Problems the kernels take: K a multiple of 64; s8 sources (u8 too when K is
// at most 256, or rewritten as s8 by the caller), or fp8 sources with K a
// multiple of 128 and at least 6 k-steps; 32-bit addressable tiles. Whether
// there are enough 256 x 256 tiles to occupy the chip is the caller's call.
static bool short_k(const gemm_params_t &p) {
    return p.K <= 4 * 64;
}

bool gemm_b8x_eligible(const gemm_params_t &p, bool f8) {
    if (p.K % 64 != 0 || p.K < 64) return false;
    // weights zero points: the kernels on 16 x 16 MFMAs (their epilogue's row path)
    if (p.rowsum && (f8 || (p.switches & GEMM_MFMA32) || p.K < 5 * 64))
        return false;
    if (f8 && (p.K % 128 != 0 || p.K < 6 * 64)) return false;
    if (p.a_is_u8 && !p.a_preflipped && !short_k(p)
            && !gemm_b8x_two_per_cu(p, f8))
        return false;
    if ((int64_t)256 * p.lda + 64 >= ((int64_t)1 << 32)) return false;
    if ((int64_t)8 * p.kb32 * 1024 >= ((int64_t)1 << 32)) return false;
    return true;
}

// Whether launch_gemm_b8x() takes the 256 x 128 kernel with two workgroups per
// CU (which also reads u8 sources as they are).
bool gemm_b8x_two_per_cu(const gemm_params_t &p, bool f8) {
    const int64_t tiles256 = (int64_t)((p.M + 255) / 256) * ((p.N + 255) / 256)
            * p.batch;
    return !f8 && !(p.switches & (GEMM_MFMA32 | GEMM_ONE_PER_CU))
            && ((p.switches & GEMM_TWO_PER_CU) || p.K <= 2048 || tiles256 <= 170
                    || (p.rowsum != nullptr
                            && (tiles256 >= 512
                                    || (p.a_is_u8 && !p.a_preflipped))));
}

// By default int8 runs on 16 x 16 x 64 MFMAs and fp8 on 16 x 16 x 128 (K a
// multiple of 256, at least 512) where they apply. int8 with an s8 source has
// two tilings: 256 x 256 with one workgroup per CU (the most MFMAs per byte
// moved into LDS: the faster main loop, 1185 against 1240 cycles per 64 MFMAs
// and SIMD) and 256 x 128 with two per CU (a workgroup's prologue, epilogue and
// dst stream run under the other's MFMAs). Measured on 4096 x K x 14336 with a
// swish / bf16 epilogue, two per CU over one per CU: K 128 0.77, 256 0.74, 512
// 0.85, 1024 0.89, 2048 0.96, 4096 1.09, 8192 1.12 of the time; on the batched
// attention scores (K 128, f32 dst bound by its write stream) 0.84; and 0.79
// where the 256 x 256 tiles number half the CUs (2048 x 4096 x 4096). So: two
// per CU up to K 2048, and beyond that where the large tiles would leave more
// than a third of the CUs without one. Weights with zero points (p.rowsum): two
// per CU at any K once every CU gets two rounds of tiles, the epilogue's
// correction pass over the staged sums then runs under the other workgroup's
// MFMAs (s8:u8:f16 with a zero point per column, 4096 x 4096 x 14336: 200
// against 213 us; 1024 rows: 66 against 63), and always for a u8 source, which
// only that kernel reads as it is. Plan-level switches override the choice
// (GEMM_MFMA32: the 32 x 32 loops; GEMM_TWO_PER_CU / GEMM_ONE_PER_CU).
void launch_gemm_b8x(const gemm_params_t &p, bool f8, hipStream_t stream) {
    const int variant = (p.switches & GEMM_MFMA32) ? 0 : 1;
    const bool two_per_cu = gemm_b8x_two_per_cu(p, f8);
    if (f8 && variant >= 1 && p.K % 256 == 0 && p.K >= 4 * 128)
        launch_b8x_fp8_mi16(p, stream);
    else if (f8)
        launch_b8x_fp8(p, stream);
    else if (two_per_cu)
        launch_b8x_int8_two_per_cu(p, stream); // any K: surplus tiles are phantom
    else if (short_k(p))
        launch_b8x_short_k(p, stream);
    else if (variant >= 1 && p.K >= 5 * 64) {
        if ((p.K / 64) & 1)
            launch_b8x_int8_mi16_odd(p, stream);
        else
            launch_b8x_int8_mi16(p, stream);
    }
    else
        launch_b8x_int8(p, stream);
}
#endif

} // namespace qmm

#if !defined(QMM_B8X_PART)
extern "C" int qmm_gemm_stamps_read(void *host, size_t bytes) {
    if (!host
            || bytes > sizeof(unsigned long long) * qmm::STAMP_TILES
                            * qmm::STAMP_SLOTS * 2)
        return QMM_INVALID_ARGUMENTS;
    return qmm::gemm_stamps_read_int8(host, bytes) ? QMM_OK : QMM_RUNTIME_ERROR;
}
#endif
