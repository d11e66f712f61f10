// hip:gfx950:mfma_b8 -- int8 (u8/s8 x s8 -> s32) and fp8 (e4m3 x e4m3 -> f32)
// GEMM on the CDNA4 matrix cores with a fused epilogue.
//
// Layout of the work:
//   * weights arrive prepacked in MFMA operand order (QMM_LAYOUT_MFMA_B8): a
//     32-column x 32-k fragment is 1 KiB, lane l holds column l%32 and the 16
//     k-bytes of half l/32, so a tile of the B operand is a plain contiguous
//     copy global -> LDS and the ds_read_b128 of a wave is conflict free;
//   * the source rows are staged row-major in LDS with an XOR swizzle of the
//     16-byte chunks, which keeps both the coalesced global load (a row's
//     BK bytes by consecutive lanes) and the fragment reads (32 rows x 16 B)
//     spread over all 64 banks;
//   * a block of 4 waves owns a BM x BN tile, each wave WM x WN of it as
//     FM x FN v_mfma_i32_32x32x32_i8 (or v_mfma_f32_32x32x64_f8f6f4)
//     accumulators; LDS is double buffered, the next tile's global loads are
//     in flight while the current one is multiplied;
//   * u8 sources are turned into s8 by flipping the top bit and the missing
//     128 * colsum(W)[n] (and the source zero point, -zp * colsum(W)[n]) is
//     added to the s32 accumulator from the column sums stored behind the
//     packed weights (identity of
//     src/cpu/matmul/gemm_x8s8s32x_matmul.cpp:165-193) -- exact in s32;
//   * the epilogue follows src/cpu/matmul/ref_matmul_int8.cpp:195-259 step by
//     step: (float)acc, * src scale, * weights scale, + bias, post-ops,
//     * 1/dst scale, + dst zero point, saturating store.
//
// Blocks are numbered so that the eight XCDs (each with its own L2) work on
// disjoint column ranges of the weights, and consecutive blocks of an XCD
// share source rows.
#include <type_traits>

#include "qmm_device.hpp"
#include "qmm_plan.hpp"

namespace qmm {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

template <bool F8>
struct acc_traits;
template <>
struct acc_traits<false> {
    typedef v16i type;
};
template <>
struct acc_traits<true> {
    typedef v16f type;
};

// compile-time loop: the body sees its index as a constant, so accumulator
// arrays indexed by it stay in registers whatever the optimizer decides about
// the loops inside the body
template <int N, typename F>
QMM_D void static_for(F &&f) {
    if constexpr (N > 0) {
        static_for<N - 1>(f);
        f(std::integral_constant<int, N - 1> {});
    }
}

// chunk swizzle of the row-major A tile: CH 16-byte chunks per row
template <int CH>
QMM_D int a_swz(int row, int q) {
    constexpr int ROWS_PER_256B = 16 / CH;
    return q ^ ((row / ROWS_PER_256B) % CH);
}

// One lane's 16 bytes from global memory straight into LDS: the wave's 64 lanes
// fill the 1 KiB at `lds_addr` (wave-uniform byte address) in lane order.
// Written as assembly on purpose: the compiler orders every later LDS read
// after a direct-to-LDS load it knows about with a full vmcnt(0), which would
// serialise the pipeline below; completion is tracked by hand with
// wait_vmcnt() + the block barrier.
QMM_D void load_to_lds16(const void *gptr, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %1\n\t"
                 "s_nop 0\n\t"
                 "global_load_lds_dwordx4 %0, off"
                 :
                 : "v"(gptr), "s"(lds_addr)
                 : "memory", "m0");
}

// s_waitcnt immediate for "at most n vector-memory operations outstanding"
// (gfx9 encoding: vmcnt in bits 3:0 and 15:14; expcnt / lgkmcnt left open)
constexpr int vmcnt_imm(int n) {
    return (n & 15) | ((n >> 4) << 14) | (7 << 4) | (15 << 8);
}

template <int BM, int BN, int BK, int WGM, int WGN, int STAGES, bool F8,
        bool U8A>
__global__ void __launch_bounds__(WGM *WGN * 64,
        (BM / WGM) * (BN / WGN) <= 128 * 64 ? 2 : 1)
gemm_b8_kernel(const gemm_params_t p) {
    constexpr int NT = WGM * WGN * 64;
    constexpr int WM = BM / WGM, WN = BN / WGN;
    constexpr int FM = WM / 32, FN = WN / 32;
    constexpr int KF = BK / 32; // k32 fragments per tile
    constexpr int CH = BK / 16; // 16-byte chunks per A row
    constexpr int A_BYTES = BM * BK, B_BYTES = BN * BK;
    constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
    constexpr int A_CH = A_BYTES / 16 / NT, B_CH = B_BYTES / 16 / NT;
    constexpr int LOADS = A_CH + B_CH; // vector loads per thread and tile
    static_assert(A_CH * 16 * NT == A_BYTES && B_CH * 16 * NT == B_BYTES, "");
    static_assert(!F8 || (KF % 2 == 0), "fp8 MFMA consumes 64 k per step");
    static_assert(STAGES >= 2 && STAGES <= 4, "");
    typedef typename acc_traits<F8>::type acc_t;
    typedef __attribute__((address_space(3))) uint8_t lds_u8;

    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm0 = (wave / WGN) * WM;
    const int wn0 = (wave % WGN) * WN;

    // ---- XCD-aware tile order ----
    // Hardware hands consecutive block ids to the 8 XCDs round robin. Give
    // XCD x the logical tiles [x*per, (x+1)*per): consecutive logical tiles
    // run on one XCD and share its L2. Logical order is n-major within groups
    // of GROUP_M row tiles, so neighbours share weight columns and src rows.
    const int ntiles = p.tiles_m * p.tiles_n;
    int lt = blockIdx.x;
    {
        const int per = (ntiles + 7) / 8;
        const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
        if (ntiles >= 64) {
            lt = xcd * per + slot;
            if (slot >= per || lt >= ntiles) return;
        }
    }
    constexpr int GROUP_M = 8;
    const int group = lt / (GROUP_M * p.tiles_n);
    const int first_m = group * GROUP_M;
    const int gsz = min(p.tiles_m - first_m, GROUP_M);
    const int tile_m = first_m + (lt % (GROUP_M * p.tiles_n)) % gsz;
    const int tile_n = (lt % (GROUP_M * p.tiles_n)) / gsz;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int bz = blockIdx.y;

    const uint8_t *__restrict__ A = p.A + (int64_t)bz * p.a_sb;
    const uint8_t *__restrict__ B = p.B + (int64_t)bz * p.b_sb;

    acc_t acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; i++)
#pragma unroll
        for (int j = 0; j < FN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                acc[i][j][r] = 0;

    // ---- global -> LDS without registers ----
    // A wave-wide global_load_lds_dwordx4 drops lane l's 16 bytes at
    // M0-base + 16*l: the LDS image of one instruction is 1 KiB contiguous and
    // any permutation has to happen on the global side. For the weights the
    // packed layout already is the LDS image. For the source tile the image is
    // [row][BK] with the 16-byte chunks of a row XOR-swizzled, so the lane that
    // fills chunk position cp of row r fetches chunk cp ^ swz(r) of that row:
    // still the same BK contiguous bytes per row, fully coalesced.
    // Loads carry no predicate: rows past M and column blocks past the packed
    // N re-read the last valid ones (their accumulators are never stored), k
    // past K re-reads the row's last 16 valid bytes, which meet the zero
    // padding of the packed weights (fp8 launches have K % BK == 0).
    const int KT = (p.K + BK - 1) / BK;
    const uint8_t *a_ptr[A_CH];
    int a_k[A_CH];
#pragma unroll
    for (int j = 0; j < A_CH; j++) {
        const int c = tid + j * NT;
        const int row = c / CH, cp = c % CH;
        const int gm = min(m0 + row, p.M - 1);
        a_ptr[j] = A + (int64_t)gm * p.lda;
        a_k[j] = a_swz<CH>(row, cp) * 16;
    }
    const uint8_t *b_ptr[B_CH];
#pragma unroll
    for (int j = 0; j < B_CH; j++) {
        const int c = tid + j * NT;
        const int nbl = c / (KF * 64), rem = c % (KF * 64);
        const int nb = min(n0 / 32 + nbl, p.nb32 - 1);
        b_ptr[j] = B + (int64_t)nb * p.kb32 * 1024 + rem * 16;
    }

    const uint32_t lds_base = __builtin_amdgcn_readfirstlane(
            (uint32_t)(uintptr_t)(lds_u8 *)lds);
    auto issue = [&](int kt) {
        const int stage = kt % STAGES;
        const uint32_t As = lds_base + stage * STAGE_BYTES;
        const uint32_t Bs = As + A_BYTES;
#pragma unroll
        for (int j = 0; j < A_CH; j++) {
            const int gk = min(kt * BK + a_k[j], p.K - 16);
            load_to_lds16(a_ptr[j] + gk, As + (j * NT + wave * 64) * 16);
        }
#pragma unroll
        for (int j = 0; j < B_CH; j++)
            load_to_lds16(b_ptr[j] + (int64_t)kt * (KF * 1024),
                    Bs + (j * NT + wave * 64) * 16);
    };

    // prologue: STAGES-1 tiles in flight
#pragma unroll
    for (int s = 0; s < STAGES - 1; s++)
        if (s < KT) issue(s);

    for (int kt = 0; kt < KT; kt++) {
        // tile kt has landed once at most the loads of the younger tiles in
        // flight remain; the barrier publishes it to the other waves and
        // guarantees everybody is done with the stage that is refilled next
        if (kt + STAGES - 2 < KT)
            __builtin_amdgcn_s_waitcnt(vmcnt_imm((STAGES - 2) * LOADS));
        else
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
        __syncthreads();
        if (kt + STAGES - 1 < KT) issue(kt + STAGES - 1);

        const uint8_t *As = lds + (kt % STAGES) * STAGE_BYTES;
        const uint8_t *Bs = As + A_BYTES;
        if constexpr (!F8) {
#pragma unroll
            for (int ki = 0; ki < KF; ki++) {
                v4i a[FM], b[FN];
#pragma unroll
                for (int i = 0; i < FM; i++) {
                    const int row = wm0 + i * 32 + (lane & 31);
                    const int q = ki * 2 + (lane >> 5);
                    uint4 v = *(const uint4 *)(As + row * BK
                            + a_swz<CH>(row, q) * 16);
                    if constexpr (U8A) { // u8 source -> s8: flip the top bits
                        v.x ^= 0x80808080u;
                        v.y ^= 0x80808080u;
                        v.z ^= 0x80808080u;
                        v.w ^= 0x80808080u;
                    }
                    a[i] = v4i {(int)v.x, (int)v.y, (int)v.z, (int)v.w};
                }
#pragma unroll
                for (int j = 0; j < FN; j++) {
                    const uint4 v = *(const uint4 *)(Bs
                            + ((((wn0 >> 5) + j) * KF + ki) * 64 + lane) * 16);
                    b[j] = v4i {(int)v.x, (int)v.y, (int)v.z, (int)v.w};
                }
#pragma unroll
                for (int i = 0; i < FM; i++)
#pragma unroll
                    for (int j = 0; j < FN; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
                                a[i], b[j], acc[i][j], 0, 0, 0);
            }
        } else {
#pragma unroll
            for (int ki = 0; ki < KF; ki += 2) {
                v8i a[FM], b[FN];
#pragma unroll
                for (int i = 0; i < FM; i++) {
                    const int row = wm0 + i * 32 + (lane & 31);
                    const int q0 = ki * 2 + (lane >> 5);
                    const uint4 v0 = *(const uint4 *)(As + row * BK
                            + a_swz<CH>(row, q0) * 16);
                    const uint4 v1 = *(const uint4 *)(As + row * BK
                            + a_swz<CH>(row, q0 + 2) * 16);
                    a[i] = v8i {(int)v0.x, (int)v0.y, (int)v0.z, (int)v0.w,
                            (int)v1.x, (int)v1.y, (int)v1.z, (int)v1.w};
                }
#pragma unroll
                for (int j = 0; j < FN; j++) {
                    const uint8_t *bp = Bs
                            + ((((wn0 >> 5) + j) * KF + ki) * 64 + lane) * 16;
                    const uint4 v0 = *(const uint4 *)bp;
                    const uint4 v1 = *(const uint4 *)(bp + 1024);
                    b[j] = v8i {(int)v0.x, (int)v0.y, (int)v0.z, (int)v0.w,
                            (int)v1.x, (int)v1.y, (int)v1.z, (int)v1.w};
                }
#pragma unroll
                for (int i = 0; i < FM; i++)
#pragma unroll
                    for (int j = 0; j < FN; j++)
                        acc[i][j]
                                = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                                        a[i], b[j], acc[i][j], 0, 0, 0, 0, 0,
                                        0);
            }
        }
    }
    __syncthreads(); // LDS is reused by the epilogue

    // ---- zero-point compensation (integer path) ----
    int comp = 0;
    if constexpr (!F8) {
        comp = p.a_is_u8 ? 128 : 0;
        if (p.src_zp) comp -= load_int(p.src_zp_dt, p.src_zp, 0);
    }

    // ---- epilogue ----
    // Accumulator register r of lane l is row 8*(r/4) + 4*(l/32) + r%4, column
    // l%32 of its 32x32 fragment: a lane owns one column. The results of one
    // 32-row band of the wave tile go through a wave-private LDS tile and come
    // back row-wise, 4 neighbouring columns per lane, so that the post-op code
    // exists once (run-time loop) and every store is a dense vector.
    float *const stg = (float *)lds + wave * (32 * WN);
    int cs[FN], zwn[FN];
    const bool has_wz = !F8 && p.rowsum != nullptr; // block uniform
#pragma unroll
    for (int j = 0; j < FN; j++) {
        cs[j] = 0;
        zwn[j] = 0;
        if constexpr (!F8) {
            const int n = n0 + wn0 + j * 32 + (lane & 31);
            if (n < p.N && comp != 0 && p.colsum)
                cs[j] = comp * p.colsum[(int64_t)bz * p.colsum_sb + n];
            // zero point of the stored (s8) weights of the lane's column
            if (has_wz && n < p.N)
                zwn[j] = (p.wei_zp ? load_int(p.wei_zp_dt, p.wei_zp,
                                  (int64_t)n * p.wei_zp_sn)
                                   : 0)
                        - p.w_off;
        }
    }
    constexpr int ROWS_PER_IT = 256 / WN; // 64 lanes x 4 columns
    // on the way back a lane owns columns ecol..ecol+3 of every row it visits
    const int ecol = (lane % (WN / 4)) * 4;
    const int en = n0 + wn0 + ecol;
    const int envalid = min(4, p.N - en);
    const bool has_ss = p.ep.src_scale.ptr != nullptr;
    const bool has_ws = p.ep.wei_scale.ptr != nullptr;
    // what depends on the lane's 4 columns only, fetched once
    ep_cols_t cols;
    epilogue_cols_load(p.ep, cols, bz, en, envalid > 0 ? envalid : 0);
    // The row interpreter indexes the post-op list at run time: it reads the
    // parameter block in the kernel argument segment (its only argument), so
    // that the by-value copy `p` stays in registers.
    const epilogue_t &epk
            = ((const gemm_params_t *)__builtin_amdgcn_kernarg_segment_ptr())->ep;
    const float ws4[4] = {cols.ws[0], cols.ws[1], cols.ws[2], cols.ws[3]};
    static_for<FM>([&](auto I) {
        constexpr int i = decltype(I)::value;
        // weights zero points: the row sums of the lane's 16 rows (s32
        // arithmetic wraps as the reference's int accumulation does)
        int rsr[16];
#pragma unroll
        for (int r = 0; r < 16; r++) rsr[r] = 0;
        if (has_wz) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int row = 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
                const int m = min(m0 + wm0 + i * 32 + row, p.M - 1);
                rsr[r] = p.rowsum[(int64_t)bz * p.M + m];
            }
        }
#pragma unroll
        for (int j = 0; j < FN; j++) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int row = 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
                float v;
                if constexpr (F8)
                    v = acc[i][j][r];
                else
                    v = (float)(int32_t)((uint32_t)acc[i][j][r]
                            + (uint32_t)cs[j]
                            - (uint32_t)zwn[j] * (uint32_t)rsr[r]);
                stg[row * WN + j * 32 + (lane & 31)] = v;
            }
        }
#pragma unroll 1
        for (int it = 0; it < 32 / ROWS_PER_IT; it++) {
            const int row = it * ROWS_PER_IT + lane / (WN / 4);
            const float4 t = *(const float4 *)&stg[row * WN + ecol];
            const int m = m0 + wm0 + i * 32 + row;
            if (m < p.M && en < p.N) {
                float v[4] = {t.x, t.y, t.z, t.w};
                const float ss = has_ss ? ep_load(p.ep.src_scale, bz, m, 0) : 1.f;
                if (p.ep.fast != EP_FAST_NONE && !p.ep.fast_ext)
                    epilogue_fast4(
                            p.ep, v, has_ss, ss, has_ws, ws4, bz, m, en, envalid);
                else
                    epilogue_rows4(epk, cols, v, has_ss, ss, bz, m, en, envalid);
            }
        }
    });
}

template <int BM, int BN, int BK, int WGM, int WGN, int STAGES, bool F8,
        bool U8A>
static void launch_cfg(const gemm_params_t &p, hipStream_t stream) {
    gemm_params_t q = p;
    q.tiles_m = (p.M + BM - 1) / BM;
    q.tiles_n = (p.N + BN - 1) / BN;
    const int ntiles = q.tiles_m * q.tiles_n;
    // with the XCD remap every XCD gets ceil(ntiles/8) slots
    const int grid_x = ntiles >= 64 ? ((ntiles + 7) / 8) * 8 : ntiles;
    constexpr size_t lds_main = (size_t)STAGES * (BM + BN) * BK;
    constexpr size_t lds_ep
            = (size_t)WGM * WGN * 32 * (BN / WGN) * sizeof(float);
    constexpr size_t lds = lds_main > lds_ep ? lds_main : lds_ep;
    auto kern = gemm_b8_kernel<BM, BN, BK, WGM, WGN, STAGES, F8, U8A>;
    ensure_dynamic_lds((const void *)kern, (int)lds);
    hipLaunchKernelGGL(kern, dim3(grid_x, p.batch), dim3(WGM * WGN * 64), lds,
            stream, q);
}

// One tile configuration and operand kind per translation unit
// (QMM_GEMM_VARIANT, QMM_GEMM_KIND), so the instantiations build in parallel;
// the unit without the macros holds the dispatcher.
#if defined(QMM_GEMM_VARIANT)
// BM, BN, BK, waves along M, waves along N, LDS stages
#if QMM_GEMM_VARIANT == 1
#define QMM_CFG 256, 128, 64, 2, 2, 3
#elif QMM_GEMM_VARIANT == 2
#define QMM_CFG 128, 128, 64, 2, 2, 3
#elif QMM_GEMM_VARIANT == 3
#define QMM_CFG 64, 64, 64, 2, 2, 3
#endif
#define QMM_CAT_(a, b) a##b
#define QMM_CAT(a, b) QMM_CAT_(a, b)
#define QMM_CAT3(a, b, c) QMM_CAT(QMM_CAT(a, b), c)
// ... and one operand kind per unit (QMM_GEMM_KIND: 0 fp8, 1 u8 source, 2 s8)
#if QMM_GEMM_KIND == 0
void QMM_CAT3(launch_gemm_b8_v, QMM_GEMM_VARIANT, _f8)(
        const gemm_params_t &p, hipStream_t stream) {
    launch_cfg<QMM_CFG, true, false>(p, stream);
}
#elif QMM_GEMM_KIND == 1
void QMM_CAT3(launch_gemm_b8_v, QMM_GEMM_VARIANT, _u8)(
        const gemm_params_t &p, hipStream_t stream) {
    launch_cfg<QMM_CFG, false, true>(p, stream);
}
#else
void QMM_CAT3(launch_gemm_b8_v, QMM_GEMM_VARIANT, _s8)(
        const gemm_params_t &p, hipStream_t stream) {
    launch_cfg<QMM_CFG, false, false>(p, stream);
}
#endif
#else
#define QMM_DECL_VARIANT(V) \
    void launch_gemm_b8_v##V##_f8(const gemm_params_t &p, hipStream_t stream); \
    void launch_gemm_b8_v##V##_u8(const gemm_params_t &p, hipStream_t stream); \
    void launch_gemm_b8_v##V##_s8(const gemm_params_t &p, hipStream_t stream); \
    static void launch_gemm_b8_v##V( \
            const gemm_params_t &p, bool f8, hipStream_t stream) { \
        if (f8) \
            launch_gemm_b8_v##V##_f8(p, stream); \
        else if (p.a_is_u8) \
            launch_gemm_b8_v##V##_u8(p, stream); \
        else \
            launch_gemm_b8_v##V##_s8(p, stream); \
    }
QMM_DECL_VARIANT(1)
QMM_DECL_VARIANT(2)
QMM_DECL_VARIANT(3)
#undef QMM_DECL_VARIANT
// 256 x 256 tile kernel with the hand-ordered main loop (qmm_gemm_b8x.hip)
bool gemm_b8x_eligible(const gemm_params_t &p, bool f8);
void launch_gemm_b8x(const gemm_params_t &p, bool f8, hipStream_t stream);

// variant: 0 = heuristic; others pick a tile configuration explicitly (used by
// the tuning sweep; 6 = the 256 x 256 kernel where it applies)
// true when launch_gemm_b8 would hand the problem to the 256 x 256 kernel
bool gemm_b8_uses_tile256(const gemm_params_t &p, bool f8, int variant) {
    if (!gemm_b8x_eligible(p, f8)) return false;
    if (variant == 6) return true;
    if (variant != 0) return false;
    const int64_t tm = (p.M + 255) / 256;
    const int64_t tiles256 = tm * ((p.N + 255) / 256) * p.batch;
    if (tiles256 >= 192) return true;
    // int8 with an s8 source also has the 256 x 128 kernel with two workgroups
    // per CU, which beats the tiles below from 32 such tiles on, unless the row
    // tiles are mostly padding and the tiles are few (measured with a swish /
    // bf16 epilogue: 256 x 4096 x 4096 29 against 37 us, 2048 x 4096 x 4096 40
    // against 67, 1024 x 512 x 1024 13 against 21; 512 x 1024 x 1024 (16 tiles)
    // 15 against 10 and 128 x 4096 x 4096 (half-empty row tiles) 29 against 18)
    if (f8 || (p.switches & (GEMM_ONE_PER_CU | GEMM_MFMA32))) return false;
    const int64_t tiles128 = tm * ((p.N + 127) / 128) * p.batch;
    const bool rows_full = 4 * (int64_t)p.M >= 3 * tm * 256;
    return tiles128 >= 32 && (rows_full || tiles128 >= 96);
}

void launch_gemm_b8(const gemm_params_t &p, bool f8, int variant,
        hipStream_t stream) {
    if (p.M <= 0 || p.N <= 0 || p.batch <= 0) return;
    if (gemm_b8_uses_tile256(p, f8, variant)) {
        launch_gemm_b8x(p, f8, stream);
        return;
    }
    if (variant == 6) variant = 0;
    if (variant == 0) {
        const int64_t big = (int64_t)((p.M + 255) / 256) * ((p.N + 127) / 128)
                * p.batch;
        const int64_t mid = (int64_t)((p.M + 127) / 128) * ((p.N + 127) / 128)
                * p.batch;
        // small problems: more, smaller tiles keep more CUs busy
        variant = big >= 256 ? 1 : (mid >= 64 ? 2 : 3);
    }
    switch (variant) {
        case 1: launch_gemm_b8_v1(p, f8, stream); break;
        case 3: launch_gemm_b8_v3(p, f8, stream); break;
        default: launch_gemm_b8_v2(p, f8, stream); break;
    }
}
#endif

} // namespace qmm
