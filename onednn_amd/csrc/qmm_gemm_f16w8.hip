// hip:gfx950:mfma_f16w8 -- f16 activations x 8-bit weights (weights-only
// quantization with one scale and one zero point per column, or per tensor) at
// many rows: the prefill entries of tests/benchdnn/inputs/matmul/
// option_set_fwks_llm_gpu with --dt=f16:u8:* --attr-scales=wei:per_oc:f16
// --attr-zero-points=wei:per_oc:u8 --attr-fpmath=f16:true. Semantics:
// src/cpu/matmul/ref_matmul.cpp:103-140 (the weights element is
// (w - zero point) x scale before it meets the activation); here the scale,
// which does not vary along K, multiplies the f32 sum in the epilogue.
//
// The kernel is gemm_b8y_kernel's design (qmm_gemm_b8x.hip: 256 x 256 block
// tile, four waves of 128 x 128, one per SIMD, 8 x 8 fragments of 16 x 16,
// LDS ring of 4 stages filled by direct global -> LDS loads three tiles ahead,
// fragments read one k-step ahead, one barrier per k-step) on
// v_mfma_f32_16x16x32_f16: a k-step is 32 k = 64 bytes of a source row, so the
// source side is byte for byte the int8 kernel's. The weights stay bytes on
// their whole way from HBM to the registers (QMM_LAYOUT_MFMA_B8: 8 KiB per
// k-step and block tile, a lane's 8 consecutive k of one column are one 8-byte
// LDS read) and become f16 operands in registers, one fragment (the next
// column of the fragment grid) during the 8 MFMAs of the current one:
//   stored byte s (s8 code; u8 weights are stored as u8 - 128)
//   u = s ^ 0x80                     = s + 128 as an unsigned byte
//   h = 0x6400 | u  (v_perm_b32)     = the f16 number 1024 + u, exactly
//   w = h - (1152 - w_off + z[n])    (v_pk_add_f16; both operands and the result
//                                     are integers below 2048: exact)
// 10 VALU instructions per fragment against 8 MFMAs of 16 cycles.
// The MFMA grid is walked column by column (weights fragment j against the 8
// source fragments), so only two converted fragments are live at a time.
#define QMM_B8X_PART 100 // helpers, main-loop pieces and the shared epilogue only
#include "qmm_gemm_b8x.hip"

namespace qmm {

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef int v2i __attribute__((ext_vector_type(2)));

namespace h16w8 {
constexpr int B_TILE = 1024; // one packed tile: 32 k x 32 columns
constexpr uint32_t FLIP = 0x80808080u, MAGIC = 0x64646464u;
constexpr uint32_t SEL_LO = 0x04010400u, SEL_HI = 0x04030402u;
} // namespace h16w8

#define QH_MF(i, j, cb, F) \
    { \
        QX_SB(); \
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16( \
                __builtin_bit_cast(v8h, fc[F]), \
                __builtin_bit_cast(v8h, fa[cb][i]), acc[i][j], 0, 0, 0); \
        QX_SB(); \
    }
#define QH_RA(nb, i) \
    { \
        fa[nb][i] = *(const v4i *)(ldsn + a_rel + (i)*1024); \
        QX_SB(); \
    }
#define QH_RB(nb, j) \
    { \
        fbr[nb][j] = *(const v2i *)(ldsn + b_rel + ((j) >> 1) * 1024 + ((j)&1) * 256); \
        QX_SB(); \
    }
// the conversion of raw fragment [RB][JN] into fc[FN], in pieces
#define QH_P01(RB, JN) \
    x0 = (uint32_t)fbr[RB][JN][0] ^ h16w8::FLIP; \
    x1 = (uint32_t)fbr[RB][JN][1] ^ h16w8::FLIP;
#define QH_P23() \
    t0 = __builtin_amdgcn_perm(h16w8::MAGIC, x0, h16w8::SEL_LO); \
    t1 = __builtin_amdgcn_perm(h16w8::MAGIC, x0, h16w8::SEL_HI);
#define QH_P45() \
    t2 = __builtin_amdgcn_perm(h16w8::MAGIC, x1, h16w8::SEL_LO); \
    t3 = __builtin_amdgcn_perm(h16w8::MAGIC, x1, h16w8::SEL_HI);
#define QH_PK(k, T, FN, JN) \
    fc[FN][k] = __builtin_bit_cast(int, __builtin_bit_cast(v2h, T) - zc[JN]);
// column j of the fragment grid: 8 MFMAs on converted fragment fc[F]; between
// them the next fragment's conversion, two LDS reads (R1, R2) and one slot of
// the direct loads (D)
#define QH_COL(j, CB, RB, JN, F, FN, R1, R2, D) \
    QH_MF(0, j, CB, F); QH_P01(RB, JN) \
    QH_MF(1, j, CB, F); QH_P23() R1; \
    QH_MF(2, j, CB, F); QH_P45() \
    QH_MF(3, j, CB, F); QH_PK(0, t0, FN, JN) R2; \
    QH_MF(4, j, CB, F); QH_PK(1, t1, FN, JN) \
    QH_MF(5, j, CB, F); QH_PK(2, t2, FN, JN) D; \
    QH_MF(6, j, CB, F); QH_PK(3, t3, FN, JN) \
    QH_MF(7, j, CB, F);
#define QH_COL_END(j, CB, F) \
    QH_MF(0, j, CB, F); QH_MF(1, j, CB, F); QH_MF(2, j, CB, F); \
    QH_MF(3, j, CB, F); QH_MF(4, j, CB, F); QH_MF(5, j, CB, F); \
    QH_MF(6, j, CB, F); QH_MF(7, j, CB, F);
// the first weights fragment of the next k-step is read first (it is converted
// during this k-step's last column), then the source fragments, which the next
// k-step's first column needs all at once
#define QH_STEP(CB, NB, DA0, DA1, DA2, DA3, DA4, DB0, DB1, DB2) \
    QH_COL(0, CB, CB, 1, 0, 1, QH_RB(NB, 0), QH_RA(NB, 0), DA0) \
    QH_COL(1, CB, CB, 2, 1, 0, QH_RA(NB, 1), QH_RA(NB, 2), DA1) \
    QH_COL(2, CB, CB, 3, 0, 1, QH_RA(NB, 3), QH_RA(NB, 4), DA2) \
    QH_COL(3, CB, CB, 4, 1, 0, QH_RA(NB, 5), QH_RA(NB, 6), DA3) \
    QH_COL(4, CB, CB, 5, 0, 1, QH_RA(NB, 7), QH_RB(NB, 1), DA4) \
    QH_COL(5, CB, CB, 6, 1, 0, QH_RB(NB, 2), QH_RB(NB, 3), DB0) \
    QH_COL(6, CB, CB, 7, 0, 1, QH_RB(NB, 4), QH_RB(NB, 5), DB1) \
    QH_COL(7, CB, NB, 0, 1, 0, QH_RB(NB, 6), QH_RB(NB, 7), DB2)
#define QH_STEP_D(CB, NB) \
    QH_STEP(CB, NB, QX_D0(a_vo, sa, dA), QX_D1(a_vo, sa, dA), \
            QX_D2(a_vo, sa, dA), QX_D3(a_vo, sa, dA), QX_D4(a_vo, sa, dA), \
            QX_M0(dB, 0 * 4096), \
            { QX_DMA(b_vo[0], sb); QX_M0(dB, 1 * 4096); }, \
            QX_DMA(b_vo[1], sb))
#define QH_STEP_ND(CB, NB) QH_STEP(CB, NB, , , , , , , , )
#define QH_LAST(CB) \
    QH_COL(0, CB, CB, 1, 0, 1, , , ) QH_COL(1, CB, CB, 2, 1, 0, , , ) \
    QH_COL(2, CB, CB, 3, 0, 1, , , ) QH_COL(3, CB, CB, 4, 1, 0, , , ) \
    QH_COL(4, CB, CB, 5, 0, 1, , , ) QH_COL(5, CB, CB, 6, 1, 0, , , ) \
    QH_COL(6, CB, CB, 7, 0, 1, , , ) QH_COL_END(7, CB, 1)

// ODD: an odd number of k-steps (one instantiation per parity, as in
// gemm_b8y_kernel).
template <bool ODD>
__global__ void __launch_bounds__(b8x::NT, 1)
gemm_f16w8_kernel(const gemm_params_t p) {
    using namespace b8x;
    typedef __attribute__((address_space(3))) uint8_t lds_u8;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm0 = (wave >> 1) * 128, wn0 = (wave & 1) * 128;

    // persistent, as gemm_b8y_kernel: workgroup w of an XCD walks the tiles
    // w, w + W, ... of the XCD's share (all in step: the late half of that
    // kernel measured 1 % slower here)
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
    const int bz = blockIdx.y;

    const int KT = p.K / 32; // host guarantees K % 32 == 0, KT >= 5 and KT % 2 == ODD
    const uint32_t lds_base = __builtin_amdgcn_readfirstlane(
            (uint32_t)(uintptr_t)(lds_u8 *)lds);

    // direct loads per k-step and thread: four 16-byte chunks of the source
    // tile (256 rows x 64 bytes, chunk-swizzled) and two of the weights (8
    // packed tiles of 1 KiB: wave w moves tiles w and w + 4)
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
        const int nbl = (tid >> 6) + 4 * j;
        const int nb = min(n0 / 32 + nbl, p.nb32 - 1) - n0 / 32;
        b_vo[j] = (uint32_t)nb * (uint32_t)p.kb32 * 1024u + lane * 16;
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
#define QH_ADV_B() \
    { \
        sb += h16w8::B_TILE; \
        dB = ((dB - lds_base + STAGE_BYTES) & (RING - 1)) + lds_base; \
    }
#define QH_FETCH_B() \
    { \
        QX_M0(dB, 0 * 4096); asm volatile("s_nop 0"); QX_DMA(b_vo[0], sb); \
        QX_M0(dB, 1 * 4096); asm volatile("s_nop 0"); QX_DMA(b_vo[1], sb); \
    }

    // fragment offsets inside a stage: lane group g = lane / 16 takes the 8 k
    // of chunk g: 16 bytes of a source row, 8 bytes of a weights column
    const int g = lane >> 4;
    const int arow = wm0 + (lane & 15);
    const int a_rel = arow * BK + a_swz16(arow, g) * 16;
    const int b_rel = A_BYTES + (wn0 >> 5) * 1024
            + ((g >> 1) * 32 + (lane & 15)) * 16 + (g & 1) * 8;

    // what is subtracted from 1024 + (stored byte ^ 0x80), per fragment column
    v2h zc[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const int n = min(n0 + wn0 + 16 * j + (lane & 15), p.N - 1);
        const int z = p.wei_zp
                ? load_int(p.wei_zp_dt, p.wei_zp, (int64_t)n * p.wei_zp_sn)
                : 0;
        const _Float16 c = (_Float16)(float)(1152 - p.w_off + z);
        zc[j] = v2h {c, c};
    }

    v4f acc[8][8];
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int j = 0; j < 8; j++)
#pragma unroll
            for (int r = 0; r < 4; r++)
                acc[i][j][r] = 0.f;
    v4i fa[2][8];
    v2i fbr[2][8];
    v4i fc[2];
    uint32_t x0, x1, t0, t1, t2, t3;

    tile_operands_stage(p, lds, tid, m0, n0, bz);

    // ---- prologue: tiles 0..3 requested (the whole ring); tile 0's fragments
    // read, its first weights fragment converted ----
    QX_FETCH(a_vo, sa, dA); QX_ADV_A();
    QH_FETCH_B(); QH_ADV_B();
    QX_FETCH(a_vo, sa, dA); QX_ADV_A();
    QH_FETCH_B(); QH_ADV_B();
    QX_FETCH(a_vo, sa, dA); QX_ADV_A();
    QH_FETCH_B(); QH_ADV_B();
    QX_FETCH(a_vo, sa, dA); QX_ADV_A();
    QH_FETCH_B(); QH_ADV_B();
    QX_WV(18);
    __syncthreads();
    uint32_t st = 0; // ring offset of the tile whose fragments are read next
    {
        const uint8_t *ldsn = lds;
        QX_SB();
        QH_RB(0, 0); QH_RA(0, 0); QH_RA(0, 1); QH_RA(0, 2); QH_RA(0, 3);
        QH_RA(0, 4); QH_RA(0, 5); QH_RA(0, 6); QH_RA(0, 7); QH_RB(0, 1);
        QH_RB(0, 2); QH_RB(0, 3); QH_RB(0, 4); QH_RB(0, 5); QH_RB(0, 6);
        QH_RB(0, 7);
        QH_P01(0, 0) QH_P23() QH_P45()
        QH_PK(0, t0, 0, 0) QH_PK(1, t1, 0, 0) QH_PK(2, t2, 0, 0)
        QH_PK(3, t3, 0, 0)
        QX_SB();
    }
    // k-step kt: multiplies tile kt-1 (buffer (kt-1)&1), reads tile kt's
    // fragments, requests tile kt+3 into the stage tile kt-1 was read from
    // during the previous k-step; 6 direct loads per tile and thread
#define QH_KSTEP(WAITV, BODY) \
    { \
        st = (st + STAGE_BYTES) & (RING - 1); \
        const uint8_t *ldsn = lds + st; \
        QX_WV(WAITV); \
        __builtin_amdgcn_s_barrier(); \
        QX_SB(); \
        BODY \
    }
    // requesting steps kt = 1 .. KT-4, in pairs; an odd KT leaves one more
    constexpr int PAIRED_END = ODD ? 6 : 5;
    for (int kt = 1; kt <= KT - PAIRED_END; kt += 2) {
        QH_KSTEP(12, QH_STEP_D(0, 1) QX_ADV_A(); QH_ADV_B();)
        QH_KSTEP(12, QH_STEP_D(1, 0) QX_ADV_A(); QH_ADV_B();)
    }
    if constexpr (ODD) {
        QH_KSTEP(12, QH_STEP_D(0, 1)) // kt = KT-4: requests tile KT-1
        QH_KSTEP(12, QH_STEP_ND(1, 0)) // kt = KT-3
        QH_KSTEP(6, QH_STEP_ND(0, 1)) // kt = KT-2
        QH_KSTEP(0, QH_STEP_ND(1, 0)) // kt = KT-1
        QH_LAST(0)
    } else {
        QH_KSTEP(12, QH_STEP_ND(0, 1)) // kt = KT-3
        QH_KSTEP(6, QH_STEP_ND(1, 0)) // kt = KT-2
        QH_KSTEP(0, QH_STEP_ND(0, 1)) // kt = KT-1
        QH_LAST(1)
    }
    __syncthreads();

    tile_epilogue<true, false>(
            p, acc, lds, lds_base, wave, lane, m0, n0, wm0, wn0, bz);
    // the staging area and the operand tables are the next tile's ring and
    // tables
    __syncthreads();
    }
}

#if QMM_F16W8_PART == 0
void launch_f16w8_even(const gemm_params_t &p, hipStream_t stream) {
    launch_b8y_persistent(gemm_f16w8_kernel<false>, p, stream);
}
#else
void launch_f16w8_odd(const gemm_params_t &p, hipStream_t stream) {
    launch_b8y_persistent(gemm_f16w8_kernel<true>, p, stream);
}
#endif

#if QMM_F16W8_PART == 0
void launch_f16w8_odd(const gemm_params_t &p, hipStream_t stream);

// Few block tiles, long K (1024 x 4096 dst over K 4096 ... 14336: 64 tiles on 256
// CUs): the K range is cut into `splits` equal slices that run as the batch
// dimension of one launch -- slice s reads the source from column s K/splits
// and the packed weights from k block s K/splits / 32, and writes its f32 sums
// to slice s of a scratch buffer -- and this kernel adds the slices in slice
// order, then applies scales, bias, post-ops and the dst conversion: one
// thread per four neighbouring columns of a row.
// (S slices, a compile-time count: a thread's S loads are all in flight before
// the first addition)
template <int S>
__global__ void __launch_bounds__(256)
f16w8_reduce_kernel(const float *part, int M, int N, int ldp,
        const epilogue_t ep) {
    const int n4 = (N + 3) / 4;
    const int64_t total = (int64_t)M * n4;
    const bool has_ss = ep.src_scale.ptr != nullptr;
    const bool has_ws = ep.wei_scale.ptr != nullptr;
    const int64_t slice = (int64_t)M * ldp;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
            i += (int64_t)gridDim.x * blockDim.x) {
        const int m = (int)(i / n4), n = (int)(i % n4) * 4;
        const float *q = part + (int64_t)m * ldp + n;
        v4f t[S];
#pragma unroll
        for (int s = 0; s < S; s++)
            t[s] = *(const v4f *)(q + s * slice);
        float v[4] = {t[0].x, t[0].y, t[0].z, t[0].w};
#pragma unroll
        for (int s = 1; s < S; s++) {
            v[0] += t[s].x;
            v[1] += t[s].y;
            v[2] += t[s].z;
            v[3] += t[s].w;
        }
        const int nvalid = min(4, N - n);
        ep_cols_t c;
        epilogue_cols_load(ep, c, 0, n, nvalid);
        const float ss = has_ss ? ep_load(ep.src_scale, 0, m, 0) : 1.f;
        if (ep.fast != EP_FAST_NONE && !ep.fast_ext)
            epilogue_fast4(ep, v, has_ss, ss, has_ws, c.ws, 0, m, n, nvalid);
        else
            epilogue_rows4(ep, c, v, has_ss, ss, 0, m, n, nvalid);
    }
}

// Problems the kernel takes: K a multiple of 32 with at least 5 k-steps, source
// rows of 16-byte granularity, tiles addressable with 32-bit offsets.
bool gemm_f16w8_eligible(const gemm_params_t &p) {
    if (p.K % 32 != 0 || p.K < 5 * 32) return false;
    if ((int64_t)256 * p.lda + 64 >= ((int64_t)1 << 32)) return false;
    if ((int64_t)8 * p.kb32 * 1024 >= ((int64_t)1 << 32)) return false;
    return true;
}

// How many K slices. Cost model in microseconds, fitted to measurements on
// 1024 x K x 4096 and 512 x 4096 x 14336: a workgroup takes 0.6 per k-step plus
// 10 for prologue and epilogue; slices add their f32 sums written (4 TB/s) and
// read back by the second kernel (3 TB/s, plus 3 for its launch). Slices must
// keep every workgroup in one round over the 256 CUs, divide the k-steps evenly
// and have at least 16 of them; they are taken when the model promises a tenth
// less time.
int gemm_f16w8_splits(int64_t M, int64_t N, int64_t K) {
    const int64_t tiles = ((M + 255) / 256) * ((N + 255) / 256);
    const int64_t kt = K / 32;
    if (tiles > 128) return 1;
    const double one = 0.6 * (double)kt + 10.0;
    double best_t = 0.9 * one;
    int best = 1;
    for (int s : {2, 3, 4, 6, 8}) {
        if (kt % s != 0 || kt / s < 16 || tiles * s > 256) continue;
        const double part = (double)s * (double)M * (double)N * 4.0;
        const double t = 0.6 * (double)(kt / s) + 10.0 + part / 4e6 + 3.0
                + (part + (double)M * (double)N * 4.0) / 3e6;
        if (t < best_t) {
            best_t = t;
            best = s;
        }
    }
    return best;
}

static void launch_one(const gemm_params_t &p, hipStream_t stream) {
    if ((p.K / 32) & 1)
        launch_f16w8_odd(p, stream);
    else
        launch_f16w8_even(p, stream);
}

// part: room for splits x M x round_up(N, 4) floats when splits > 1
void launch_gemm_f16w8(const gemm_params_t &p, int splits, float *part,
        hipStream_t stream) {
    if (splits <= 1) {
        launch_one(p, stream);
        return;
    }
    const int ldp = (p.N + 3) / 4 * 4;
    gemm_params_t q = p;
    q.K = p.K / splits;
    q.batch = splits;
    q.a_sb = (int64_t)q.K * 2;
    q.b_sb = (int64_t)(q.K / 32) * 1024;
    std::memset(&q.ep, 0, sizeof(q.ep));
    q.ep.dst.ptr = part;
    q.ep.dst.dt = dt_f32;
    q.ep.dst.sb = (int64_t)p.M * ldp;
    q.ep.dst.sm = ldp;
    q.ep.dst.sn = 1;
    q.ep.fast = EP_FAST_PLAIN;
    launch_one(q, stream);
    const int64_t total = (int64_t)p.M * (ldp / 4);
    int64_t blocks = (total + 255) / 256;
    if (blocks > 65535) blocks = 65535;
#define QH_REDUCE(S) \
    case S: \
        hipLaunchKernelGGL(f16w8_reduce_kernel<S>, dim3((unsigned)blocks), \
                dim3(256), 0, stream, (const float *)part, p.M, p.N, ldp, p.ep); \
        break;
    switch (splits) {
        QH_REDUCE(2)
        QH_REDUCE(3)
        QH_REDUCE(4)
        QH_REDUCE(6)
        default: QH_REDUCE(8)
    }
#undef QH_REDUCE
}
#endif

} // namespace qmm
