// hip:gfx950:mfma_b8, at most 64 source rows (the decode step of a W8A8 linear
// layer, one token or a small batch of them): the launch is one read of the weights, so the kernel is organised
// around memory parallelism instead of tiles. A workgroup owns 32 columns (one
// block of QMM_LAYOUT_MFMA_B8, whose 1 KiB fragments already are the MFMA
// operand per lane); its 8 waves cut K between them and each streams its
// fragments straight into registers, 16 requested at a time together with the
// matching source bytes, and multiplies them with v_mfma_i32_32x32x32_i8 (the
// first M rows of the 32 x 32 result are the source rows; the others repeat the
// last row and are dropped: MR = 4 keeps only registers 0..3 of lanes 0..31,
// MR = 32 everything, MR = 64 two such
// blocks of rows). The waves' s32 sums are added through LDS -- integer
// addition, so the result does not depend on the cut -- and the epilogue of
// qmm_gemm_b8.hip runs per element:
//   (float)(P + comp * colsum[n] - z_w'[n] * (rowsum[m] + K * comp)),
// source scale, weights scale, bias, post-ops, dst quantization
// (src/cpu/matmul/ref_matmul_int8.cpp:165-259). The row sums that a weights
// zero point needs come from dot products of the source fragments with ones.
#include "qmm_device.hpp"
#include "qmm_plan.hpp"

namespace qmm {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));

constexpr int GB8_WAVES = 8;
constexpr int GB8_CH = 16; // fragments in flight per wave

// MR = 32 / 64 (one or two blocks of 32 rows against the same weights
// fragments): the source bytes of a chunk go through a wave-private piece of LDS --
// requested as whole 256-byte row pieces (16 lanes a row, 4 rows an
// instruction) instead of one 16-byte piece per lane out of 32 different rows
// -- and come back in operand order. The same bytes hold the wave's results
// for the sum across waves afterwards.
constexpr int GB8_CH32 = 8; // fragments per chunk with 32 rows
constexpr int GB8_APITCH = GB8_CH32 * 32 + 16; // bytes of a staged row
constexpr int gb8_wave_lds(int mr) { // >= mr x 32 s32 of results + row sums
    return mr >= 32 ? mr * GB8_APITCH : (4 * 32 + 4) * 4;
}
static_assert(gb8_wave_lds(64) >= 64 * 32 * 4 + 64 * 4, "");

template <int MR>
__global__ void __launch_bounds__(GB8_WAVES * 64)
gemv_b8_kernel(const gemm_params_t p) {
    constexpr int CH = MR >= 32 ? GB8_CH32 : GB8_CH;
    constexpr int RB = MR >= 32 ? MR / 32 : 1; // blocks of 32 rows
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    constexpr int WAVE_LDS = gb8_wave_lds(MR);
    // a wave's results [MR][32] and row sums [MR], s32
    auto red = [&](int w, int r, int c) -> int & {
        return ((int *)(lds_raw + w * WAVE_LDS))[r * 32 + c];
    };
    auto red_rs = [&](int w, int r) -> int & {
        return ((int *)(lds_raw + w * WAVE_LDS))[MR * 32 + r];
    };
    const int nb = blockIdx.x;
    // the wave's fragments (32 k each): an even cut of the K / 32 that hold data
    const int nfrag = (p.K + 31) / 32;
    const int per = (nfrag + GB8_WAVES - 1) / GB8_WAVES;
    const int f0 = min(wave * per, nfrag), f1 = min(f0 + per, nfrag);
    const v4u *bsrc = (const v4u *)(p.B + (int64_t)nb * p.kb32 * 1024) + lane;
    // A operand: lane l is row l % 32, bytes 16 (l / 32) .. + 15 of the fragment
    const int row = min(lane & 31, p.M - 1);
    const uint8_t *arow = p.A + (int64_t)row * p.lda;
    const uint32_t flip = p.a_is_u8 && !p.a_preflipped ? 0x80808080u : 0u;
    const bool need_rs = p.wei_zp != nullptr || p.w_off != 0;
    uint8_t *const stage = lds_raw + wave * WAVE_LDS;

    v16i acc[RB];
    int rsum[RB];
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
        rsum[rb] = 0;
#pragma unroll
        for (int r = 0; r < 16; r++) acc[rb][r] = 0;
    }
    for (int fb = f0; fb < f1; fb += CH) {
        v4u bq[CH];
        uint4 av[RB][CH];
        // every request of the chunk before the first use; fragments past the
        // wave's end repeat its last one and are skipped below
        if constexpr (MR >= 32) {
            // piece l % 16 of rows l / 16 + 4 i (K is a multiple of 16: a piece
            // is inside the row or past it)
            static_assert(CH == 8, "a block of 32 rows is 8 row quadruples");
            const int k = fb * 32 + (lane & 15) * 16;
#pragma unroll
            for (int rb = 0; rb < RB; rb++)
#pragma unroll
                for (int i = 0; i < CH; i++) {
                    const int r = min(32 * rb + 4 * i + (lane >> 4), p.M - 1);
                    av[rb][i] = *(const uint4 *)(p.A + (int64_t)r * p.lda
                            + min(k, p.K - 16));
                }
#pragma unroll
            for (int j = 0; j < CH; j++)
                bq[j] = __builtin_nontemporal_load(bsrc + (int64_t)min(fb + j, f1 - 1) * 64);
#pragma unroll
            for (int rb = 0; rb < RB; rb++)
#pragma unroll
                for (int i = 0; i < CH; i++)
                    *(uint4 *)(stage + (32 * rb + 4 * i + (lane >> 4)) * GB8_APITCH
                            + (lane & 15) * 16)
                            = k >= p.K ? make_uint4(flip, flip, flip, flip) // zero after the flip
                                       : av[rb][i];
#pragma unroll
            for (int rb = 0; rb < RB; rb++)
#pragma unroll
                for (int j = 0; j < CH; j++)
                    av[rb][j] = *(const uint4 *)(stage
                            + (32 * rb + (lane & 31)) * GB8_APITCH + j * 32
                            + (lane >> 5) * 16);
        } else {
#pragma unroll
            for (int j = 0; j < CH; j++) {
                const int f = min(fb + j, f1 - 1);
                bq[j] = __builtin_nontemporal_load(bsrc + (int64_t)f * 64);
                // K is a multiple of 16: a half fragment is inside the row or past it
                const int k = f * 32 + (lane >> 5) * 16;
                av[0][j] = *(const uint4 *)(arow + min(k, p.K - 16));
                if (k >= p.K) av[0][j] = make_uint4(flip, flip, flip, flip); // zero after the flip
            }
        }
#pragma unroll
        for (int j = 0; j < CH; j++) {
            if (fb + j < f1) {
                const v4i b = {(int)bq[j].x, (int)bq[j].y, (int)bq[j].z,
                        (int)bq[j].w};
#pragma unroll
                for (int rb = 0; rb < RB; rb++) {
                    const v4i a = {(int)(av[rb][j].x ^ flip), (int)(av[rb][j].y ^ flip),
                            (int)(av[rb][j].z ^ flip), (int)(av[rb][j].w ^ flip)};
                    if (need_rs) {
                        int t = rsum[rb];
                        t = __builtin_amdgcn_sdot4(a[0], 0x01010101, t, false);
                        t = __builtin_amdgcn_sdot4(a[1], 0x01010101, t, false);
                        t = __builtin_amdgcn_sdot4(a[2], 0x01010101, t, false);
                        t = __builtin_amdgcn_sdot4(a[3], 0x01010101, t, false);
                        rsum[rb] = t;
                    }
                    acc[rb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc[rb], 0, 0, 0);
                }
            }
        }
    }
    // accumulator register r of lane l is row 8 (r / 4) + 4 (l / 32) + r % 4,
    // column l % 32; the two k halves of row r's sum sit in lanes r and r + 32
    if constexpr (MR == 4) {
        if (lane < 32) {
#pragma unroll
            for (int r = 0; r < 4; r++) red(wave, r, lane) = acc[0][r];
        }
    } else {
#pragma unroll
        for (int rb = 0; rb < RB; rb++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                red(wave, 32 * rb + 8 * (r / 4) + 4 * (lane >> 5) + r % 4, lane & 31)
                        = acc[rb][r];
    }
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
        const int tot = rsum[rb] + __shfl_xor(rsum[rb], 32);
        if (lane < (MR < 32 ? MR : 32)) red_rs(wave, 32 * rb + lane) = tot;
    }
    __syncthreads();
    // one thread per element: column t % 32, rows t / 32 + 16 i
    const int tid = threadIdx.x;
    const int n = nb * 32 + (tid & 31);
    if (n >= p.N) return;
    int comp = p.a_is_u8 ? 128 : 0;
    if (p.src_zp) comp -= load_int(p.src_zp_dt, p.src_zp, 0);
    const int cs = comp != 0 && p.colsum ? comp * p.colsum[n] : 0;
    const int zw = need_rs
            ? (p.wei_zp ? load_int(p.wei_zp_dt, p.wei_zp, (int64_t)n * p.wei_zp_sn) : 0)
                    - p.w_off
            : 0;
#pragma unroll
    for (int i = 0; i < (MR + 15) / 16; i++) {
        const int r = (tid >> 5) + 16 * i;
        if (r < p.M && r < MR) {
            uint32_t v = 0, rs = 0;
#pragma unroll
            for (int w = 0; w < GB8_WAVES; w++) {
                v += (uint32_t)red(w, r, tid & 31);
                rs += (uint32_t)red_rs(w, r);
            }
            // s32 arithmetic that wraps as the reference's int accumulation
            v += (uint32_t)cs - (uint32_t)zw * (rs + (uint32_t)p.K * (uint32_t)comp);
            epilogue_apply_store(p.ep, (float)(int32_t)v, 0, r, n);
        }
    }
}

} // namespace

// p.M <= 64, one batch, integer operands (the caller checks)
void launch_gemv_b8(const gemm_params_t &p, hipStream_t stream) {
    if (p.M <= 0 || p.N <= 0) return;
    if (p.M <= 4) {
        hipLaunchKernelGGL(gemv_b8_kernel<4>, dim3((unsigned)p.nb32),
                dim3(GB8_WAVES * 64), GB8_WAVES * (4 * 32 + 4) * 4, stream, p);
    } else if (p.M <= 32) {
        constexpr int lds = GB8_WAVES * gb8_wave_lds(32);
        ensure_dynamic_lds((const void *)gemv_b8_kernel<32>, lds);
        hipLaunchKernelGGL(gemv_b8_kernel<32>, dim3((unsigned)p.nb32),
                dim3(GB8_WAVES * 64), lds, stream, p);
    } else {
        constexpr int lds = GB8_WAVES * gb8_wave_lds(64);
        ensure_dynamic_lds((const void *)gemv_b8_kernel<64>, lds);
        hipLaunchKernelGGL(gemv_b8_kernel<64>, dim3((unsigned)p.nb32),
                dim3(GB8_WAVES * 64), lds, stream, p);
    }
}

} // namespace qmm
