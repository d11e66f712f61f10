// hip:gfx950:decode_w4 at many rows (the prefill step of a weights-only
// quantized linear layer): 16-bit activations [M,K] x 4-bit or 8-bit weights
// [K,N] with K-grouped scales and zero points, f32 accumulation -- the
// arithmetic of qmm_gemv_w4.hip (src/cpu/matmul/ref_matmul.cpp:140-173 with
// fpmath_mode apply_to_int), tiled so that a weights tile is unpacked once for
// BM rows:
//   * a workgroup of 8 waves owns BM rows x 256 columns; a wave owns 32
//     columns (two 16-column tiles of QMM_LAYOUT_MFMA_W4 / _W8 per 128 k,
//     loaded straight into registers one k tile ahead) and all BM rows;
//   * the activations of a k tile (BM x 128, 16-bit) are shared by the eight
//     waves through LDS, double buffered, one barrier per k tile; they cross
//     the CU's load path once per 256 columns;
//   * per k tile and column: P = sum a * (offset + w) and S = sum a from
//     16 x 16 x 32 MFMAs (the nibble -> float trick of the decode kernel: no
//     integer-to-float conversion), then out += scale * (P - (offset + zp) * S);
//     for 8-bit weights both nibble planes add into P, the high one behind
//     the exponent of 16 * offset (P = sum a * (17 offset + w)).
// One 16-bit scale and at most one byte-sized zero point per column and k tile
// (group widths 128 << s or all of K), as in the decode kernel's fast variant.
#include <type_traits>

#include "qmm_device.hpp"
#include "qmm_plan.hpp"

// The kernel is instantiated per activation type and weights width in
// translation units of their own (QMM_W4F_PART = 0..3: bit 0 f16 activations,
// bit 1 8-bit weights), so that they compile in parallel; the unit without the
// macro holds the launcher that picks one.
namespace qmm {
#if defined(QMM_W4F_PART)
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));

constexpr int WF_WAVES = 8;
constexpr int WF_PITCH = 256 + 16; // bytes of a staged activation row

template <bool F16>
QMM_D v4f mfma16(const v4u &a, const v4u &b, const v4f &c) {
    if constexpr (F16)
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(
                __builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0,
                0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                __builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0,
                0, 0);
}

QMM_D uint4 ld_stream(const uint8_t *ptr) {
    const v4u v = __builtin_nontemporal_load((const v4u *)ptr);
    return make_uint4(v.x, v.y, v.z, v.w);
}

// flags_m / shifts: as gemv_w4_fast_kernel (qmm_gemv_w4.hip)
// BM rows (32 or 64) x 16 * CBW * 8 columns per workgroup; CBW = 1 where the
// problem has too few columns to fill the chip with 256-column blocks
template <bool F16, bool WSIGNED, bool W8, int BM, int CBW>
__global__ void __launch_bounds__(WF_WAVES * 64)
gemm_w4f_kernel(const gemv_params_t p, const int shifts, const int flags_m) {
    constexpr int RB = BM / 16; // row blocks of the MFMA
    constexpr int NP = W8 ? 2 : 1;
    constexpr int TILE_BYTES = 1024 * NP;
    // two activation buffers; after the k loop the same bytes stage the results
    constexpr int A_BUF = BM * WF_PITCH, STG_PITCH = 16 * CBW + 4; // floats per staged row
    constexpr int STG_WAVE = 32 * STG_PITCH * 4; // 32 rows x the wave's columns
    constexpr int LDS_BYTES
            = 2 * A_BUF > WF_WAVES * STG_WAVE ? 2 * A_BUF : WF_WAVES * STG_WAVE;
    __shared__ __attribute__((aligned(16))) uint8_t lds_raw[LDS_BYTES];
    uint8_t *const lds_a[2] = {lds_raw, lds_raw + A_BUF};
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c = lane >> 4, r = lane & 15;
    const int N = p.N, K = p.K, M = p.M;
    const int m0 = blockIdx.y * BM;
    const int nb16 = p.nb16, tiles = p.kg128;
    const int nb0 = (blockIdx.x * WF_WAVES + wave) * CBW; // first 16-column block
    const int gs_shift = (int8_t)(shifts & 0xff), gz_shift = (int8_t)(shifts >> 8);
    const bool scale_per_n = flags_m & 1, zp_per_n = flags_m & 2;
    const bool zp4 = flags_m & 4, zp_signed = flags_m & 8, sc_f16 = flags_m & 16;
    const bool has_zp = flags_m & 64;
    constexpr float OFFSET = F16 ? 1024.f : 128.f;
    constexpr uint32_t ONE2 = F16 ? 0x3C003C00u : 0x3F803F80u;
    const v4u ones = {ONE2, ONE2, ONE2, ONE2};
    constexpr uint32_t sflip = WSIGNED ? 0x88888888u : 0u;
    constexpr float soff = WSIGNED ? 8.f : 0.f;
    constexpr uint32_t MAGIC = F16 ? 0x64006400u : 0x43004300u;
    // 8-bit weights: the high nibbles behind the exponent of 16 * offset, where
    // one unit of the last mantissa bit is 16 (f16: 0x7400 | h = 16384 + 16 h;
    // bf16: 0x4500 | h = 2048 + 16 h), so both planes add into one accumulator:
    // sum a * (16 (offset + h) + (offset + l)) = sum a * (17 offset + w)
    constexpr uint32_t MAGIC_HI = W8 ? (F16 ? 0x74007400u : 0x45004500u) : MAGIC;
    constexpr uint32_t NIB = 0x000F000Fu;

    // column blocks past the last one repeat it and are never stored
    const uint8_t *Bt[CBW];
    const uint16_t *scn[CBW];
    int zcol[CBW];
    const int64_t sN = scale_per_n ? N : 0, zN = zp_per_n ? N : 0;
    const uint8_t *pZP = p.zps ? (const uint8_t *)p.zps : p.B;
#pragma unroll
    for (int cb = 0; cb < CBW; cb++) {
        Bt[cb] = p.B + ((int64_t)min(nb0 + cb, nb16 - 1) * tiles) * TILE_BYTES
                + lane * 16;
        const int nn = min((nb0 + cb) * 16 + r, N - 1);
        scn[cb] = (const uint16_t *)p.scales + (scale_per_n ? nn : 0);
        zcol[cb] = zp_per_n ? nn : 0;
    }

    // activations: thread t stages 16-byte chunk t % 16 of rows t / 16 + 32 i
    // (a row of a k tile is 256 bytes = 16 chunks); rows past M repeat the
    // last row, chunks past K are zero
    constexpr int A_LD = BM * 16 / (WF_WAVES * 64);
    static_assert(A_LD >= 1, "");
    const int a_chunk = tid & 15, a_row = tid >> 4;
    const uint16_t *a_src[A_LD];
#pragma unroll
    for (int i = 0; i < A_LD; i++)
        a_src[i] = p.A + (int64_t)min(m0 + a_row + WF_WAVES * 4 * i, M - 1) * p.lda;
    // two request slots: a tile's operands are asked for two k tiles before
    // they are used (one k tile of arithmetic is shorter than a trip to memory)
    uint4 a_reg[2][A_LD], wt[2][CBW][NP];
    // kept in their storage types: widening them here would make the request
    // wait for the values
    uint16_t scp[2][CBW];
    uint8_t zpp[2][CBW];
    auto request = [&](int kt, auto slot_tag) { // global -> registers, tile kt
        constexpr int sl = decltype(slot_tag)::value;
        const int tc = min(kt, tiles - 1);
#pragma unroll
        for (int cb = 0; cb < CBW; cb++)
#pragma unroll
            for (int pl = 0; pl < NP; pl++)
                wt[sl][cb][pl] = ld_stream(
                        Bt[cb] + (int64_t)tc * TILE_BYTES + pl * 1024);
        const int k = tc * 128 + a_chunk * 8;
#pragma unroll
        for (int i = 0; i < A_LD; i++) // (chunks past K are zeroed when staged:
            // touching the value here would make the request wait for it)
            a_reg[sl][i] = *(const uint4 *)(a_src[i] + min(k, K - 8));
        const int gsc = gs_shift < 0 ? 0 : tc >> gs_shift;
        const int gzp = gz_shift < 0 ? 0 : tc >> gz_shift;
#pragma unroll
        for (int cb = 0; cb < CBW; cb++) {
            scp[sl][cb] = scn[cb][(int64_t)gsc * sN];
            const int64_t zi = has_zp ? (int64_t)gzp * zN + zcol[cb] : 0;
            zpp[sl][cb] = pZP[zp4 ? zi >> 1 : zi];
        }
    };

    v4f out[RB][CBW];
#pragma unroll
    for (int rb = 0; rb < RB; rb++)
#pragma unroll
        for (int cb = 0; cb < CBW; cb++) out[rb][cb] = v4f {0.f, 0.f, 0.f, 0.f};

    // one k tile; its operands sit in request slot kt % 2 (= LDS buffer)
    auto k_tile = [&](int kt, auto slot_tag) {
        constexpr int sl = decltype(slot_tag)::value;
        // this tile's operands leave the request registers: activations to
        // LDS, weights / scales / zero points to the compute registers
        const bool past_k = kt * 128 + a_chunk * 8 >= K;
#pragma unroll
        for (int i = 0; i < A_LD; i++)
            *(uint4 *)(lds_a[sl] + (a_row + WF_WAVES * 4 * i) * WF_PITCH + a_chunk * 16)
                    = past_k ? make_uint4(0, 0, 0, 0) : a_reg[sl][i];
        uint4 w_cur[CBW][NP];
        uint16_t sc_cur[CBW];
        uint8_t zp_cur[CBW];
#pragma unroll
        for (int cb = 0; cb < CBW; cb++) {
#pragma unroll
            for (int pl = 0; pl < NP; pl++) w_cur[cb][pl] = wt[sl][cb][pl];
            sc_cur[cb] = scp[sl][cb];
            zp_cur[cb] = zpp[sl][cb];
        }
        // the tile is staged; every wave is past its reads of the other buffer
        __syncthreads();
        // unconditional (past the end: the last tile again, never used): a
        // branch around the loads makes the compiler wait for them at its end
        request(kt + 2, slot_tag);

        // scale and zero point of the tile's group, per column block
        const int gzp = gz_shift < 0 ? 0 : kt >> gz_shift;
        float sc[CBW], zp[CBW];
#pragma unroll
        for (int cb = 0; cb < CBW; cb++) {
            sc[cb] = sc_f16 ? (float)__builtin_bit_cast(_Float16, sc_cur[cb])
                            : u2f((uint32_t)sc_cur[cb] << 16);
            const int odd = zp4 ? (int)(((int64_t)gzp * zN + zcol[cb]) & 1) : 0;
            const int zbits = zp4 ? 4 : 8;
            const uint32_t zraw
                    = ((uint32_t)zp_cur[cb] >> (4 * odd)) & ((1u << zbits) - 1u);
            const int zsx = (int)(zraw << (32 - zbits)) >> (32 - zbits);
            zp[cb] = has_zp ? (float)(zp_signed ? zsx : (int)zraw) : 0.f;
        }
        // f16: the offsets leave the weights before the MFMA -- (1024 + w) -
        // (1024 + z) and (16384 + 16 h) - 16384 are small integers, exact in a
        // packed f16 subtraction -- so the products sum to a * (w - z) and no
        // activation sums are needed. bf16 has no packed subtraction: there
        // the sums S of the activations come from an MFMA against ones and the
        // offsets leave in the fold, P - (offset + z) S.
        uint32_t sub_hi[CBW], sub_lo[CBW];
#pragma unroll
        for (int cb = 0; cb < CBW; cb++) {
            if constexpr (F16) {
                const float lo = OFFSET + (W8 ? 0.f : soff) + zp[cb];
                const float hi = W8 ? 16.f * OFFSET + 16.f * soff : lo;
                const uint32_t l16 = __builtin_bit_cast(uint16_t, (_Float16)lo);
                const uint32_t h16 = __builtin_bit_cast(uint16_t, (_Float16)hi);
                sub_lo[cb] = l16 | (l16 << 16);
                sub_hi[cb] = h16 | (h16 << 16);
            } else {
                sub_lo[cb] = sub_hi[cb] = 0;
            }
        }
        auto pk_sub = [](uint32_t x, uint32_t y) {
            return __builtin_bit_cast(uint32_t,
                    __builtin_bit_cast(v2h, x) - __builtin_bit_cast(v2h, y));
        };

        v4f Pu[RB][CBW], Su[RB];
#pragma unroll
        for (int rb = 0; rb < RB; rb++) {
            Su[rb] = v4f {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int cb = 0; cb < CBW; cb++) {
                Pu[rb][cb] = v4f {0.f, 0.f, 0.f, 0.f};
            }
        }
#pragma unroll
        for (int s4 = 0; s4 < 4; s4++) {
            v4u b[CBW], bl[CBW];
#pragma unroll
            for (int cb = 0; cb < CBW; cb++) {
                const uint32_t d = (s4 == 0 ? w_cur[cb][0].x
                                : s4 == 1   ? w_cur[cb][0].y
                                : s4 == 2   ? w_cur[cb][0].z
                                            : w_cur[cb][0].w)
                        ^ sflip;
                b[cb].x = (d & NIB) | MAGIC_HI;
                b[cb].y = ((d >> 4) & NIB) | MAGIC_HI;
                b[cb].z = ((d >> 8) & NIB) | MAGIC_HI;
                b[cb].w = ((d >> 12) & NIB) | MAGIC_HI;
                if constexpr (F16) {
#pragma unroll
                    for (int e = 0; e < 4; e++) b[cb][e] = pk_sub(b[cb][e], sub_hi[cb]);
                }
                bl[cb] = b[cb];
                if constexpr (W8) {
                    const uint32_t dl = s4 == 0 ? w_cur[cb][NP - 1].x
                            : s4 == 1           ? w_cur[cb][NP - 1].y
                            : s4 == 2           ? w_cur[cb][NP - 1].z
                                                : w_cur[cb][NP - 1].w;
                    bl[cb].x = (dl & NIB) | MAGIC;
                    bl[cb].y = ((dl >> 4) & NIB) | MAGIC;
                    bl[cb].z = ((dl >> 8) & NIB) | MAGIC;
                    bl[cb].w = ((dl >> 12) & NIB) | MAGIC;
                    if constexpr (F16) {
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            bl[cb][e] = pk_sub(bl[cb][e], sub_lo[cb]);
                    }
                }
            }
#pragma unroll
            for (int rb = 0; rb < RB; rb++) {
                // A operand: lane (r, c) holds row 16 rb + r, k = 32 s4 + 8 c ..
                const uint4 v = *(const uint4 *)(lds_a[sl]
                        + (16 * rb + r) * WF_PITCH + (32 * s4 + 8 * c) * 2);
                const v4u a = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int cb = 0; cb < CBW; cb++) {
                    Pu[rb][cb] = mfma16<F16>(a, b[cb], Pu[rb][cb]);
                    if constexpr (W8)
                        Pu[rb][cb] = mfma16<F16>(a, bl[cb], Pu[rb][cb]);
                }
                if constexpr (!F16) Su[rb] = mfma16<F16>(a, ones, Su[rb]);
            }
        }
#pragma unroll
        for (int cb = 0; cb < CBW; cb++) {
            const float off = W8 ? 17.f * OFFSET + 16.f * soff + zp[cb]
                                 : OFFSET + soff + zp[cb];
#pragma unroll
            for (int rb = 0; rb < RB; rb++)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    out[rb][cb][j] = F16
                            ? __builtin_fmaf(sc[cb], Pu[rb][cb][j], out[rb][cb][j])
                            : __builtin_fmaf(sc[cb],
                                      Pu[rb][cb][j] - off * Su[rb][j], out[rb][cb][j]);
        }
    };
    request(0, std::integral_constant<int, 0> {});
    request(1, std::integral_constant<int, 1> {});
    for (int kt = 0; kt < tiles; kt += 2) {
        k_tile(kt, std::integral_constant<int, 0> {});
        if (kt + 1 < tiles) k_tile(kt + 1, std::integral_constant<int, 1> {});
    }

    // Epilogue: the wave's results go through a wave-private LDS tile, 32 rows
    // at a time, and come back as four neighbouring columns of a row per lane,
    // so that bias / post-ops / dst conversion exist once and every store is a
    // vector. MFMA output: register j of lane l is row 4 * (l / 16) + j,
    // column l % 16.
    __syncthreads(); // every wave is done with the activation buffers
    float *const stg = (float *)(lds_raw + wave * STG_WAVE);
    const int n_w = nb0 * 16; // the wave's first column
    static_assert(RB == 2 || RB == 4, "halves of 32 rows");
    constexpr int QPR = 4 * CBW; // lanes (four columns each) per staged row
    auto flush = [&](auto h_tag) { // rows 32 h .. 32 h + 31 (h a constant:
        // the accumulators must stay in registers)
        constexpr int h = decltype(h_tag)::value;
#pragma unroll
        for (int rb2 = 0; rb2 < 2; rb2++)
#pragma unroll
            for (int cb = 0; cb < CBW; cb++)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    stg[(16 * rb2 + 4 * c + j) * STG_PITCH + 16 * cb + r]
                            = out[2 * h + rb2][cb][j];
        // (wave-private: the LDS writes above are ordered before the reads
        // below by the compiler's waitcnt, no barrier needed)
#pragma unroll 1
        for (int it = 0; it < 32 * QPR / 64; it++) {
            const int row = it * (64 / QPR) + lane / QPR, cg = (lane % QPR) * 4;
            const float4 t = *(const float4 *)&stg[row * STG_PITCH + cg];
            const int m = m0 + 32 * h + row, n = n_w + cg;
            if (m < M && n < N) {
                float v[4] = {t.x, t.y, t.z, t.w};
                epilogue_apply_store4(p.ep, v, 0, m, n, min(4, N - n));
            }
        }
    };
    flush(std::integral_constant<int, 0> {});
    if constexpr (RB == 4) flush(std::integral_constant<int, 1> {});
}

} // namespace

// Which shape a problem runs as: 64 x 256 blocks where they fill at least half
// the chip, else 128-column blocks of 32 or 64 rows.
static void w4f_shape(const gemv_params_t &p, int &bm, int &cbw) {
    const int64_t wide = (int64_t)((p.M + 63) / 64) * ((p.N + 255) / 256);
    cbw = p.M > 64 && wide >= 128 ? 2 : 1;
    bm = cbw == 1 && p.M <= 32 ? 32 : 64;
}

#define QMM_W4F_NAME2(n) launch_gemm_w4f_part##n
#define QMM_W4F_NAME(n) QMM_W4F_NAME2(n)
void QMM_W4F_NAME(QMM_W4F_PART)(const gemv_params_t &p, int shifts, int flags_m,
        hipStream_t stream) {
    int bm, cbw;
    w4f_shape(p, bm, cbw);
    const int bn = 16 * cbw * WF_WAVES;
    const dim3 grid((unsigned)((p.N + bn - 1) / bn), (unsigned)((p.M + bm - 1) / bm));
    auto go = [&](auto kern) {
        hipLaunchKernelGGL(kern, grid, dim3(WF_WAVES * 64), 0, stream, p, shifts,
                flags_m);
    };
    constexpr bool F = (QMM_W4F_PART & 1) != 0, W = (QMM_W4F_PART & 2) != 0;
    auto by_bm = [&](auto sgn) {
        constexpr bool S = decltype(sgn)::value;
        if (cbw == 2) go(gemm_w4f_kernel<F, S, W, 64, 2>);
        else if (bm == 64) go(gemm_w4f_kernel<F, S, W, 64, 1>);
        else go(gemm_w4f_kernel<F, S, W, 32, 1>);
    };
    if (p.wei_signed) by_bm(std::true_type {});
    else by_bm(std::false_type {});
}

#else // the launcher

void launch_gemm_w4f_part0(const gemv_params_t &, int, int, hipStream_t);
void launch_gemm_w4f_part1(const gemv_params_t &, int, int, hipStream_t);
void launch_gemm_w4f_part2(const gemv_params_t &, int, int, hipStream_t);
void launch_gemm_w4f_part3(const gemv_params_t &, int, int, hipStream_t);

// Whether the tiled kernel is the better way to run p.M > 16 rows, against the
// decode kernel once per block of 16 rows. Both walk K at about the same pace;
// measured at K = 4096: a pass of the decode kernel over 4096 columns 4.3 us, a
// round of 128-column workgroups 26 us (32 rows) or 40 us (64 rows).
bool gemm_w4f_wins(const gemv_params_t &p) {
    if (p.M <= 16) return false;
    const int64_t wide = (int64_t)((p.M + 63) / 64) * ((p.N + 255) / 256);
    if (p.M > 64 && wide >= 128) return true;
    const int bm = p.M <= 32 ? 32 : 64;
    const double wgs = (double)((p.M + bm - 1) / bm) * ((p.N + 127) / 128);
    const double rounds = wgs <= 256 ? 1.0 : wgs / 256;
    const double tiled = (bm == 32 ? 26.0 : 40.0) * rounds;
    const double passes = (double)((p.M + 15) / 16) * 4.3 * p.N / 4096.0;
    return tiled < passes;
}

// more than 16 rows (the caller decides with gemm_w4f_wins), fast-variant
// attribute set (the caller checks); flags_m and shifts as for
// gemv_w4_fast_kernel
void launch_gemm_w4f(const gemv_params_t &p, int shifts, int flags_m,
        hipStream_t stream) {
    switch ((p.act_f16 ? 1 : 0) | (p.w8 ? 2 : 0)) {
        case 0: launch_gemm_w4f_part0(p, shifts, flags_m, stream); break;
        case 1: launch_gemm_w4f_part1(p, shifts, flags_m, stream); break;
        case 2: launch_gemm_w4f_part2(p, shifts, flags_m, stream); break;
        default: launch_gemm_w4f_part3(p, shifts, flags_m, stream); break;
    }
}

#endif

} // namespace qmm
