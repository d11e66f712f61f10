// hip:gfx950:mfma_w4a8 -- s8 activations x 4-bit weights (s4 / u4) on the int8
// matrix cores, with scales that vary along K in groups on both operands
// (dynamically quantized activations, group-quantized weights) and optional
// grouped weights zero points.
//
// The arithmetic is that of src/cpu/matmul/ref_matmul_int8.cpp:139-219 with the
// group as the unit: inside a K group the products are summed in s32, the
// group's sum is converted to f32, multiplied by the source scale of (row,
// group) and the weights scale of (group, column) and added to an f32
// accumulator; bias / post-ops / dst quantization follow once at the end.
//
//   * weights are prepacked (QMM_LAYOUT_MFMA_W4K64): a 32-column x 64-k tile is
//     1 KiB, a lane's 16 bytes are its two 32-k operand fragments as nibbles.
//     Every nibble is a signed value w' (s4 as is, u4 minus 8) and is expanded
//     to the byte 16 * w' with one shift and two ANDs per eight values, so the
//     MFMA accumulates 16 * sum(s * w'): the factor is a power of two and is
//     folded into the weights scales;
//   * zero points and the u4 offset leave the dot product through the row sums
//     of the source: sum(s * (w - z)) = sum(s * w') - (z - off) * sum(s), all in
//     s32 (off = 8 for u4, 0 for s4);
//   * source zero points and u8 sources (read as s' = s - 128 by flipping the
//     top bit of each byte, zero point z_s' = z_s - 128) add the mirror term
//     through the column sums of the stored nibbles per group:
//     16 sum((s' - z_s')(w' - z_w')) = 16 sum(s' w') - 16 z_w' sum(s')
//         - z_s' * 16 (sum(w') - group * z_w');
//   * a pre-pass (w4a8_prep_kernel) rewrites the scale and zero-point buffers of
//     the launch, whatever their data types and strides, as f32 / s32 arrays
//     [group][row] and [group][column] in the scratchpad and computes the row
//     sums, so the GEMM fetches the 1 KiB of each that a group of its tile needs
//     with one direct-to-LDS load;
//   * a workgroup owns BM x BN of dst; tiles of 64 k are streamed global -> LDS
//     through a ring of STAGES, one barrier per tile (the scheme of
//     qmm_gemm_b8.hip). Each wave keeps two accumulator sets: s32 for the
//     running group (the first MFMA of a group starts from zero) and f32 for
//     the result. Two workgroups share a CU so that one can rescale while the
//     other multiplies.
#include <type_traits>

#include "qmm_device.hpp"
#include "qmm_plan.hpp"

namespace qmm {
namespace w4a8 {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));

template <int N, typename F>
QMM_D void static_for(F &&f) {
    if constexpr (N > 0) {
        static_for<N - 1>(f);
        f(std::integral_constant<int, N - 1> {});
    }
}

// 16-byte chunk q of row `row` of the row-major 64-byte-wide source tile
QMM_D int a_swz(int row, int q) {
    return q ^ ((row >> 2) & 3);
}

// lane l's 16 bytes go to lds_addr + 16 * l (wave-uniform lds_addr)
QMM_D void load_to_lds16(const void *gptr, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %1\n\t"
                 "s_nop 0\n\t"
                 "global_load_lds_dwordx4 %0, off"
                 :
                 : "v"(gptr), "s"(lds_addr)
                 : "memory", "m0");
}

constexpr int vmcnt_imm(int n) {
    return (n & 15) | ((n >> 4) << 14) | (7 << 4) | (15 << 8);
}

constexpr int BK = 64;
constexpr int X_BYTES = 1024; // one per-group array slice in LDS

// Scale / zero-point fetch of the small-row kernel in two steps without any
// control flow, so that a thread issues all its loads before it looks at the
// first value. SC: bytes of a scale (2: f16 or bf16, 4: f32). ZPK: storage of a
// zero point (1: s8 / u8, 2: s4 / u4, two per byte).
template <int SC>
QMM_D uint32_t scale_raw(const void *p, int64_t idx) {
    if constexpr (SC == 4)
        return ((const uint32_t *)p)[idx];
    else
        return ((const uint16_t *)p)[idx];
}
template <int SC>
QMM_D float scale_value(int dt, uint32_t raw) {
    if constexpr (SC == 4) {
        return u2f(raw);
    } else {
        const float h = (float)__builtin_bit_cast(_Float16, (uint16_t)raw);
        const float b = u2f(raw << 16);
        return dt == dt_f16 ? h : b;
    }
}
template <int ZPK>
QMM_D uint32_t zp_raw(const void *p, int64_t idx) {
    return ((const uint8_t *)p)[ZPK == 2 ? (idx >> 1) : idx];
}
template <int ZPK>
QMM_D int zp_value(int dt, uint32_t raw, int64_t idx) {
    if constexpr (ZPK == 2) {
        const int nib = (int)((raw >> (4 * (int)(idx & 1))) & 0xf);
        return dt == dt_s4 ? ((nib ^ 8) - 8) : nib;
    } else {
        return dt == dt_s8 ? (int)(int8_t)raw : (int)raw;
    }
}

// ZPM: 0 no zero points and s4 weights; 1 weights zero points or u4 weights
// (the group's source row sums take part); 2 also source zero points or a u8
// source (the group's weights column sums take part, and the source bytes
// are shifted to s8 by flipping their top bit).
// HALF: groups of 32 k, two per 64-k tile (each MFMA is a group of its own and
// the group end runs after it); the per-group arrays then travel with the
// tile, two slices each.
template <int BM, int BN, int WGM, int WGN, int STAGES, int ZPM, bool HALF = false>
__global__ void __launch_bounds__(WGM *WGN * 64, 2)
gemm_w4a8_kernel(const w4a8_params_t p) {
    constexpr bool HAS_ZP = ZPM >= 1, SRC_ZP = ZPM == 2;
    static_assert(!(HALF && SRC_ZP), "");
    constexpr int NW = WGM * WGN;
    constexpr int WM = BM / WGM, WN = BN / WGN;
    constexpr int FM = WM / 32, FN = WN / 32;
    constexpr int A_BYTES = BM * BK, B_BYTES = BN * BK / 2;
    constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
    // per-group arrays: ss, sw [, rs, zw [, zs, c2]]
    constexpr int NX = SRC_ZP ? 6 : HAS_ZP ? 4 : 2;
    constexpr int XSLOT = (HALF ? 2 : 1) * NX * X_BYTES;
    constexpr int X_OFF = STAGES * STAGE_BYTES;
    // wave-wide 1 KiB loads per tile / per group, spread over the waves; a
    // wave whose share runs past the end repeats earlier ones (same bytes to
    // the same place), so that every wave issues the same number
    constexpr int A_W = A_BYTES / 1024, B_W = B_BYTES / 1024;
    constexpr int TILE_W = A_W + B_W;
    constexpr int PER_T = (TILE_W + NW - 1) / NW;
    constexpr int PER_X = (NX + NW - 1) / NW;
    static_assert(A_W * 1024 == A_BYTES && B_W * 1024 == B_BYTES, "");
    static_assert(BM <= 256 && BN <= 256, "group arrays are 1 KiB of f32");
    static_assert(STAGES >= 3 && STAGES <= 6, "");
    typedef __attribute__((address_space(3))) uint8_t lds_u8;

    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm0 = (wave / WGN) * WM;
    const int wn0 = (wave % WGN) * WN;

    // XCD-aware tile order: consecutive logical tiles run on one XCD
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

    // ---- addresses of this wave's loads ----
    // Tile loads: index x < A_W is 16 source rows (4 chunks of 16 bytes each,
    // XOR-swizzled in LDS), the others one packed 32-column weights block.
    const uint8_t *t_ptr[PER_T];
    int t_step[PER_T];
    uint32_t t_lds[PER_T];
#pragma unroll
    for (int j = 0; j < PER_T; j++) {
        const int x = (wave * PER_T + j) % TILE_W; // wave-uniform
        if (x < A_W) {
            const int c = x * 64 + lane;
            const int row = c >> 2, cp = c & 3;
            const int gm = min(m0 + row, p.M - 1);
            t_ptr[j] = p.A + (int64_t)gm * p.lda + a_swz(row, cp) * 16;
            t_step[j] = BK;
            t_lds[j] = x * 1024;
        } else {
            const int y = x - A_W;
            const int nb = min(n0 / 32 + y, p.nb32 - 1);
            t_ptr[j] = p.B + (int64_t)nb * p.kt64 * 1024 + lane * 16;
            t_step[j] = 1024;
            t_lds[j] = A_BYTES + y * 1024;
        }
    }
    // Group loads: 256 consecutive f32 / s32 of the transposed arrays from the
    // tile's first row / column on (the arrays are padded so this stays inside)
    const uint8_t *x_ptr[PER_X];
    int64_t x_step[PER_X];
    uint32_t x_lds[PER_X];
#pragma unroll
    for (int j = 0; j < PER_X; j++) {
        const int x = (wave * PER_X + j) % NX;
        // 0: ss, 1: sw, 2: rs, 3: zw, 4: zs, 5: c2
        const bool row_side = (x & 1) == 0;
        const void *base = x == 0 ? (const void *)p.ssT
                : x == 1          ? (const void *)p.swT
                : x == 2          ? (const void *)p.rsT
                : x == 3          ? (const void *)p.zwT
                : x == 4          ? (const void *)p.zsT
                                  : (const void *)p.c2T;
        x_ptr[j] = (const uint8_t *)base
                + ((int64_t)(row_side ? m0 : n0) + lane * 4) * 4;
        x_step[j] = (int64_t)(row_side ? p.Mpad : p.Npad) * 4;
        x_lds[j] = x * X_BYTES;
    }

    const uint32_t lds_base = __builtin_amdgcn_readfirstlane(
            (uint32_t)(uintptr_t)(lds_u8 *)lds);
    const int KT = p.kt64;
    // issue state: tile number, its position in its group, the group
    int is_kt = 0, is_t = 0, is_g = 0;
    auto issue = [&]() {
        if constexpr (HALF) {
            const uint32_t xs = lds_base + X_OFF + (is_kt % STAGES) * XSLOT;
#pragma unroll
            for (int h = 0; h < 2; h++)
#pragma unroll
                for (int j = 0; j < PER_X; j++)
                    load_to_lds16(x_ptr[j] + (2 * is_kt + h) * x_step[j],
                            xs + h * NX * X_BYTES + x_lds[j]);
        } else if (is_t == 0) {
            const uint32_t xs = lds_base + X_OFF + (is_g % STAGES) * XSLOT;
#pragma unroll
            for (int j = 0; j < PER_X; j++)
                load_to_lds16(x_ptr[j] + is_g * x_step[j], xs + x_lds[j]);
        }
        const uint32_t st = lds_base + (is_kt % STAGES) * STAGE_BYTES;
#pragma unroll
        for (int j = 0; j < PER_T; j++)
            load_to_lds16(t_ptr[j] + (int64_t)is_kt * t_step[j], st + t_lds[j]);
        is_kt++;
        if (++is_t == p.tpg) {
            is_t = 0;
            is_g++;
        }
    };

    v16i acc[FM][FN];
    v16f res[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; i++)
#pragma unroll
        for (int j = 0; j < FN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                acc[i][j][r] = 0;
                res[i][j][r] = 0.f;
            }

#pragma unroll
    for (int s = 0; s < STAGES - 1; s++)
        if (s < KT) issue();

    // ---- group end: res += (float)(acc [+ zw * rowsum [+ zs * c2]]) * ss * sw
    auto group_end = [&](const uint8_t *xs) {
        // (zw = -16 (z_w - offset); c2 = -16 (column sum - group * (z_w - offset)))
        // Accumulator register r of lane l is row 8*(r/4) + 4*(l/32) + r%4,
        // column l%32 of its fragment.
        const float *ssl = (const float *)xs;
        const float *swl = (const float *)(xs + X_BYTES);
        const int32_t *rsl = (const int32_t *)(xs + 2 * X_BYTES);
        const int32_t *zwl = (const int32_t *)(xs + 3 * X_BYTES);
        const int32_t *zsl = (const int32_t *)(xs + 4 * X_BYTES);
        const int32_t *c2l = (const int32_t *)(xs + 5 * X_BYTES);
        float sw[FN];
        int zw[FN], c2[FN];
#pragma unroll
        for (int j = 0; j < FN; j++) {
            sw[j] = swl[wn0 + j * 32 + (lane & 31)];
            zw[j] = HAS_ZP ? zwl[wn0 + j * 32 + (lane & 31)] : 0;
            c2[j] = SRC_ZP ? c2l[wn0 + j * 32 + (lane & 31)] : 0;
        }
        static_for<FM>([&](auto I) {
            constexpr int i = decltype(I)::value;
            float ss[16];
            int rs[16], zs[16];
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int row = wm0 + i * 32 + 8 * q + 4 * (lane >> 5);
                if constexpr (SRC_ZP) {
                    const int4 z4 = *(const int4 *)&zsl[row];
                    zs[4 * q + 0] = z4.x;
                    zs[4 * q + 1] = z4.y;
                    zs[4 * q + 2] = z4.z;
                    zs[4 * q + 3] = z4.w;
                }
                const float4 s4 = *(const float4 *)&ssl[row];
                ss[4 * q + 0] = s4.x;
                ss[4 * q + 1] = s4.y;
                ss[4 * q + 2] = s4.z;
                ss[4 * q + 3] = s4.w;
                if constexpr (HAS_ZP) {
                    const int4 r4 = *(const int4 *)&rsl[row];
                    rs[4 * q + 0] = r4.x;
                    rs[4 * q + 1] = r4.y;
                    rs[4 * q + 2] = r4.z;
                    rs[4 * q + 3] = r4.w;
                }
            }
#pragma unroll
            for (int j = 0; j < FN; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    int t = acc[i][j][r];
                    if constexpr (HAS_ZP) t += __mul24(zw[j], rs[r]);
                    if constexpr (SRC_ZP) t += __mul24(zs[r], c2[j]);
                    res[i][j][r] = __builtin_fmaf(
                            (float)t * ss[r], sw[j], res[i][j][r]);
                }
        });
    };

    // one 64-k tile: FIRST starts the group's s32 accumulators from zero
    auto tile_mma = [&](int kt, auto first_tag) {
        constexpr bool FIRST = decltype(first_tag)::value;
        // the tile has landed once only younger tiles' loads are in flight (a
        // younger tile may carry group loads too: then this waits a little
        // longer than needed, never shorter)
        if (kt + STAGES - 2 < KT)
            __builtin_amdgcn_s_waitcnt(vmcnt_imm((STAGES - 2) * PER_T));
        else
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
        __syncthreads();
        if (kt + STAGES - 1 < KT) issue();

        const uint8_t *As = lds + (kt % STAGES) * STAGE_BYTES;
        const uint8_t *Bs = As + A_BYTES;
        uint4 braw[FN];
#pragma unroll
        for (int j = 0; j < FN; j++)
            braw[j] = *(const uint4 *)(Bs + (((wn0 >> 5) + j) * 64 + lane) * 16);
#pragma unroll
        for (int ki = 0; ki < 2; ki++) {
            v4i a[FM], b[FN];
#pragma unroll
            for (int i = 0; i < FM; i++) {
                const int row = wm0 + i * 32 + (lane & 31);
                const int q = ki * 2 + (lane >> 5);
                const uint4 v = *(const uint4 *)(As + row * BK
                        + a_swz(row, q) * 16);
                if constexpr (SRC_ZP) // u8 source: s - 128 as s8
                    a[i] = v4i {(int)(v.x ^ p.a_flip), (int)(v.y ^ p.a_flip),
                            (int)(v.z ^ p.a_flip), (int)(v.w ^ p.a_flip)};
                else
                    a[i] = v4i {(int)v.x, (int)v.y, (int)v.z, (int)v.w};
            }
#pragma unroll
            for (int j = 0; j < FN; j++) {
                const uint32_t w0 = ki ? braw[j].z : braw[j].x;
                const uint32_t w1 = ki ? braw[j].w : braw[j].y;
                b[j] = v4i {(int)((w0 << 4) & 0xF0F0F0F0u),
                        (int)(w0 & 0xF0F0F0F0u), (int)((w1 << 4) & 0xF0F0F0F0u),
                        (int)(w1 & 0xF0F0F0F0u)};
            }
#pragma unroll
            for (int i = 0; i < FM; i++)
#pragma unroll
                for (int j = 0; j < FN; j++) {
                    if (HALF || (FIRST && ki == 0)) {
                        const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0,
                                0, 0, 0};
                        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
                                a[i], b[j], zero, 0, 0, 0);
                    } else {
                        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
                                a[i], b[j], acc[i][j], 0, 0, 0);
                    }
                }
            if constexpr (HALF)
                group_end(lds + X_OFF + (kt % STAGES) * XSLOT
                        + ki * NX * X_BYTES);
        }
    };

    int kt = 0;
    if constexpr (HALF) {
        for (; kt < KT; kt++)
            tile_mma(kt, std::true_type {});
    } else
    for (int g = 0; g < p.ng; g++) {
        tile_mma(kt++, std::true_type {});
        for (int t = 1; t < p.tpg; t++)
            tile_mma(kt++, std::false_type {});

        group_end(lds + X_OFF + (g % STAGES) * XSLOT);
    }
    __syncthreads(); // LDS is reused by the epilogue

    // ---- epilogue: rows back through a wave-private LDS tile, 4 neighbouring
    // columns per lane, then bias / post-ops / dst conversion ----
    float *const stg = (float *)lds + wave * (32 * WN);
    constexpr int ROWS_PER_IT = 256 / WN;
    const int ecol = (lane % (WN / 4)) * 4;
    const int en = n0 + wn0 + ecol;
    const int envalid = min(4, p.N - en);
    const float one4[4] = {1.f, 1.f, 1.f, 1.f};
    ep_cols_t cols;
    epilogue_cols_load(p.ep, cols, 0, en, envalid > 0 ? envalid : 0);
    // the row interpreter reads the parameter block where it lies (the kernel
    // argument segment): its run-time indexing must not drag `p` into memory
    const epilogue_t &epk
            = ((const w4a8_params_t *)__builtin_amdgcn_kernarg_segment_ptr())->ep;
    static_for<FM>([&](auto I) {
        constexpr int i = decltype(I)::value;
#pragma unroll
        for (int j = 0; j < FN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int row = 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
                stg[row * WN + j * 32 + (lane & 31)] = res[i][j][r];
            }
#pragma unroll 1
        for (int it = 0; it < 32 / ROWS_PER_IT; it++) {
            const int row = it * ROWS_PER_IT + lane / (WN / 4);
            const float4 t = *(const float4 *)&stg[row * WN + ecol];
            const int m = m0 + wm0 + i * 32 + row;
            if (m < p.M && en < p.N) {
                float v[4] = {t.x, t.y, t.z, t.w};
                if (p.ep.fast != EP_FAST_NONE && !p.ep.fast_ext)
                    epilogue_fast4(
                            p.ep, v, false, 1.f, false, one4, 0, m, en, envalid);
                else
                    epilogue_rows4(epk, cols, v, false, 1.f, 0, m, en, envalid);
            }
        }
    });
}

#if !defined(QMM_W4A8_PART)
// ---- pre-pass ----
// One thread per (group, row) and per (group, column).
__global__ void __launch_bounds__(256) w4a8_prep_kernel(const w4a8_prep_t p) {
    const int64_t rows = (int64_t)p.ng * p.M, cols = (int64_t)p.ng * p.N;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
            i < rows + cols; i += (int64_t)gridDim.x * blockDim.x) {
        if (i < rows) {
            const int g = (int)(i / p.M), m = (int)(i % p.M);
            const int k0 = g * p.gk;
            p.ssT[(int64_t)g * p.Mpad + m] = p.ss
                    ? load_float(p.ss_dt, p.ss,
                            m * p.ss_sm + (k0 / p.ss_g) * p.ss_sk)
                    : 1.f;
            if (p.zsT) // source zero point of the (row, group), as s8 counts
                p.zsT[(int64_t)g * p.Mpad + m]
                        = (p.zs ? load_int(p.zs_dt, p.zs,
                                   m * p.zs_sm + (k0 / p.zs_g) * p.zs_sk)
                                : 0)
                        - (p.a_flip ? 128 : 0);
            if (p.rsT) {
                const uint8_t *a = p.A + (int64_t)m * p.lda + k0;
                int sum = 0;
                for (int k = 0; k < p.gk; k += 16) {
                    const uint4 v = *(const uint4 *)(a + k);
                    const uint32_t w[4] = {v.x ^ p.a_flip, v.y ^ p.a_flip,
                            v.z ^ p.a_flip, v.w ^ p.a_flip};
#pragma unroll
                    for (int d = 0; d < 4; d++)
                        sum += (int)(int8_t)(w[d] & 0xff)
                                + (int)(int8_t)((w[d] >> 8) & 0xff)
                                + (int)(int8_t)((w[d] >> 16) & 0xff)
                                + (int)(int8_t)(w[d] >> 24);
                }
                p.rsT[(int64_t)g * p.Mpad + m] = sum;
            }
        } else {
            const int64_t c = i - rows;
            const int g = (int)(c / p.N), n = (int)(c % p.N);
            const int k0 = g * p.gk;
            const float s = p.sw ? load_float(p.sw_dt, p.sw,
                                    (k0 / p.sw_g) * p.sw_sk + n * p.sw_sn)
                                 : 1.f;
            p.swT[(int64_t)g * p.Npad + n] = s * 0.0625f;
            if (p.zwT) {
                const int z = p.zw ? load_int(p.zw_dt, p.zw,
                                      (k0 / p.zw_g) * p.zw_sk + n * p.zw_sn)
                                   : 0;
                p.zwT[(int64_t)g * p.Npad + n] = -16 * (z - p.w_off);
                if (p.c2T) {
                    // column sum of the group's stored nibbles w' (signed):
                    // the 64 k of a tile are the 16-byte pieces of lanes
                    // n % 32 and n % 32 + 32 of the column block's tile
                    const int tpg = p.gk / 64;
                    const uint8_t *b = p.B
                            + (((int64_t)(n >> 5) * p.kt64 + (int64_t)g * tpg) * 64
                                      + (n & 31))
                                    * 16;
                    int sum = 0;
                    for (int t = 0; t < tpg; t++) {
#pragma unroll
                        for (int h = 0; h < 2; h++) {
                            const uint4 v = *(const uint4 *)(b + (int64_t)t * 1024
                                    + h * 512);
                            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                            for (int d = 0; d < 4; d++) {
                                // nibble ^ 8 is w' + 8: bytewise sums of the
                                // low and high nibbles, then of the four bytes
                                const uint32_t y = w[d] ^ 0x88888888u;
                                const uint32_t e = (y & 0x0F0F0F0Fu)
                                        + ((y >> 4) & 0x0F0F0F0Fu);
                                sum += (int)((e * 0x01010101u) >> 24) - 64;
                            }
                        }
                    }
                    p.c2T[(int64_t)g * p.Npad + n]
                            = -16 * sum + p.gk * 16 * (z - p.w_off);
                }
            }
        }
    }
}

#endif // pre-pass

// ---- rows <= 64: split-K streaming kernel ----
// At these sizes the launch is one read of the weights and nothing else
// matters, so the kernel is built around memory-level parallelism: 128 columns
// x FM*32 rows per workgroup of four waves, each wave owning 32 columns. The
// packed layout already is the MFMA operand order per lane, so a wave loads
// its weights fragments straight into registers, SM_CH tiles (1 KiB each) at
// a time (the host cuts K so that a slice is one chunk where it can), all
// requested first thing in the kernel; behind them the scales / zero points of
// the slice (converted once into LDS) and the source rows of the chunk (staged
// in LDS, shared by the four waves), so the whole workgroup costs one memory
// round trip. Row sums come from v_dot4 on the source fragments. No pre-pass,
// no direct-to-LDS loads.
constexpr int SM_CH = 16; // 64-k tiles per chunk

// HAS_ZP: zero points or u4 weights (row-sum path); ZPK: 0 = no zero-point
// buffer (the constant u4 offset only), else its storage class. MODE 1: groups
// of 32 k (p.tpg == 0): every MFMA is a group of its own, twice the groups per
// slice. MODE 2: source zero points / u8 source (with HAS_ZP), as in the
// single-token kernel below: the source bytes are flipped to s8, the column
// sums of the stored nibbles come from dot products of the weights operand
// with ones, and the group end adds z_s' * -(16 sum w' + group * zw).
constexpr int sm_maxg(int mode) { // groups per slice
    return mode == 1 ? 2 * W4A8_SMALL_MAX_GPS : W4A8_SMALL_MAX_GPS;
}
constexpr size_t sm_lds_bytes(int fm, int mode) {
    return (size_t)SM_CH * fm * 32 * BK
            + (size_t)sm_maxg(mode) * (fm * 32 * 4 * (mode == 2 ? 2 : 1) + 128 * 4 + 128 * 4)
            + 4 * fm * 32 * 4;
}

template <int FM, int SC, bool HAS_ZP, int ZPK, int MODE = 0>
__global__ void __launch_bounds__(256)
w4a8_small_kernel(const w4a8_small_t p) {
    constexpr bool HALF = MODE == 1, SZP = MODE == 2;
    static_assert(!SZP || HAS_ZP, "");
    constexpr int BM = FM * 32, BN = 128, NT = 256;
    constexpr int MAXG = sm_maxg(MODE);
    constexpr int A_BYTES = SM_CH * BM * BK; // [tile][row][64 B], swizzled
    constexpr int SS_OFF = A_BYTES;
    constexpr int ZS_OFF = SS_OFF + MAXG * BM * 4; // SZP only
    constexpr int SW_OFF = ZS_OFF + (SZP ? MAXG * BM * 4 : 0);
    constexpr int ZW_OFF = SW_OFF + MAXG * BN * 4;
    constexpr int RS_OFF = ZW_OFF + MAXG * BN * 4; // [4 waves][BM] s32
    constexpr int A_PER = SM_CH * BM * 4 / NT; // 16-byte pieces per thread
    constexpr int SS_PER = MAXG * BM / NT, SW_PER = MAXG * BN / NT;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const w4a8_prep_t &q = p.q;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n0 = blockIdx.x * BN;
    const int m0 = blockIdx.z * BM;
    const int split = blockIdx.y;
    const int g_begin = split * p.gps; // p.gps is even with groups of 32 k
    const int g_cnt = min(p.gps, q.ng - g_begin);
    const int T0 = HALF ? g_begin / 2 : g_begin * p.tpg; // first 64-k tile of the slice
    const int KT = HALF ? g_cnt / 2 : g_cnt * p.tpg; // tiles of this workgroup

    // Request order = order of use: source rows, scales, then the weights tile
    // by tile, so that every wait below leaves the younger requests in flight.
    // source rows of a chunk: piece = 16 bytes, 64 pieces per row
    uint4 av[A_PER];
    auto load_rows = [&](int t0, int cnt) {
#pragma unroll
        for (int j = 0; j < A_PER; j++) {
            const int pc = tid + j * NT;
            const int row = pc >> 6, c16 = pc & 63;
            av[j] = make_uint4(0, 0, 0, 0);
            if (m0 + row < q.M && (c16 >> 2) < cnt)
                av[j] = *(const uint4 *)(q.A + (int64_t)(m0 + row) * q.lda
                        + (int64_t)(T0 + t0) * BK + c16 * 16);
        }
    };
    auto stage_rows = [&]() {
#pragma unroll
        for (int j = 0; j < A_PER; j++) {
            const int pc = tid + j * NT;
            const int row = pc >> 6, c16 = pc & 63;
            const int tl = c16 >> 2, cp = c16 & 3;
            *(uint4 *)(lds + (tl * BM + row) * BK + a_swz(row, cp) * 16) = av[j];
        }
    };
    // this wave's 32-column block of the packed weights; tiles past the end of
    // a chunk repeat its last one
    const int nb = min(n0 / 32 + wave, p.nb32 - 1);
    const v4u *bsrc = (const v4u *)(p.B + (int64_t)nb * p.kt64 * 1024) + lane;
    v4u bq[SM_CH];
    auto load_weights = [&](int t0, int cnt) {
#pragma unroll
        for (int j = 0; j < SM_CH; j++)
            bq[j] = __builtin_nontemporal_load(
                    bsrc + (int64_t)(T0 + t0 + min(j, cnt - 1)) * 64);
    };

    load_rows(0, min(SM_CH, KT));
    // scales and zero points of the slice (f32 / s32 in LDS, [group][row or
    // column]): all loads of a thread before the first conversion
    uint32_t rs_[SS_PER], rzs_[SS_PER], rw_[SW_PER], rz_[SW_PER];
    int64_t iz_[SW_PER];
    const bool has_ss = q.ss != nullptr, has_sw = q.sw != nullptr;
#pragma unroll
    for (int j = 0; j < SS_PER; j++)
        rs_[j] = rzs_[j] = 0;
#pragma unroll
    for (int j = 0; j < SW_PER; j++) {
        rw_[j] = rz_[j] = 0;
        iz_[j] = 0;
    }
    if (has_ss) {
#pragma unroll
        for (int j = 0; j < SS_PER; j++) {
            const int i = tid + j * NT;
            const int gl = min(i / BM, g_cnt - 1), r = i % BM;
            const int k0 = (g_begin + gl) * q.gk;
            const int m = min(m0 + r, q.M - 1);
            rs_[j] = scale_raw<SC>(q.ss, m * q.ss_sm + (k0 / q.ss_g) * q.ss_sk);
        }
    }
    if constexpr (SZP) {
        if (q.zs) { // one byte per value: s8 or u8 (host-checked)
#pragma unroll
            for (int j = 0; j < SS_PER; j++) {
                const int i = tid + j * NT;
                const int gl = min(i / BM, g_cnt - 1), r = i % BM;
                const int k0 = (g_begin + gl) * q.gk;
                const int m = min(m0 + r, q.M - 1);
                rzs_[j] = ((const uint8_t *)q.zs)[m * q.zs_sm + (k0 / q.zs_g) * q.zs_sk];
            }
        }
    }
    if (has_sw) {
#pragma unroll
        for (int j = 0; j < SW_PER; j++) {
            const int i = tid + j * NT;
            const int gl = min(i / BN, g_cnt - 1), c = i % BN;
            const int k0 = (g_begin + gl) * q.gk;
            const int n = min(n0 + c, q.N - 1);
            rw_[j] = scale_raw<SC>(q.sw, (k0 / q.sw_g) * q.sw_sk + n * q.sw_sn);
        }
    }
    if constexpr (ZPK != 0) {
#pragma unroll
        for (int j = 0; j < SW_PER; j++) {
            const int i = tid + j * NT;
            const int gl = min(i / BN, g_cnt - 1), c = i % BN;
            const int k0 = (g_begin + gl) * q.gk;
            const int n = min(n0 + c, q.N - 1);
            iz_[j] = (k0 / q.zw_g) * q.zw_sk + n * q.zw_sn;
            rz_[j] = zp_raw<ZPK>(q.zw, iz_[j]);
        }
    }
    load_weights(0, min(SM_CH, KT));

    stage_rows();
    {
        float *ssl = (float *)(lds + SS_OFF);
        float *swl = (float *)(lds + SW_OFF);
        int32_t *zwl = (int32_t *)(lds + ZW_OFF);
#pragma unroll
        for (int j = 0; j < SS_PER; j++) {
            const int i = tid + j * NT;
            const float v = scale_value<SC>(q.ss_dt, rs_[j]);
            if (i < g_cnt * BM) {
                ssl[i] = has_ss ? v : 1.f;
                if constexpr (SZP) {
                    const int z = !q.zs      ? 0
                            : q.zs_dt == dt_s8 ? (int)(int8_t)rzs_[j]
                                               : (int)rzs_[j];
                    ((int32_t *)(lds + ZS_OFF))[i] = z - (q.a_flip ? 128 : 0);
                }
            }
        }
#pragma unroll
        for (int j = 0; j < SW_PER; j++) {
            const int i = tid + j * NT;
            const float v = scale_value<SC>(q.sw_dt, rw_[j]);
            if (i < g_cnt * BN) {
                swl[i] = (has_sw ? v : 1.f) * 0.0625f;
                if constexpr (HAS_ZP) {
                    int z = 0;
                    if constexpr (ZPK != 0)
                        z = zp_value<ZPK>(q.zw_dt, rz_[j], iz_[j]);
                    zwl[i] = -16 * (z - q.w_off);
                }
            }
        }
    }
    __syncthreads();

    v16i acc[FM];
    v16f res[FM];
    int rsum[FM], csum = 0;
#pragma unroll
    for (int i = 0; i < FM; i++) {
        rsum[i] = 0;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            acc[i][r] = 0;
            res[i][r] = 0.f;
        }
    }
    const float *ssl = (const float *)(lds + SS_OFF);
    const float *swl = (const float *)(lds + SW_OFF);
    const int32_t *zwl = (const int32_t *)(lds + ZW_OFF);
    int32_t *rsw = (int32_t *)(lds + RS_OFF) + wave * BM;
    const int32_t *zsl = (const int32_t *)(lds + ZS_OFF);
    int t_in_g = 0, gl = 0; // position of the next tile in its group; the group
    const int mrows = min(BM, q.M - m0);
    // group end: res += (float)(acc [+ zw * rowsum [+ zs * c2]]) * ss * sw
    auto group_end = [&]() {
        const float sw = swl[gl * BN + wave * 32 + (lane & 31)];
        int zw = 0, c2 = 0;
        if constexpr (HAS_ZP) {
            zw = zwl[gl * BN + wave * 32 + (lane & 31)];
#pragma unroll
            for (int i = 0; i < FM; i++) {
                // both k halves of a row: lanes l and l ^ 32
                const int tot = rsum[i] + __shfl_xor(rsum[i], 32);
                rsw[i * 32 + (lane & 31)] = tot;
                rsum[i] = 0;
            }
        }
        if constexpr (SZP) {
            // the column's 16 * sum w' of the group, both k halves
            const int ctot = csum + __shfl_xor(csum, 32);
            csum = 0;
            c2 = -ctot - q.gk * zw;
        }
#pragma unroll
        for (int i = 0; i < FM; i++) {
#pragma unroll
            for (int c = 0; c < 4; c++) {
                // registers 4c..4c+3 are rows 8c..8c+7 of the fragment: skip
                // those past the last row
                if (i * 32 + 8 * c >= mrows) continue;
                const int row = i * 32 + 8 * c + 4 * (lane >> 5);
                const float4 s4 = *(const float4 *)&ssl[gl * BM + row];
                const float ss[4] = {s4.x, s4.y, s4.z, s4.w};
                int rs[4] = {0, 0, 0, 0}, zs[4] = {0, 0, 0, 0};
                if constexpr (HAS_ZP) {
                    const int4 r4 = *(const int4 *)&rsw[row];
                    rs[0] = r4.x;
                    rs[1] = r4.y;
                    rs[2] = r4.z;
                    rs[3] = r4.w;
                }
                if constexpr (SZP) {
                    const int4 z4 = *(const int4 *)&zsl[gl * BM + row];
                    zs[0] = z4.x;
                    zs[1] = z4.y;
                    zs[2] = z4.z;
                    zs[3] = z4.w;
                }
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    int t = acc[i][4 * c + e];
                    if constexpr (HAS_ZP) t += __mul24(zw, rs[e]);
                    if constexpr (SZP) t += __mul24(zs[e], c2);
                    res[i][4 * c + e] = __builtin_fmaf(
                            (float)t * ss[e], sw, res[i][4 * c + e]);
                }
            }
        }
        gl++;
    };

    for (int t0 = 0; t0 < KT; t0 += SM_CH) {
        const int cnt = min(SM_CH, KT - t0);
        if (t0 > 0) {
            load_rows(t0, cnt);
            load_weights(t0, cnt);
            __syncthreads(); // everybody is done with the previous chunk's rows
            stage_rows();
            __syncthreads();
        }
#pragma unroll
        for (int j = 0; j < SM_CH; j++) {
            if (j < cnt) {
                const uint8_t *As = lds + j * BM * BK;
                const bool first = t_in_g == 0; // the group's accumulators start at 0
#pragma unroll
                for (int ki = 0; ki < 2; ki++) {
                    const uint32_t w0 = ki ? bq[j].z : bq[j].x;
                    const uint32_t w1 = ki ? bq[j].w : bq[j].y;
                    const v4i b = {(int)((w0 << 4) & 0xF0F0F0F0u),
                            (int)(w0 & 0xF0F0F0F0u),
                            (int)((w1 << 4) & 0xF0F0F0F0u),
                            (int)(w1 & 0xF0F0F0F0u)};
                    if constexpr (SZP) {
                        int t = csum;
                        t = __builtin_amdgcn_sdot4(b[0], 0x01010101, t, false);
                        t = __builtin_amdgcn_sdot4(b[1], 0x01010101, t, false);
                        t = __builtin_amdgcn_sdot4(b[2], 0x01010101, t, false);
                        t = __builtin_amdgcn_sdot4(b[3], 0x01010101, t, false);
                        csum = t;
                    }
#pragma unroll
                    for (int i = 0; i < FM; i++) {
                        const int row = i * 32 + (lane & 31);
                        const int cq = ki * 2 + (lane >> 5);
                        const uint4 v = *(const uint4 *)(As + row * BK
                                + a_swz(row, cq) * 16);
                        v4i a = {(int)v.x, (int)v.y, (int)v.z, (int)v.w};
                        if constexpr (SZP) // u8 source: s - 128 as s8
                            a = v4i {(int)(v.x ^ q.a_flip), (int)(v.y ^ q.a_flip),
                                    (int)(v.z ^ q.a_flip), (int)(v.w ^ q.a_flip)};
                        if constexpr (HAS_ZP) {
                            int t = rsum[i];
                            t = __builtin_amdgcn_sdot4(a[0], 0x01010101, t, false);
                            t = __builtin_amdgcn_sdot4(a[1], 0x01010101, t, false);
                            t = __builtin_amdgcn_sdot4(a[2], 0x01010101, t, false);
                            t = __builtin_amdgcn_sdot4(a[3], 0x01010101, t, false);
                            rsum[i] = t;
                        }
                        if (HALF || (ki == 0 && first)) {
                            const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0,
                                    0, 0, 0, 0};
                            acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
                                    a, b, zero, 0, 0, 0);
                        } else {
                            acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
                                    a, b, acc[i], 0, 0, 0);
                        }
                    }
                    if constexpr (HALF) group_end();
                }
                if constexpr (!HALF) {
                    if (++t_in_g == p.tpg) {
                        t_in_g = 0;
                        group_end();
                    }
                }
            }
        }
    }

    // slice result -> part[split][m][n]
    const int n = n0 + wave * 32 + (lane & 31);
    if (n < q.N) {
        float *out = p.part + (int64_t)split * q.M * p.ldp + n;
#pragma unroll
        for (int i = 0; i < FM; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int m = m0 + i * 32 + 8 * (r / 4) + 4 * (lane >> 5) + r % 4;
                if (m < q.M) out[(int64_t)m * p.ldp] = res[i][r];
            }
    }
}

// ---- rows <= 4 (single-token decode): one launch, no partial results ----
// A workgroup owns 32 columns; its NWV waves cut K between them (whole groups),
// each wave exactly as a wave of the kernel above but with everything it
// stages (its rows of the source, the scales of its groups) in a wave-private
// piece of LDS, so there is no barrier before the end. The waves' results are
// summed through LDS in wave order (= K order) by wave 0, which also runs the
// epilogue. Accumulator registers 0..3 of lanes 0..31 are rows 0..3: the only
// ones looked at.
// MODE 1: groups of 32 k (p.tpg == 0): every MFMA is a group of its own, twice
// the groups per wave. MODE 2: source zero points / u8 source (with HAS_ZP):
// the source bytes are flipped to s8, the column sums of the stored nibbles
// come from dot products of the weights operand with ones, and the group end
// adds z_s' * -(16 sum w' + group * zw) (see gemm_w4a8_kernel).
constexpr int TN_ROWS = 4;
constexpr int TN_AROW = SM_CH * BK + 16; // staged row, padded against conflicts
constexpr int tn_maxg(int mode) { // groups per wave
    return mode == 1 ? 32 : 16;
}
constexpr int tn_wave_bytes(int mode) {
    // rows, source scales [, source zero points], weights scales, zero points
    return TN_ROWS * TN_AROW + tn_maxg(mode) * 4 * 4 * (mode == 2 ? 2 : 1)
            + tn_maxg(mode) * 32 * 4 + tn_maxg(mode) * 32 * 4;
}

template <int NWV, int SC, bool HAS_ZP, int ZPK, int MODE = 0>
__global__ void __launch_bounds__(NWV * 64)
w4a8_tiny_kernel(const w4a8_small_t p) {
    constexpr bool HALF = MODE == 1, SZP = MODE == 2;
    static_assert(!SZP || HAS_ZP, "");
    constexpr int TN_MAXG = tn_maxg(MODE), TN_WAVE_BYTES = tn_wave_bytes(MODE);
    constexpr int SW_PER = TN_MAXG * 32 / 64, SS_PER = TN_MAXG * 4 / 64;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const w4a8_prep_t &q = p.q;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n0 = blockIdx.x * 32;
    const int g_begin = wave * p.gps; // p.gps is even with groups of 32 k
    const int g_cnt = max(0, min(p.gps, q.ng - g_begin));
    const int T0 = HALF ? g_begin / 2 : g_begin * p.tpg;
    const int KT = HALF ? g_cnt / 2 : g_cnt * p.tpg; // tiles of this wave
    uint8_t *wA = lds + wave * TN_WAVE_BYTES;
    float *wss = (float *)(wA + TN_ROWS * TN_AROW);
    int32_t *wzs = (int32_t *)(wss + TN_MAXG * 4); // SZP only
    float *wsw = wss + TN_MAXG * 4 * (SZP ? 2 : 1);
    int32_t *wzw = (int32_t *)(wsw + TN_MAXG * 32);
    float *red = (float *)(lds + NWV * TN_WAVE_BYTES); // [NWV][4][32]

    float res[4] = {0.f, 0.f, 0.f, 0.f};
    if (KT > 0) {
        // request order = order of use: rows, scales, weights tile by tile
        uint4 av[TN_ROWS];
        auto load_rows = [&](int t0, int cnt) {
#pragma unroll
            for (int r = 0; r < TN_ROWS; r++) {
                av[r] = make_uint4(0, 0, 0, 0);
                if (r < q.M && (lane >> 2) < cnt)
                    av[r] = *(const uint4 *)(q.A + (int64_t)r * q.lda
                            + (int64_t)(T0 + t0) * BK + lane * 16);
            }
        };
        auto stage_rows = [&]() {
#pragma unroll
            for (int r = 0; r < TN_ROWS; r++)
                *(uint4 *)(wA + r * TN_AROW + lane * 16) = av[r];
        };
        const int nb = min(n0 / 32, p.nb32 - 1);
        const v4u *bsrc
                = (const v4u *)(p.B + (int64_t)nb * p.kt64 * 1024) + lane;
        v4u bq[SM_CH];
        auto load_weights = [&](int t0, int cnt) {
#pragma unroll
            for (int j = 0; j < SM_CH; j++)
                bq[j] = __builtin_nontemporal_load(
                        bsrc + (int64_t)(T0 + t0 + min(j, cnt - 1)) * 64);
        };

        load_rows(0, min(SM_CH, KT));
        const bool has_ss = q.ss != nullptr, has_sw = q.sw != nullptr;
        uint32_t rs_[SS_PER], rzs_[SS_PER], rw_[SW_PER], rz_[SW_PER];
        int64_t iz_[SW_PER];
#pragma unroll
        for (int j = 0; j < SS_PER; j++)
            rs_[j] = rzs_[j] = 0;
#pragma unroll
        for (int j = 0; j < SW_PER; j++) {
            rw_[j] = rz_[j] = 0;
            iz_[j] = 0;
        }
#pragma unroll
        for (int j = 0; j < SS_PER; j++) {
            const int i = lane + j * 64;
            const int gl = min(i >> 2, g_cnt - 1), r = min(i & 3, q.M - 1);
            const int k0 = (g_begin + gl) * q.gk;
            if (has_ss)
                rs_[j] = scale_raw<SC>(
                        q.ss, r * q.ss_sm + (k0 / q.ss_g) * q.ss_sk);
            if constexpr (SZP) {
                if (q.zs) // one byte: s8 or u8 (host-checked)
                    rzs_[j] = ((const uint8_t *)q.zs)[r * q.zs_sm
                            + (k0 / q.zs_g) * q.zs_sk];
            }
        }
        if (has_sw) {
#pragma unroll
            for (int j = 0; j < SW_PER; j++) {
                const int i = lane + j * 64;
                const int gl = min(i >> 5, g_cnt - 1), c = i & 31;
                const int k0 = (g_begin + gl) * q.gk;
                const int n = min(n0 + c, q.N - 1);
                rw_[j] = scale_raw<SC>(
                        q.sw, (k0 / q.sw_g) * q.sw_sk + n * q.sw_sn);
            }
        }
        if constexpr (ZPK != 0) {
#pragma unroll
            for (int j = 0; j < SW_PER; j++) {
                const int i = lane + j * 64;
                const int gl = min(i >> 5, g_cnt - 1), c = i & 31;
                const int k0 = (g_begin + gl) * q.gk;
                const int n = min(n0 + c, q.N - 1);
                iz_[j] = (k0 / q.zw_g) * q.zw_sk + n * q.zw_sn;
                rz_[j] = zp_raw<ZPK>(q.zw, iz_[j]);
            }
        }
        load_weights(0, min(SM_CH, KT));

        stage_rows();
#pragma unroll
        for (int j = 0; j < SS_PER; j++) {
            const float v = scale_value<SC>(q.ss_dt, rs_[j]);
            wss[lane + j * 64] = has_ss ? v : 1.f;
            if constexpr (SZP) {
                const int z = !q.zs ? 0
                        : q.zs_dt == dt_s8 ? (int)(int8_t)rzs_[j]
                                           : (int)rzs_[j];
                wzs[lane + j * 64] = z - (q.a_flip ? 128 : 0);
            }
        }
#pragma unroll
        for (int j = 0; j < SW_PER; j++) {
            const int i = lane + j * 64;
            const float v = scale_value<SC>(q.sw_dt, rw_[j]);
            wsw[i] = (has_sw ? v : 1.f) * 0.0625f;
            if constexpr (HAS_ZP) {
                int z = 0;
                if constexpr (ZPK != 0) z = zp_value<ZPK>(q.zw_dt, rz_[j], iz_[j]);
                wzw[i] = -16 * (z - q.w_off);
            }
        }

        v16i acc;
#pragma unroll
        for (int r = 0; r < 16; r++)
            acc[r] = 0;
        int rsum = 0, csum = 0;
        int t_in_g = 0, gl = 0;
        const int arow = min(lane & 31, q.M - 1) * TN_AROW + (lane >> 5) * 16;
        // group end: res += (float)(acc [+ zw * rowsum [+ zs * c2]]) * ss * sw
        auto group_end = [&]() {
            const float sw = wsw[gl * 32 + (lane & 31)];
            const float4 s4 = *(const float4 *)&wss[gl * 4];
            const float ss[4] = {s4.x, s4.y, s4.z, s4.w};
            int zw = 0, tot = 0, c2 = 0;
            int zs[4] = {0, 0, 0, 0};
            if constexpr (HAS_ZP) {
                zw = wzw[gl * 32 + (lane & 31)];
                // both k halves of a row: lanes l and l ^ 32;
                // row r of the source sits in lane r
                tot = rsum + __shfl_xor(rsum, 32);
                rsum = 0;
            }
            if constexpr (SZP) {
                // the column's 16 * sum w' of the group, both k halves
                const int ctot = csum + __shfl_xor(csum, 32);
                csum = 0;
                c2 = -ctot - q.gk * zw;
                const int4 z4 = *(const int4 *)&wzs[gl * 4];
                zs[0] = z4.x;
                zs[1] = z4.y;
                zs[2] = z4.z;
                zs[3] = z4.w;
            }
#pragma unroll
            for (int r = 0; r < 4; r++) {
                int t = acc[r];
                if constexpr (HAS_ZP)
                    t += __mul24(zw, __builtin_amdgcn_readlane(tot, r));
                if constexpr (SZP) t += __mul24(zs[r], c2);
                res[r] = __builtin_fmaf((float)t * ss[r], sw, res[r]);
            }
            gl++;
        };
        for (int t0 = 0; t0 < KT; t0 += SM_CH) {
            const int cnt = min(SM_CH, KT - t0);
            if (t0 > 0) {
                load_rows(t0, cnt);
                load_weights(t0, cnt);
                stage_rows();
            }
#pragma unroll
            for (int j = 0; j < SM_CH; j++) {
                if (j < cnt) {
                    const bool first = t_in_g == 0;
#pragma unroll
                    for (int ki = 0; ki < 2; ki++) {
                        const uint32_t w0 = ki ? bq[j].z : bq[j].x;
                        const uint32_t w1 = ki ? bq[j].w : bq[j].y;
                        const v4i b = {(int)((w0 << 4) & 0xF0F0F0F0u),
                                (int)(w0 & 0xF0F0F0F0u),
                                (int)((w1 << 4) & 0xF0F0F0F0u),
                                (int)(w1 & 0xF0F0F0F0u)};
                        const uint4 v = *(const uint4 *)(wA + arow
                                + (j * 4 + ki * 2) * 16);
                        v4i a = {(int)v.x, (int)v.y, (int)v.z, (int)v.w};
                        if constexpr (SZP) {
                            // u8 source: s - 128 as s8
                            a = v4i {(int)(v.x ^ q.a_flip), (int)(v.y ^ q.a_flip),
                                    (int)(v.z ^ q.a_flip), (int)(v.w ^ q.a_flip)};
                            int t = csum;
                            t = __builtin_amdgcn_sdot4(b[0], 0x01010101, t, false);
                            t = __builtin_amdgcn_sdot4(b[1], 0x01010101, t, false);
                            t = __builtin_amdgcn_sdot4(b[2], 0x01010101, t, false);
                            t = __builtin_amdgcn_sdot4(b[3], 0x01010101, t, false);
                            csum = t;
                        }
                        if constexpr (HAS_ZP) {
                            int t = rsum;
                            t = __builtin_amdgcn_sdot4(a[0], 0x01010101, t, false);
                            t = __builtin_amdgcn_sdot4(a[1], 0x01010101, t, false);
                            t = __builtin_amdgcn_sdot4(a[2], 0x01010101, t, false);
                            t = __builtin_amdgcn_sdot4(a[3], 0x01010101, t, false);
                            rsum = t;
                        }
                        if (HALF || (ki == 0 && first)) {
                            const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0,
                                    0, 0, 0, 0};
                            acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(
                                    a, b, zero, 0, 0, 0);
                        } else {
                            acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(
                                    a, b, acc, 0, 0, 0);
                        }
                        if constexpr (HALF) group_end();
                    }
                    if constexpr (!HALF) {
                        if (++t_in_g == p.tpg) {
                            t_in_g = 0;
                            group_end();
                        }
                    }
                }
            }
        }
    }

    if (lane < 32) {
#pragma unroll
        for (int r = 0; r < 4; r++)
            red[(wave * 4 + r) * 32 + lane] = res[r];
    }
    __syncthreads();
    if (wave == 0 && lane < 32) {
        const int n = n0 + lane;
        for (int r = 0; r < q.M; r++) {
            float v = red[r * 32 + lane];
            for (int w = 1; w < NWV; w++)
                v += red[(w * 4 + r) * 32 + lane];
            if (n < q.N) epilogue_apply_store(p.ep, v, 0, r, n);
        }
    }
}

template <int NWV, int SC, bool HAS_ZP, int ZPK, int MODE = 0>
static void launch_tiny_cfg(const w4a8_small_t &p, hipStream_t stream) {
    constexpr size_t lds = (size_t)NWV * tn_wave_bytes(MODE) + NWV * 4 * 32 * 4;
    auto kern = w4a8_tiny_kernel<NWV, SC, HAS_ZP, ZPK, MODE>;
    ensure_dynamic_lds((const void *)kern, (int)lds);
    hipLaunchKernelGGL(kern, dim3((p.q.N + 31) / 32), dim3(NWV * 64), lds,
            stream, p);
}

template <int NWV, int SC, int MODE = 0>
static void launch_tiny_zp(const w4a8_small_t &p, bool has_zp, int zpk,
        hipStream_t stream) {
    if constexpr (MODE != 2) {
        if (!has_zp) {
            launch_tiny_cfg<NWV, SC, false, 0, MODE>(p, stream);
            return;
        }
    }
    if (zpk == 0)
        launch_tiny_cfg<NWV, SC, true, 0, MODE>(p, stream);
    else if (zpk == 1)
        launch_tiny_cfg<NWV, SC, true, 1, MODE>(p, stream);
    else
        launch_tiny_cfg<NWV, SC, true, 2, MODE>(p, stream);
}

// ---- 5 .. 64 rows of one matrix: one launch, no partial results ----
// The batched decode step (a few tens of tokens): still one read of the weights,
// so the single-token kernel's shape with whole 32-row MFMA blocks. A workgroup
// owns 32 columns; its NWV waves cut K between them in whole groups, and a wave
// walks its range in chunks of MD_CH(RB) tiles: per chunk it requests the
// weights tiles (straight into registers: the packed layout is the operand
// order), its source rows as whole row pieces (16 lanes a row) and the chunk's
// scales / zero points, one chunk ahead of the arithmetic; rows and tables wait
// in a wave-private piece of LDS (no barrier before the end) and come back in
// operand order. Group ends as in the kernels above. The waves' f32 results are
// added through LDS in wave order (= K order) and every thread runs the
// epilogue of a few elements. RB: blocks of 32 rows (1 or 2).
// MODE as above: 1 groups of 32 k, 2 source zero points / u8 source.
constexpr int md_ch(int rb) { return 4 / rb; } // 64-k tiles per chunk
constexpr int md_gpc(int rb, int mode) { // most groups a chunk can hold
    return (mode == 1 ? 2 : 1) * md_ch(rb);
}
constexpr int md_apitch(int rb) { return md_ch(rb) * BK + 16; } // staged row, bytes
constexpr int md_wave_bytes(int rb, int mode, int gpc) {
    // rows; source scales [, source zero points]; weights scales, zero points
    // of the gpc groups a chunk holds; row sums
    return rb * 32 * md_apitch(rb)
            + gpc * (rb * 32 * 4 * (mode == 2 ? 2 : 1) + 32 * 4 * 2) + rb * 32 * 4;
}
static_assert(32 * md_apitch(1) >= 32 * 32 * 4 && 64 * md_apitch(2) >= 64 * 32 * 4,
        "a wave's results fit where its rows were staged");

template <int NWV, int RB, int SC, bool HAS_ZP, int ZPK, int MODE = 0>
__global__ void __launch_bounds__(NWV * 64)
w4a8_mid_kernel(const w4a8_small_t p) {
    constexpr bool HALF = MODE == 1, SZP = MODE == 2;
    static_assert(!SZP || HAS_ZP, "");
    constexpr int R = RB * 32, CH = md_ch(RB), GPC = md_gpc(RB, MODE);
    constexpr int APITCH = md_apitch(RB);
    // p.splits: groups per full chunk (CH / p.tpg, or 2 CH of 32 k): the size of
    // the wave's tables
    const int gpc = p.splits;
    const int WAVE_BYTES = md_wave_bytes(RB, MODE, gpc);
    constexpr int PPR = CH * 4; // 16-byte pieces of a staged row
    constexpr int A_PER = R * PPR / 64; // row pieces per lane and chunk
    constexpr int SS_PER = GPC * R / 64, SW_PER = GPC * 32 / 64;
    static_assert(A_PER == 8 && SS_PER >= 1 && SW_PER >= 1, "");
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const w4a8_prep_t &q = p.q;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n0 = blockIdx.x * 32;
    const int g_begin = wave * p.gps; // p.gps: groups per wave, whole chunks' worth of tiles
    const int g_cnt = max(0, min(p.gps, q.ng - g_begin));
    const int T0 = HALF ? g_begin / 2 : g_begin * p.tpg; // first tile of the wave
    const int KT = HALF ? g_cnt / 2 : g_cnt * p.tpg; // tiles of this wave
    uint8_t *wA = lds + wave * WAVE_BYTES;
    float *wss = (float *)(wA + R * APITCH); // [gpc][R]
    int32_t *wzs = (int32_t *)(wss + gpc * R); // SZP only
    float *wsw = wss + gpc * R * (SZP ? 2 : 1); // [gpc][32]
    int32_t *wzw = (int32_t *)(wsw + gpc * 32);
    int32_t *rsw = wzw + gpc * 32; // [R]
    const int mrows = min(R, q.M);

    v16f res[RB];
#pragma unroll
    for (int i = 0; i < RB; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) res[i][r] = 0.f;

    if (KT > 0) {
        const bool has_ss = q.ss != nullptr, has_sw = q.sw != nullptr;
        const int nb = min(n0 / 32, p.nb32 - 1);
        const v4u *bsrc = (const v4u *)(p.B + (int64_t)nb * p.kt64 * 1024) + lane;
        // what a chunk asks for, one chunk ahead of its use
        uint4 av[A_PER];
        v4u bn[CH];
        uint32_t rs_[SS_PER], rzs_[SS_PER], rw_[SW_PER], rz_[SW_PER];
        int64_t iz_[SW_PER];
#pragma unroll
        for (int j = 0; j < SS_PER; j++) rs_[j] = rzs_[j] = 0;
#pragma unroll
        for (int j = 0; j < SW_PER; j++) {
            rw_[j] = rz_[j] = 0;
            iz_[j] = 0;
        }
        // groups of the chunk that starts at tile t0 of the wave
        auto first_group = [&](int t0) { return HALF ? 2 * t0 : t0 / p.tpg; };
        auto request = [&](int t0, int cnt) {
            // source rows: piece l % PPR of rows l / PPR + (64 / PPR) i
#pragma unroll
            for (int i = 0; i < A_PER; i++) {
                const int row = min(lane / PPR + (64 / PPR) * i, q.M - 1);
                const int pc = lane % PPR;
                av[i] = make_uint4(0, 0, 0, 0);
                if ((pc >> 2) < cnt)
                    av[i] = *(const uint4 *)(q.A + (int64_t)row * q.lda
                            + (int64_t)(T0 + t0) * BK + pc * 16);
            }
            const int gl0 = first_group(t0);
#pragma unroll
            for (int j = 0; j < SS_PER; j++) {
                const int i = lane + j * 64;
                const int gl = min(gl0 + i / R, g_cnt - 1), r = min(i % R, q.M - 1);
                const int k0 = (g_begin + gl) * q.gk;
                if (has_ss)
                    rs_[j] = scale_raw<SC>(q.ss, r * q.ss_sm + (k0 / q.ss_g) * q.ss_sk);
                if constexpr (SZP) {
                    if (q.zs) // one byte: s8 or u8 (host-checked)
                        rzs_[j] = ((const uint8_t *)q.zs)[r * q.zs_sm
                                + (k0 / q.zs_g) * q.zs_sk];
                }
            }
#pragma unroll
            for (int j = 0; j < SW_PER; j++) {
                const int i = lane + j * 64;
                const int gl = min(gl0 + (i >> 5), g_cnt - 1), c = i & 31;
                const int k0 = (g_begin + gl) * q.gk;
                const int n = min(n0 + c, q.N - 1);
                if (has_sw)
                    rw_[j] = scale_raw<SC>(q.sw, (k0 / q.sw_g) * q.sw_sk + n * q.sw_sn);
                if constexpr (ZPK != 0) {
                    iz_[j] = (k0 / q.zw_g) * q.zw_sk + n * q.zw_sn;
                    rz_[j] = zp_raw<ZPK>(q.zw, iz_[j]);
                }
            }
#pragma unroll
            for (int j = 0; j < CH; j++)
                bn[j] = __builtin_nontemporal_load(
                        bsrc + (int64_t)(T0 + t0 + min(j, cnt - 1)) * 64);
        };
        auto stage = [&]() {
#pragma unroll
            for (int i = 0; i < A_PER; i++)
                *(uint4 *)(wA + (lane / PPR + (64 / PPR) * i) * APITCH + (lane % PPR) * 16)
                        = av[i];
#pragma unroll
            for (int j = 0; j < SS_PER; j++) {
                const float v = scale_value<SC>(q.ss_dt, rs_[j]);
                if (lane + j * 64 < gpc * R) {
                    wss[lane + j * 64] = has_ss ? v : 1.f;
                    if constexpr (SZP) {
                        const int z = !q.zs ? 0
                                : q.zs_dt == dt_s8 ? (int)(int8_t)rzs_[j]
                                                   : (int)rzs_[j];
                        wzs[lane + j * 64] = z - (q.a_flip ? 128 : 0);
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < SW_PER; j++) {
                const int i = lane + j * 64;
                const float v = scale_value<SC>(q.sw_dt, rw_[j]);
                if (i < gpc * 32) {
                    wsw[i] = (has_sw ? v : 1.f) * 0.0625f;
                    if constexpr (HAS_ZP) {
                        int z = 0;
                        if constexpr (ZPK != 0) z = zp_value<ZPK>(q.zw_dt, rz_[j], iz_[j]);
                        wzw[i] = -16 * (z - q.w_off);
                    }
                }
            }
        };

        v16i acc[RB];
        int rsum[RB], csum = 0;
#pragma unroll
        for (int i = 0; i < RB; i++) {
            rsum[i] = 0;
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][r] = 0;
        }
        int t_in_g = 0, gl = 0; // position in the group; group of the chunk
        // group end: res += (float)(acc [+ zw * rowsum [+ zs * c2]]) * ss * sw
        auto group_end = [&]() {
            const float sw = wsw[gl * 32 + (lane & 31)];
            int zw = 0, c2 = 0;
            if constexpr (HAS_ZP) {
                zw = wzw[gl * 32 + (lane & 31)];
#pragma unroll
                for (int i = 0; i < RB; i++) {
                    // both k halves of a row: lanes l and l ^ 32
                    const int tot = rsum[i] + __shfl_xor(rsum[i], 32);
                    rsw[i * 32 + (lane & 31)] = tot;
                    rsum[i] = 0;
                }
            }
            if constexpr (SZP) {
                // the column's 16 * sum w' of the group, both k halves
                const int ctot = csum + __shfl_xor(csum, 32);
                csum = 0;
                c2 = -ctot - q.gk * zw;
            }
#pragma unroll
            for (int i = 0; i < RB; i++) {
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    // registers 4c .. 4c+3 are rows 8c + 4 (l / 32) .. + 3 of the block
                    if (i * 32 + 8 * c >= mrows) continue;
                    const int row = i * 32 + 8 * c + 4 * (lane >> 5);
                    const float4 s4 = *(const float4 *)&wss[gl * R + row];
                    const float ss[4] = {s4.x, s4.y, s4.z, s4.w};
                    int rs[4] = {0, 0, 0, 0}, zs[4] = {0, 0, 0, 0};
                    if constexpr (HAS_ZP) {
                        const int4 r4 = *(const int4 *)&rsw[row];
                        rs[0] = r4.x, rs[1] = r4.y, rs[2] = r4.z, rs[3] = r4.w;
                    }
                    if constexpr (SZP) {
                        const int4 z4 = *(const int4 *)&wzs[gl * R + row];
                        zs[0] = z4.x, zs[1] = z4.y, zs[2] = z4.z, zs[3] = z4.w;
                    }
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        int t = acc[i][4 * c + e];
                        if constexpr (HAS_ZP) t += __mul24(zw, rs[e]);
                        if constexpr (SZP) t += __mul24(zs[e], c2);
                        res[i][4 * c + e] = __builtin_fmaf(
                                (float)t * ss[e], sw, res[i][4 * c + e]);
                    }
                }
            }
            gl++;
        };

        request(0, min(CH, KT));
        for (int t0 = 0; t0 < KT; t0 += CH) {
            const int cnt = min(CH, KT - t0);
            stage();
            v4u bq[CH];
#pragma unroll
            for (int j = 0; j < CH; j++) bq[j] = bn[j];
            if (t0 + CH < KT) request(t0 + CH, min(CH, KT - t0 - CH));
            gl = 0;
#pragma unroll
            for (int j = 0; j < CH; j++) {
                if (j < cnt) {
                    const bool first = t_in_g == 0; // the group's accumulators start at 0
#pragma unroll
                    for (int ki = 0; ki < 2; ki++) {
                        const uint32_t w0 = ki ? bq[j].z : bq[j].x;
                        const uint32_t w1 = ki ? bq[j].w : bq[j].y;
                        const v4i b = {(int)((w0 << 4) & 0xF0F0F0F0u),
                                (int)(w0 & 0xF0F0F0F0u),
                                (int)((w1 << 4) & 0xF0F0F0F0u),
                                (int)(w1 & 0xF0F0F0F0u)};
                        if constexpr (SZP) {
                            int t = csum;
                            t = __builtin_amdgcn_sdot4(b[0], 0x01010101, t, false);
                            t = __builtin_amdgcn_sdot4(b[1], 0x01010101, t, false);
                            t = __builtin_amdgcn_sdot4(b[2], 0x01010101, t, false);
                            t = __builtin_amdgcn_sdot4(b[3], 0x01010101, t, false);
                            csum = t;
                        }
#pragma unroll
                        for (int i = 0; i < RB; i++) {
                            const uint4 v = *(const uint4 *)(wA
                                    + (i * 32 + (lane & 31)) * APITCH
                                    + (j * 4 + ki * 2 + (lane >> 5)) * 16);
                            v4i a = {(int)v.x, (int)v.y, (int)v.z, (int)v.w};
                            if constexpr (SZP) // u8 source: s - 128 as s8
                                a = v4i {(int)(v.x ^ q.a_flip), (int)(v.y ^ q.a_flip),
                                        (int)(v.z ^ q.a_flip), (int)(v.w ^ q.a_flip)};
                            if constexpr (HAS_ZP) {
                                int t = rsum[i];
                                t = __builtin_amdgcn_sdot4(a[0], 0x01010101, t, false);
                                t = __builtin_amdgcn_sdot4(a[1], 0x01010101, t, false);
                                t = __builtin_amdgcn_sdot4(a[2], 0x01010101, t, false);
                                t = __builtin_amdgcn_sdot4(a[3], 0x01010101, t, false);
                                rsum[i] = t;
                            }
                            if (HALF || (ki == 0 && first)) {
                                const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0,
                                        0, 0, 0, 0};
                                acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
                                        a, b, zero, 0, 0, 0);
                            } else {
                                acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
                                        a, b, acc[i], 0, 0, 0);
                            }
                        }
                        if constexpr (HALF) group_end();
                    }
                    if constexpr (!HALF) {
                        if (++t_in_g == p.tpg) {
                            t_in_g = 0;
                            group_end();
                        }
                    }
                }
            }
        }
    }

    // register r of lane l is row 8 (r / 4) + 4 (l / 32) + r % 4 of its block,
    // column l % 32; a wave's results go where its rows were staged
    float *red = (float *)wA; // [R][32]
#pragma unroll
    for (int i = 0; i < RB; i++)
#pragma unroll
        for (int r = 0; r < 16; r++)
            red[(i * 32 + 8 * (r / 4) + 4 * (lane >> 5) + r % 4) * 32 + (lane & 31)]
                    = res[i][r];
    __syncthreads();
    const int n = n0 + (threadIdx.x & 31);
    if (n >= q.N) return;
#pragma unroll 1
    for (int row = threadIdx.x >> 5; row < mrows; row += NWV * 2) {
        float v = ((const float *)lds)[row * 32 + (threadIdx.x & 31)];
        for (int w = 1; w < NWV; w++)
            v += ((const float *)(lds + w * WAVE_BYTES))[row * 32 + (threadIdx.x & 31)];
        epilogue_apply_store(p.ep, v, 0, row, n);
    }
}

template <int NWV, int RB, int SC, bool HAS_ZP, int ZPK, int MODE>
static void launch_mid_cfg(const w4a8_small_t &p, hipStream_t stream) {
    const size_t lds = (size_t)NWV * md_wave_bytes(RB, MODE, p.splits);
    auto kern = w4a8_mid_kernel<NWV, RB, SC, HAS_ZP, ZPK, MODE>;
    ensure_dynamic_lds((const void *)kern, (int)lds);
    hipLaunchKernelGGL(kern, dim3((p.q.N + 31) / 32), dim3(NWV * 64), lds, stream, p);
}

template <int NWV, int RB, int SC, int MODE>
static void launch_mid_zp(const w4a8_small_t &p, bool has_zp, int zpk,
        hipStream_t stream) {
    if constexpr (MODE != 2) {
        if (!has_zp) {
            launch_mid_cfg<NWV, RB, SC, false, 0, MODE>(p, stream);
            return;
        }
    }
    if (zpk == 0)
        launch_mid_cfg<NWV, RB, SC, true, 0, MODE>(p, stream);
    else if (zpk == 1)
        launch_mid_cfg<NWV, RB, SC, true, 1, MODE>(p, stream);
    else
        launch_mid_cfg<NWV, RB, SC, true, 2, MODE>(p, stream);
}

// by waves per workgroup, rows (one or two blocks of 32) and scale size
template <int MODE>
static void launch_mid_mode(const w4a8_small_t &p, bool has_zp, int zpk, bool sc4,
        int nwv, hipStream_t stream) {
    auto by_sc = [&](auto W, auto B) {
        constexpr int NWV = decltype(W)::value, RB = decltype(B)::value;
        if (sc4)
            launch_mid_zp<NWV, RB, 4, MODE>(p, has_zp, zpk, stream);
        else
            launch_mid_zp<NWV, RB, 2, MODE>(p, has_zp, zpk, stream);
    };
    auto by_rows = [&](auto W) {
        if (p.q.M > 32) by_sc(W, std::integral_constant<int, 2> {});
        else by_sc(W, std::integral_constant<int, 1> {});
    };
    if (nwv == 8) by_rows(std::integral_constant<int, 8> {});
    else by_rows(std::integral_constant<int, 4> {});
}

#if defined(QMM_W4A8_PART) && QMM_W4A8_PART == 3
// sum of the slices in slice order, then bias / post-ops / dst conversion:
// one thread per four neighbouring columns of a row
__global__ void __launch_bounds__(256)
w4a8_reduce_kernel(const float *part, int splits, int M, int N, int ldp,
        const epilogue_t ep) {
    const int n4 = (N + 3) / 4;
    const int64_t total = (int64_t)M * n4;
    const float one4[4] = {1.f, 1.f, 1.f, 1.f};
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
            i += (int64_t)gridDim.x * blockDim.x) {
        const int m = (int)(i / n4), n = (int)(i % n4) * 4;
        float v[4] = {0.f, 0.f, 0.f, 0.f};
        for (int s = 0; s < splits; s++) {
            const float4 t
                    = *(const float4 *)&part[((int64_t)s * M + m) * ldp + n];
            if (s == 0) {
                v[0] = t.x;
                v[1] = t.y;
                v[2] = t.z;
                v[3] = t.w;
            } else {
                v[0] += t.x;
                v[1] += t.y;
                v[2] += t.z;
                v[3] += t.w;
            }
        }
        const int nvalid = min(4, N - n);
        if (ep.fast != EP_FAST_NONE && !ep.fast_ext)
            epilogue_fast4(ep, v, false, 1.f, false, one4, 0, m, n, nvalid);
        else
            epilogue_apply_store4(ep, v, 0, m, n, nvalid);
    }
}

#endif // reduction

template <int FM, int SC, bool HAS_ZP, int ZPK, int MODE>
static void launch_small_cfg(const w4a8_small_t &p, hipStream_t stream) {
    constexpr int BM = FM * 32;
    constexpr size_t lds = sm_lds_bytes(FM, MODE);
    auto kern = w4a8_small_kernel<FM, SC, HAS_ZP, ZPK, MODE>;
    ensure_dynamic_lds((const void *)kern, (int)lds);
    hipLaunchKernelGGL(kern,
            dim3((p.q.N + 127) / 128, p.splits, (p.q.M + BM - 1) / BM),
            dim3(256), lds, stream, p);
}

template <int FM, int SC, int MODE>
static void launch_small_zp(const w4a8_small_t &p, bool has_zp, int zpk,
        hipStream_t stream) {
    if constexpr (MODE != 2) {
        if (!has_zp) {
            launch_small_cfg<FM, SC, false, 0, MODE>(p, stream);
            return;
        }
    }
    if (zpk == 0)
        launch_small_cfg<FM, SC, true, 0, MODE>(p, stream);
    else if (zpk == 1)
        launch_small_cfg<FM, SC, true, 1, MODE>(p, stream);
    else
        launch_small_cfg<FM, SC, true, 2, MODE>(p, stream);
}

// by rows (one or two 32-row fragments) and scale size
template <int MODE>
static void launch_small_mode(const w4a8_small_t &p, bool has_zp, int zpk,
        bool sc4, hipStream_t stream) {
    if (p.q.M > 32) {
        if (sc4)
            launch_small_zp<2, 4, MODE>(p, has_zp, zpk, stream);
        else
            launch_small_zp<2, 2, MODE>(p, has_zp, zpk, stream);
    } else {
        if (sc4)
            launch_small_zp<1, 4, MODE>(p, has_zp, zpk, stream);
        else
            launch_small_zp<1, 2, MODE>(p, has_zp, zpk, stream);
    }
}

template <int BM, int BN, int WGM, int WGN, int ZPM, bool HALF = false>
static void launch_cfg(const w4a8_params_t &p, hipStream_t stream) {
    // a tile is only 8 MFMAs per wave: five stages (four tiles in flight) are
    // what it takes to cover the L2 / HBM latency; two workgroups still fit
    // (four stages with the six per-group arrays of ZPM = 2, three where every
    // tile carries two slices of each array)
    constexpr int STAGES = HALF ? 3 : ZPM == 2 ? 4 : 5;
    w4a8_params_t q = p;
    q.tiles_m = (p.M + BM - 1) / BM;
    q.tiles_n = (p.N + BN - 1) / BN;
    const int ntiles = q.tiles_m * q.tiles_n;
    const int grid_x = ntiles >= 64 ? ((ntiles + 7) / 8) * 8 : ntiles;
    constexpr size_t lds_main = (size_t)STAGES
            * (BM * BK + BN * BK / 2
                    + (HALF ? 2 : 1) * (ZPM == 2 ? 6 : ZPM == 1 ? 4 : 2) * X_BYTES);
    constexpr size_t lds_ep
            = (size_t)WGM * WGN * 32 * (BN / WGN) * sizeof(float);
    constexpr size_t lds = lds_main > lds_ep ? lds_main : lds_ep;
    auto kern = gemm_w4a8_kernel<BM, BN, WGM, WGN, STAGES, ZPM, HALF>;
    ensure_dynamic_lds((const void *)kern, (int)lds);
    hipLaunchKernelGGL(kern, dim3(grid_x), dim3(WGM * WGN * 64), lds, stream, q);
}

template <int ZPM, bool HALF = false>
static void launch_zp(const w4a8_params_t &p, int variant, hipStream_t stream) {
    switch (variant) {
        case 1: launch_cfg<128, 128, 2, 2, ZPM, HALF>(p, stream); break;
        case 2: launch_cfg<64, 128, 2, 2, ZPM, HALF>(p, stream); break;
        default: launch_cfg<32, 64, 1, 2, ZPM, HALF>(p, stream); break;
    }
}

} // namespace w4a8

// The kernel families build in translation units of their own (QMM_W4A8_PART:
// 1, 2 the tiled GEMM without / with zero points, 3 the split-K kernel and its
// reduction, 4 the single-token kernel, 5 the tiled GEMM with source zero
// points, 6 and 7 the tiled GEMM with groups of 32 k without / with zero
// points, 8 and 9 the single-token kernel and 10 and 11 the split-K kernel with
// groups of 32 k / source zero points, 12 to 14 the one-launch kernel for 5 to 64
// rows in its three modes); the unit without the macro holds the pre-pass and
// the dispatch.
#if defined(QMM_W4A8_PART)
#if QMM_W4A8_PART == 1
void launch_gemm_w4a8_nozp(const w4a8_params_t &p, int variant,
        hipStream_t stream) {
    w4a8::launch_zp<0>(p, variant, stream);
}
#elif QMM_W4A8_PART == 2
void launch_gemm_w4a8_zp(const w4a8_params_t &p, int variant,
        hipStream_t stream) {
    w4a8::launch_zp<1>(p, variant, stream);
}
#elif QMM_W4A8_PART == 5
void launch_gemm_w4a8_szp(const w4a8_params_t &p, int variant,
        hipStream_t stream) {
    w4a8::launch_zp<2>(p, variant, stream);
}
#elif QMM_W4A8_PART == 6
void launch_gemm_w4a8_half_nozp(const w4a8_params_t &p, int variant,
        hipStream_t stream) {
    w4a8::launch_zp<0, true>(p, variant, stream);
}
#elif QMM_W4A8_PART == 7
void launch_gemm_w4a8_half_zp(const w4a8_params_t &p, int variant,
        hipStream_t stream) {
    w4a8::launch_zp<1, true>(p, variant, stream);
}
#elif QMM_W4A8_PART == 10
void launch_gemm_w4a8_small_half_part(const w4a8_small_t &p, bool has_zp,
        int zpk, bool sc4, hipStream_t stream) {
    w4a8::launch_small_mode<1>(p, has_zp, zpk, sc4, stream);
}
#elif QMM_W4A8_PART == 11
void launch_gemm_w4a8_small_szp_part(const w4a8_small_t &p, bool has_zp,
        int zpk, bool sc4, hipStream_t stream) {
    w4a8::launch_small_mode<2>(p, has_zp, zpk, sc4, stream);
}
#elif QMM_W4A8_PART == 3
void launch_gemm_w4a8_small_part(const w4a8_small_t &p, bool has_zp, int zpk,
        bool sc4, hipStream_t stream) {
    w4a8::launch_small_mode<0>(p, has_zp, zpk, sc4, stream);
}
// the slices' partial results -> dst
void launch_gemm_w4a8_reduce(const w4a8_small_t &p, hipStream_t stream) {
    const int64_t total = (int64_t)p.q.M * ((p.q.N + 3) / 4);
    int64_t blocks = (total + 255) / 256;
    if (blocks > 65535) blocks = 65535;
    hipLaunchKernelGGL(w4a8::w4a8_reduce_kernel, dim3((unsigned)blocks),
            dim3(256), 0, stream, (const float *)p.part, p.splits, p.q.M, p.q.N,
            p.ldp, p.ep);
}
#elif QMM_W4A8_PART == 12
void launch_gemm_w4a8_mid_part(const w4a8_small_t &p, bool has_zp, int zpk,
        bool sc4, int nwv, hipStream_t stream) {
    w4a8::launch_mid_mode<0>(p, has_zp, zpk, sc4, nwv, stream);
}
#elif QMM_W4A8_PART == 13
void launch_gemm_w4a8_mid_half_part(const w4a8_small_t &p, bool has_zp, int zpk,
        bool sc4, int nwv, hipStream_t stream) {
    w4a8::launch_mid_mode<1>(p, has_zp, zpk, sc4, nwv, stream);
}
#elif QMM_W4A8_PART == 14
void launch_gemm_w4a8_mid_szp_part(const w4a8_small_t &p, bool has_zp, int zpk,
        bool sc4, int nwv, hipStream_t stream) {
    w4a8::launch_mid_mode<2>(p, true, zpk, sc4, nwv, stream);
}
#elif QMM_W4A8_PART == 4 || QMM_W4A8_PART == 8 || QMM_W4A8_PART == 9
// the single-token kernel: whole tiles per group (4), groups of 32 k (8),
// source zero points / u8 source (9)
#if QMM_W4A8_PART == 4
#define QMM_TINY_NAME launch_gemm_w4a8_tiny_part
#define QMM_TINY_MODE 0
#elif QMM_W4A8_PART == 8
#define QMM_TINY_NAME launch_gemm_w4a8_tiny_half_part
#define QMM_TINY_MODE 1
#else
#define QMM_TINY_NAME launch_gemm_w4a8_tiny_szp_part
#define QMM_TINY_MODE 2
#endif
void QMM_TINY_NAME(const w4a8_small_t &p, bool has_zp, int zpk, bool sc4,
        int nwv, hipStream_t stream) {
    if (nwv == 8) {
        if (sc4)
            w4a8::launch_tiny_zp<8, 4, QMM_TINY_MODE>(p, has_zp, zpk, stream);
        else
            w4a8::launch_tiny_zp<8, 2, QMM_TINY_MODE>(p, has_zp, zpk, stream);
    } else {
        if (sc4)
            w4a8::launch_tiny_zp<4, 4, QMM_TINY_MODE>(p, has_zp, zpk, stream);
        else
            w4a8::launch_tiny_zp<4, 2, QMM_TINY_MODE>(p, has_zp, zpk, stream);
    }
}
#endif
#else
void launch_gemm_w4a8_nozp(const w4a8_params_t &p, int variant,
        hipStream_t stream);
void launch_gemm_w4a8_zp(const w4a8_params_t &p, int variant,
        hipStream_t stream);
void launch_gemm_w4a8_szp(const w4a8_params_t &p, int variant,
        hipStream_t stream);
void launch_gemm_w4a8_half_nozp(const w4a8_params_t &p, int variant,
        hipStream_t stream);
void launch_gemm_w4a8_half_zp(const w4a8_params_t &p, int variant,
        hipStream_t stream);
void launch_gemm_w4a8_small_part(const w4a8_small_t &p, bool has_zp, int zpk,
        bool sc4, hipStream_t stream);
void launch_gemm_w4a8_small_half_part(const w4a8_small_t &p, bool has_zp,
        int zpk, bool sc4, hipStream_t stream);
void launch_gemm_w4a8_small_szp_part(const w4a8_small_t &p, bool has_zp,
        int zpk, bool sc4, hipStream_t stream);
void launch_gemm_w4a8_reduce(const w4a8_small_t &p, hipStream_t stream);
void launch_gemm_w4a8_tiny_part(const w4a8_small_t &p, bool has_zp, int zpk,
        bool sc4, int nwv, hipStream_t stream);
void launch_gemm_w4a8_tiny_half_part(const w4a8_small_t &p, bool has_zp,
        int zpk, bool sc4, int nwv, hipStream_t stream);
void launch_gemm_w4a8_tiny_szp_part(const w4a8_small_t &p, bool has_zp,
        int zpk, bool sc4, int nwv, hipStream_t stream);
void launch_gemm_w4a8_mid_part(const w4a8_small_t &p, bool has_zp, int zpk,
        bool sc4, int nwv, hipStream_t stream);
void launch_gemm_w4a8_mid_half_part(const w4a8_small_t &p, bool has_zp, int zpk,
        bool sc4, int nwv, hipStream_t stream);
void launch_gemm_w4a8_mid_szp_part(const w4a8_small_t &p, bool has_zp, int zpk,
        bool sc4, int nwv, hipStream_t stream);

void launch_w4a8_prep(const w4a8_prep_t &p, hipStream_t stream) {
    const int64_t total = (int64_t)p.ng * ((int64_t)p.M + p.N);
    int64_t blocks = (total + 255) / 256;
    if (blocks > 65535) blocks = 65535;
    hipLaunchKernelGGL(w4a8::w4a8_prep_kernel, dim3((unsigned)blocks), dim3(256),
            0, stream, p);
}

// Data types the small-row kernels read directly: both scales of one size
// (f16 / bf16, or f32) and zero points of one byte or less.
bool gemm_w4a8_small_takes(const w4a8_prep_t &q) {
    auto two = [](int dt) { return dt == dt_f16 || dt == dt_bf16; };
    const int sdt = q.ss ? q.ss_dt : q.sw_dt, wdt = q.sw ? q.sw_dt : q.ss_dt;
    if ((q.ss || q.sw)
            && !((two(sdt) && two(wdt)) || (sdt == dt_f32 && wdt == dt_f32)))
        return false;
    if (q.zw && q.zw_dt == dt_s32) return false;
    return true;
}

static bool scales_are_f32(const w4a8_prep_t &q) {
    const int sdt = q.ss ? q.ss_dt : q.sw_dt;
    return (q.ss || q.sw) && sdt == dt_f32;
}
static int zp_storage(const w4a8_prep_t &q) {
    return !q.zw ? 0 : ((q.zw_dt == dt_s4 || q.zw_dt == dt_u4) ? 2 : 1);
}

// Single-token decode kernel: nwv waves per workgroup (4 or 8), p.gps groups
// per wave; p.part / p.splits are unused. p.tpg == 0: groups of 32 k;
// p.q.zsT != nullptr stands for "source zero points / u8 source" (the pointer
// itself is not used by this kernel).
void launch_gemm_w4a8_tiny(const w4a8_small_t &p, bool has_zp, int nwv,
        hipStream_t stream) {
    if (p.q.M <= 0 || p.q.N <= 0) return;
    if (p.tpg == 0)
        launch_gemm_w4a8_tiny_half_part(
                p, has_zp, zp_storage(p.q), scales_are_f32(p.q), nwv, stream);
    else if (p.q.zsT)
        launch_gemm_w4a8_tiny_szp_part(
                p, true, zp_storage(p.q), scales_are_f32(p.q), nwv, stream);
    else
        launch_gemm_w4a8_tiny_part(
                p, has_zp, zp_storage(p.q), scales_are_f32(p.q), nwv, stream);
}

// 5 .. 64 rows in one launch: nwv waves per workgroup (4 or 8), p.gps groups per
// wave. The kernel's chunks hold whole groups: groups of 32 k, or of 1, 2 or 4
// tiles with at most 32 rows (1 or 2 tiles with more).
bool gemm_w4a8_mid_takes(int M, int group_k) {
    if (M <= 4 || M > 64) return false;
    if (group_k == 32) return true;
    if (group_k % 64 != 0) return false;
    const int tpg = group_k / 64, ch = w4a8::md_ch(M > 32 ? 2 : 1);
    return tpg <= ch && ch % tpg == 0;
}
// groups per chunk (the kernel's p.splits) and the LDS a wave needs
int gemm_w4a8_mid_gpc(int M, int group_k) {
    const int ch = w4a8::md_ch(M > 32 ? 2 : 1);
    return group_k == 32 ? 2 * ch : ch / (group_k / 64);
}
int gemm_w4a8_mid_wave_bytes(int M, int group_k, bool src_zp) {
    return w4a8::md_wave_bytes(M > 32 ? 2 : 1, group_k == 32 ? 1 : (src_zp ? 2 : 0),
            gemm_w4a8_mid_gpc(M, group_k));
}
void launch_gemm_w4a8_mid(const w4a8_small_t &p, bool has_zp, int nwv,
        hipStream_t stream) {
    if (p.q.M <= 0 || p.q.N <= 0) return;
    if (p.tpg == 0)
        launch_gemm_w4a8_mid_half_part(
                p, has_zp, zp_storage(p.q), scales_are_f32(p.q), nwv, stream);
    else if (p.q.zsT)
        launch_gemm_w4a8_mid_szp_part(
                p, true, zp_storage(p.q), scales_are_f32(p.q), nwv, stream);
    else
        launch_gemm_w4a8_mid_part(
                p, has_zp, zp_storage(p.q), scales_are_f32(p.q), nwv, stream);
}

// groups one wave of the single-token kernel can hold (its LDS tables)
int gemm_w4a8_tiny_max_groups(bool half) {
    return w4a8::tn_maxg(half ? 1 : 0);
}

void launch_gemm_w4a8_small(const w4a8_small_t &p, bool has_zp,
        hipStream_t stream) {
    if (p.q.M <= 0 || p.q.N <= 0) return;
    // p.tpg == 0: groups of 32 k; p.q.zsT != nullptr: source zero points / u8
    // source (as for the single-token kernel)
    if (p.tpg == 0)
        launch_gemm_w4a8_small_half_part(
                p, has_zp, zp_storage(p.q), scales_are_f32(p.q), stream);
    else if (p.q.zsT)
        launch_gemm_w4a8_small_szp_part(
                p, true, zp_storage(p.q), scales_are_f32(p.q), stream);
    else
        launch_gemm_w4a8_small_part(
                p, has_zp, zp_storage(p.q), scales_are_f32(p.q), stream);
    launch_gemm_w4a8_reduce(p, stream);
}

// variant: 0 = by problem size; 1: 128 x 128, 2: 64 x 128, 3: 32 x 64 tiles
void launch_gemm_w4a8(const w4a8_params_t &p, int variant, hipStream_t stream) {
    if (p.M <= 0 || p.N <= 0) return;
    if (variant < 1 || variant > 3) {
        const int64_t big = (int64_t)((p.M + 127) / 128) * ((p.N + 127) / 128);
        const int64_t mid = (int64_t)((p.M + 63) / 64) * ((p.N + 127) / 128);
        variant = big >= 256 ? 1 : ((mid >= 128 && p.M > 32) ? 2 : 3);
        if (variant == 3 && p.M > 64) variant = 2;
    }
    if (p.tpg == 0) { // groups of 32 k
        if (p.zwT)
            launch_gemm_w4a8_half_zp(p, variant, stream);
        else
            launch_gemm_w4a8_half_nozp(p, variant, stream);
    } else if (p.zsT)
        launch_gemm_w4a8_szp(p, variant, stream);
    else if (p.zwT)
        launch_gemm_w4a8_zp(p, variant, stream);
    else
        launch_gemm_w4a8_nozp(p, variant, stream);
}
#endif

} // namespace qmm
