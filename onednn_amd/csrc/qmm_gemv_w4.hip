// hip:gfx950:decode_w4 -- weights-decompression matmul for small M (the decode
// step of an LLM linear layer): 16-bit activations [M,K] x 4-bit weights [K,N]
// with K-grouped scales and zero points, f32 accumulation
// (semantics: src/cpu/matmul/ref_matmul.cpp:140-173 with
// fpmath_mode apply_to_int).
//
// The kernel is bound by the HBM stream of the packed weights, so everything
// is arranged around one 128-bit load per lane:
//   * weights are prepacked (QMM_LAYOUT_MFMA_W4) in 1 KiB tiles of 16 columns
//     x 128 k; lane 16*c + n holds, per 32-k step s, the eight nibbles of
//     column n for k = 32*s + 8*c + 0..7, ordered so that
//     (dword >> 4i) & 0x000F000F is the pair (2i, 2i+1);
//   * a pair of nibbles becomes a pair of bf16 (or f16) values 128+w
//     (1024+w) with a single v_and_or_b32 on the exponent pattern -- no
//     integer-to-float conversions in the stream;
//   * the 16 x 16 x 32 MFMA multiplies 16 activation rows by the 16 columns of
//     the tile; a second MFMA against a vector of ones yields the row sums of
//     the activations, which remove both the magic offset and the zero point
//     when a scale group closes:
//         out += scale[g,n] * (P - (offset + zp[g,n]) * S);
//   * a block owns 16 columns and all of K; its waves take the k tiles round
//     robin and issue their loads before touching the activations, which are
//     staged once per block in LDS in MFMA operand order.
#include <type_traits>

#include "qmm_device.hpp"
#include "qmm_plan.hpp"

namespace qmm {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));

constexpr int GEMV_WAVES = 8;
constexpr int GEMV_LDS_BUDGET = 128 * 1024;

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

// lane i of every row of 16 lanes takes the value of lane i + S of that row
// (zero past the row's end)
template <int S>
QMM_D uint32_t row_shl(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(
            0, (int)v, 0x100 + S, 0xf, 0xf, true);
}

// weights are read exactly once: keep them from displacing reusable lines
QMM_D uint4 ld_stream(const uint8_t *ptr) {
    const v4u v = __builtin_nontemporal_load((const v4u *)ptr);
    return make_uint4(v.x, v.y, v.z, v.w);
}

// Cross-wave reduction of the partial sums and the epilogue, shared by the two
// kernels: every wave leaves its 4 values per lane in LDS, wave 0 adds them in
// wave order and stores. Register j of lane l is row 4 * (l / 16) + j of the
// MFMA result. ROWS = 16: every row is an activation row; ROWS = 8: the even
// rows (registers 0 and 2) are activation rows 0..7; ROWS = 4 and 1: rows 0,
// 4, 8, 12 (register 0) are activation rows 0..3. `plain` (wave-uniform): nothing follows the accumulation (no scales,
// bias, post-ops, dst scale or zero point) and dst is dense along n, so the
// value is converted and stored without the post-op interpreter; `dst` and
// `dst_sm` are then the dst pointer and row pitch, read by the caller long
// before (the parameter block is cold, its first touch costs a trip to memory).
template <int ROWS>
QMM_D void gemv_reduce_store(const gemv_params_t &p, float *red, const v4f &out,
        int wave, int lane, int m_base, int rows, int n, bool plain = false,
        void *dst = nullptr, int64_t dst_sm = 0, int dst_dt = 0) {
    constexpr int SPL = ROWS == 16 ? 1 : ROWS == 8 ? 2 : 4; // MFMA rows per activation row
    constexpr int NJ = 4 / SPL;
#pragma unroll
    for (int j = 0; j < NJ; j++)
        red[(wave * 64 + lane) * NJ + j] = out[j * SPL];
    __syncthreads();
    if (wave == 0) {
        const int c = lane >> 4;
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < GEMV_WAVES; w++)
                v += red[(w * 64 + lane) * NJ + j];
            // MFMA output: register j of lane l is row 4*(l/16)+j, column l%16
            const int row = (4 * c + j * SPL) / SPL;
            const int m = m_base + row;
            if (m < p.M && n < p.N && row < rows) {
                if (plain)
                    store_float(dst_dt, v, dst, m * dst_sm + n);
                else
                    epilogue_apply_store(p.ep, v, 0, m, n);
            }
        }
    }
}

// General kernel: any group sizes and scale / zero-point types the
// implementation accepts; activations staged in LDS, K walked in a loop.
template <bool F16>
__global__ void __launch_bounds__(GEMV_WAVES * 64)
gemv_w4_kernel(const gemv_params_t p, const int MR, const int KC) {
    constexpr int FAST = 0;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    // lds: activations [KC/8 chunks][MR rows][16 bytes]; later reused for the
    // cross-wave reduction [GEMV_WAVES][64 lanes][4 floats]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // consecutive workgroups run on the 8 XCDs in turn: give each XCD a
    // contiguous range of column blocks, so that a scale / zero-point line
    // (64 and more neighbouring columns) is fetched into one L2 only
    const int nb = (gridDim.x & 7) == 0
            ? (int)((blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3))
            : (int)blockIdx.x;
    const int m_base = p.m0 + blockIdx.y * 16;
    const int rows = min(16, p.M - m_base);
    const int c = lane >> 4; // k chunk of the lane
    const int r = lane & 15; // activation row (A operand) / column (B operand)
    const int n = nb * 16 + r;

    constexpr uint32_t MAGIC = F16 ? 0x64006400u : 0x43004300u;
    constexpr float OFFSET = F16 ? 1024.f : 128.f;
    constexpr uint32_t ONE2 = F16 ? 0x3C003C00u : 0x3F803F80u;
    const v4u ones = {ONE2, ONE2, ONE2, ONE2};
    const uint32_t sflip = p.wei_signed ? 0x88888888u : 0u;
    const float soff = p.wei_signed ? 8.f : 0.f;

    // flush granularity: the scale and zero-point groups both close there
    // (the fast variant folds once per 128-k tile and does not need it)
    int fl = p.gs;
    if (!FAST && p.gz > 0) {
        int a = p.gs, b = p.gz;
        while (b) {
            const int t = a % b;
            a = b;
            b = t;
        }
        fl = a;
    }

    v4f out = {0.f, 0.f, 0.f, 0.f};
    v4f P = {0.f, 0.f, 0.f, 0.f}, S = {0.f, 0.f, 0.f, 0.f};

    const uint8_t *__restrict__ Bt
            = p.B + ((int64_t)nb * p.kg128) * 1024 + lane * 16;
    const int Kpad = p.kg128 * 128;

    // Scale / zero point of the group that contains k (this lane's column).
    // Loading and decoding are split: the raw bits are fetched without any
    // dependent instruction, so the compiler can leave the loads in flight
    // next to the weights stream and convert when the value is needed.
    const int64_t sN = p.scale_per_n ? p.N : 0, zN = p.zp_per_n ? p.N : 0;
    const bool lane_ok = n < p.N;
    auto scale_raw = [&](int kq) -> uint32_t {
        if (!p.scales || !lane_ok) return 0u;
        const int64_t idx = (int64_t)(kq / p.gs) * (p.scale_per_n ? p.N : 1)
                + (p.scale_per_n ? n : 0);
        return p.scale_dt == dt_f32 ? ((const uint32_t *)p.scales)[idx]
                                    : (uint32_t)((const uint16_t *)p.scales)[idx];
    };
    auto scale_cvt = [&](uint32_t raw) -> float {
        if (!p.scales || !lane_ok) return 1.f;
        if (p.scale_dt == dt_f32) return u2f(raw);
        if (p.scale_dt == dt_bf16) return u2f(raw << 16);
        return f16_to_f32((uint16_t)raw);
    };
    auto zp_index = [&](int kq) -> int64_t {
        const int64_t g = p.gz > 0 ? kq / p.gz : 0;
        return g * (p.zp_per_n ? p.N : 1) + (p.zp_per_n ? n : 0);
    };
    auto zp_raw = [&](int kq) -> uint32_t {
        if (!p.zps || !lane_ok) return 0u;
        const int64_t idx = zp_index(kq);
        if (p.zp_dt == dt_s32) return ((const uint32_t *)p.zps)[idx];
        if (p.zp_dt == dt_s4 || p.zp_dt == dt_u4)
            return ((const uint8_t *)p.zps)[idx >> 1];
        return ((const uint8_t *)p.zps)[idx];
    };
    auto zp_cvt = [&](uint32_t raw, int kq) -> float {
        if (!p.zps || !lane_ok) return 0.f;
        switch (p.zp_dt) {
            case dt_s32: return (float)(int32_t)raw;
            case dt_s8: return (float)(int8_t)raw;
            case dt_u8: return (float)(uint8_t)raw;
            default: {
                const int nib = (zp_index(kq) & 1) ? (raw >> 4) & 0xf : raw & 0xf;
                return (float)(p.zp_dt == dt_s4 ? s4_value(nib) : nib);
            }
        }
    };
    // When no group closes inside a 128-k tile, a tile has one scale and one
    // zero point per column: they are fetched together with the tile so that
    // their latency overlaps the weights stream instead of following it.
    const bool per_tile = FAST || fl % 128 == 0;
    const uint16_t *const fast_sc = (const uint16_t *)p.scales;
    const uint8_t *const fast_zp = p.zps ? (const uint8_t *)p.zps : p.B;
    const bool zp4 = p.zp_dt == dt_s4 || p.zp_dt == dt_u4;

    {
        for (int kc0 = 0; kc0 < Kpad; kc0 += KC) {
            const int kc_len = min(KC, Kpad - kc0);
            const int tiles = kc_len / 128;
            const int g0 = kc0 / 128;
            constexpr int UNR = 4;
            uint4 wt[UNR];
            uint32_t scp[UNR], zpp[UNR]; // raw scale / zero-point bits per tile
            auto fetch = [&](int tb) {
#pragma unroll
                for (int u = 0; u < UNR; u++) {
                    const int t = tb + wave + u * GEMV_WAVES;
                    wt[u] = make_uint4(0, 0, 0, 0);
                    scp[u] = 0u;
                    zpp[u] = 0u;
                    if (t < tiles) {
                        wt[u] = ld_stream(Bt + (int64_t)(g0 + t) * 1024);
                        if (per_tile) {
                            const int kq = min(kc0 + (t + 1) * 128, p.K) - 1;
                            scp[u] = scale_raw(kq);
                            zpp[u] = zp_raw(kq);
                        }
                    }
                }
            };
            // Vector-memory results return in issue order, so the activation
            // chunks this thread stages are requested first and the weights right
            // behind them: waiting for the activations then leaves the weights in
            // flight. Chunk kc (8 values) of row m lands at (kc*MR + m)*16.
            if (kc0 > 0) __syncthreads(); // previous chunk fully consumed
            const int nchunks = (kc_len / 8) * MR;
            auto act_load = [&](int i) -> uint4 {
                const int kc = i / MR, m = i % MR;
                const int k = kc0 + kc * 8;
                uint4 v = make_uint4(0, 0, 0, 0);
                if (i < nchunks && m < rows && k < p.K)
                    v = *(const uint4 *)(p.A + (int64_t)(m_base + m) * p.lda + k);
                return v;
            };
            constexpr int ACT_PRE = 2;
            uint4 areg[ACT_PRE];
#pragma unroll
            for (int q = 0; q < ACT_PRE; q++)
                areg[q] = act_load(tid + q * GEMV_WAVES * 64);
            fetch(0);
#pragma unroll
            for (int q = 0; q < ACT_PRE; q++) {
                const int i = tid + q * GEMV_WAVES * 64;
                if (i < nchunks) *(uint4 *)(lds + (size_t)i * 16) = areg[q];
            }
            for (int i = tid + ACT_PRE * GEMV_WAVES * 64; i < nchunks;
                    i += GEMV_WAVES * 64)
                *(uint4 *)(lds + (size_t)i * 16) = act_load(i);
            __syncthreads();

            for (int tb = 0; tb < tiles; tb += UNR * GEMV_WAVES) {
                if (tb > 0) fetch(tb);
#pragma unroll
                for (int u = 0; u < UNR; u++) {
                    const int t = tb + wave + u * GEMV_WAVES;
                    if (t >= tiles) break;
                    const uint32_t wd[4] = {wt[u].x ^ sflip, wt[u].y ^ sflip,
                            wt[u].z ^ sflip, wt[u].w ^ sflip};
#pragma unroll
                    for (int s = 0; s < 4; s++) {
                        const uint32_t d = wd[s];
                        v4u b;
                        b.x = (d & 0x000F000Fu) | MAGIC;
                        b.y = ((d >> 4) & 0x000F000Fu) | MAGIC;
                        b.z = ((d >> 8) & 0x000F000Fu) | MAGIC;
                        b.w = ((d >> 12) & 0x000F000Fu) | MAGIC;
                        v4u a = {0u, 0u, 0u, 0u};
                        if (r < MR) {
                            const uint4 av = *(const uint4 *)(lds
                                    + ((size_t)(t * 16 + s * 4 + c) * MR + r) * 16);
                            a = v4u {av.x, av.y, av.z, av.w};
                        }
                        P = mfma16<F16>(a, b, P);
                        S = mfma16<F16>(a, ones, S);
                        const int k_end = kc0 + t * 128 + (s + 1) * 32;
                        // A wave's tiles are not adjacent in k, so the partial
                        // sums are folded at every tile end as well as where a
                        // scale / zero-point group closes inside a tile (folding
                        // early is exact in structure: both factors are constant
                        // over the folded range).
                        if (s == 3 || (!per_tile && k_end % fl == 0)) {
                            // the range just folded contains k_end - 1
                            float sc, zp;
                            if (per_tile) {
                                const int kq = min(kc0 + (t + 1) * 128, p.K) - 1;
                                sc = scale_cvt(scp[u]);
                                zp = zp_cvt(zpp[u], kq);
                            } else {
                                const int kq = min(k_end, p.K) - 1;
                                sc = scale_cvt(scale_raw(kq));
                                zp = zp_cvt(zp_raw(kq), kq);
                            }
                            const float off = OFFSET + soff + zp;
#pragma unroll
                            for (int j = 0; j < 4; j++) {
                                out[j] = __builtin_fmaf(
                                        sc, P[j] - off * S[j], out[j]);
                                P[j] = 0.f;
                                S[j] = 0.f;
                            }
                        }
                    }
                }
            }
        }

    }

    // ---- reduce the waves' partial sums and finish ----
    __syncthreads(); // the staged activations are dead
    gemv_reduce_store<16>(p, (float *)lds, out, wave, lane, m_base, rows, n);
}

// Fast kernel: one 16-bit scale and at most one byte-sized (4- or 8-bit) zero
// point per column and 128-k tile, group widths 128 << s (or all of K). Every
// load is unconditional (out-of-range tiles re-read the last valid one, an
// absent zero-point buffer is replaced by the weights pointer), so the number
// of loads in flight is known at compile time and no wait drains the whole
// queue. ROWS: 16 activation rows per workgroup (four activation loads per
// lane and tile, one per MFMA step), at most 8 with two loads, or at most 4 /
// exactly 1 with ONE load per lane and tile. With SPL = 4, 2, 1 steps per
// load, load h of lane (r, c) fetches, for activation row r / SPL, the chunk
// that MFMA step h SPL + r % SPL multiplies; in step s the operand row SPL j
// takes it from lane SPL j + s % SPL (a shift within the 16 lanes), so every
// SPL-th row of the MFMA is an activation row and the others are never stored.
//
// A launch of this kernel lives a few microseconds, and the first of them
// passes before its first load is issued. Part of that was the kernel waiting
// for its own arguments: the parameter block arrived through three dependent
// rounds of scalar loads before the first weights address existed. Everything
// the load addresses depend on is therefore passed as 14 leading scalar
// arguments, which the hardware preloads into registers while the wave is
// launched (the build enables this for this file); the rest of the parameter
// block is only needed for the epilogue and is fetched under the weights'
// latency.
//   shifts: gs_shift | gz_shift << 8 (as bytes; 0xff: one group over all of K)
//   flags_m: bit 0 scale per column, 1 zero point per column, 2 zero points
//     4-bit, 3 zero points signed, 4 scales f16 (else bf16), 5 weights signed,
//     6 zero points present, 7 plain store (see gemv_reduce_store);
//     bits 8..: M
// W8: 8-bit weights as two planes of nibbles (QMM_LAYOUT_MFMA_W8: a tile is
// its high-nibble KiB followed by its low-nibble KiB). Both planes go through
// the 4-bit arithmetic, w = 16 hi + lo, the high nibbles as 16 * (offset + hi)
// so that both planes add into one accumulator:
//     sum a * (w - z) = P - (17 * offset + 16 * [8 if signed] + z) * S,
// the sign of an s8 weight living in its high nibble.
constexpr int GEMV_UNR = 4; // tiles of a wave in flight
constexpr int GEMV_APITCH = 256 + 16; // bytes of a staged activation row of a tile
constexpr int GEMV_STAGE_BYTES = GEMV_WAVES * GEMV_UNR * 16 * GEMV_APITCH;

template <bool F16, int ROWS, bool WSIGNED, bool W8, bool STAGED = false>
__global__ void __launch_bounds__(GEMV_WAVES * 64)
gemv_w4_fast_kernel(const uint8_t *__restrict__ pB,
        const uint16_t *__restrict__ pA, const uint16_t *__restrict__ pSC,
        const uint8_t *__restrict__ pZP, const int kg128, const int N,
        const int K, const int lda, const int shifts, const int flags_m,
        const gemv_params_t p) {
    __shared__ __attribute__((aligned(16))) float red[GEMV_WAVES * 64 * 4];
    // STAGED: the activations of a wave's tiles pass through a wave-private
    // piece of LDS (see below)
    extern __shared__ __attribute__((aligned(16))) uint8_t act_lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int uw = __builtin_amdgcn_readfirstlane(tid >> 6);
    // consecutive workgroups run on the 8 XCDs in turn: give each XCD a
    // contiguous range of column blocks, so that a scale / zero-point line
    // (64 and more neighbouring columns) is fetched into one L2 only
    const int nb16 = (N + 15) >> 4;
    const int bx = blockIdx.x;
    const int nb = (nb16 & 7) == 0 ? (bx & 7) * (nb16 >> 3) + (bx >> 3) : bx;
    const int M = (uint32_t)flags_m >> 8;
    const int m_base = blockIdx.y * 16;
    const int rows = min(16, M - m_base);
    const int c = lane >> 4; // k chunk of the lane
    const int r = lane & 15; // activation row (A operand) / column (B operand)
    const int n = nb * 16 + r;
    const int gs_shift = (int8_t)(shifts & 0xff), gz_shift = (int8_t)(shifts >> 8);
    const bool scale_per_n = flags_m & 1, zp_per_n = flags_m & 2;
    const bool zp4 = flags_m & 4, zp_signed = flags_m & 8, sc_f16 = flags_m & 16;
    const bool has_zp = flags_m & 64;

    constexpr float OFFSET = F16 ? 1024.f : 128.f;
    constexpr uint32_t ONE2 = F16 ? 0x3C003C00u : 0x3F803F80u;
    const v4u ones = {ONE2, ONE2, ONE2, ONE2};
    constexpr uint32_t sflip = WSIGNED ? 0x88888888u : 0u;
    constexpr float soff = WSIGNED ? 8.f : 0.f;
    // the exponent pattern lives in a vector register and the nibble mask in a
    // scalar one: (d >> 4 i) & mask | magic is then a shift and one
    // v_and_or_b32 (an instruction takes one scalar or literal operand only)
    uint32_t MAGIC = F16 ? 0x64006400u : 0x43004300u;
    asm volatile("" : "+v"(MAGIC));
    // 8-bit weights: the high nibbles behind the exponent of 16 * offset, where
    // one unit of the last mantissa bit is 16 (f16: 0x7400 | h = 16384 + 16 h;
    // bf16: 0x4500 | h = 2048 + 16 h), so both planes add into one accumulator
    uint32_t MAGIC_HI = W8 ? (F16 ? 0x74007400u : 0x45004500u) : MAGIC;
    if constexpr (W8) asm volatile("" : "+v"(MAGIC_HI));
    uint32_t NIB = 0x000F000Fu;
    asm volatile("" : "+s"(NIB));

    v4f out = {0.f, 0.f, 0.f, 0.f};
    constexpr int NP = W8 ? 2 : 1; // planes per tile
    constexpr int TILE_BYTES = 1024 * NP;
    const uint8_t *__restrict__ Bt
            = pB + ((int64_t)nb * kg128) * TILE_BYTES + lane * 16;
    const int64_t sN = scale_per_n ? N : 0, zN = zp_per_n ? N : 0;

    // Waves are independent until the final reduction: each one fetches its
    // weight tiles, their scales / zero points AND its activation fragments
    // (lane (r, c) holds row r, k = 32 s + 8 c .. + 7 of a tile) straight into
    // registers, every load unconditional (clamped addresses), all issued
    // before the first use. No LDS staging, no barrier before the arithmetic.
    // Tile and group indices are wave uniform (scalar arithmetic, shifts
    // instead of divisions). Rows past M compute on a repeated row and are
    // never stored; only k past K has to be zeroed (the padded weights decode
    // to the magic offset, not 0).
    const int tiles = kg128;
    constexpr int SPL = ROWS == 16 ? 1 : ROWS == 8 ? 2 : 4; // steps per load
    constexpr int NA = 4 / SPL; // activation loads per tile
    // STAGED (16 rows, a launch of at most one workgroup per CU -- the 136 KiB
    // leave room for one): requested as whole 256-byte row pieces (16 lanes a
    // row, 4 rows an instruction: load h of lane l is piece l % 16 of row
    // 4 h + l / 16) instead of 64-byte pieces of 16 different rows, and read
    // back from LDS in operand order; wave-private, so no barrier. 4096 x 4096
    // at 16 rows: 6.7 us against 7.5 us; with more workgroups than CUs the
    // second resident workgroup is worth more (14336 columns: 19 against 21 us).
    static_assert(!STAGED || ROWS == 16, "");
    const int rr = ROWS == 1 ? 0 : STAGED ? 0 : min(r / SPL, rows - 1);
    const uint16_t *__restrict__ Arow = pA + (int64_t)(m_base + rr) * lda;
    uint8_t *const stage_w = act_lds + uw * (GEMV_UNR * 16 * GEMV_APITCH);
    const int nn = min(n, N - 1);
    const uint16_t *const scn = pSC + (scale_per_n ? nn : 0);
    const int zcol = zp_per_n ? nn : 0;
    const bool k_tail = (K & 127) != 0;
    constexpr int UNR = GEMV_UNR;
    void *dst_ptr = nullptr;
    int64_t dst_sm = 0;
    int dst_dt = 0;
    // steps past the end repeat the last tile and are folded with scale 0
    auto tile_of = [&](int t) { return min(t, tiles - 1); };
    for (int tb = 0; tb < tiles; tb += UNR * GEMV_WAVES) {
        // Loads are issued tile by tile (weights, activations, scale, zero
        // point) and consumed in the same order below: results return in
        // issue order, so tile u is unpacked and multiplied while tiles
        // u + 1 .. are still arriving. (Requesting all activations first and
        // the scales last, so that only the weights order the arithmetic, was
        // measured slower: the first weights request leaves later.)
        uint4 wt[UNR][NP], av[UNR][NA];
        uint32_t scp[UNR], zpp[UNR];
#pragma unroll
        for (int u = 0; u < UNR; u++) {
            const int tc = tile_of(tb + uw + u * GEMV_WAVES);
#pragma unroll
            for (int pl = 0; pl < NP; pl++)
                wt[u][pl] = ld_stream(Bt + (int64_t)tc * TILE_BYTES + pl * 1024);
#pragma unroll
            for (int h = 0; h < NA; h++) {
                // chunks past the row's end re-read its last one, rows past M
                // the last row
                if constexpr (STAGED) {
                    const int row = min(4 * h + (lane >> 4), rows - 1);
                    const int k = min(tc * 128 + (lane & 15) * 8, K - 8);
                    av[u][h] = *(const uint4 *)(pA + (int64_t)(m_base + row) * lda + k);
                } else {
                    const int k = min(
                            tc * 128 + (h * SPL + r % SPL) * 32 + c * 8, K - 8);
                    av[u][h] = *(const uint4 *)(Arow + k);
                }
            }
            const int gsc = gs_shift < 0 ? 0 : tc >> gs_shift;
            scp[u] = scn[(int64_t)gsc * sN];
            const int gzp = gz_shift < 0 ? 0 : tc >> gz_shift;
            const int64_t zi = has_zp ? (int64_t)gzp * zN + zcol : 0;
            zpp[u] = pZP[zp4 ? zi >> 1 : zi];
        }
        if (k_tail && tb + UNR * GEMV_WAVES >= tiles) {
            // zero the activations past K (last tile of the matrix)
#pragma unroll
            for (int u = 0; u < UNR; u++) {
                const int tc = tile_of(tb + uw + u * GEMV_WAVES);
#pragma unroll
                for (int h = 0; h < NA; h++)
                    if ((STAGED ? tc * 128 + (lane & 15) * 8
                                : tc * 128 + (h * SPL + r % SPL) * 32 + c * 8)
                            >= K)
                        av[u][h] = make_uint4(0, 0, 0, 0);
            }
        }
        // what the final store needs from the (cold) parameter block is
        // requested here, behind the loads and ahead of the arithmetic
        if (tb == 0) {
            dst_ptr = (void *)p.ep.dst.ptr;
            dst_sm = p.ep.dst.sm;
            dst_dt = p.ep.dst.dt;
            asm volatile("" ::"s"(dst_ptr), "s"(dst_sm), "s"(dst_dt));
        }
        if constexpr (STAGED) {
#pragma unroll
            for (int u = 0; u < UNR; u++)
#pragma unroll
                for (int h = 0; h < NA; h++)
                    *(uint4 *)(stage_w + ((u * 16 + 4 * h + (lane >> 4)) * GEMV_APITCH)
                            + (lane & 15) * 16)
                            = av[u][h];
        }
        // the four tiles are independent accumulation chains: a tile past
        // the end is a repeat of the last one and is folded with scale 0
#pragma unroll
        for (int u = 0; u < UNR; u++) {
            v4f Pu = {0.f, 0.f, 0.f, 0.f}, Su = {0.f, 0.f, 0.f, 0.f};
            if constexpr (STAGED) {
                // lane (r, c): row r, k = 32 s + 8 c .. + 7 of the tile
#pragma unroll
                for (int h = 0; h < NA; h++)
                    av[u][h] = *(const uint4 *)(stage_w + (u * 16 + r) * GEMV_APITCH
                            + h * 64 + c * 16);
            }
#pragma unroll
            for (int s4 = 0; s4 < 4; s4++) {
                const uint32_t d = (s4 == 0 ? wt[u][0].x
                                : s4 == 1   ? wt[u][0].y
                                : s4 == 2   ? wt[u][0].z
                                            : wt[u][0].w)
                        ^ sflip;
                v4u b;
                b.x = (d & NIB) | MAGIC_HI;
                b.y = ((d >> 4) & NIB) | MAGIC_HI;
                b.z = ((d >> 8) & NIB) | MAGIC_HI;
                b.w = ((d >> 12) & NIB) | MAGIC_HI;
                v4u bl = b;
                if constexpr (W8) {
                    const uint32_t dl = s4 == 0 ? wt[u][NP - 1].x
                            : s4 == 1           ? wt[u][NP - 1].y
                            : s4 == 2           ? wt[u][NP - 1].z
                                                : wt[u][NP - 1].w;
                    bl.x = (dl & NIB) | MAGIC;
                    bl.y = ((dl >> 4) & NIB) | MAGIC;
                    bl.z = ((dl >> 8) & NIB) | MAGIC;
                    bl.w = ((dl >> 12) & NIB) | MAGIC;
                }
                v4u a;
                {
                    // operand row SPL j takes step s4's chunk from lane
                    // (SPL j + s4 % SPL, c) of load s4 / SPL
                    const uint4 v = av[u][s4 / SPL];
                    if (s4 % SPL == 0)
                        a = v4u {v.x, v.y, v.z, v.w};
                    else if (s4 % SPL == 1)
                        a = v4u {row_shl<1>(v.x), row_shl<1>(v.y),
                                row_shl<1>(v.z), row_shl<1>(v.w)};
                    else if (s4 % SPL == 2)
                        a = v4u {row_shl<2>(v.x), row_shl<2>(v.y),
                                row_shl<2>(v.z), row_shl<2>(v.w)};
                    else
                        a = v4u {row_shl<3>(v.x), row_shl<3>(v.y),
                                row_shl<3>(v.z), row_shl<3>(v.w)};
                }
                Pu = mfma16<F16>(a, b, Pu);
                if constexpr (W8) Pu = mfma16<F16>(a, bl, Pu);
                Su = mfma16<F16>(a, ones, Su);
            }
            const int t = tb + uw + u * GEMV_WAVES;
            const int tc = tile_of(t);
            // one scale and one zero point per column and tile
            float sc = sc_f16
                    ? (float)__builtin_bit_cast(_Float16, (uint16_t)scp[u])
                    : u2f(scp[u] << 16);
            if (t >= tiles) sc = 0.f;
            // zero point: byte or nibble, signed or not, by shifts and selects
            // (wave-uniform branches here cost more than the arithmetic)
            const int gzp = gz_shift < 0 ? 0 : tc >> gz_shift;
            const int odd = zp4 ? (int)(((int64_t)gzp * zN + zcol) & 1) : 0;
            const int zbits = zp4 ? 4 : 8;
            const uint32_t zraw = (zpp[u] >> (4 * odd)) & ((1u << zbits) - 1u);
            const int zsx = (int)(zraw << (32 - zbits)) >> (32 - zbits);
            const float zp = has_zp ? (float)(zp_signed ? zsx : (int)zraw) : 0.f;
            const float off = W8 ? 17.f * OFFSET + 16.f * soff + zp
                                 : OFFSET + soff + zp;
            // a single row: only register 0 (row 0) is stored
#pragma unroll
            for (int j = 0; j < 4; j += SPL)
                out[j] = __builtin_fmaf(sc,
                        Pu[j] - off * Su[j],
                        out[j]);
        }
    }
    gemv_reduce_store<ROWS>(p, red, out, uw, lane, m_base, rows, n,
            (flags_m & 128) != 0, dst_ptr, dst_sm, dst_dt);
}

// gemv_w4_fast_kernel for wide weight matrices (4-bit weights, activations
// straight from global memory): a workgroup owns CB column blocks of 16. The
// activation fragments, their sums and the unpacking constants serve all of
// them, and the launch has 1 / CB as many workgroups, each with CB times the
// weights in flight: with more column blocks than the chip holds workgroups at
// once that is fewer rounds of workgroups and 1 / CB of the activation traffic
// (4096 x 14336 at 16 rows: 20.3 us with one block, 18.3 with two, 17.5 with four).
template <bool F16, int ROWS, bool WSIGNED, int CB>
__global__ void __launch_bounds__(GEMV_WAVES * 64)
gemv_w4_fast_cb_kernel(const uint8_t *__restrict__ pB,
        const uint16_t *__restrict__ pA, const uint16_t *__restrict__ pSC,
        const uint8_t *__restrict__ pZP, const int kg128, const int N,
        const int K, const int lda, const int shifts, const int flags_m,
        const gemv_params_t p) {
    constexpr bool W8 = false, STAGED = false;
    __shared__ __attribute__((aligned(16))) float red[GEMV_WAVES * 64 * 4];
    // STAGED: the activations of a wave's tiles pass through a wave-private
    // piece of LDS (see below)
    extern __shared__ __attribute__((aligned(16))) uint8_t act_lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int uw = __builtin_amdgcn_readfirstlane(tid >> 6);
    // consecutive workgroups run on the 8 XCDs in turn: give each XCD a
    // contiguous range of column blocks, so that a scale / zero-point line
    // (64 and more neighbouring columns) is fetched into one L2 only
    const int nbg = ((N + 15) >> 4) / CB; // groups of CB blocks (the host checks divisibility)
    const int bx = blockIdx.x;
    const int nb = ((nbg & 7) == 0 ? (bx & 7) * (nbg >> 3) + (bx >> 3) : bx) * CB;
    const int M = (uint32_t)flags_m >> 8;
    const int m_base = blockIdx.y * 16;
    const int rows = min(16, M - m_base);
    const int c = lane >> 4; // k chunk of the lane
    const int r = lane & 15; // activation row (A operand) / column (B operand)
    const int n = nb * 16 + r;
    const int gs_shift = (int8_t)(shifts & 0xff), gz_shift = (int8_t)(shifts >> 8);
    const bool scale_per_n = flags_m & 1, zp_per_n = flags_m & 2;
    const bool zp4 = flags_m & 4, zp_signed = flags_m & 8, sc_f16 = flags_m & 16;
    const bool has_zp = flags_m & 64;

    constexpr float OFFSET = F16 ? 1024.f : 128.f;
    constexpr uint32_t ONE2 = F16 ? 0x3C003C00u : 0x3F803F80u;
    const v4u ones = {ONE2, ONE2, ONE2, ONE2};
    constexpr uint32_t sflip = WSIGNED ? 0x88888888u : 0u;
    constexpr float soff = WSIGNED ? 8.f : 0.f;
    // the exponent pattern lives in a vector register and the nibble mask in a
    // scalar one: (d >> 4 i) & mask | magic is then a shift and one
    // v_and_or_b32 (an instruction takes one scalar or literal operand only)
    uint32_t MAGIC = F16 ? 0x64006400u : 0x43004300u;
    asm volatile("" : "+v"(MAGIC));
    // 8-bit weights: the high nibbles behind the exponent of 16 * offset, where
    // one unit of the last mantissa bit is 16 (f16: 0x7400 | h = 16384 + 16 h;
    // bf16: 0x4500 | h = 2048 + 16 h), so both planes add into one accumulator
    uint32_t MAGIC_HI = W8 ? (F16 ? 0x74007400u : 0x45004500u) : MAGIC;
    if constexpr (W8) asm volatile("" : "+v"(MAGIC_HI));
    uint32_t NIB = 0x000F000Fu;
    asm volatile("" : "+s"(NIB));

    v4f out[CB];
#pragma unroll
    for (int cb = 0; cb < CB; cb++) out[cb] = v4f {0.f, 0.f, 0.f, 0.f};
    constexpr int NP = W8 ? 2 : 1; // planes per tile
    constexpr int TILE_BYTES = 1024 * NP;
    const uint8_t *__restrict__ Bt
            = pB + ((int64_t)nb * kg128) * TILE_BYTES + lane * 16;
    const int64_t BSTEP = (int64_t)kg128 * TILE_BYTES; // to the next column block
    const int64_t sN = scale_per_n ? N : 0, zN = zp_per_n ? N : 0;

    // Waves are independent until the final reduction: each one fetches its
    // weight tiles, their scales / zero points AND its activation fragments
    // (lane (r, c) holds row r, k = 32 s + 8 c .. + 7 of a tile) straight into
    // registers, every load unconditional (clamped addresses), all issued
    // before the first use. No LDS staging, no barrier before the arithmetic.
    // Tile and group indices are wave uniform (scalar arithmetic, shifts
    // instead of divisions). Rows past M compute on a repeated row and are
    // never stored; only k past K has to be zeroed (the padded weights decode
    // to the magic offset, not 0).
    const int tiles = kg128;
    constexpr int SPL = ROWS == 16 ? 1 : ROWS == 8 ? 2 : 4; // steps per load
    constexpr int NA = 4 / SPL; // activation loads per tile
    // STAGED (16 rows, a launch of at most one workgroup per CU -- the 136 KiB
    // leave room for one): requested as whole 256-byte row pieces (16 lanes a
    // row, 4 rows an instruction: load h of lane l is piece l % 16 of row
    // 4 h + l / 16) instead of 64-byte pieces of 16 different rows, and read
    // back from LDS in operand order; wave-private, so no barrier. 4096 x 4096
    // at 16 rows: 6.7 us against 7.5 us; with more workgroups than CUs the
    // second resident workgroup is worth more (14336 columns: 19 against 21 us).
    static_assert(!STAGED || ROWS == 16, "");
    const int rr = ROWS == 1 ? 0 : STAGED ? 0 : min(r / SPL, rows - 1);
    const uint16_t *__restrict__ Arow = pA + (int64_t)(m_base + rr) * lda;
    uint8_t *const stage_w = act_lds + uw * (GEMV_UNR * 16 * GEMV_APITCH);
    // column of block cb: n + 16 cb
    const uint16_t *scn[CB];
    int zcol[CB];
#pragma unroll
    for (int cb = 0; cb < CB; cb++) {
        const int nn = min(n + 16 * cb, N - 1);
        scn[cb] = pSC + (scale_per_n ? nn : 0);
        zcol[cb] = zp_per_n ? nn : 0;
    }
    const bool k_tail = (K & 127) != 0;
    constexpr int UNR = GEMV_UNR;
    void *dst_ptr = nullptr;
    int64_t dst_sm = 0;
    int dst_dt = 0;
    // steps past the end repeat the last tile and are folded with scale 0
    auto tile_of = [&](int t) { return min(t, tiles - 1); };
    for (int tb = 0; tb < tiles; tb += UNR * GEMV_WAVES) {
        // Loads are issued tile by tile (weights, activations, scale, zero
        // point) and consumed in the same order below: results return in
        // issue order, so tile u is unpacked and multiplied while tiles
        // u + 1 .. are still arriving. (Requesting all activations first and
        // the scales last, so that only the weights order the arithmetic, was
        // measured slower: the first weights request leaves later.)
        uint4 wt[CB][UNR][NP], av[UNR][NA];
        uint32_t scp[CB][UNR], zpp[CB][UNR];
#pragma unroll
        for (int u = 0; u < UNR; u++) {
            const int tc = tile_of(tb + uw + u * GEMV_WAVES);
#pragma unroll
            for (int cb = 0; cb < CB; cb++)
#pragma unroll
                for (int pl = 0; pl < NP; pl++)
                    wt[cb][u][pl] = ld_stream(Bt + cb * BSTEP
                            + (int64_t)tc * TILE_BYTES + pl * 1024);
#pragma unroll
            for (int h = 0; h < NA; h++) {
                // chunks past the row's end re-read its last one, rows past M
                // the last row
                if constexpr (STAGED) {
                    const int row = min(4 * h + (lane >> 4), rows - 1);
                    const int k = min(tc * 128 + (lane & 15) * 8, K - 8);
                    av[u][h] = *(const uint4 *)(pA + (int64_t)(m_base + row) * lda + k);
                } else {
                    const int k = min(
                            tc * 128 + (h * SPL + r % SPL) * 32 + c * 8, K - 8);
                    av[u][h] = *(const uint4 *)(Arow + k);
                }
            }
            const int gsc = gs_shift < 0 ? 0 : tc >> gs_shift;
            const int gzp = gz_shift < 0 ? 0 : tc >> gz_shift;
#pragma unroll
            for (int cb = 0; cb < CB; cb++) {
                scp[cb][u] = scn[cb][(int64_t)gsc * sN];
                const int64_t zi = has_zp ? (int64_t)gzp * zN + zcol[cb] : 0;
                zpp[cb][u] = pZP[zp4 ? zi >> 1 : zi];
            }
        }
        if (k_tail && tb + UNR * GEMV_WAVES >= tiles) {
            // zero the activations past K (last tile of the matrix)
#pragma unroll
            for (int u = 0; u < UNR; u++) {
                const int tc = tile_of(tb + uw + u * GEMV_WAVES);
#pragma unroll
                for (int h = 0; h < NA; h++)
                    if ((STAGED ? tc * 128 + (lane & 15) * 8
                                : tc * 128 + (h * SPL + r % SPL) * 32 + c * 8)
                            >= K)
                        av[u][h] = make_uint4(0, 0, 0, 0);
            }
        }
        // what the final store needs from the (cold) parameter block is
        // requested here, behind the loads and ahead of the arithmetic
        if (tb == 0) {
            dst_ptr = (void *)p.ep.dst.ptr;
            dst_sm = p.ep.dst.sm;
            dst_dt = p.ep.dst.dt;
            asm volatile("" ::"s"(dst_ptr), "s"(dst_sm), "s"(dst_dt));
        }
        if constexpr (STAGED) {
#pragma unroll
            for (int u = 0; u < UNR; u++)
#pragma unroll
                for (int h = 0; h < NA; h++)
                    *(uint4 *)(stage_w + ((u * 16 + 4 * h + (lane >> 4)) * GEMV_APITCH)
                            + (lane & 15) * 16)
                            = av[u][h];
        }
        // the four tiles are independent accumulation chains: a tile past
        // the end is a repeat of the last one and is folded with scale 0
#pragma unroll
        for (int u = 0; u < UNR; u++) {
            v4f Pu[CB], Su = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int cb = 0; cb < CB; cb++) Pu[cb] = v4f {0.f, 0.f, 0.f, 0.f};
            if constexpr (STAGED) {
                // lane (r, c): row r, k = 32 s + 8 c .. + 7 of the tile
#pragma unroll
                for (int h = 0; h < NA; h++)
                    av[u][h] = *(const uint4 *)(stage_w + (u * 16 + r) * GEMV_APITCH
                            + h * 64 + c * 16);
            }
#pragma unroll
            for (int s4 = 0; s4 < 4; s4++) {
                v4u a;
                {
                    // operand row SPL j takes step s4's chunk from lane
                    // (SPL j + s4 % SPL, c) of load s4 / SPL
                    const uint4 v = av[u][s4 / SPL];
                    if (s4 % SPL == 0)
                        a = v4u {v.x, v.y, v.z, v.w};
                    else if (s4 % SPL == 1)
                        a = v4u {row_shl<1>(v.x), row_shl<1>(v.y),
                                row_shl<1>(v.z), row_shl<1>(v.w)};
                    else if (s4 % SPL == 2)
                        a = v4u {row_shl<2>(v.x), row_shl<2>(v.y),
                                row_shl<2>(v.z), row_shl<2>(v.w)};
                    else
                        a = v4u {row_shl<3>(v.x), row_shl<3>(v.y),
                                row_shl<3>(v.z), row_shl<3>(v.w)};
                }
#pragma unroll
                for (int cb = 0; cb < CB; cb++) {
                    const uint32_t d = (s4 == 0 ? wt[cb][u][0].x
                                    : s4 == 1   ? wt[cb][u][0].y
                                    : s4 == 2   ? wt[cb][u][0].z
                                                : wt[cb][u][0].w)
                            ^ sflip;
                    v4u b;
                    b.x = (d & NIB) | MAGIC_HI;
                    b.y = ((d >> 4) & NIB) | MAGIC_HI;
                    b.z = ((d >> 8) & NIB) | MAGIC_HI;
                    b.w = ((d >> 12) & NIB) | MAGIC_HI;
                    v4u bl = b;
                    if constexpr (W8) {
                        const uint32_t dl = s4 == 0 ? wt[cb][u][NP - 1].x
                                : s4 == 1           ? wt[cb][u][NP - 1].y
                                : s4 == 2           ? wt[cb][u][NP - 1].z
                                                    : wt[cb][u][NP - 1].w;
                        bl.x = (dl & NIB) | MAGIC;
                        bl.y = ((dl >> 4) & NIB) | MAGIC;
                        bl.z = ((dl >> 8) & NIB) | MAGIC;
                        bl.w = ((dl >> 12) & NIB) | MAGIC;
                    }
                    Pu[cb] = mfma16<F16>(a, b, Pu[cb]);
                    if constexpr (W8) Pu[cb] = mfma16<F16>(a, bl, Pu[cb]);
                }
                Su = mfma16<F16>(a, ones, Su);
            }
            const int t = tb + uw + u * GEMV_WAVES;
            const int tc = tile_of(t);
            const int gzp = gz_shift < 0 ? 0 : tc >> gz_shift;
#pragma unroll
            for (int cb = 0; cb < CB; cb++) {
                // one scale and one zero point per column and tile
                float sc = sc_f16
                        ? (float)__builtin_bit_cast(_Float16, (uint16_t)scp[cb][u])
                        : u2f(scp[cb][u] << 16);
                if (t >= tiles) sc = 0.f;
                // zero point: byte or nibble, signed or not, by shifts and selects
                // (wave-uniform branches here cost more than the arithmetic)
                const int odd = zp4 ? (int)(((int64_t)gzp * zN + zcol[cb]) & 1) : 0;
                const int zbits = zp4 ? 4 : 8;
                const uint32_t zraw = (zpp[cb][u] >> (4 * odd)) & ((1u << zbits) - 1u);
                const int zsx = (int)(zraw << (32 - zbits)) >> (32 - zbits);
                const float zp = has_zp ? (float)(zp_signed ? zsx : (int)zraw) : 0.f;
                const float off = W8 ? 17.f * OFFSET + 16.f * soff + zp
                                     : OFFSET + soff + zp;
                // a single row: only register 0 (row 0) is stored
#pragma unroll
                for (int j = 0; j < 4; j += SPL)
                    out[cb][j] = __builtin_fmaf(sc,
                            Pu[cb][j] - off * Su[j],
                            out[cb][j]);
            }
        }
    }
#pragma unroll
    for (int cb = 0; cb < CB; cb++) {
        if (cb) __syncthreads(); // wave 0 has read the previous block's sums
        gemv_reduce_store<ROWS>(p, red, out[cb], uw, lane, m_base, rows,
                n + 16 * cb, (flags_m & 128) != 0, dst_ptr, dst_sm, dst_dt);
    }
}

void launch_gemm_w4f(const gemv_params_t &p, int shifts, int flags_m,
        hipStream_t stream);
bool gemm_w4f_wins(const gemv_params_t &p);

// Returns false when no kernel takes the problem (nothing is launched then).
bool launch_gemv_w4(const gemv_params_t &p, hipStream_t stream) {
    if (p.M <= 0 || p.N <= 0) return true;
    const int rows = p.M < 16 ? p.M : 16;
    int MR = 1;
    while (MR < rows) MR *= 2;
    const int Kpad = p.kg128 * 128;
    int KC = GEMV_LDS_BUDGET / (2 * MR);
    KC = KC / 128 * 128;
    if (KC > Kpad) KC = Kpad;
    size_t lds = (size_t)KC * 2 * MR;
    const size_t red = (size_t)GEMV_WAVES * 64 * 4 * sizeof(float);
    if (lds < red) lds = red;
    dim3 grid(p.nb16, (p.M + 15) / 16);
    // the all-unconditional-loads variant (see the kernel's FAST parameter)
    int fl = p.gs;
    if (p.gz > 0) {
        int a = p.gs, b = p.gz;
        while (b) {
            const int t = a % b;
            a = b;
            b = t;
        }
        fl = a;
    }
    // group widths of the form 128 << s (or one group over all of K)
    auto shift_of = [&](int g, int &sh) {
        if (g >= Kpad) {
            sh = -1;
            return true;
        }
        if (g % 128 != 0) return false;
        int q = g / 128;
        sh = 0;
        while (q > 1 && q % 2 == 0) {
            q /= 2;
            sh++;
        }
        return q == 1;
    };
    gemv_params_t q = p;
    // 8-bit weights exist in the fast variant only (host-checked at creation)
    const bool fast = p.scales && fl % 128 == 0
            && (p.scale_dt == dt_f16 || p.scale_dt == dt_bf16)
            && (!p.zps || p.zp_dt != dt_s32) && shift_of(p.gs, q.gs_shift)
            && (p.gz > 0 ? shift_of(p.gz, q.gz_shift)
                         : ((q.gz_shift = -1), true));
    if (fast && p.m0 == 0 && p.lda < ((int64_t)1 << 31) && p.M < (1 << 23)) {
        // nothing between the accumulation and a dense dst row
        const bool plain = !p.ep.src_scale.ptr && !p.ep.wei_scale.ptr
                && !p.ep.bias.ptr && p.ep.npo == 0 && !p.ep.dst_scale
                && !p.ep.dst_zp && p.ep.dst.sn == 1;
        const int flags_m = (p.scale_per_n ? 1 : 0) | (p.zp_per_n ? 2 : 0)
                | (p.zp_dt == dt_s4 || p.zp_dt == dt_u4 ? 4 : 0)
                | (p.zp_dt == dt_s4 || p.zp_dt == dt_s8 ? 8 : 0)
                | (p.scale_dt == dt_f16 ? 16 : 0) | (p.wei_signed ? 32 : 0)
                | (p.zps ? 64 : 0) | (plain ? 128 : 0) | (p.M << 8);
        const int shifts = (q.gs_shift & 0xff) | ((q.gz_shift & 0xff) << 8);
        // an absent zero-point buffer is never dereferenced past its first
        // byte: the weights stand in for it
        const uint8_t *zp = p.zps ? (const uint8_t *)p.zps : p.B;
        // More than 16 rows: the tiled kernel (a weights tile unpacked once
        // for 32 or 64 rows) where it beats this one once per block of 16 rows.
        if (gemm_w4f_wins(p)) {
            launch_gemm_w4f(q, shifts, flags_m, stream);
            return true;
        }
        // more than 8 rows in at most one workgroup per CU: the variant that
        // stages its activations in LDS
        const bool staged = p.M > 8 && (int64_t)grid.x * grid.y <= 256;
        const int lds = staged ? GEMV_STAGE_BYTES : 0;
        // two column blocks per workgroup where one block each would be more
        // workgroups than the chip holds at once (two per CU)
        // (5 .. 8 rows keep one block: with two, the 8-row form spills registers)
        const bool two = !p.w8 && !staged && (p.nb16 & 1) == 0 && p.nb16 >= 512
                && !(p.M > 4 && p.M <= 8);
        // more than 8 rows: four blocks, for a quarter of the activation traffic
        const bool four = two && p.M > 8 && (p.nb16 & 3) == 0 && p.nb16 >= 768;
        auto go = [&](auto kern) {
            if (lds) ensure_dynamic_lds((const void *)kern, lds);
            hipLaunchKernelGGL(kern,
                    four       ? dim3(grid.x / 4, grid.y)
                            : two ? dim3(grid.x / 2, grid.y)
                                  : grid,
                    dim3(GEMV_WAVES * 64), lds, stream, p.B,
                    p.A, (const uint16_t *)p.scales, zp, p.kg128, p.N, p.K,
                    (int)p.lda, shifts, flags_m, q);
        };
        // template arguments from the run-time choices, one level each
        auto by_w8 = [&](auto f16, auto rows, auto sgn) {
            constexpr bool F = decltype(f16)::value, S = decltype(sgn)::value;
            constexpr int R = decltype(rows)::value;
            if constexpr (R == 16) {
                if (staged) {
                    if (p.w8)
                        go(gemv_w4_fast_kernel<F, R, S, true, true>);
                    else
                        go(gemv_w4_fast_kernel<F, R, S, false, true>);
                    return;
                }
            }
            if constexpr (R == 16) {
                if (four) {
                    go(gemv_w4_fast_cb_kernel<F, R, S, 4>);
                    return;
                }
            }
            if (p.w8)
                go(gemv_w4_fast_kernel<F, R, S, true>);
            else if (two)
                go(gemv_w4_fast_cb_kernel<F, R, S, 2>);
            else
                go(gemv_w4_fast_kernel<F, R, S, false>);
        };
        auto by_sign = [&](auto f16, auto rows) {
            if (p.wei_signed)
                by_w8(f16, rows, std::true_type {});
            else
                by_w8(f16, rows, std::false_type {});
        };
        auto by_rows = [&](auto f16) {
            if (p.M == 1)
                by_sign(f16, std::integral_constant<int, 1> {});
            else if (p.M <= 4)
                by_sign(f16, std::integral_constant<int, 4> {});
            else if (p.M <= 8)
                by_sign(f16, std::integral_constant<int, 8> {});
            else
                by_sign(f16, std::integral_constant<int, 16> {});
        };
        if (p.act_f16)
            by_rows(std::true_type {});
        else
            by_rows(std::false_type {});
        return true;
    }
    // 8-bit weights exist in the all-unconditional-loads form only; creation
    // admits nothing else, and a drift between the two checks must not pass
    // as a launch that wrote nothing
    if (p.w8) return false;
    auto launch = [&](auto kern) {
        ensure_dynamic_lds((const void *)kern, GEMV_LDS_BUDGET);
        hipLaunchKernelGGL(kern, grid, dim3(GEMV_WAVES * 64), lds, stream, q,
                MR, KC);
    };
    if (p.act_f16)
        launch(gemv_w4_kernel<true>);
    else
        launch(gemv_w4_kernel<false>);
    return true;
}

} // namespace qmm
