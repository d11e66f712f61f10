// hip:gfx950:mfma_f16 -- plain 16-bit matmul (f16 x f16 or bf16 x bf16, f32
// accumulation; src/cpu/matmul/ref_matmul.cpp:130-233 with no quantization
// attributes), batched: the unfused attention products that sit next to the
// quantized linear layers in an LLM (scores = Q x K^T, context = P x V) and
// that would otherwise fall to the per-element kernel.
//
// Source rows K-contiguous, weights rows N-contiguous (the reference's plain
// `ab` / `abcd` weights), any K and N: operands that are not 16-byte granular
// are staged element by element. A workgroup of four waves owns a 64 x 64 tile
// of dst; per 32-k step the source tile [64][32] and the weights tile [32][64]
// go through LDS (double buffered, one barrier per step). The weights are the
// MFMA's FIRST operand, transposed on the way out of LDS by
// ds_read_b64_tr_b16 (lane i of a 16-lane group receives element i & 3 of the
// 8-byte chunks that lanes (i >> 2) + 4 t addressed), so lane (r, c) holds
// column n = r for k = 4 c .. 4 c + 3 and 16 + 4 c .. 16 + 4 c + 3, and the
// source fragment is read in the same k order. With the weights first,
// register i of lane (r, c) is dst[m = r][n = 4 c + i]: four neighbouring
// columns of a row, which is what the common epilogue takes.
#include "qmm_device.hpp"
#include "qmm_plan.hpp"

#include <type_traits>

namespace qmm {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef short v4s __attribute__((ext_vector_type(4)));
typedef short v8s __attribute__((ext_vector_type(8)));

constexpr int F16_BK = 32;
// Tile shapes: BM x BN of dst per workgroup of four waves arranged WGM x WGN.
//   64 x 64, waves 1 x 4 (a wave owns 64 rows x 16 columns): small problems;
//   128 x 128, waves 2 x 2 (64 x 64 per wave: 16 MFMAs per 32-k step for 8
//   transposing and 8 plain fragment reads, four times the MFMAs per LDS read of
//   the small tile): problems with enough such tiles to fill the chip.
template <int BM_, int BN_, int WGM_, int WGN_>
struct f16_tile {
    static constexpr int BM = BM_, BN = BN_, WGM = WGM_, WGN = WGN_;
    static constexpr int WM = BM / WGM, WN = BN / WGN; // wave tile
    static constexpr int MF = WM / 16, NF = WN / 16; // 16 x 16 fragments of a wave
    static constexpr int A_PITCH = F16_BK * 2 + 16; // bytes of a staged source row
    static constexpr int B_PITCH = BN * 2 + 16; // bytes of a staged weights row
    static constexpr int A_BYTES = BM * A_PITCH, B_BYTES = F16_BK * B_PITCH;
    static constexpr int CA = BM * 4 / 256, CB = F16_BK * (BN / 8) / 256; // chunks a thread stages
    static constexpr int OUT_PITCH = BN + 4; // words of a staged dst row
    static constexpr int OUT_ROWS = WM; // dst rows staged at a time: one wave row
    static constexpr int LDS_BYTES = 2 * (A_BYTES + B_BYTES) > OUT_ROWS * OUT_PITCH * 4
            ? 2 * (A_BYTES + B_BYTES)
            : OUT_ROWS * OUT_PITCH * 4;
    static_assert(WM == 64 && CA >= 1 && CB >= 1, "tile shape");
};
typedef f16_tile<64, 64, 1, 4> f16_small_t;
typedef f16_tile<128, 128, 2, 2> f16_big_t;

template <bool BF>
QMM_D v4f mma16(const v8s &a, const v8s &b, const v4f &c) {
    if constexpr (BF)
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                __builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(
                __builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
}

// Eight neighbouring 16-bit elements of a row of `len` elements, starting at
// element `at` (a multiple of 8), in two steps so that nothing touches the
// loaded registers before the tile is staged: `request8` only issues loads,
// `finish8` zeroes what lies at or past `len` (or in a row that is not there).
//   G = 8: rows start on 16-byte boundaries and `len` is a multiple of 8, so a
//     chunk is inside the row or past it: one aligned 16-byte load.
//   G = 0: any alignment, `len` >= 8: one 16-byte load that need not be aligned
//     (global loads take any address), at min(at, len - 8); where that moved the
//     window back, the chunk's elements are the window's upper ones and
//     `finish8` shifts them down, which also zero-fills what is past `len`.
//   G = 1: rows shorter than 8: element loads.
typedef unsigned v4u_any __attribute__((ext_vector_type(4), aligned(2)));

template <int G>
struct req8_t {
    uint32_t w[G == 1 ? 8 : 4];
};

template <int G>
QMM_D void request8(req8_t<G> &r, const uint16_t *row, int at, int len) {
    if constexpr (G == 8) {
        const uint4 v = *(const uint4 *)(row + (at < len ? at : 0));
        r.w[0] = v.x, r.w[1] = v.y, r.w[2] = v.z, r.w[3] = v.w;
    } else if constexpr (G == 0) {
        const auto v = *(const v4u_any *)(row + min(at, len - 8));
        r.w[0] = v[0], r.w[1] = v[1], r.w[2] = v[2], r.w[3] = v[3];
    } else {
#pragma unroll
        for (int j = 0; j < 8; j++) r.w[j] = row[at + j < len ? at + j : 0];
    }
}

template <int G>
QMM_D uint4 finish8(const req8_t<G> &r, int at, int len, bool row_ok) {
    uint32_t w[4];
    if constexpr (G == 8) {
        const bool ok = row_ok && at < len;
#pragma unroll
        for (int j = 0; j < 4; j++) w[j] = ok ? r.w[j] : 0u;
    } else if constexpr (G == 0) {
        // the window started `back` elements before the chunk: shift the 128
        // bits right by 16 * back (0 .. 112)
        const int back = at - min(at, len - 8);
        const uint64_t lo = (uint64_t)r.w[0] | ((uint64_t)r.w[1] << 32);
        const uint64_t hi = (uint64_t)r.w[2] | ((uint64_t)r.w[3] << 32);
        const int sh = 16 * (back & 3);
        const uint64_t a = back < 4 ? lo : hi, b = back < 4 ? hi : 0ull;
        const uint64_t nlo = sh ? (a >> sh) | (b << (64 - sh)) : a;
        const uint64_t nhi = b >> sh;
        const bool ok = row_ok && at < len;
        w[0] = ok ? (uint32_t)nlo : 0u;
        w[1] = ok ? (uint32_t)(nlo >> 32) : 0u;
        w[2] = ok ? (uint32_t)nhi : 0u;
        w[3] = ok ? (uint32_t)(nhi >> 32) : 0u;
    } else {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t lo = row_ok && at + 2 * j < len ? r.w[2 * j] : 0u;
            const uint32_t hi = row_ok && at + 2 * j + 1 < len ? r.w[2 * j + 1] : 0u;
            w[j] = lo | (hi << 16);
        }
    }
    return make_uint4(w[0], w[1], w[2], w[3]);
}

constexpr int F16_AHEAD = 4; // steps between an operand's request and its staging

template <int N, typename F>
QMM_D void static_for(F &&f) {
    if constexpr (N > 0) {
        static_for<N - 1>(f);
        f(std::integral_constant<int, N - 1> {});
    }
}

// LIGHT: nothing follows the accumulation but at most one relu / linear / clip
// (what the attention products carry). Everything else goes through the
// post-op interpreter, whose register needs halve the waves a SIMD can hold.
QMM_HD bool light_epilogue(const epilogue_t &ep) {
    if (ep.bias.ptr || ep.src_scale.ptr || ep.wei_scale.ptr || ep.dst_scale || ep.dst_zp)
        return false;
    if (ep.npo == 0) return true;
    return ep.npo == 1 && ep.po[0].kind == pk_eltwise
            && (ep.po[0].alg == alg_relu || ep.po[0].alg == alg_linear
                    || ep.po[0].alg == alg_clip || ep.po[0].alg == alg_clip_v2);
}

template <bool BF, bool LIGHT, int GA, int GB, typename T>
__global__ void __launch_bounds__(256)
gemm_f16_kernel(const gemm16_params_t p) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[T::LDS_BYTES];
    uint8_t *const lds_a = lds, *const lds_b = lds + 2 * T::A_BYTES;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wrow = wave / T::WGN, wcol = wave % T::WGN;
    const int r = lane & 15, c = lane >> 4;
    // Consecutive workgroups start on the 8 XCDs in turn. The launch is a flat
    // list of tiles (columns fastest, then rows, then batch entries); XCD j takes
    // the j-th eighth of it, so the tiles one L2 sees are neighbours: a few
    // batch entries (attention heads) or a few row panels of one matrix, and
    // their operands are fetched into that L2 only.
    const int gx = (p.N + T::BN - 1) / T::BN, gy = (p.M + T::BM - 1) / T::BM;
    int id = blockIdx.x;
    {
        const int total = gridDim.x;
        if ((total & 7) == 0) id = (id & 7) * (total >> 3) + (id >> 3);
    }
    const int m0 = ((id / gx) % gy) * T::BM, n0 = (id % gx) * T::BN;
    const int64_t bz = id / (gx * gy);
    const uint16_t *A = p.A + bz * p.a_sb, *B = p.B + bz * p.b_sb;
    // staging: chunk q = tid + 256 i (8 elements each) is chunk q % 4 of source
    // row q / 4, and chunk q % (BN / 8) of weights row q / (BN / 8) of the step
    constexpr int BCH = T::BN / 8;
    const int steps = (p.K + F16_BK - 1) / F16_BK;

    // operands are requested F16_AHEAD steps before they are staged: one slot
    // of registers per step in flight, named statically (the loop is unrolled
    // by the slot count)
    req8_t<GA> ra[F16_AHEAD][T::CA];
    req8_t<GB> rb[F16_AHEAD][T::CB];
    auto request = [&](int kt, auto S) {
        constexpr int sl = decltype(S)::value;
        const int k0 = min(kt, steps - 1) * F16_BK; // (the prologue may ask past a short K)
#pragma unroll
        for (int i = 0; i < T::CA; i++) {
            const int q = tid + 256 * i, ar = q >> 2, ak = (q & 3) * 8;
            request8<GA>(ra[sl][i], A + (int64_t)min(m0 + ar, p.M - 1) * p.lda, k0 + ak, p.K);
        }
#pragma unroll
        for (int i = 0; i < T::CB; i++) {
            const int q = tid + 256 * i, bk = q / BCH, bn = (q % BCH) * 8;
            request8<GB>(rb[sl][i], B + (int64_t)min(k0 + bk, p.K - 1) * p.ldb, n0 + bn, p.N);
        }
    };
    auto stage = [&](int kt, auto S) {
        constexpr int sl = decltype(S)::value;
        const int k0 = kt * F16_BK, buf = kt & 1;
#pragma unroll
        for (int i = 0; i < T::CA; i++) {
            const int q = tid + 256 * i, ar = q >> 2, ak = (q & 3) * 8;
            *(uint4 *)(lds_a + buf * T::A_BYTES + ar * T::A_PITCH + ak * 2)
                    = finish8<GA>(ra[sl][i], k0 + ak, p.K, m0 + ar < p.M);
        }
#pragma unroll
        for (int i = 0; i < T::CB; i++) {
            const int q = tid + 256 * i, bk = q / BCH, bn = (q % BCH) * 8;
            *(uint4 *)(lds_b + buf * T::B_BYTES + bk * T::B_PITCH + bn * 2)
                    = finish8<GB>(rb[sl][i], n0 + bn, p.N, k0 + bk < p.K);
        }
    };

    v4f acc[T::MF][T::NF];
#pragma unroll
    for (int mf = 0; mf < T::MF; mf++)
#pragma unroll
        for (int nf = 0; nf < T::NF; nf++) acc[mf][nf] = v4f {0.f, 0.f, 0.f, 0.f};

    auto step = [&](int kt, auto S) {
        constexpr int sl = decltype(S)::value;
        const int buf = kt & 1;
        // the slot's tile kt was staged a step ago (short K: nothing left to ask
        // for, and a dst-bound launch should not read its operands twice)
        if (kt + F16_AHEAD < steps) request(kt + F16_AHEAD, S);
        // weights fragments of the wave's columns, transposed out of LDS
        v8s bf[T::NF];
#pragma unroll
        for (int nf = 0; nf < T::NF; nf++) {
            const uint8_t *vb = lds_b + buf * T::B_BYTES + (4 * c + (r >> 2)) * T::B_PITCH
                    + (T::WN * wcol + 16 * nf + 4 * (r & 3)) * 2;
            const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (v4s __attribute__((address_space(3))) *)vb);
            const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (v4s __attribute__((address_space(3))) *)(vb + 16 * T::B_PITCH));
            bf[nf] = v8s {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
#pragma unroll
        for (int mf = 0; mf < T::MF; mf++) {
            // source fragment: row 16 mf + r of the wave's rows, the same eight k
            const uint8_t *pa = lds_a + buf * T::A_BYTES
                    + (T::WM * wrow + 16 * mf + r) * T::A_PITCH;
            const v4s x = *(const v4s *)(pa + (4 * c) * 2);
            const v4s y = *(const v4s *)(pa + (16 + 4 * c) * 2);
            const v8s af = {x[0], x[1], x[2], x[3], y[0], y[1], y[2], y[3]};
#pragma unroll
            for (int nf = 0; nf < T::NF; nf++)
                acc[mf][nf] = mma16<BF>(bf[nf], af, acc[mf][nf]);
        }
        if (kt + 1 < steps)
            stage(kt + 1, std::integral_constant<int, (sl + 1) % F16_AHEAD> {});
        __syncthreads();
    };

    static_for<F16_AHEAD>([&](auto S) { request(decltype(S)::value, S); });
    stage(0, std::integral_constant<int, 0> {});
    __syncthreads();
    for (int kt = 0; kt < steps; kt += F16_AHEAD)
        static_for<F16_AHEAD>([&](auto S) {
            if (kt + decltype(S)::value < steps) step(kt + decltype(S)::value, S);
        });

    // register i of lane (r, c) is dst[16 mf + r][16 nf + 4 c + i] of the wave
    // tile. One wave row (64 dst rows) at a time goes through LDS, so that
    // neighbouring lanes store whole row pieces of BN columns instead of 16
    // rows with 8 bytes each.
    float *out = (float *)lds;
    constexpr int TPR = T::BN / 4, RPI = 256 / TPR; // threads per row, rows per pass
    const int n = n0 + (tid % TPR) * 4;
#pragma unroll 1
    for (int h = 0; h < T::WGM; h++) {
        if (h) __syncthreads();
        if (wrow == h) {
#pragma unroll
            for (int mf = 0; mf < T::MF; mf++)
#pragma unroll
                for (int nf = 0; nf < T::NF; nf++)
                    *(v4f *)(out + (16 * mf + r) * T::OUT_PITCH + T::WN * wcol + 16 * nf + 4 * c)
                            = acc[mf][nf];
        }
        __syncthreads();
        // one copy of the interpreter is enough; the light form is four stores
#pragma unroll 1
        for (int i = 0; i < T::OUT_ROWS / RPI; i++) {
            const int row = RPI * i + tid / TPR, m = m0 + T::WM * h + row;
            if (m < p.M && n < p.N) {
                const v4f t = *(const v4f *)(out + row * T::OUT_PITCH + (tid % TPR) * 4);
                float v[4] = {t[0], t[1], t[2], t[3]};
                if constexpr (LIGHT) {
                    if (p.ep.npo) {
                        const int alg = p.ep.po[0].alg;
                        const float al = p.ep.po[0].alpha, be = p.ep.po[0].beta,
                                    sc = p.ep.po[0].scale;
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            const float e = alg == alg_relu ? eltwise_one<alg_relu>(v[j], al, be)
                                    : alg == alg_linear     ? eltwise_one<alg_linear>(v[j], al, be)
                                    : alg == alg_clip       ? eltwise_one<alg_clip>(v[j], al, be)
                                                      : eltwise_one<alg_clip_v2>(v[j], al, be);
                            v[j] = e * sc;
                        }
                    }
                    epilogue_store4(p.ep, v, bz * p.ep.dst.sb + (int64_t)m * p.ep.dst.sm + n,
                            min(4, p.N - n));
                } else {
                    epilogue_apply_store4(p.ep, v, bz, m, n, min(4, p.N - n));
                }
            }
        }
    }
}

// ---- short K over many columns (the attention scores: K = 64 / 128) ----------
// Such a launch is its dst stream, and time stamps inside the kernels show where
// it goes: a CU retires a store instruction of a wave only every 85 to 100
// cycles whatever it carries, so the time is the number of store instructions --
// four 16-bit results (8 bytes) a lane took 13.5 k cycles per 128 x 128 tile
// against 4.4 k for its four k-steps; eight results (16 bytes) a lane 5.4 k. The
// rest of this kernel keeps the CU storing: a workgroup owns 128 rows of one
// batch entry, keeps them in LDS for all of K (at most 128) and WALKS a range
// of column tiles; only the weights tiles stream (the next tile's k-step kt is
// requested while this tile's is multiplied), so the next tile is never waited
// for and a byte of dst costs half a byte of loads. A wave stores its 64 x 64
// through a wave-private slice of LDS, 16 rows at a time (eight lanes a row
// piece of 128 bytes), without a barrier. LIGHT epilogues only (what these
// products carry). 32 x (2048 x 128 x 2048): 124 us against 165 us for the
// 64 x 64 tiles (1000: 26 against 38 us).
// A barrier that orders LDS traffic only. __syncthreads() also waits for every
// global store the wave has issued (its fence covers global memory), which in a
// kernel that keeps storing tiles while it multiplies the next one puts the full
// latency of the stores in front of every k-step: 165 us instead of the time below.
QMM_D void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}
constexpr int F16_WALK_K = 128; // most k the resident rows hold
constexpr int F16_WALK_APITCH = F16_WALK_K * 2 + 16; // bytes of a resident row
constexpr int F16_WALK_SPITCH = 64 + 4; // words of a wave's staged dst row
constexpr int F16_WALK_A = 128 * F16_WALK_APITCH;
constexpr int F16_WALK_LDS
        = F16_WALK_A + 2 * f16_big_t::B_BYTES + 4 * 16 * F16_WALK_SPITCH * 4;
// STEPS: k-steps of a tile (2: K <= 64, 4: K <= 128; k past K multiplies zeros).
// The weights of k-step kt of the NEXT tile are requested while this tile's are
// multiplied: request slot and LDS buffer of a step are compile-time values.
template <bool BF, int GA, int GB, int STEPS>
__global__ void __launch_bounds__(256)
gemm_f16_walk_kernel(const gemm16_params_t p, const int nseg) {
    using T = f16_big_t;
    static_assert(STEPS == 2 || STEPS == 4, "");
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[]; // F16_WALK_LDS bytes
    uint8_t *const lds_a = lds, *const lds_b = lds + F16_WALK_A;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wrow = wave / T::WGN, wcol = wave % T::WGN;
    const int r = lane & 15, c = lane >> 4;
    float *const wout = (float *)(lds + F16_WALK_A + 2 * T::B_BYTES) + wave * 16 * F16_WALK_SPITCH;
    // workgroup -> (batch entry, row block, segment of the column tiles); the
    // XCDs take contiguous eighths of that list, as above
    const int gx = (p.N + T::BN - 1) / T::BN, gy = (p.M + T::BM - 1) / T::BM;
    int id = blockIdx.x;
    {
        const int total = gridDim.x;
        if ((total & 7) == 0) id = (id & 7) * (total >> 3) + (id >> 3);
    }
    const int tps = (gx + nseg - 1) / nseg; // tiles per segment
    const int tile0 = (id % nseg) * tps, ntile = min(tps, gx - tile0);
    if (ntile <= 0) return; // (workgroup-uniform, before any barrier)
    const int m0 = ((id / nseg) % gy) * T::BM;
    const int64_t bz = id / (nseg * gy);
    const uint16_t *A = p.A + bz * p.a_sb, *B = p.B + bz * p.b_sb;
    constexpr int BCH = T::BN / 8;

    req8_t<GB> rb[STEPS][T::CB];
    auto request = [&](int n0, auto KT) __attribute__((always_inline)) {
        constexpr int kt = decltype(KT)::value, k0 = kt * F16_BK;
#pragma unroll
        for (int i = 0; i < T::CB; i++) {
            const int q = tid + 256 * i, bk = q / BCH, bn = (q % BCH) * 8;
            request8<GB>(rb[kt][i], B + (int64_t)min(k0 + bk, p.K - 1) * p.ldb, n0 + bn, p.N);
        }
    };
    auto stage = [&](int n0, auto KT) __attribute__((always_inline)) {
        constexpr int kt = decltype(KT)::value, k0 = kt * F16_BK, buf = kt & 1;
#pragma unroll
        for (int i = 0; i < T::CB; i++) {
            const int q = tid + 256 * i, bk = q / BCH, bn = (q % BCH) * 8;
            *(uint4 *)(lds_b + buf * T::B_BYTES + bk * T::B_PITCH + bn * 2)
                    = finish8<GB>(rb[kt][i], n0 + bn, p.N, k0 + bk < p.K);
        }
    };
    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;
    using S2 = std::integral_constant<int, 2>;
    using S3 = std::integral_constant<int, 3>;

    int n0 = tile0 * T::BN;
    request(n0, S0 {});
    request(n0, S1 {});
    if constexpr (STEPS == 4) {
        request(n0, S2 {});
        request(n0, S3 {});
    }
    // the workgroup's rows, all of K: chunk q = tid + 256 i is chunk q % 16 of row q / 16
    {
        constexpr int NA = 128 * (STEPS * F16_BK / 8) / 256, CPR = STEPS * F16_BK / 8;
        req8_t<GA> ra[NA];
#pragma unroll
        for (int i = 0; i < NA; i++) {
            const int q = tid + 256 * i, ar = q / CPR, ak = (q % CPR) * 8;
            request8<GA>(ra[i], A + (int64_t)min(m0 + ar, p.M - 1) * p.lda, ak, p.K);
        }
#pragma unroll
        for (int i = 0; i < NA; i++) {
            const int q = tid + 256 * i, ar = q / CPR, ak = (q % CPR) * 8;
            *(uint4 *)(lds_a + ar * F16_WALK_APITCH + ak * 2)
                    = finish8<GA>(ra[i], ak, p.K, m0 + ar < p.M);
        }
    }
    stage(n0, S0 {});
    lds_barrier();

    v4f acc[T::MF][T::NF];
    const int alg = p.ep.npo ? p.ep.po[0].alg : -1;
    const float al = p.ep.po[0].alpha, be = p.ep.po[0].beta, sc = p.ep.po[0].scale;
    const bool dst_bf = p.ep.dst.dt == dt_bf16;
    const bool wide16 = (dst_bf || p.ep.dst.dt == dt_f16) && p.ep.dst.sn == 1;

    // one k-step: the next tile's weights for this k-step requested, the MFMAs,
    // the next step's weights staged, one barrier
    auto step = [&](bool more, auto KT) __attribute__((always_inline)) {
        constexpr int kt = decltype(KT)::value, buf = kt & 1;
        constexpr bool last = kt == STEPS - 1;
        if (more) request(n0 + T::BN, KT); // the slot's weights were staged a step ago
        v8s bf[T::NF];
#pragma unroll
        for (int nf = 0; nf < T::NF; nf++) {
            const uint8_t *vb = lds_b + buf * T::B_BYTES + (4 * c + (r >> 2)) * T::B_PITCH
                    + (T::WN * wcol + 16 * nf + 4 * (r & 3)) * 2;
            const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (v4s __attribute__((address_space(3))) *)vb);
            const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (v4s __attribute__((address_space(3))) *)(vb + 16 * T::B_PITCH));
            bf[nf] = v8s {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
#pragma unroll
        for (int mf = 0; mf < T::MF; mf++) {
            const uint8_t *pa = lds_a + (T::WM * wrow + 16 * mf + r) * F16_WALK_APITCH
                    + kt * (F16_BK * 2);
            const v4s x = *(const v4s *)(pa + (4 * c) * 2);
            const v4s y = *(const v4s *)(pa + (16 + 4 * c) * 2);
            const v8s af = {x[0], x[1], x[2], x[3], y[0], y[1], y[2], y[3]};
#pragma unroll
            for (int nf = 0; nf < T::NF; nf++)
                acc[mf][nf] = mma16<BF>(bf[nf], af,
                        kt == 0 ? v4f {0.f, 0.f, 0.f, 0.f} : acc[mf][nf]);
        }
        if constexpr (!last)
            stage(n0, std::integral_constant<int, kt + 1> {});
        else if (more)
            stage(n0 + T::BN, S0 {});
        lds_barrier();
    };

    for (int tile = 0; tile < ntile; tile++, n0 += T::BN) {
        const bool more = tile + 1 < ntile;
        step(more, S0 {});
        step(more, S1 {});
        if constexpr (STEPS == 4) {
            step(more, S2 {});
            step(more, S3 {});
        }
        // the wave's 64 x 64 results, 16 rows at a time through its own slice of
        // LDS: lane (r, c) holds dst[16 mf + r][16 nf + 4 c + i]; 16 lanes then
        // store a 64-column row piece
        // (a fragment row per call with a compile-time index: left as a loop over
        // mf the compiler kept it rolled and the accumulators in memory)
        auto store_rows = [&](auto MFI) __attribute__((always_inline)) {
            constexpr int mf = decltype(MFI)::value;
#pragma unroll
            for (int nf = 0; nf < T::NF; nf++)
                *(v4f *)(wout + r * F16_WALK_SPITCH + 16 * nf + 4 * c) = acc[mf][nf];
            // eight lanes a row, eight columns (16 bytes of a 16-bit dst) a lane:
            // what a CU stores per cycle depends on the bytes per instruction
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const int row = 8 * i + (lane >> 3), m = m0 + T::WM * wrow + 16 * mf + row;
                const int n8 = n0 + T::WN * wcol + (lane & 7) * 8;
                const v4f t0 = *(const v4f *)(wout + row * F16_WALK_SPITCH + (lane & 7) * 8);
                const v4f t1 = *(const v4f *)(wout + row * F16_WALK_SPITCH + (lane & 7) * 8 + 4);
                if (m < p.M && n8 < p.N) {
                    float v[8] = {t0[0], t0[1], t0[2], t0[3], t1[0], t1[1], t1[2], t1[3]};
                    if (alg >= 0) {
#pragma unroll
                        for (int j = 0; j < 8; j++) {
                            const float e = alg == alg_relu ? eltwise_one<alg_relu>(v[j], al, be)
                                    : alg == alg_linear     ? eltwise_one<alg_linear>(v[j], al, be)
                                    : alg == alg_clip       ? eltwise_one<alg_clip>(v[j], al, be)
                                                      : eltwise_one<alg_clip_v2>(v[j], al, be);
                            v[j] = e * sc;
                        }
                    }
                    const int64_t off = bz * p.ep.dst.sb + (int64_t)m * p.ep.dst.sm + n8;
                    if (wide16 && n8 + 8 <= p.N) {
                        uint16_t h[8];
                        bool nan = false;
#pragma unroll
                        for (int j = 0; j < 8; j++) nan = nan || v[j] != v[j];
                        if (dst_bf) {
#pragma unroll
                            for (int j = 0; j < 8; j++) h[j] = f32_to_bf16(v[j]);
                        } else if (nan) { // (the reference's conversion of a NaN keeps its payload)
#pragma unroll
                            for (int j = 0; j < 8; j++) h[j] = f32_to_f16(v[j]);
                        } else {
#pragma unroll
                            for (int j = 0; j < 8; j++) h[j] = f32_to_f16_hw(v[j]);
                        }
                        uint32_t w[4];
#pragma unroll
                        for (int j = 0; j < 4; j++)
                            w[j] = (uint32_t)h[2 * j] | ((uint32_t)h[2 * j + 1] << 16);
                        typedef unsigned v4u_any2 __attribute__((ext_vector_type(4), aligned(2)));
                        *(v4u_any2 *)((uint16_t *)p.ep.dst.ptr + off) = v4u_any2 {w[0], w[1], w[2], w[3]};
                    } else {
                        const float a4[4] = {v[0], v[1], v[2], v[3]}, b4[4] = {v[4], v[5], v[6], v[7]};
                        epilogue_store4(p.ep, a4, off, min(4, p.N - n8));
                        if (n8 + 4 < p.N) epilogue_store4(p.ep, b4, off + 4, min(4, p.N - n8 - 4));
                    }
                }
            }
        };
        static_assert(T::MF == 4, "");
        store_rows(S0 {});
        store_rows(S1 {});
        store_rows(S2 {});
        store_rows(S3 {});
    }
}

// ---- few rows per batch (M <= 4): the decode-time attention products ---------
// One token's scores (1 x 128 by 128 x keys) and context (1 x keys by
// keys x 128) per head are a few MB of weights read once; a 64 x 64 MFMA tile
// would leave most of the chip idle. Here a workgroup owns `cw` columns of one
// batch entry: `tpr` neighbouring lanes cover a weights row of the chunk (V
// elements each: one 16-byte load at any address, or one element for rows
// shorter than 32), the 256 / tpr lane groups take every
// (256 / tpr)-th k, requests run one unrolled block ahead of the arithmetic,
// the activations wait in LDS as f32, and the partial sums of the lane groups
// meet through lane permutes (within a wave) and LDS (across the four waves).
constexpr int GV_THREADS = 256;
constexpr int GV_MAX_ACT = 8192; // staged activation elements (rows x K)

template <bool BF>
QMM_D float up16(uint32_t h) {
    if constexpr (BF) return __builtin_bit_cast(float, h << 16);
    return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}

template <bool BF, int V, int MR>
__global__ void __launch_bounds__(GV_THREADS)
gemv_f16_kernel(const gemm16_params_t p, const int tpr_log2) {
    constexpr int U = V == 8 ? 8 : 16; // loads per lane and block
    // (16-byte loads at any address: rows of any length and alignment)
    typedef typename std::conditional<V == 8, v4u_any, uint16_t>::type wv_t;
    extern __shared__ __attribute__((aligned(16))) float gv_lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int tpr = 1 << tpr_log2, cw = tpr * V, rpp = GV_THREADS >> tpr_log2;
    const int col_l = (tid & (tpr - 1)) * V, phase = tid >> tpr_log2;
    // V = 8: the last chunk moves back inside the row (N >= cw, the host
    // checks), recomputing a few columns of its neighbour with the same result
    const int n0 = V == 8 ? min((int)blockIdx.x * cw, p.N - cw) : blockIdx.x * cw;
    const int n = n0 + col_l;
    const int64_t bz = blockIdx.y;
    const int K = p.K;
    float *qtab = gv_lds; // [MR][K]
    float *red = gv_lds + MR * K; // [4][MR][cw]
    const uint16_t *wcol = p.B + bz * p.b_sb + (n < p.N ? n : 0);

    auto request = [&](wv_t (&w)[U], int kb) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int k = min(kb + u * rpp + phase, K - 1);
            w[u] = *(const wv_t *)(wcol + (int64_t)k * p.ldb);
        }
    };
    wv_t wc[U], wn[U];
    request(wc, 0);

    // activations -> f32 table; rows past M stay zero
    const uint16_t *A = p.A + bz * p.a_sb;
#pragma unroll
    for (int m = 0; m < MR; m++) {
        const bool row_ok = m < p.M;
        const uint16_t *arow = A + (int64_t)(row_ok ? m : 0) * p.lda;
        for (int k0 = 0; k0 < K; k0 += 4 * GV_THREADS) {
            uint16_t t[4];
#pragma unroll
            for (int j = 0; j < 4; j++)
                t[j] = arow[min(k0 + j * GV_THREADS + tid, K - 1)];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int k = k0 + j * GV_THREADS + tid;
                if (k < K) qtab[m * K + k] = row_ok ? up16<BF>(t[j]) : 0.f;
            }
        }
    }
    __syncthreads();

    float acc[MR][V];
#pragma unroll
    for (int m = 0; m < MR; m++)
#pragma unroll
        for (int i = 0; i < V; i++) acc[m][i] = 0.f;

    const int block = U * rpp;
    for (int kb = 0; kb < K; kb += block) {
        request(wn, min(kb + block, K - 1)); // clamped: past K it re-reads the last row
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int k = kb + u * rpp + phase;
            const bool ok = k < K;
            float q[MR];
#pragma unroll
            for (int m = 0; m < MR; m++) q[m] = ok ? qtab[m * K + min(k, K - 1)] : 0.f;
            float wf[V];
            if constexpr (V == 8) {
                const uint32_t d[4] = {wc[u][0], wc[u][1], wc[u][2], wc[u][3]};
#pragma unroll
                for (int i = 0; i < 8; i++)
                    wf[i] = up16<BF>((d[i / 2] >> (16 * (i % 2))) & 0xffffu);
            } else {
                wf[0] = up16<BF>(wc[u]);
            }
#pragma unroll
            for (int i = 0; i < V; i++) {
                const float w = ok ? wf[i] : 0.f; // a clamped re-read counts as zero
#pragma unroll
                for (int m = 0; m < MR; m++) acc[m][i] = fmaf(q[m], w, acc[m][i]);
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) wc[u] = wn[u];
    }

    // lanes l, l + tpr, l + 2 tpr ... of a wave hold the same columns
    for (int s = tpr; s < 64; s <<= 1) {
#pragma unroll
        for (int m = 0; m < MR; m++)
#pragma unroll
            for (int i = 0; i < V; i++) acc[m][i] += __shfl_xor(acc[m][i], s);
    }
    if (lane < tpr) {
#pragma unroll
        for (int m = 0; m < MR; m++)
#pragma unroll
            for (int i = 0; i < V; i++)
                red[(wave * MR + m) * cw + col_l + i] = acc[m][i];
    }
    __syncthreads();
    // A workgroup stores only the columns from blockIdx.x * cw on: where the
    // load window moved back, the columns in front of that belong to the
    // neighbour, and an epilogue that reads dst (sum) must see each element once.
    const int quads = cw >> 2;
    if (tid < MR * quads) {
        const int m = tid / quads, c4 = (tid - m * quads) * 4;
        const int own0 = blockIdx.x * cw, shift = own0 - n0;
        const int nn = own0 + c4;
        if (m < p.M && nn < p.N) {
            float v[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                float t = 0.f;
                const int c = min(shift + c4 + i, cw - 1);
#pragma unroll
                for (int w = 0; w < 4; w++) t += red[(w * MR + m) * cw + c];
                v[i] = t;
            }
            epilogue_apply_store4(p.ep, v, bz, m, nn, min(4, p.N - nn));
        }
    }
}

template <bool BF, int V, int MR>
void launch_gemv_f16_as(const gemm16_params_t &p, int tpr_log2, hipStream_t stream) {
    const int cw = (1 << tpr_log2) * V;
    const size_t lds = sizeof(float) * ((size_t)MR * p.K + 4 * MR * cw);
    hipLaunchKernelGGL((gemv_f16_kernel<BF, V, MR>),
            dim3((unsigned)((p.N + cw - 1) / cw), (unsigned)p.batch),
            dim3(GV_THREADS), lds, stream, p, tpr_log2);
}

} // namespace

void launch_gemm_f16(const gemm16_params_t &p, hipStream_t stream) {
    if (p.M <= 0 || p.N <= 0 || p.batch <= 0) return;
    const int mr = p.M == 1 ? 1 : 4;
    if (p.M <= 4 && (int64_t)mr * p.K <= GV_MAX_ACT) {
        // 16-byte loads (8 columns a lane) wherever a 32-column chunk fits the row
        const bool vec = p.N >= 32;
        int tpr_log2 = 6; // one element per lane: 64 columns per workgroup
        if (vec) {
            // the widest chunk (32 .. 256 columns) that still gives 256 workgroups
            tpr_log2 = 5;
            while (tpr_log2 > 2
                    && ((int64_t)p.batch * ((p.N + (8 << tpr_log2) - 1) >> (tpr_log2 + 3)) < 256
                            || (8 << tpr_log2) > p.N))
                tpr_log2--;
        }
        auto go = [&](auto bf, auto v) {
            if (mr == 1)
                launch_gemv_f16_as<decltype(bf)::value, decltype(v)::value, 1>(
                        p, tpr_log2, stream);
            else
                launch_gemv_f16_as<decltype(bf)::value, decltype(v)::value, 4>(
                        p, tpr_log2, stream);
        };
        auto by_bf = [&](auto v) {
            if (p.bf) go(std::true_type {}, v);
            else go(std::false_type {}, v);
        };
        if (vec) by_bf(std::integral_constant<int, 8> {});
        else by_bf(std::integral_constant<int, 1> {});
        return;
    }
    // aligned 16-byte loads where rows start on 16-byte boundaries and hold a
    // multiple of 8 elements, else unaligned ones (rows of 8 elements and
    // more), else element loads
    auto pick = [](int g, int len) { return g >= 8 && len % 8 == 0 ? 8 : len >= 8 ? 0 : 1; };
    int ga = pick(p.a_vec, p.K), gb = pick(p.b_vec, p.N);
    const bool light = light_epilogue(p.ep) && p.ep.dst.sn == 1;
    // the interpreter form exists three times: aligned, any alignment, short rows
    if (!light && !(ga == 8 && gb == 8)) ga = gb = (ga != 1 && gb != 1) ? 0 : 1;
    // 128 x 128 tiles once they give every CU a workgroup (the small tile's four
    // times as many workgroups spread better below that) and K is long enough
    // for the main loop to matter: 4096^3 421 -> 241 us, 32 x (2048 x 2048 x 128)
    // 137 -> 80 us; with K = 128 (attention scores) a launch is its dst stream
    // and the small tile's higher occupancy wins (998: 52 against 74 us). Not
    // for the element-load forms.
    const int64_t big_tiles = (int64_t)((p.M + 127) / 128) * ((p.N + 127) / 128) * p.batch;
    const bool big = p.tile != 1 && ga != 1 && gb != 1 && p.M > 64 && p.N > 64
            && (p.tile == 2 || (big_tiles >= 256 && p.K >= 256));
    // short K over many column tiles with a light epilogue: the walking kernel,
    // with the column tiles of a row block cut into as few segments as give
    // every CU two workgroups
    const int gx128 = (p.N + 127) / 128, gy128 = (p.M + 127) / 128;
    // (by default only where a lane's eight results make one aligned 16-byte
    // store: rows of a 16-bit dst that start on 16-byte boundaries; with rows of
    // 998 elements the wide stores split and the kernel is no faster than the
    // 64 x 64 tiles, 47.7 against 46.4 us)
    const bool dst16 = (p.ep.dst.dt == dt_f16 || p.ep.dst.dt == dt_bf16) && p.ep.dst.sm % 8 == 0
            && p.ep.dst.sb % 8 == 0 && (uintptr_t)p.ep.dst.ptr % 16 == 0;
    const bool walk = p.tile != 1
            && ((p.tile == 3 && p.K <= F16_WALK_K)
                    || (p.tile == 0 && p.K <= F16_WALK_K && gx128 >= 4
                            && (int64_t)gy128 * p.batch >= 64 && dst16))
            && light && ga != 1 && gb != 1 && p.M > 64;
    if (walk) {
        int nseg = 1;
        while ((int64_t)gy128 * p.batch * nseg < 512 && nseg * 2 <= gx128 / 2) nseg *= 2;
        const dim3 grid((unsigned)(gy128 * p.batch * nseg));
        auto gow = [&](auto bf, auto a, auto b) {
            auto launch = [&](auto st) {
                auto kern = gemm_f16_walk_kernel<decltype(bf)::value, decltype(a)::value,
                        decltype(b)::value, decltype(st)::value>;
                ensure_dynamic_lds((const void *)kern, F16_WALK_LDS);
                hipLaunchKernelGGL(kern, grid, dim3(256), F16_WALK_LDS, stream, p, nseg);
            };
            if (p.K <= 64) launch(std::integral_constant<int, 2> {});
            else launch(std::integral_constant<int, 4> {});
        };
        using W8 = std::integral_constant<int, 8>;
        using W0 = std::integral_constant<int, 0>;
        auto by_bfw = [&](auto a, auto b) {
            if (p.bf) gow(std::true_type {}, a, b);
            else gow(std::false_type {}, a, b);
        };
        if (ga == 8 && gb == 8) by_bfw(W8 {}, W8 {});
        else if (ga == 8) by_bfw(W8 {}, W0 {});
        else if (gb == 8) by_bfw(W0 {}, W8 {});
        else by_bfw(W0 {}, W0 {});
        return;
    }
    auto go = [&](auto bf, auto lt, auto a, auto b) {
        if (big) {
            const dim3 grid((unsigned)(((p.N + 127) / 128) * ((p.M + 127) / 128) * p.batch));
            if constexpr (decltype(a)::value != 1 && decltype(b)::value != 1)
                hipLaunchKernelGGL((gemm_f16_kernel<decltype(bf)::value, decltype(lt)::value,
                                           decltype(a)::value, decltype(b)::value, f16_big_t>),
                        grid, dim3(256), 0, stream, p);
        } else {
            const dim3 grid((unsigned)(((p.N + 63) / 64) * ((p.M + 63) / 64) * p.batch));
            hipLaunchKernelGGL((gemm_f16_kernel<decltype(bf)::value, decltype(lt)::value,
                                       decltype(a)::value, decltype(b)::value, f16_small_t>),
                    grid, dim3(256), 0, stream, p);
        }
    };
    auto by_bf = [&](auto lt, auto a, auto b) {
        if (p.bf) go(std::true_type {}, lt, a, b);
        else go(std::false_type {}, lt, a, b);
    };
    using I8 = std::integral_constant<int, 8>;
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    if (!light) {
        if (ga == 8) by_bf(std::false_type {}, I8 {}, I8 {});
        else if (ga == 0) by_bf(std::false_type {}, I0 {}, I0 {});
        else by_bf(std::false_type {}, I1 {}, I1 {});
        return;
    }
    auto by_b = [&](auto a) {
        if (gb == 8) by_bf(std::true_type {}, a, I8 {});
        else if (gb == 0) by_bf(std::true_type {}, a, I0 {});
        else by_bf(std::true_type {}, a, I1 {});
    };
    if (ga == 8) by_b(I8 {});
    else if (ga == 0) by_b(I0 {});
    else by_b(I1 {});
}

} // namespace qmm
