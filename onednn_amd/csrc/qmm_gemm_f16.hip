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

namespace qmm {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef short v4s __attribute__((ext_vector_type(4)));
typedef short v8s __attribute__((ext_vector_type(8)));

constexpr int F16_BM = 64, F16_BN = 64, F16_BK = 32;
constexpr int F16_A_PITCH = F16_BK * 2 + 16; // bytes of a staged source row
constexpr int F16_B_PITCH = F16_BN * 2 + 16; // bytes of a staged weights row

template <bool BF>
QMM_D v4f mma16(const v8s &a, const v8s &b, const v4f &c) {
    if constexpr (BF)
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                __builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(
                __builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
}

// eight neighbouring 16-bit elements p[0..7] of a row of `len` elements
// starting at element `at`: one 16-byte load where the row allows it, else
// element by element; elements at or past `len` (or a row that is not there)
// read as zero
QMM_D uint4 load8(const uint16_t *row, int64_t at, int64_t len, bool row_ok,
        bool vec) {
    if (row_ok && vec && at + 8 <= len) return *(const uint4 *)(row + at);
    uint32_t w[4] = {0, 0, 0, 0};
    if (row_ok) {
#pragma unroll
        for (int i = 0; i < 8; i++)
            if (at + i < len) w[i / 2] |= (uint32_t)row[at + i] << (16 * (i % 2));
    }
    return make_uint4(w[0], w[1], w[2], w[3]);
}

template <bool BF>
__global__ void __launch_bounds__(256)
gemm_f16_kernel(const gemm16_params_t p) {
    __shared__ __attribute__((aligned(16))) uint8_t lds_a[2][F16_BM * F16_A_PITCH];
    __shared__ __attribute__((aligned(16))) uint8_t lds_b[2][F16_BK * F16_B_PITCH];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, c = lane >> 4;
    const int m0 = blockIdx.y * F16_BM, n0 = blockIdx.x * F16_BN;
    const int64_t bz = blockIdx.z;
    const uint16_t *A = p.A + bz * p.a_sb, *B = p.B + bz * p.b_sb;
    // staging: thread t copies chunk (t % 4) of source row t / 4, and chunk
    // (t % 8) of weights row t / 8 of the step (8 elements each)
    const int ar = tid >> 2, ak = (tid & 3) * 8;
    const int bk = tid >> 3, bn = (tid & 7) * 8;
    const bool a_row_ok = m0 + ar < p.M;
    const uint16_t *a_row = A + (int64_t)min(m0 + ar, p.M - 1) * p.lda;
    const bool b_cols_ok = n0 + bn < p.N;
    const int steps = (p.K + F16_BK - 1) / F16_BK;

    uint4 ra, rb;
    auto request = [&](int kt) {
        const int k0 = kt * F16_BK;
        ra = load8(a_row, k0 + ak, p.K, a_row_ok, p.a_vec != 0);
        const bool b_row_ok = k0 + bk < p.K && b_cols_ok;
        rb = load8(B + (int64_t)min(k0 + bk, p.K - 1) * p.ldb, n0 + bn, p.N,
                b_row_ok, p.b_vec != 0);
    };
    auto stage = [&](int buf) {
        *(uint4 *)(lds_a[buf] + ar * F16_A_PITCH + ak * 2) = ra;
        *(uint4 *)(lds_b[buf] + bk * F16_B_PITCH + bn * 2) = rb;
    };

    v4f acc[4];
#pragma unroll
    for (int mf = 0; mf < 4; mf++) acc[mf] = v4f {0.f, 0.f, 0.f, 0.f};

    request(0);
    stage(0);
    __syncthreads();
    for (int kt = 0; kt < steps; kt++) {
        const int buf = kt & 1;
        if (kt + 1 < steps) request(kt + 1);
        // weights fragment of the wave's 16 columns, transposed out of LDS
        const uint8_t *vb = lds_b[buf] + (4 * c + (r >> 2)) * F16_B_PITCH
                + (16 * wave + 4 * (r & 3)) * 2;
        const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (v4s __attribute__((address_space(3))) *)vb);
        const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (v4s __attribute__((address_space(3))) *)(vb + 16 * F16_B_PITCH));
        const v8s bf = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
#pragma unroll
        for (int mf = 0; mf < 4; mf++) {
            // source fragment: row 16 mf + r, the same eight k
            const uint8_t *pa = lds_a[buf] + (16 * mf + r) * F16_A_PITCH;
            const v4s x = *(const v4s *)(pa + (4 * c) * 2);
            const v4s y = *(const v4s *)(pa + (16 + 4 * c) * 2);
            const v8s af = {x[0], x[1], x[2], x[3], y[0], y[1], y[2], y[3]};
            acc[mf] = mma16<BF>(bf, af, acc[mf]);
        }
        if (kt + 1 < steps) stage(buf ^ 1);
        __syncthreads();
    }

    // register i of lane (r, c): dst[m0 + 16 mf + r][n0 + 16 wave + 4 c + i]
    const int n = n0 + 16 * wave + 4 * c;
#pragma unroll
    for (int mf = 0; mf < 4; mf++) {
        const int m = m0 + 16 * mf + r;
        if (m < p.M && n < p.N) {
            float v[4] = {acc[mf][0], acc[mf][1], acc[mf][2], acc[mf][3]};
            epilogue_apply_store4(p.ep, v, bz, m, n, min(4, p.N - n));
        }
    }
}

} // namespace

void launch_gemm_f16(const gemm16_params_t &p, hipStream_t stream) {
    if (p.M <= 0 || p.N <= 0 || p.batch <= 0) return;
    const dim3 grid((unsigned)((p.N + F16_BN - 1) / F16_BN),
            (unsigned)((p.M + F16_BM - 1) / F16_BM), (unsigned)p.batch);
    if (p.bf)
        hipLaunchKernelGGL(gemm_f16_kernel<true>, grid, dim3(256), 0, stream, p);
    else
        hipLaunchKernelGGL(gemm_f16_kernel<false>, grid, dim3(256), 0, stream, p);
}

} // namespace qmm
