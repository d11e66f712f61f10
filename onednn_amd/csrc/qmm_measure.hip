// Measurement aids. (1) A kernel that only reads. It pulls up to three byte ranges
// through 16-byte vector loads with the launch shape of the decode kernel
// (256 workgroups of 512 lanes) and stores one word per wave, so that a timing
// harness can put a read-only floor next to a memory-bound kernel's figure.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "qmm_hip.h"

namespace {

struct read_seg_t {
    const uint4 *p[3];
    uint32_t n16[3]; // 16-byte words
};

__device__ inline void fold(uint4 &acc, const uint4 &v, bool keep) {
    const uint32_t m = keep ? 0xFFFFFFFFu : 0u;
    acc.x ^= v.x & m;
    acc.y ^= v.y & m;
    acc.z ^= v.z & m;
    acc.w ^= v.w & m;
}

// Each workgroup reads one contiguous slab of every range, as the decode
// kernel reads the weights, scales and zero points of its columns. The first
// four loads of range 0 and the first load of ranges 1 and 2 are issued
// back to back before any is consumed (indices past a slab's end are clamped
// and their data dropped, so that no load waits on a branch); what a slab
// holds beyond that is read by the loops that follow.
__global__ __launch_bounds__(512) void stream_read_kernel(
        read_seg_t s, uint32_t *sink) {
    uint32_t lo[3], hi[3];
#pragma unroll
    for (int g = 0; g < 3; g++) {
        const uint32_t n = s.n16[g];
        const uint32_t slab = (n + gridDim.x - 1) / gridDim.x;
        lo[g] = blockIdx.x * slab < n ? blockIdx.x * slab : n;
        hi[g] = lo[g] + slab < n ? lo[g] + slab : n;
    }
    const uint32_t t = threadIdx.x;
    uint4 v0[4], v1, v2;
    const bool any0 = hi[0] > lo[0], any1 = hi[1] > lo[1], any2 = hi[2] > lo[2];
#pragma unroll
    for (int u = 0; u < 4; u++) {
        const uint32_t j = lo[0] + t + u * 512;
        if (any0) v0[u] = s.p[0][j < hi[0] ? j : hi[0] - 1];
    }
    if (any1) v1 = s.p[1][lo[1] + t < hi[1] ? lo[1] + t : hi[1] - 1];
    if (any2) v2 = s.p[2][lo[2] + t < hi[2] ? lo[2] + t : hi[2] - 1];
    uint4 acc = {0, 0, 0, 0};
#pragma unroll
    for (int u = 0; u < 4; u++)
        if (any0) fold(acc, v0[u], lo[0] + t + u * 512 < hi[0]);
    if (any1) fold(acc, v1, lo[1] + t < hi[1]);
    if (any2) fold(acc, v2, lo[2] + t < hi[2]);
    for (uint32_t i = lo[0] + t + 4 * 512; i < hi[0]; i += 512)
        fold(acc, s.p[0][i], true);
    for (uint32_t i = lo[1] + t + 512; i < hi[1]; i += 512)
        fold(acc, s.p[1][i], true);
    for (uint32_t i = lo[2] + t + 512; i < hi[2]; i += 512)
        fold(acc, s.p[2][i], true);
    uint32_t v = acc.x ^ acc.y ^ acc.z ^ acc.w;
#pragma unroll
    for (int o = 32; o; o >>= 1) v ^= __shfl_xor(v, o);
    if ((t & 63) == 0) sink[(blockIdx.x * 512u + t) >> 6] = v;
}

} // namespace

extern "C" int qmm_stream_read(const void *p0, size_t n0, const void *p1,
        size_t n1, const void *p2, size_t n2, void *sink, void *stream) {
    const void *ps[3] = {p0, p1, p2};
    const size_t ns[3] = {n0, n1, n2};
    read_seg_t s;
    for (int g = 0; g < 3; g++) {
        if (ns[g] && (!ps[g] || ((uintptr_t)ps[g] & 15) || (ns[g] >> 35)))
            return QMM_INVALID_ARGUMENTS;
        s.p[g] = (const uint4 *)ps[g];
        s.n16[g] = (uint32_t)(ns[g] / 16);
    }
    if (!sink) return QMM_INVALID_ARGUMENTS;
    hipLaunchKernelGGL(stream_read_kernel, dim3(QMM_STREAM_READ_GROUPS),
            dim3(512), 0, (hipStream_t)stream, s, (uint32_t *)sink);
    return hipGetLastError() == hipSuccess ? QMM_OK : QMM_RUNTIME_ERROR;
}

// (3) below: a kernel that only writes (the ceiling of a launch bound by its
// destination stream).
// (2) Matrix-core ceiling: a kernel that issues nothing but the MFMAs of the
// 256 x 256 GEMM kernels' main loop -- one wave per SIMD, 256 accumulator
// registers, 8 + 8 operand fragments held in registers and filled with
// pseudo-random bytes, two operand sets alternating per k-step as the double
// buffering of the real loop does -- with no LDS, no global memory and no
// barrier in the loop. What it sustains is what the matrix cores deliver on
// data that toggles like real operands at the clock the card settles at under
// that load: the practical ceiling a full kernel is measured against.
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

__device__ inline uint32_t mix32(uint32_t x) {
    x ^= x >> 16;
    x *= 0x7feb352du;
    x ^= x >> 15;
    x *= 0x846ca68bu;
    x ^= x >> 16;
    return x;
}
// e4m3: keep every byte away from the NaN codes 0x7f / 0xff
__device__ inline uint32_t no_nan_e4m3(uint32_t w) {
    const uint32_t m = w & 0x7f7f7f7fu;
    const uint32_t is7f = ((m + 0x01010101u) >> 7) & 0x01010101u; // byte == 0x7f
    return w ^ is7f;
}

// two standard normal deviates from two 32-bit words (Box-Muller)
__device__ inline void normal2(uint32_t u, uint32_t v, float &x, float &y) {
    const float a = ((u >> 8) + 1) * (1.f / 16777216.f); // (0, 1]
    const float r = __builtin_sqrtf(-2.f * __logf(a));
    const float t = (v >> 8) * (6.28318530718f / 16777216.f);
    x = r * __cosf(t);
    y = r * __sinf(t);
}
// One operand dword (four k values) of the benchmark configurations' data:
// int8 A: clip(round(N(0,1) * 32), +-127); int8 B: uniform in [-127, 127];
// fp8 (both operands): e4m3 of clip(N(0,1) * 4, +-448).
__device__ inline uint32_t config_dword(bool f8, bool is_b, uint32_t h) {
    const uint32_t h2 = mix32(h ^ 0x68bc21ebu), h3 = mix32(h + 0x02e5be93u),
                   h4 = mix32(h ^ 0x1b56c4e9u);
    if (!f8 && is_b) {
        uint32_t w = 0;
        for (int i = 0; i < 4; i++) {
            const int v = (int)((mix32(h + i) >> 8) % 255u) - 127;
            w |= (uint32_t)(v & 0xff) << (8 * i);
        }
        return w;
    }
    float g[4];
    normal2(h, h2, g[0], g[1]);
    normal2(h3, h4, g[2], g[3]);
    if (f8) {
        for (int i = 0; i < 4; i++)
            g[i] = fminf(fmaxf(g[i] * 4.f, -448.f), 448.f);
        int w = __builtin_amdgcn_cvt_pk_fp8_f32(g[0], g[1], 0, false);
        w = __builtin_amdgcn_cvt_pk_fp8_f32(g[2], g[3], w, true);
        return (uint32_t)w;
    }
    uint32_t w = 0;
    for (int i = 0; i < 4; i++) {
        const int v = (int)fminf(fmaxf(__builtin_rintf(g[i] * 32.f), -127.f), 127.f);
        w |= (uint32_t)(v & 0xff) << (8 * i);
    }
    return w;
}

// KIND 0: v_mfma_i32_16x16x64_i8, 1: v_mfma_i32_32x32x32_i8,
//      2: v_mfma_f32_16x16x128_f8f6f4, 3: v_mfma_f32_32x32x64_f8f6f4 (e4m3).
// data 0: uniformly random bytes; 1: all-zero operands (what the same loop
// reaches when nothing toggles); 2: the distributions of the benchmark
// configurations (config_dword).
// KIND 4: KIND 0 (int8 16 x 16 x 64) walking the fragment grid column by column:
// eight consecutive MFMAs keep the weights fragment and change the source
// fragment, where KIND 0 keeps the source fragment and changes the weights.
template <int KIND0>
__global__ void __launch_bounds__(256, 1)
mfma_ceiling_kernel(uint32_t seed, int ksteps, int data, uint32_t *sink) {
    constexpr int KIND = KIND0 == 4 ? 0 : KIND0;
    constexpr bool BY_COLUMN = KIND0 == 4;
    constexpr bool F8 = KIND >= 2;
    constexpr bool SMALL = KIND == 0 || KIND == 2; // 16 x 16 fragments
    constexpr int NF = SMALL ? 8 : 4; // fragment grid NF x NF
    constexpr int OPW = F8 ? 8 : 4; // dwords of one operand
    constexpr int ACCW = SMALL ? 4 : 16;
    typedef typename std::conditional<F8, v8i, v4i>::type op_t;
    typedef typename std::conditional<F8,
            typename std::conditional<SMALL, v4f, v16f>::type,
            typename std::conditional<SMALL, v4i, v16i>::type>::type acc_t;
    const uint32_t gid = blockIdx.x * 256u + threadIdx.x;
    op_t fa[2][NF], fb[2][NF];
#pragma unroll 1
    for (int s = 0; s < 2; s++)
#pragma unroll
        for (int i = 0; i < NF; i++)
#pragma unroll
            for (int w = 0; w < OPW; w++) {
                const uint32_t ha = mix32(seed ^ (gid * 977u + (s * NF + i) * 64u + w));
                const uint32_t hb = mix32(~seed ^ (gid * 1031u + (s * NF + i) * 64u + w + 32u));
                uint32_t a = ha, b = hb;
                if (data == 2) a = config_dword(F8, false, ha), b = config_dword(F8, true, hb);
                if (F8) a = no_nan_e4m3(a), b = no_nan_e4m3(b);
                if (data == 1) a = b = 0;
                // (the operand arrays are indexed with constants only)
                if (s == 0) fa[0][i][w] = (int)a, fb[0][i][w] = (int)b;
                else fa[1][i][w] = (int)a, fb[1][i][w] = (int)b;
            }
    acc_t acc[NF][NF];
#pragma unroll
    for (int i = 0; i < NF; i++)
#pragma unroll
        for (int j = 0; j < NF; j++)
#pragma unroll
            for (int r = 0; r < ACCW; r++) acc[i][j][r] = 0;
    for (int k = 0; k < ksteps; k += 2) {
#pragma unroll
        for (int s = 0; s < 2; s++)
#pragma unroll
            for (int i0 = 0; i0 < NF; i0++)
#pragma unroll
                for (int j0 = 0; j0 < NF; j0++) {
                    const int i = BY_COLUMN ? j0 : i0, j = BY_COLUMN ? i0 : j0;
                    if constexpr (KIND == 0)
                        // accumulators pinned to the accumulator file: with the
                        // builtin the allocator moves part of them through
                        // vector registers inside the loop
                        asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0"
                                     : "+a"(acc[i][j])
                                     : "v"(fb[s][j]), "v"(fa[s][i]));
                    else if constexpr (KIND == 1)
                        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
                                fa[s][i], fb[s][j], acc[i][j], 0, 0, 0);
                    else if constexpr (KIND == 2)
                        // as in the GEMM kernel, only fragments 0..3 have a
                        // second register set (8-dword operands: two full sets
                        // do not fit next to 256 accumulators)
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                                fb[j < 4 ? s : 0][j], fa[i < 4 ? s : 0][i],
                                acc[i][j], 0, 0, 0, 0, 0, 0);
                    else
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                                fa[s][i], fb[s][j], acc[i][j], 0, 0, 0, 0, 0, 0);
                }
    }
    uint32_t v = 0;
#pragma unroll
    for (int i = 0; i < NF; i++)
#pragma unroll
        for (int j = 0; j < NF; j++)
#pragma unroll
            for (int r = 0; r < ACCW; r++)
                v += __builtin_bit_cast(uint32_t, acc[i][j][r]);
    sink[gid] = v;
}

} // namespace

extern "C" int qmm_mfma_ceiling(int kind, int ksteps, int groups, int data,
        void *sink, void *stream, double *ops_per_launch) {
    if (kind < 0 || kind > 4 || data < 0 || data > 2 || ksteps < 2 || (ksteps & 1) || groups < 1 || !sink)
        return QMM_INVALID_ARGUMENTS;
    // operations of one k-step of one wave: the fragment grid covers 128 x 128
    // outputs; a k-step contracts 64 k (int8, fp8 32 x 32 x 64) or 128 k
    const double kdepth = kind == 2 ? 128.0 : (kind == 1 ? 32.0 : 64.0);
    if (ops_per_launch)
        *ops_per_launch = 2.0 * 128 * 128 * kdepth * ksteps * 4.0 * groups;
    const dim3 g(groups), b(256);
    hipStream_t st = (hipStream_t)stream;
    uint32_t *out = (uint32_t *)sink;
    switch (kind) {
        case 0: hipLaunchKernelGGL(mfma_ceiling_kernel<0>, g, b, 0, st, 0x9e3779b9u, ksteps, data, out); break;
        case 1: hipLaunchKernelGGL(mfma_ceiling_kernel<1>, g, b, 0, st, 0x9e3779b9u, ksteps, data, out); break;
        case 2: hipLaunchKernelGGL(mfma_ceiling_kernel<2>, g, b, 0, st, 0x9e3779b9u, ksteps, data, out); break;
        case 3: hipLaunchKernelGGL(mfma_ceiling_kernel<3>, g, b, 0, st, 0x9e3779b9u, ksteps, data, out); break;
        default: hipLaunchKernelGGL(mfma_ceiling_kernel<4>, g, b, 0, st, 0x9e3779b9u, ksteps, data, out); break;
    }
    return hipGetLastError() == hipSuccess ? QMM_OK : QMM_RUNTIME_ERROR;
}

// (3) A kernel that only writes: every lane stores 16-byte vectors with a
// grid-stride loop, rows of a workgroup contiguous, as an epilogue that streams
// a large destination does.
namespace {
__global__ void __launch_bounds__(256) stream_write_kernel(
        uint4 *dst, size_t n16, uint32_t seed) {
    const size_t stride = (size_t)gridDim.x * 256;
    uint4 v = {seed, seed ^ threadIdx.x, seed + blockIdx.x, ~seed};
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += stride) {
        dst[i] = v;
        v.x += 0x9e3779b9u;
    }
}
__global__ void __launch_bounds__(256) stream_copy_kernel(
        uint4 *dst, const uint4 *src, size_t n16) {
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += stride)
        dst[i] = src[i];
}
} // namespace

extern "C" int qmm_stream_copy(void *dst, const void *src, size_t bytes,
        int groups, void *stream) {
    if (!dst || !src || (((uintptr_t)dst | (uintptr_t)src) & 15) || groups < 1)
        return QMM_INVALID_ARGUMENTS;
    hipLaunchKernelGGL(stream_copy_kernel, dim3(groups), dim3(256), 0,
            (hipStream_t)stream, (uint4 *)dst, (const uint4 *)src, bytes / 16);
    return hipGetLastError() == hipSuccess ? QMM_OK : QMM_RUNTIME_ERROR;
}

extern "C" int qmm_stream_write(void *dst, size_t bytes, int groups, void *stream) {
    if (!dst || ((uintptr_t)dst & 15) || groups < 1) return QMM_INVALID_ARGUMENTS;
    hipLaunchKernelGGL(stream_write_kernel, dim3(groups), dim3(256), 0,
            (hipStream_t)stream, (uint4 *)dst, bytes / 16, 0x12345u);
    return hipGetLastError() == hipSuccess ? QMM_OK : QMM_RUNTIME_ERROR;
}
