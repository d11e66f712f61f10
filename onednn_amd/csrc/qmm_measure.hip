// Measurement aid: a kernel that only reads. It pulls up to three byte ranges
// through 16-byte vector loads with the launch shape of the decode kernel
// (256 workgroups of 512 lanes) and stores one word per wave, so that a timing
// harness can put a read-only floor next to a memory-bound kernel's figure.
#include <hip/hip_runtime.h>
#include <stdint.h>

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
