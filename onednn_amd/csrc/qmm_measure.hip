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

__global__ __launch_bounds__(512) void stream_read_kernel(
        read_seg_t s, uint32_t *sink) {
    const uint32_t t = blockIdx.x * 512u + threadIdx.x;
    const uint32_t stride = gridDim.x * 512u;
    uint4 acc = {0, 0, 0, 0};
#pragma unroll
    for (int g = 0; g < 3; g++) {
        const uint4 *p = s.p[g];
        const uint32_t n = s.n16[g];
        uint32_t i = t;
        // four loads in flight per lane
        for (; i + 3 * stride < n; i += 4 * stride) {
            const uint4 a = p[i];
            const uint4 b = p[i + stride];
            const uint4 c = p[i + 2 * stride];
            const uint4 d = p[i + 3 * stride];
            acc.x ^= a.x ^ b.x ^ c.x ^ d.x;
            acc.y ^= a.y ^ b.y ^ c.y ^ d.y;
            acc.z ^= a.z ^ b.z ^ c.z ^ d.z;
            acc.w ^= a.w ^ b.w ^ c.w ^ d.w;
        }
        for (; i < n; i += stride) {
            const uint4 a = p[i];
            acc.x ^= a.x;
            acc.y ^= a.y;
            acc.z ^= a.z;
            acc.w ^= a.w;
        }
    }
    uint32_t v = acc.x ^ acc.y ^ acc.z ^ acc.w;
#pragma unroll
    for (int o = 32; o; o >>= 1) v ^= __shfl_xor(v, o);
    if ((threadIdx.x & 63) == 0) sink[t >> 6] = v;
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
