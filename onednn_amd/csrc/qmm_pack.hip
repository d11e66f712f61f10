// Weights prepacking: plain strided tensors -> the MFMA operand layouts
// (QMM_LAYOUT_MFMA_B8 with s32 column sums, QMM_LAYOUT_MFMA_W4,
// QMM_LAYOUT_MFMA_W4K64) and back.
// This is the reorder a user runs once per weights tensor after asking the
// matmul primitive descriptor for its weights layout through format_tag any
// (the role of src/cpu/x64/matmul/brgemm_matmul_reorders.cpp:29-53 in the
// reference). Values are copied bit for bit (u4 in the W4K64 layout: minus 8,
// undone on the way back); padding is zero.
#include "qmm_device.hpp"
#include "qmm_plan.hpp"

namespace qmm {

struct pack_params_t {
    const uint8_t *src;
    uint8_t *dst;
    int64_t batch, K, N;
    int64_t sb, sk, sn; // plain side strides, elements
    int32_t dt;
    int32_t pad_;
};

// one thread per 16-byte chunk of the packed tensor
__global__ void __launch_bounds__(256)
pack_b8_kernel(const pack_params_t p, const b8_geom_t g) {
    const int64_t chunks = p.batch * g.batch_bytes / 16;
    for (int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; c < chunks;
            c += (int64_t)gridDim.x * blockDim.x) {
        const int64_t per_b = g.batch_bytes / 16;
        const int64_t b = c / per_b, cb = c % per_b;
        const int lane = (int)(cb % 64);
        const int64_t frag = cb / 64;
        const int64_t nb = frag / g.kb32, kb = frag % g.kb32;
        const int64_t n = nb * 32 + (lane & 31);
        const int64_t k0 = kb * 32 + (lane >> 5) * 16;
        const uint32_t flip = p.dt == dt_u8 ? 0x80u : 0u;
        uint32_t w[4] = {0, 0, 0, 0};
        if (n < p.N) {
            const uint8_t *s = p.src + b * p.sb + n * p.sn;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int64_t k = k0 + i;
                // u8 weights are stored as s8 = u8 - 128 (top bit flipped);
                // the padding stays 0
                const uint32_t v
                        = k < p.K ? (uint32_t)s[k * p.sk] ^ flip : 0u;
                w[i / 4] |= v << (8 * (i % 4));
            }
        }
        *(uint4 *)(p.dst + c * 16) = make_uint4(w[0], w[1], w[2], w[3]);
    }
}

// column sums of the 8-bit weights as the kernels see them (s8; u8 weights
// minus 128): blockIdx.y cuts K into
// chunks of COLSUM_KCHUNK rows, a thread sums one column of its chunk and adds
// the partial sum to the (zeroed) s32 result -- integer atomics, so the result
// does not depend on the order
constexpr int COLSUM_KCHUNK = 128;

__global__ void __launch_bounds__(256)
colsum_zero_kernel(const pack_params_t p, const b8_geom_t g) {
    const int64_t total = p.batch * g.Npad;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
            i += (int64_t)gridDim.x * blockDim.x)
        ((int32_t *)(p.dst + g.colsum_off))[i] = 0;
}

__global__ void __launch_bounds__(256)
colsum_kernel(const pack_params_t p, const b8_geom_t g) {
    const int64_t total = p.batch * g.Npad;
    const int64_t k0 = (int64_t)blockIdx.y * COLSUM_KCHUNK;
    const int64_t k1 = k0 + COLSUM_KCHUNK < p.K ? k0 + COLSUM_KCHUNK : p.K;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
            i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t b = i / g.Npad, n = i % g.Npad;
        if (n >= p.N) continue;
        const uint8_t *s = p.src + b * p.sb + n * p.sn;
        int32_t acc = 0;
        for (int64_t k = k0; k < k1; k++) {
            const uint8_t v = s[k * p.sk];
            acc += p.dt == dt_s8 ? (int32_t)(int8_t)v
                    : p.dt == dt_u8 ? (int32_t)v - 128
                                    : (int32_t)v;
        }
        atomicAdd((int32_t *)(p.dst + g.colsum_off) + i, acc);
    }
}

__global__ void __launch_bounds__(256)
unpack_b8_kernel(const pack_params_t p, const b8_geom_t g) {
    // p.src: packed, p.dst: plain
    const int64_t total = p.batch * p.K * p.N;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
            i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t n = i % p.N, k = (i / p.N) % p.K, b = i / (p.N * p.K);
        p.dst[b * p.sb + k * p.sk + n * p.sn]
                = p.src[b * g.batch_bytes + b8_offset(g, k, n)]
                ^ (p.dt == dt_u8 ? 0x80 : 0);
    }
}

// one thread per packed dword (8 nibbles)
__global__ void __launch_bounds__(256)
pack_w4_kernel(const pack_params_t p, const w4_geom_t g) {
    const int64_t dwords = p.batch * g.batch_bytes / 4;
    for (int64_t d = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; d < dwords;
            d += (int64_t)gridDim.x * blockDim.x) {
        const int64_t per_b = g.batch_bytes / 4;
        const int64_t b = d / per_b, db = d % per_b;
        const int s = (int)(db % 4);
        const int lane = (int)((db / 4) % 64);
        const int64_t tile = db / 256;
        const int64_t nbk = tile / g.kg128, kg = tile % g.kg128;
        const int64_t n = nbk * 16 + (lane & 15);
        const int64_t kbase = kg * 128 + 32 * s + 8 * (lane >> 4);
        uint32_t w = 0;
        if (n < p.N) {
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const int64_t k = kbase + j;
                if (k >= p.K) continue;
                const int64_t e = b * p.sb + k * p.sk + n * p.sn;
                const uint32_t nib = (uint32_t)nibble_at(p.src, e);
                const int pos = j / 2 + 4 * (j % 2);
                w |= nib << (4 * pos);
            }
        }
        ((uint32_t *)p.dst)[d] = w;
    }
}

// QMM_LAYOUT_MFMA_W8: one thread per packed dword (the high or the low
// nibbles of 8 weights bytes); g is the 4-bit geometry of the same K and N, a
// tile being its two 1 KiB planes
__global__ void __launch_bounds__(256)
pack_w8_kernel(const pack_params_t p, const w4_geom_t g) {
    const int64_t per_b = g.batch_bytes / 2; // dwords: 2 planes of batch_bytes
    const int64_t dwords = p.batch * per_b;
    for (int64_t d = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; d < dwords;
            d += (int64_t)gridDim.x * blockDim.x) {
        const int64_t b = d / per_b, db = d % per_b;
        const int s = (int)(db % 4);
        const int lane = (int)((db / 4) % 64);
        const int plane = (int)((db / 256) % 2);
        const int64_t tile = db / 512;
        const int64_t nbk = tile / g.kg128, kg = tile % g.kg128;
        const int64_t n = nbk * 16 + (lane & 15);
        const int64_t kbase = kg * 128 + 32 * s + 8 * (lane >> 4);
        uint32_t w = 0;
        if (n < p.N) {
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const int64_t k = kbase + j;
                if (k >= p.K) continue;
                const uint32_t v = p.src[b * p.sb + k * p.sk + n * p.sn];
                const uint32_t nib = plane ? (v & 15u) : (v >> 4);
                const int pos = j / 2 + 4 * (j % 2);
                w |= nib << (4 * pos);
            }
        }
        ((uint32_t *)p.dst)[d] = w;
    }
}

// one thread per destination byte
__global__ void __launch_bounds__(256)
unpack_w8_kernel(const pack_params_t p, const w4_geom_t g) {
    const int64_t total = p.batch * p.K * p.N;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
            i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t n = i % p.N, k = (i / p.N) % p.K, b = i / (p.N * p.K);
        // nibble index inside the 4-bit layout: 2048 nibbles per tile plane
        const int64_t ni = w4_nibble_index(g, k, n);
        const int64_t tile = ni / 2048, off = ni % 2048;
        const uint8_t *t = p.src + b * g.batch_bytes * 2 + tile * 2048;
        const int hi = nibble_at(t, off), lo = nibble_at(t + 1024, off);
        p.dst[b * p.sb + k * p.sk + n * p.sn] = (uint8_t)((hi << 4) | lo);
    }
}

// one thread per destination byte: the two nibbles are neighbours along the
// plain tensor's stride-1 dim (n for ab, k for ba)
__global__ void __launch_bounds__(256)
unpack_w4_kernel(const pack_params_t p, const w4_geom_t g) {
    const bool n_inner = p.sn == 1;
    const int64_t total = p.batch * p.K * p.N / 2;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
            i += (int64_t)gridDim.x * blockDim.x) {
        uint8_t out = 0;
        int64_t e0 = 0;
        for (int h = 0; h < 2; h++) {
            const int64_t l = 2 * i + h;
            int64_t b, k, n;
            if (n_inner) {
                n = l % p.N;
                k = (l / p.N) % p.K;
                b = l / (p.N * p.K);
            } else {
                k = l % p.K;
                n = (l / p.K) % p.N;
                b = l / (p.N * p.K);
            }
            const int64_t e = b * p.sb + k * p.sk + n * p.sn;
            if (h == 0) e0 = e;
            const int64_t ni = b * g.batch_bytes * 2 + w4_nibble_index(g, k, n);
            out |= (uint8_t)(nibble_at(p.src, ni) << (4 * (int)(e & 1)));
        }
        p.dst[e0 >> 1] = out;
    }
}

// QMM_LAYOUT_MFMA_W4K64, one thread per packed dword (8 nibbles). u4 values are
// stored as u - 8 (nibble ^ 8): the int8 GEMM reads every nibble as signed.
__global__ void __launch_bounds__(256)
pack_w4k_kernel(const pack_params_t p, const w4k_geom_t g) {
    const int64_t dwords = p.batch * g.batch_bytes / 4;
    const uint32_t flip = p.dt == dt_u4 ? 8u : 0u;
    for (int64_t d = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; d < dwords;
            d += (int64_t)gridDim.x * blockDim.x) {
        const int64_t per_b = g.batch_bytes / 4;
        const int64_t b = d / per_b, db = d % per_b;
        const int dw = (int)(db % 4);
        const int lane = (int)((db / 4) % 64);
        const int64_t tile = db / 256;
        const int64_t nb = tile / g.kt64, kt = tile % g.kt64;
        const int64_t n = nb * 32 + (lane & 31);
        const int64_t kbase
                = kt * 64 + 32 * (dw / 2) + 16 * (lane >> 5) + 8 * (dw % 2);
        uint32_t w = 0;
        if (n < p.N) {
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const int64_t k = kbase + j;
                if (k >= p.K) continue;
                const int64_t e = b * p.sb + k * p.sk + n * p.sn;
                const uint32_t nib = (uint32_t)nibble_at(p.src, e) ^ flip;
                const int pos = 2 * (j % 4) + j / 4;
                w |= nib << (4 * pos);
            }
        }
        ((uint32_t *)p.dst)[d] = w;
    }
}

__global__ void __launch_bounds__(256)
unpack_w4k_kernel(const pack_params_t p, const w4k_geom_t g) {
    const bool n_inner = p.sn == 1;
    const int64_t total = p.batch * p.K * p.N / 2;
    const int flip = p.dt == dt_u4 ? 8 : 0;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
            i += (int64_t)gridDim.x * blockDim.x) {
        uint8_t out = 0;
        int64_t e0 = 0;
        for (int h = 0; h < 2; h++) {
            const int64_t l = 2 * i + h;
            int64_t b, k, n;
            if (n_inner) {
                n = l % p.N;
                k = (l / p.N) % p.K;
                b = l / (p.N * p.K);
            } else {
                k = l % p.K;
                n = (l / p.K) % p.N;
                b = l / (p.N * p.K);
            }
            const int64_t e = b * p.sb + k * p.sk + n * p.sn;
            if (h == 0) e0 = e;
            const int64_t ni = b * g.batch_bytes * 2 + w4k_nibble_index(g, k, n);
            out |= (uint8_t)((nibble_at(p.src, ni) ^ flip) << (4 * (int)(e & 1)));
        }
        p.dst[e0 >> 1] = out;
    }
}

static unsigned grid_for(int64_t n) {
    int64_t b = (n + 255) / 256;
    if (b < 1) b = 1;
    if (b > 262144) b = 262144;
    return (unsigned)b;
}

void launch_pack_b8(const void *src, void *dst, int dt, int64_t batch,
        int64_t K, int64_t N, int64_t sb, int64_t sk, int64_t sn,
        bool with_colsum, hipStream_t stream) {
    const b8_geom_t g = b8_geom(batch, K, N);
    pack_params_t p {(const uint8_t *)src, (uint8_t *)dst, batch, K, N, sb, sk,
            sn, dt, 0};
    hipLaunchKernelGGL(pack_b8_kernel, dim3(grid_for(batch * g.batch_bytes / 16)),
            dim3(256), 0, stream, p, g);
    if (with_colsum) {
        hipLaunchKernelGGL(colsum_zero_kernel, dim3(grid_for(batch * g.Npad)),
                dim3(256), 0, stream, p, g);
        const int64_t cols = (batch * g.Npad + 255) / 256;
        const unsigned kchunks
                = (unsigned)((K + COLSUM_KCHUNK - 1) / COLSUM_KCHUNK);
        hipLaunchKernelGGL(colsum_kernel,
                dim3((unsigned)(cols < 65535 ? cols : 65535),
                        kchunks ? kchunks : 1),
                dim3(256), 0, stream, p, g);
    }
}

// u8 activations -> s8 (x ^ 0x80) into a dense [batch][M][K] buffer: the
// pre-pass of the 256 x 256 GEMM kernel for u8 sources (the +128 * colsum
// correction is applied in its epilogue). One thread per 16 bytes.
__global__ void __launch_bounds__(256)
flip_u8_kernel(const uint8_t *src, uint8_t *dst, int64_t rows, int64_t K16,
        int64_t M, int64_t lda, int64_t a_sb) {
    const int64_t total = rows * K16;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
            i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t r = i / K16, c = i % K16;
        const int64_t b = r / M, m = r % M;
        uint4 v = *(const uint4 *)(src + b * a_sb + m * lda + c * 16);
        v.x ^= 0x80808080u;
        v.y ^= 0x80808080u;
        v.z ^= 0x80808080u;
        v.w ^= 0x80808080u;
        *(uint4 *)(dst + i * 16) = v;
    }
}

void launch_flip_u8(const void *src, void *dst, int64_t batch, int64_t M,
        int64_t K, int64_t lda, int64_t a_sb, hipStream_t stream) {
    hipLaunchKernelGGL(flip_u8_kernel, dim3(grid_for(batch * M * K / 16)),
            dim3(256), 0, stream, (const uint8_t *)src, (uint8_t *)dst,
            batch * M, K / 16, M, lda, a_sb);
}

// Row sums of the 8-bit source as the kernels see it (s8; a u8 source minus
// 128), plus K times the source compensation (128 for a u8 source, minus the
// source zero point): what a weights zero point multiplies,
//   sum_k (s - z_s)(w - z_w) = P + comp * colsum[n] - z_w' * (rowsum[m] + K * comp)
// with P the s8 x s8 product sum and z_w' the zero point of the stored s8
// weights. One wave per row.
__global__ void __launch_bounds__(256)
rowsum_b8_kernel(const uint8_t *src, int32_t *dst, int64_t rows, int64_t M,
        int64_t K, int64_t lda, int64_t a_sb, int a_is_u8, const void *src_zp,
        int src_zp_dt) {
    const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= rows) return;
    const int lane = threadIdx.x & 63;
    const uint8_t *a = src + (r / M) * a_sb + (r % M) * lda;
    const uint32_t flip = a_is_u8 ? 0x80808080u : 0u;
    int sum = 0;
    for (int64_t k = lane * 16; k < K; k += 64 * 16) { // K % 16 == 0
        const uint4 v = *(const uint4 *)(a + k);
        const uint32_t w[4] = {v.x ^ flip, v.y ^ flip, v.z ^ flip, v.w ^ flip};
#pragma unroll
        for (int d = 0; d < 4; d++)
            sum += (int)(int8_t)(w[d] & 0xff) + (int)(int8_t)((w[d] >> 8) & 0xff)
                    + (int)(int8_t)((w[d] >> 16) & 0xff) + (int)(int8_t)(w[d] >> 24);
    }
#pragma unroll
    for (int o = 32; o; o >>= 1) sum += __shfl_xor(sum, o);
    if (lane == 0) {
        int comp = a_is_u8 ? 128 : 0;
        if (src_zp) comp -= load_int(src_zp_dt, src_zp, 0);
        dst[r] = sum + (int)K * comp;
    }
}

void launch_rowsum_b8(const void *src, int32_t *dst, int64_t batch, int64_t M,
        int64_t K, int64_t lda, int64_t a_sb, bool a_is_u8, const void *src_zp,
        int src_zp_dt, hipStream_t stream) {
    const int64_t rows = batch * M;
    hipLaunchKernelGGL(rowsum_b8_kernel, dim3((unsigned)((rows + 3) / 4)),
            dim3(256), 0, stream, (const uint8_t *)src, dst, rows, M, K, lda,
            a_sb, a_is_u8 ? 1 : 0, src_zp, src_zp_dt);
}

void launch_unpack_b8(const void *src, void *dst, int dt, int64_t batch,
        int64_t K, int64_t N, int64_t sb, int64_t sk, int64_t sn,
        hipStream_t stream) {
    const b8_geom_t g = b8_geom(batch, K, N);
    pack_params_t p {(const uint8_t *)src, (uint8_t *)dst, batch, K, N, sb, sk,
            sn, dt, 0};
    hipLaunchKernelGGL(unpack_b8_kernel, dim3(grid_for(batch * K * N)),
            dim3(256), 0, stream, p, g);
}

void launch_pack_w4(const void *src, void *dst, int dt, int64_t batch,
        int64_t K, int64_t N, int64_t sb, int64_t sk, int64_t sn,
        hipStream_t stream) {
    const w4_geom_t g = w4_geom(batch, K, N);
    pack_params_t p {(const uint8_t *)src, (uint8_t *)dst, batch, K, N, sb, sk,
            sn, dt, 0};
    hipLaunchKernelGGL(pack_w4_kernel, dim3(grid_for(batch * g.batch_bytes / 4)),
            dim3(256), 0, stream, p, g);
}

void launch_unpack_w4(const void *src, void *dst, int dt, int64_t batch,
        int64_t K, int64_t N, int64_t sb, int64_t sk, int64_t sn,
        hipStream_t stream) {
    const w4_geom_t g = w4_geom(batch, K, N);
    pack_params_t p {(const uint8_t *)src, (uint8_t *)dst, batch, K, N, sb, sk,
            sn, dt, 0};
    hipLaunchKernelGGL(unpack_w4_kernel, dim3(grid_for(batch * K * N / 2)),
            dim3(256), 0, stream, p, g);
}

void launch_pack_w8(const void *src, void *dst, int dt, int64_t batch,
        int64_t K, int64_t N, int64_t sb, int64_t sk, int64_t sn,
        hipStream_t stream) {
    const w4_geom_t g = w4_geom(batch, K, N);
    pack_params_t p {(const uint8_t *)src, (uint8_t *)dst, batch, K, N, sb, sk,
            sn, dt, 0};
    hipLaunchKernelGGL(pack_w8_kernel, dim3(grid_for(batch * g.batch_bytes / 2)),
            dim3(256), 0, stream, p, g);
}

void launch_unpack_w8(const void *src, void *dst, int dt, int64_t batch,
        int64_t K, int64_t N, int64_t sb, int64_t sk, int64_t sn,
        hipStream_t stream) {
    const w4_geom_t g = w4_geom(batch, K, N);
    pack_params_t p {(const uint8_t *)src, (uint8_t *)dst, batch, K, N, sb, sk,
            sn, dt, 0};
    hipLaunchKernelGGL(unpack_w8_kernel, dim3(grid_for(batch * K * N)),
            dim3(256), 0, stream, p, g);
}

void launch_pack_w4k(const void *src, void *dst, int dt, int64_t batch,
        int64_t K, int64_t N, int64_t sb, int64_t sk, int64_t sn,
        hipStream_t stream) {
    const w4k_geom_t g = w4k_geom(batch, K, N);
    pack_params_t p {(const uint8_t *)src, (uint8_t *)dst, batch, K, N, sb, sk,
            sn, dt, 0};
    hipLaunchKernelGGL(pack_w4k_kernel,
            dim3(grid_for(batch * g.batch_bytes / 4)), dim3(256), 0, stream, p,
            g);
}

void launch_unpack_w4k(const void *src, void *dst, int dt, int64_t batch,
        int64_t K, int64_t N, int64_t sb, int64_t sk, int64_t sn,
        hipStream_t stream) {
    const w4k_geom_t g = w4k_geom(batch, K, N);
    pack_params_t p {(const uint8_t *)src, (uint8_t *)dst, batch, K, N, sb, sk,
            sn, dt, 0};
    hipLaunchKernelGGL(unpack_w4k_kernel, dim3(grid_for(batch * K * N / 2)),
            dim3(256), 0, stream, p, g);
}

} // namespace qmm
