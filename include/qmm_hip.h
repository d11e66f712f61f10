/*
 * Thin C ABI over the gfx950 HIP kernels of the quantized matmul path.
 *
 * This is the only interface the .hip translation units export. The dnnl_*
 * entry points (include/oneapi/dnnl/dnnl.h) are host C++ on top of it: a
 * primitive descriptor picks an implementation with qmm_matmul_impl_supports(),
 * a primitive owns a plan, and execute() is one qmm_matmul_launch() on the
 * stream's HIP stream. Plain-old-data only: dims, strides, data-type codes,
 * masks, groups, the post-op list and device pointers. No call here allocates
 * except plan creation (one small device copy of the descriptor).
 *
 * Reference interfaces this layer stands in for:
 *   - primitive_t::execute(const exec_ctx_t &) of a matmul implementation
 *     (src/common/primitive.hpp:43-80, src/gpu/amd/miopen_matmul.hpp:35-165),
 *   - pd_t::init() returning status::unimplemented for unsupported cases so
 *     the implementation list falls through
 *     (src/common/primitive_desc_iterator.hpp:67-94,
 *      src/gpu/gpu_matmul_list.cpp:45-62),
 *   - the reorder implementation list entry used for weights prepacking
 *     (src/cpu/x64/matmul/brgemm_matmul_reorders.hpp:28-76).
 *
 * Data-type, algorithm and primitive-kind codes are the dnnl ones
 * (dnnl_data_type_t, dnnl_alg_kind_t, dnnl_primitive_kind_t).
 */
#ifndef QMM_HIP_H
#define QMM_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define QMM_MAX_NDIMS 12
#define QMM_MAX_POST_OPS 32
#define QMM_API __attribute__((visibility("default")))

/* status codes: 0 ok; the rest map 1:1 onto dnnl_status_t */
enum {
    QMM_OK = 0,
    QMM_OUT_OF_MEMORY = 1,
    QMM_INVALID_ARGUMENTS = 2,
    QMM_UNIMPLEMENTED = 3,
    QMM_RUNTIME_ERROR = 5
};

/* Physical layouts of a weights tensor. */
enum {
    QMM_LAYOUT_PLAIN = 0, /* strided, strides in elements */
    /* 1-byte elements (s8/u8/f8) in MFMA operand order: per batch,
     * [N/32][K/32][64 lanes][16 bytes], lane = 32*((k%32)/16) + n%32,
     * byte = k%16; K padded to 128 and N to 32 with zeros; followed (256-byte
     * aligned) by s32 column sums [batch][Npad] for integer weights. */
    QMM_LAYOUT_MFMA_B8 = 1,
    /* 4-bit elements for the decode kernel: per batch,
     * [N/16][K/128][64 lanes][16 bytes], lane = 16*c + n%16 holds
     * k = 128*g + 32*s + 8*c + j for dword s = 0..3, and inside a dword the
     * nibble at bits 4*p..4*p+3 is j = perm(p) = (p%2)*4 + p/2 ... see
     * qmm_w4_nibble_pos(); K padded to 128 and N to 16 with zeros. */
    QMM_LAYOUT_MFMA_W4 = 2,
    /* 4-bit elements for the int8-activation GEMM: per batch,
     * [N/32][K/64][64 lanes][16 bytes]; lane = 32*h + n%32 holds, in dword
     * 2*i + q, the eight values k = 64*t + 32*i + 16*h + 8*q + j (j = 0..7),
     * value j in the nibble at bits 4*p..4*p+3 with p = 2*(j%4) + j/4, so that
     * (dword << 4) & 0xF0F0F0F0 and dword & 0xF0F0F0F0 are j = 0..3 and
     * j = 4..7 as bytes holding 16 * value. Values are stored as signed
     * nibbles: s4 as is, u4 as (u - 8). K padded to 64 and N to 32 with
     * zeros. */
    QMM_LAYOUT_MFMA_W4K64 = 3,
    /* 8-bit elements for the decode kernel, as two planes of nibbles: per
     * batch, [N/16][K/128][2 planes][64 lanes][16 bytes]; plane 0 holds the
     * high nibbles and plane 1 the low nibbles of the bytes, each in the
     * order of QMM_LAYOUT_MFMA_W4. K padded to 128 and N to 16 with zeros. */
    QMM_LAYOUT_MFMA_W8 = 4
};

typedef struct {
    int32_t dt;
    int32_t ndims;
    int64_t dims[QMM_MAX_NDIMS];
    int64_t strides[QMM_MAX_NDIMS]; /* elements; ignored for packed layouts */
} qmm_tensor_t;

/* One scales or zero-points entry (dnnl_primitive_attr_set_scales /
 * _set_zero_points): the buffer is a dense row-major tensor over the masked
 * dims of the quantized tensor with its last two dims divided by the groups
 * (src/cpu/matmul/matmul_utils.hpp:156-196). */
typedef struct {
    int32_t set; /* 0: default value (scale 1, zero point 0) */
    int32_t mask;
    int32_t dt;
    int32_t has_groups;
    int64_t g0, g1; /* groups over the last two dims; 1 when absent */
} qmm_quant_t;

typedef struct {
    int32_t kind; /* dnnl_sum / dnnl_eltwise / dnnl_binary / dnnl_prelu */
    int32_t alg;
    float alpha, beta, scale;
    int32_t zero_point;
    int32_t dt; /* sum: data type dst is read as (0 = dst's own) */
    int32_t mask; /* prelu */
    qmm_tensor_t src1; /* binary operand descriptor (plain) */
} qmm_postop_t;

enum { QMM_SRC = 0, QMM_WEI = 1, QMM_DST = 2 };

typedef struct {
    qmm_tensor_t src, wei, bias, dst; /* bias.ndims == 0: no bias */
    int32_t wei_layout;
    int32_t apply_to_int; /* fpmath_mode apply_to_int */
    qmm_quant_t scales[3];
    qmm_quant_t zps[3];
    int32_t npo;
    int32_t reserved;
    qmm_postop_t po[QMM_MAX_POST_OPS];
} qmm_matmul_desc_t;

typedef struct {
    const void *src, *wei, *bias;
    void *dst;
    const void *scales[3];
    const void *zps[3];
    const void *po_arg[QMM_MAX_POST_OPS]; /* binary src1 / prelu weights */
    void *scratch; /* qmm_matmul_scratch_size() bytes, or NULL when 0 */
} qmm_matmul_args_t;

typedef struct qmm_plan qmm_plan_t;

/* ---- matmul implementations, in dispatch order ---- */
QMM_API int qmm_matmul_impl_count(void);
QMM_API const char *qmm_matmul_impl_name(int impl);
/* QMM_OK if implementation `impl` computes `desc`; QMM_UNIMPLEMENTED if not */
QMM_API int qmm_matmul_impl_supports(int impl, const qmm_matmul_desc_t *desc);
QMM_API size_t qmm_matmul_scratch_size(int impl, const qmm_matmul_desc_t *desc);
QMM_API int qmm_matmul_plan_create(
        qmm_plan_t **plan, int impl, const qmm_matmul_desc_t *desc);
QMM_API void qmm_matmul_plan_destroy(qmm_plan_t *plan);
/* Enqueue on `hip_stream` (a hipStream_t); asynchronous. */
QMM_API int qmm_matmul_launch(const qmm_plan_t *plan,
        const qmm_matmul_args_t *args, void *hip_stream);

/* qmm_matmul_launch() for callers that cannot allocate device memory (code
 * under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc). No counterpart in the reference: there the scratchpad is always
 * a memory object the user or the library allocates. args->scratch is ignored;
 * the kernels' scratch (weights packed on the fly, the s8 copy of a u8 source,
 * per-group scale arrays) is a buffer of QMM_STATIC_SCRATCH_BYTES that the
 * library holds on every GPU it runs on from load to process end. The call
 * allocates nothing and fails with QMM_INVALID_ARGUMENTS (qmm_last_error()
 * says why) when qmm_matmul_scratch_size() exceeds that size. All calls on one
 * GPU share the buffer: calls that overlap in time on one GPU (different
 * streams or threads) race; calls on one stream do not. Every kernel writes
 * the part of the buffer it later reads, so nothing has to be cleared between
 * calls. The buffer is the one of the stream's device (the current device for
 * the null stream); its address is looked up once per device, when a plan that
 * fits is created with that device current, else at the first such launch
 * there (a mutex and one hipGetSymbolAddress). */
#define QMM_STATIC_SCRATCH_BYTES (32u << 20)
QMM_API int qmm_matmul_launch_static_scratch(const qmm_plan_t *plan,
        const qmm_matmul_args_t *args, void *hip_stream);

/* ---- packed weights layouts ---- */
/* Bytes a weights tensor [batch..., K, N] of type dt occupies in `layout`. */
QMM_API size_t qmm_packed_size(int layout, int dt, int64_t batch, int64_t K, int64_t N);
/* Layout format_tag any resolves to for this problem, or QMM_LAYOUT_PLAIN. */
QMM_API int qmm_matmul_preferred_wei_layout(const qmm_matmul_desc_t *desc);
/* The same for one implementation (the packed layout `impl` takes this problem
 * in, or QMM_LAYOUT_PLAIN): what format_tag any resolves to when the
 * implementation list is walked past the first that applies. */
QMM_API int qmm_matmul_impl_preferred_wei_layout(int impl, const qmm_matmul_desc_t *desc);

/* ---- reorder ---- */
typedef struct {
    qmm_tensor_t src, dst; /* same logical dims */
    int32_t src_layout, dst_layout;
    qmm_quant_t src_scale, dst_scale, src_zp, dst_zp;
} qmm_reorder_desc_t;

typedef struct {
    const void *src;
    void *dst;
    const void *src_scale, *dst_scale, *src_zp, *dst_zp;
} qmm_reorder_args_t;

QMM_API int qmm_reorder_supports(const qmm_reorder_desc_t *desc);
/* Name of the implementation qmm_reorder_launch() runs for `desc`:
 * "hip:gfx950:prepack" (to / from a packed weights layout),
 * "hip:gfx950:quantize" (row-wise element pass with scales / zero points) or
 * "hip:gfx950:reorder" (any strides, one element per thread). */
QMM_API const char *qmm_reorder_impl_name(const qmm_reorder_desc_t *desc);
QMM_API int qmm_reorder_launch(const qmm_reorder_desc_t *desc,
        const qmm_reorder_args_t *args, void *hip_stream);

/* ---- softmax (forward) ----
 * The step between the two matmuls of an attention block. Stands in for
 * ref_softmax_fwd_t::execute (src/cpu/ref_softmax.cpp:40-312). Plain strided
 * tensors of equal dims; alg is dnnl_softmax_accurate or dnnl_softmax_log;
 * scales are single values (mask 0). */
typedef struct {
    qmm_tensor_t src, dst;
    int32_t axis;
    int32_t alg;
    qmm_quant_t src_scale, dst_scale;
} qmm_softmax_desc_t;

typedef struct {
    const void *src;
    void *dst;
    const void *src_scale, *dst_scale;
} qmm_softmax_args_t;

QMM_API int qmm_softmax_supports(const qmm_softmax_desc_t *desc);
QMM_API const char *qmm_softmax_impl_name(const qmm_softmax_desc_t *desc);
QMM_API int qmm_softmax_launch(const qmm_softmax_desc_t *desc,
        const qmm_softmax_args_t *args, void *hip_stream);

/* ---- scaled dot-product attention ----
 * dst = softmax(scale * Q x K + mask) x V in one kernel. Stands in for the
 * reference's internal sdpa primitive (src/common/sdpa_types.hpp:38-80,
 * sdpa_utils.hpp:116-180; execute arguments src/gpu/intel/ocl/micro_sdpa.cpp:
 * 674-690). q [.., Q, D], k [.., D, S] (the transposed view of a [S, D]
 * cache), v [.., S, D], dst [.., Q, D]; mask: ndims 0 when absent, else dims
 * equal to the scores' [.., Q, S] or 1; scale_dt 0 when there is no scale
 * tensor; k / v may be s8 / u8 with one scale and zero point per key. */
typedef struct {
    qmm_tensor_t q, k, v, dst, mask;
    int32_t scale_dt;
    int32_t invert_scale; /* multiply by 1 / scale */
    int32_t causal; /* key index > query index is masked out */
    int32_t reserved;
    int64_t kv_head_number;
    qmm_quant_t k_scale, k_zp, v_scale, v_zp;
} qmm_sdpa_desc_t;

typedef struct {
    const void *q, *k, *v;
    void *dst;
    const void *mask, *scale;
    const void *k_scale, *k_zp, *v_scale, *v_zp;
    void *scratch; /* qmm_sdpa_scratch_size() bytes, or NULL when 0 */
} qmm_sdpa_args_t;

QMM_API int qmm_sdpa_supports(const qmm_sdpa_desc_t *desc);
QMM_API const char *qmm_sdpa_impl_name(const qmm_sdpa_desc_t *desc);
/* Bytes of scratch a launch needs: non-zero only for at most 16 queries with
 * enough keys to be cut into several ranges (partial results per range). */
QMM_API size_t qmm_sdpa_scratch_size(const qmm_sdpa_desc_t *desc);
QMM_API int qmm_sdpa_launch(const qmm_sdpa_desc_t *desc,
        const qmm_sdpa_args_t *args, void *hip_stream);

/* ---- kernel-selection overrides ----
 * For A/B measurements and for tests that must reach a particular kernel at
 * sizes the oracle finishes quickly. Environment variables, read once when a
 * plan is created (qmm_matmul_plan_create) and fixed for that plan's life; a
 * launch reads no process-wide state. Production code leaves them unset.
 *   QMM_GEMM_VARIANT: 0 by problem size (default); 1..3 a tile configuration of
 *     the general mfma_b8 kernel; 6 the 256 x 256 kernels wherever eligible;
 *     for mfma_f16 plans 1 = 64 x 64 tiles, 2 = 128 x 128 tiles, 3 = 128-row
 *     workgroups that walk the column tiles (short K); for mfma_f16w8 plans
 *     1 = K in one pass (no slices with a second, reducing kernel)
 *   QMM_W4A8_VARIANT: 0 by problem size (default); 1..3 a tile configuration;
 *     4 as 0 but with the split-K kernel instead of the one-launch kernel at
 *     5 .. 64 rows, 5 as 0 but with the one-launch kernel wherever it applies
 *   QMM_B8X_VARIANT: the 256-row int8 / fp8 kernels: 1 = by shape (default: 16 x 16
 *     MFMAs; int8 with 256 x 128 tiles and two workgroups per CU up to K 2048,
 *     256 x 256 tiles and one per CU beyond), 2 = 256 x 128 two per CU wherever it
 *     applies, 3 = 256 x 256 one per CU, 4 = as 3 with one workgroup per tile
 *     instead of one per CU walking its tiles, 5 = as 3 with every workgroup
 *     starting at once (no half-tile stagger), 0 = the loops on 32 x 32 MFMAs */

/* ---- measurement switches of the 256 x 256 GEMM kernels ----
 * QMM_MEASURE (environment, read at plan creation like the overrides above):
 * bit 0: the int8 kernel with 256 x 256 tiles on 16 x 16 x 64 MFMAs (even number
 * of k-steps; QMM_B8X_VARIANT=3 selects it at any K) ends after its main loop
 * and stores nothing (what the loop alone costs); bit 1: the first lane of every workgroup records (core clock counter,
 * 100 MHz counter) at kernel entry, main-loop entry, main-loop exit and the end
 * of the epilogue (slots 0..3), and inside the epilogue after each half of the
 * tile is staged (slots 4, 6) and after the first half's rows are stored (5). qmm_gemm_stamps_read() copies the records of the last such
 * launch out: 8 slots x 2 x uint64 per block tile, tile = (blockIdx.x + gridDim.x *
 * blockIdx.y) % 4096, at most 4096 * 128 bytes. No counterpart in the
 * reference. */
QMM_API int qmm_gemm_stamps_read(void *host, size_t bytes);

/* ---- measurement aid ----
 * Launches a kernel that only reads: up to three byte ranges (16-byte aligned,
 * lengths rounded down to 16), pulled with 16-byte vector loads by
 * QMM_STREAM_READ_GROUPS workgroups of 512 lanes (the decode kernel's launch
 * shape), one word stored per wave into `sink` (QMM_STREAM_READ_GROUPS * 32
 * bytes). No counterpart in the reference; benchmarks use it to put a
 * read-only floor next to the decode kernel's time. */
#define QMM_STREAM_READ_GROUPS 256
QMM_API int qmm_stream_read(const void *p0, size_t n0, const void *p1,
        size_t n1, const void *p2, size_t n2, void *sink, void *stream);

/* Launches a kernel that only writes: `groups` workgroups of 256 lanes store
 * 16-byte vectors over `bytes` of dst (16-byte aligned) with a grid-stride
 * loop. Benchmarks time it to state what a launch bound by its destination
 * stream can reach on this card. No counterpart in the reference. */
QMM_API int qmm_stream_write(void *dst, size_t bytes, int groups, void *hip_stream);

/* Launches a plain copy kernel: `groups` workgroups of 256 lanes move `bytes`
 * (both pointers 16-byte aligned) from src to dst, one 16-byte vector per lane
 * and pass. A kernel of known traffic: profiler counters of HBM bytes are scaled
 * by what they read for it. No counterpart in the reference. */
QMM_API int qmm_stream_copy(void *dst, const void *src, size_t bytes, int groups,
        void *hip_stream);

/* Launches `groups` workgroups of four waves that issue nothing but the MFMAs
 * of the 256 x 256 GEMM kernels' main loop (`ksteps` k-steps, even, of the
 * 128 x 128 wave tile) on register-resident operands (data 0: uniformly random
 * bytes, 1: zeros, 2: the value distributions of the int8 / fp8 benchmark
 * configurations): kind 0 = v_mfma_i32_16x16x64_i8, 1 = v_mfma_i32_32x32x32_i8,
 * 2 = v_mfma_f32_16x16x128_f8f6f4, 3 = v_mfma_f32_32x32x64_f8f6f4 (e4m3), 4 = kind 0
 * with the weights fragment instead of the source fragment held over eight
 * consecutive MFMAs. One word
 * per lane goes to `sink` (groups * 1024 bytes); *ops_per_launch receives the
 * multiply-add operations (x 2) of a launch. No counterpart in the reference;
 * benchmarks time it to state what the matrix cores sustain on this card next
 * to the published peak. */
QMM_API int qmm_mfma_ceiling(int kind, int ksteps, int groups, int data,
        void *sink, void *hip_stream, double *ops_per_launch);

/* ---- device queries used by the engine ---- */
QMM_API int qmm_device_count(void);
QMM_API const char *qmm_last_error(void);

#ifdef __cplusplus
}
#endif
#endif
