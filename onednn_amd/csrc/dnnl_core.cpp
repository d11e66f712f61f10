// Engine, stream, memory descriptor, memory, attribute and post-ops entry
// points of the dnnl C API subset (include/oneapi/dnnl/dnnl.h). Host-only.
// Error behaviour follows the reference: null handles and malformed
// descriptors give dnnl_invalid_arguments, resource failures
// dnnl_out_of_memory / dnnl_runtime_error.
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <new>

#include "dnnl_objects.hpp"
#include "oneapi/dnnl/dnnl_debug.h"

namespace host {

size_t dt_bits(dnnl_data_type_t dt) {
    switch (dt) {
        case dnnl_f16:
        case dnnl_bf16: return 16;
        case dnnl_f32:
        case dnnl_s32: return 32;
        case dnnl_f64: return 64;
        case dnnl_s8:
        case dnnl_u8:
        case dnnl_boolean:
        case dnnl_f8_e5m2:
        case dnnl_f8_e4m3:
        case dnnl_e8m0: return 8;
        case dnnl_s4:
        case dnnl_u4:
        case dnnl_f4_e2m1:
        case dnnl_f4_e3m0: return 4;
        default: return 0;
    }
}

static bool dims_ok(int ndims, const dnnl_dims_t dims) {
    if (ndims < 0 || ndims > DNNL_MAX_NDIMS) return false;
    if (ndims > 0 && !dims) return false;
    for (int d = 0; d < ndims; d++)
        if (dims[d] < 0 && dims[d] != DNNL_RUNTIME_DIM_VAL) return false;
    return true;
}

// Strides must describe a non-overlapping layout
// (memory_desc_strides_check, src/common/memory_desc.cpp).
static bool strides_ok(int ndims, const dnnl_dims_t dims, const dnnl_dims_t s) {
    int perm[DNNL_MAX_NDIMS], n = 0;
    for (int d = 0; d < ndims; d++) {
        if (dims[d] == DNNL_RUNTIME_DIM_VAL || s[d] == DNNL_RUNTIME_DIM_VAL)
            return true;
        if (dims[d] == 0) return true;
        if (s[d] < 0) return false;
        if (dims[d] > 1) perm[n++] = d;
    }
    std::sort(perm, perm + n, [&](int a, int b) {
        return s[a] != s[b] ? s[a] < s[b] : dims[a] < dims[b];
    });
    int64_t min_next = 1;
    for (int i = 0; i < n; i++) {
        const int d = perm[i];
        if (s[d] < min_next) return false;
        min_next = s[d] * dims[d];
    }
    return true;
}

bool md_init_plain(dnnl_memory_desc &md, int ndims, const dnnl_dims_t dims,
        dnnl_data_type_t dt, const dnnl_dims_t strides) {
    md = dnnl_memory_desc();
    if (ndims == 0) return true;
    if (!dims_ok(ndims, dims) || dt_bits(dt) == 0) return false;
    md.ndims = ndims;
    std::copy(dims, dims + ndims, md.dims);
    md.data_type = dt;
    md.format_kind = dnnl_blocked;
    if (strides) {
        if (!strides_ok(ndims, dims, strides)) return false;
        std::copy(strides, strides + ndims, md.strides);
    } else {
        bool runtime = false;
        md.strides[ndims - 1] = 1;
        for (int d = ndims - 2; d >= 0; d--) {
            if (dims[d + 1] == DNNL_RUNTIME_DIM_VAL) runtime = true;
            md.strides[d] = runtime
                    ? DNNL_RUNTIME_DIM_VAL
                    : md.strides[d + 1] * std::max<int64_t>(dims[d + 1], 1);
        }
    }
    return true;
}

bool md_equal(const dnnl_memory_desc &a, const dnnl_memory_desc &b) {
    if (a.ndims != b.ndims) return false;
    if (a.ndims == 0) return true;
    if (a.data_type != b.data_type || a.format_kind != b.format_kind)
        return false;
    for (int d = 0; d < a.ndims; d++)
        if (a.dims[d] != b.dims[d]) return false;
    if (a.format_kind == dnnl_blocked) {
        for (int d = 0; d < a.ndims; d++)
            if (a.strides[d] != b.strides[d]) return false;
        return a.offset0 == b.offset0;
    }
    if (a.format_kind == dnnl_format_kind_opaque)
        return a.packed_layout == b.packed_layout
                && a.packed_bytes == b.packed_bytes
                && a.packed_transposed == b.packed_transposed;
    return true;
}

size_t md_size(const dnnl_memory_desc &md) {
    if (md.ndims == 0 || md.has_zero_dim()) return 0;
    if (md.has_runtime_dims()) return DNNL_RUNTIME_SIZE_VAL;
    if (md.format_kind == dnnl_format_kind_opaque) return md.packed_bytes;
    if (md.format_kind != dnnl_blocked) return 0;
    int64_t max_off = md.offset0;
    for (int d = 0; d < md.ndims; d++)
        max_off += (md.dims[d] - 1) * md.strides[d];
    const size_t n = (size_t)max_off + 1;
    const size_t bits = dt_bits(md.data_type);
    return bits == 4 ? (n + 1) / 2 : n * (bits / 8);
}

void md_to_tensor(qmm_tensor_t &t, const dnnl_memory_desc &md) {
    std::memset(&t, 0, sizeof(t));
    t.dt = md.data_type;
    t.ndims = md.ndims;
    for (int d = 0; d < md.ndims; d++) {
        t.dims[d] = md.dims[d];
        t.strides[d] = md.format_kind == dnnl_blocked ? md.strides[d] : 0;
    }
}

dnnl_status_t from_qmm(int st) {
    switch (st) {
        case QMM_OK: return dnnl_success;
        case QMM_OUT_OF_MEMORY: return dnnl_out_of_memory;
        case QMM_INVALID_ARGUMENTS: return dnnl_invalid_arguments;
        case QMM_UNIMPLEMENTED: return dnnl_unimplemented;
        default: return dnnl_runtime_error;
    }
}

} // namespace host

using namespace host;

namespace {

// physical dim order of the plain tags, outermost first; index = tag - dnnl_a
const char *const tag_names[] = {"a", "ab", "abc", "abcd", "abcde", "abcdef",
        "abcdefg", "abcdefgh", "abcdefghi", "abcdefghij", "abcdefghijk",
        "abcdefghijkl", "ba", "acb", "bac", "bca", "cab", "cba", "abdc", "acbd",
        "acdb", "adbc", "adcb", "bacd", "bcda", "cdab", "cdba", "dcab", "abced",
        "abdec", "acbde", "acdeb", "adecb", "bacde", "bcdea", "cdeab", "cdeba",
        "decab", "abcdfe", "abdefc", "abdfce", "acbdef", "adefcb", "defcab",
        "abcdegf", "abcdefhg", "abcdefgih", "abcdefghji", "abcdefghikj",
        "abcdefghijlk"};

dnnl_fpmath_mode_t g_default_fpmath = dnnl_fpmath_mode_strict;
int g_verbose = -1;

bool set_device(const dnnl_engine *e) {
    if (!e || e->device < 0) return false;
    return hipSetDevice(e->device) == hipSuccess;
}

bool eltwise_ok(dnnl_alg_kind_t alg, float alpha, float beta) {
    // post-op form of is_eltwise_ok (src/common/math_utils.hpp:418-450)
    const int a = alg;
    const bool use_src = a >= dnnl_eltwise_relu && a <= dnnl_eltwise_hardswish;
    if (use_src) {
        if ((a == dnnl_eltwise_clip || a == dnnl_eltwise_clip_v2)
                && !(beta >= alpha))
            return false;
        return true;
    }
    const bool use_dst = a >= dnnl_eltwise_relu_use_dst_for_bwd
            && a <= dnnl_eltwise_clip_v2_use_dst_for_bwd;
    if (!use_dst) return false;
    if ((a == dnnl_eltwise_relu_use_dst_for_bwd
                || a == dnnl_eltwise_elu_use_dst_for_bwd)
            && !(alpha >= 0))
        return false;
    if (a == dnnl_eltwise_clip_v2_use_dst_for_bwd && !(beta >= alpha))
        return false;
    return true;
}

bool is_runtime_f32(float v) {
    uint32_t u;
    std::memcpy(&u, &v, 4);
    return u == 0x7fc000d0u;
}

} // namespace

int dnnl_amd_verbose_level() {
    if (g_verbose < 0) {
        const char *e = std::getenv("ONEDNN_VERBOSE");
        if (!e) e = std::getenv("DNNL_VERBOSE");
        g_verbose = e ? std::atoi(e) : 0;
    }
    return g_verbose;
}

extern "C" {

// ======================= engine =============================================
size_t dnnl_engine_get_count(dnnl_engine_kind_t kind) {
    if (kind != dnnl_gpu) return 0;
    return (size_t)qmm_device_count();
}

dnnl_status_t dnnl_engine_create(
        dnnl_engine_t *engine, dnnl_engine_kind_t kind, size_t index) {
    if (!engine) return dnnl_invalid_arguments;
    if (kind != dnnl_gpu) return dnnl_invalid_arguments; // no CPU runtime
    int device = (int)index;
    if (index >= (size_t)qmm_device_count()) {
        // Descriptor-only engine: primitive descriptors can be created and
        // queried on a host without a GPU; anything touching device memory
        // fails with dnnl_runtime_error.
        const char *e = std::getenv("DNNL_AMD_DESCRIPTOR_ONLY");
        if (!(e && e[0] == '1' && index == 0)) return dnnl_invalid_arguments;
        device = -1;
    }
    dnnl_engine *p = new (std::nothrow) dnnl_engine {kind, device};
    if (!p) return dnnl_out_of_memory;
    *engine = p;
    return dnnl_success;
}

dnnl_status_t dnnl_engine_get_kind(
        dnnl_engine_t engine, dnnl_engine_kind_t *kind) {
    if (!engine || !kind) return dnnl_invalid_arguments;
    *kind = engine->kind;
    return dnnl_success;
}

dnnl_status_t dnnl_engine_destroy(dnnl_engine_t engine) {
    if (engine && --engine->refs == 0) delete engine;
    return dnnl_success;
}

// ======================= stream =============================================
dnnl_status_t dnnl_stream_create(
        dnnl_stream_t *stream, dnnl_engine_t engine, unsigned flags) {
    if (!stream || !engine) return dnnl_invalid_arguments;
    if (!(flags & (dnnl_stream_in_order | dnnl_stream_out_of_order)))
        return dnnl_invalid_arguments;
    if (!set_device(engine)) return dnnl_runtime_error;
    hipStream_t s = nullptr;
    // default priority, does not synchronize with the null stream
    if (hipStreamCreateWithFlags(&s, hipStreamNonBlocking) != hipSuccess)
        return dnnl_runtime_error;
    dnnl_stream *p = new (std::nothrow) dnnl_stream {engine, s, true, flags};
    if (!p) {
        (void)hipStreamDestroy(s);
        return dnnl_out_of_memory;
    }
    engine->refs++;
    *stream = p;
    return dnnl_success;
}

dnnl_status_t dnnl_stream_get_engine(
        const_dnnl_stream_t stream, dnnl_engine_t *engine) {
    if (!stream || !engine) return dnnl_invalid_arguments;
    *engine = stream->engine;
    return dnnl_success;
}

dnnl_status_t dnnl_stream_wait(dnnl_stream_t stream) {
    if (!stream) return dnnl_invalid_arguments;
    if (!set_device(stream->engine)) return dnnl_runtime_error;
    return hipStreamSynchronize((hipStream_t)stream->hip_stream) == hipSuccess
            ? dnnl_success
            : dnnl_runtime_error;
}

dnnl_status_t dnnl_stream_destroy(dnnl_stream_t stream) {
    if (!stream) return dnnl_success;
    if (stream->owns_stream && stream->hip_stream && set_device(stream->engine))
        (void)hipStreamDestroy((hipStream_t)stream->hip_stream);
    dnnl_engine_destroy(stream->engine);
    delete stream;
    return dnnl_success;
}

// HIP interop (no counterpart in the reference, which reaches AMD GPUs through
// SYCL): wrap a caller-owned hipStream_t, e.g. the framework's current stream.
DNNL_API dnnl_status_t dnnl_hip_interop_stream_create(
        dnnl_stream_t *stream, dnnl_engine_t engine, void *hip_stream) {
    if (!stream || !engine) return dnnl_invalid_arguments;
    if (engine->device < 0) return dnnl_runtime_error;
    dnnl_stream *p = new (std::nothrow)
            dnnl_stream {engine, hip_stream, false, dnnl_stream_in_order};
    if (!p) return dnnl_out_of_memory;
    engine->refs++;
    *stream = p;
    return dnnl_success;
}

DNNL_API dnnl_status_t dnnl_hip_interop_stream_get_stream(
        dnnl_stream_t stream, void **hip_stream) {
    if (!stream || !hip_stream) return dnnl_invalid_arguments;
    *hip_stream = stream->hip_stream;
    return dnnl_success;
}

// ======================= library-wide =======================================
dnnl_status_t dnnl_get_default_fpmath_mode(dnnl_fpmath_mode_t *mode) {
    if (!mode) return dnnl_invalid_arguments;
    *mode = g_default_fpmath;
    return dnnl_success;
}
dnnl_status_t dnnl_set_default_fpmath_mode(dnnl_fpmath_mode_t mode) {
    if ((int)mode < 0 || mode > dnnl_fpmath_mode_tf32)
        return dnnl_invalid_arguments;
    g_default_fpmath = mode;
    return dnnl_success;
}
dnnl_status_t dnnl_set_verbose(int level) {
    if (level < 0 || level > 2) return dnnl_invalid_arguments;
    g_verbose = level;
    return dnnl_success;
}
const dnnl_version_t *dnnl_version(void) {
    static const dnnl_version_t v = {DNNL_VERSION_MAJOR, DNNL_VERSION_MINOR,
            DNNL_VERSION_PATCH, "mi355x-qmatmul", DNNL_CPU_RUNTIME,
            DNNL_GPU_RUNTIME};
    return &v;
}

// ======================= memory descriptors =================================
dnnl_status_t dnnl_memory_desc_destroy(dnnl_memory_desc_t md) {
    delete md;
    return dnnl_success;
}

dnnl_status_t dnnl_memory_desc_clone(
        dnnl_memory_desc_t *md, const_dnnl_memory_desc_t existing) {
    if (!md || !existing) return dnnl_invalid_arguments;
    *md = new (std::nothrow) dnnl_memory_desc(*existing);
    return *md ? dnnl_success : dnnl_out_of_memory;
}

dnnl_status_t dnnl_memory_desc_create_with_strides(dnnl_memory_desc_t *md,
        int ndims, const dnnl_dims_t dims, dnnl_data_type_t data_type,
        const dnnl_dims_t strides) {
    if (!md) return dnnl_invalid_arguments;
    dnnl_memory_desc tmp;
    if (!md_init_plain(tmp, ndims, dims, data_type, strides))
        return dnnl_invalid_arguments;
    *md = new (std::nothrow) dnnl_memory_desc(tmp);
    return *md ? dnnl_success : dnnl_out_of_memory;
}

dnnl_status_t dnnl_memory_desc_create_with_tag(dnnl_memory_desc_t *md,
        int ndims, const dnnl_dims_t dims, dnnl_data_type_t data_type,
        dnnl_format_tag_t tag) {
    if (!md) return dnnl_invalid_arguments;
    dnnl_memory_desc tmp;
    if (ndims == 0) {
        *md = new (std::nothrow) dnnl_memory_desc();
        return *md ? dnnl_success : dnnl_out_of_memory;
    }
    if (!dims_ok(ndims, dims) || dt_bits(data_type) == 0)
        return dnnl_invalid_arguments;
    if (tag == dnnl_format_tag_any || tag == dnnl_format_tag_undef) {
        tmp.ndims = ndims;
        std::copy(dims, dims + ndims, tmp.dims);
        tmp.data_type = data_type;
        tmp.format_kind = tag == dnnl_format_tag_any ? dnnl_format_kind_any
                                                     : dnnl_format_kind_undef;
    } else {
        if (tag < dnnl_a || tag >= dnnl_format_tag_last)
            return dnnl_invalid_arguments;
        const char *name = tag_names[tag - dnnl_a];
        if ((int)std::strlen(name) != ndims) return dnnl_invalid_arguments;
        dnnl_dims_t strides;
        int64_t s = 1;
        for (int i = ndims - 1; i >= 0; i--) {
            const int d = name[i] - 'a';
            strides[d] = s;
            if (dims[d] == DNNL_RUNTIME_DIM_VAL || s == DNNL_RUNTIME_DIM_VAL)
                s = DNNL_RUNTIME_DIM_VAL;
            else if (dims[d] != 0)
                s *= dims[d];
        }
        if (!md_init_plain(tmp, ndims, dims, data_type, strides))
            return dnnl_invalid_arguments;
    }
    *md = new (std::nothrow) dnnl_memory_desc(tmp);
    return *md ? dnnl_success : dnnl_out_of_memory;
}

dnnl_status_t dnnl_memory_desc_reshape(dnnl_memory_desc_t *out,
        const_dnnl_memory_desc_t in, int ndims, const dnnl_dims_t dims) {
    if (!out || !in || !dims_ok(ndims, dims)) return dnnl_invalid_arguments;
    if (!in->is_plain() || in->has_runtime_dims()) return dnnl_invalid_arguments;
    int64_t n = 1;
    for (int d = 0; d < ndims; d++)
        n *= dims[d];
    if (n != in->nelems()) return dnnl_invalid_arguments;
    // only dense row-major tensors reshape freely; otherwise dims of one may
    // be inserted or dropped
    dnnl_memory_desc dense;
    md_init_plain(dense, in->ndims, in->dims, in->data_type, nullptr);
    dnnl_memory_desc tmp;
    if (md_equal(dense, *in)) {
        if (!md_init_plain(tmp, ndims, dims, in->data_type, nullptr))
            return dnnl_invalid_arguments;
    } else {
        dnnl_dims_t strides;
        int i = 0;
        for (int d = 0; d < ndims; d++) {
            while (i < in->ndims && in->dims[i] == 1 && dims[d] != 1)
                i++;
            if (dims[d] == 1 && !(i < in->ndims && in->dims[i] == 1)) {
                strides[d] = i < in->ndims ? in->strides[i] * in->dims[i] : 1;
                continue;
            }
            if (i >= in->ndims || in->dims[i] != dims[d])
                return dnnl_invalid_arguments;
            strides[d] = in->strides[i++];
        }
        while (i < in->ndims && in->dims[i] == 1)
            i++;
        if (i != in->ndims) return dnnl_invalid_arguments;
        tmp = *in;
        tmp.ndims = ndims;
        std::copy(dims, dims + ndims, tmp.dims);
        std::copy(strides, strides + ndims, tmp.strides);
    }
    *out = new (std::nothrow) dnnl_memory_desc(tmp);
    return *out ? dnnl_success : dnnl_out_of_memory;
}

dnnl_status_t dnnl_memory_desc_permute_axes(dnnl_memory_desc_t *out,
        const_dnnl_memory_desc_t in, const int *perm) {
    if (!out || !in || !perm) return dnnl_invalid_arguments;
    if (!in->is_plain() && !in->is_any()) return dnnl_invalid_arguments;
    bool seen[DNNL_MAX_NDIMS] = {};
    for (int d = 0; d < in->ndims; d++) {
        if (perm[d] < 0 || perm[d] >= in->ndims || seen[perm[d]])
            return dnnl_invalid_arguments;
        seen[perm[d]] = true;
    }
    // axis d of the input becomes axis perm[d] of the output
    dnnl_memory_desc tmp = *in;
    for (int d = 0; d < in->ndims; d++) {
        tmp.dims[perm[d]] = in->dims[d];
        tmp.strides[perm[d]] = in->strides[d];
    }
    *out = new (std::nothrow) dnnl_memory_desc(tmp);
    return *out ? dnnl_success : dnnl_out_of_memory;
}

dnnl_status_t dnnl_memory_desc_query(
        const_dnnl_memory_desc_t md, dnnl_query_t what, void *result) {
    if (!md || !result) return dnnl_invalid_arguments;
    static const dnnl_dims_t zeros = {};
    switch (what) {
        case dnnl_query_ndims_s32: *(int32_t *)result = md->ndims; break;
        case dnnl_query_dims: *(const dnnl_dims_t **)result = &md->dims; break;
        case dnnl_query_padded_dims:
            *(const dnnl_dims_t **)result = &md->dims;
            break;
        case dnnl_query_padded_offsets:
            *(const dnnl_dims_t **)result = &zeros;
            break;
        case dnnl_query_data_type:
            *(dnnl_data_type_t *)result = md->data_type;
            break;
        case dnnl_query_submemory_offset_s64:
            *(int64_t *)result = md->offset0;
            break;
        case dnnl_query_format_kind:
            *(dnnl_format_kind_t *)result = md->format_kind;
            break;
        case dnnl_query_strides:
            if (!md->is_plain()) return dnnl_invalid_arguments;
            *(const dnnl_dims_t **)result = &md->strides;
            break;
        case dnnl_query_inner_nblks_s32:
            if (!md->is_plain()) return dnnl_invalid_arguments;
            *(int32_t *)result = 0;
            break;
        case dnnl_query_inner_blks:
        case dnnl_query_inner_idxs:
            if (!md->is_plain()) return dnnl_invalid_arguments;
            *(const dnnl_dims_t **)result = &zeros;
            break;
        default: return dnnl_unimplemented;
    }
    return dnnl_success;
}

int dnnl_memory_desc_equal(
        const_dnnl_memory_desc_t lhs, const_dnnl_memory_desc_t rhs) {
    if (lhs == rhs) return 1;
    if (!lhs || !rhs) return 0;
    return md_equal(*lhs, *rhs);
}

size_t dnnl_memory_desc_get_size(const_dnnl_memory_desc_t md) {
    return md ? md_size(*md) : 0;
}

size_t dnnl_data_type_size(dnnl_data_type_t dt) {
    const size_t bits = dt_bits(dt);
    if (bits == 0) return (size_t)-1;
    return bits < 8 ? 1 : bits / 8; // 4-bit types report one byte
}

// ======================= memory =============================================
dnnl_status_t dnnl_memory_create(dnnl_memory_t *memory,
        const_dnnl_memory_desc_t md, dnnl_engine_t engine, void *handle) {
    if (!memory || !md || !engine) return dnnl_invalid_arguments;
    if (md->is_any() || md->has_runtime_dims()) return dnnl_invalid_arguments;
    void *ptr = handle;
    bool owns = false;
    if (handle == DNNL_MEMORY_ALLOCATE) {
        ptr = nullptr;
        const size_t sz = md_size(*md);
        if (sz) {
            if (!set_device(engine)) return dnnl_runtime_error;
            if (hipMalloc(&ptr, sz) != hipSuccess) return dnnl_out_of_memory;
            owns = true;
        }
    }
    dnnl_memory *m
            = new (std::nothrow) dnnl_memory {engine, *md, ptr, owns, nullptr};
    if (!m) {
        if (owns) (void)hipFree(ptr);
        return dnnl_out_of_memory;
    }
    engine->refs++;
    *memory = m;
    return dnnl_success;
}

dnnl_status_t dnnl_memory_get_memory_desc(
        const_dnnl_memory_t memory, const_dnnl_memory_desc_t *md) {
    if (!memory || !md) return dnnl_invalid_arguments;
    *md = &memory->md;
    return dnnl_success;
}

dnnl_status_t dnnl_memory_get_engine(
        const_dnnl_memory_t memory, dnnl_engine_t *engine) {
    if (!memory || !engine) return dnnl_invalid_arguments;
    *engine = memory->engine;
    return dnnl_success;
}

dnnl_status_t dnnl_memory_map_data(const_dnnl_memory_t memory, void **mapped) {
    if (!memory || !mapped) return dnnl_invalid_arguments;
    dnnl_memory *m = const_cast<dnnl_memory *>(memory);
    const size_t sz = md_size(m->md);
    *mapped = nullptr;
    if (sz == 0 || !m->handle) return dnnl_success;
    if (m->mapped) return dnnl_runtime_error;
    if (!set_device(m->engine)) return dnnl_runtime_error;
    void *host_ptr = nullptr;
    if (hipHostMalloc(&host_ptr, sz, hipHostMallocDefault) != hipSuccess)
        return dnnl_out_of_memory;
    // all streams of the engine are drained first: the map is a sync point
    if (hipDeviceSynchronize() != hipSuccess
            || hipMemcpy(host_ptr, m->handle, sz, hipMemcpyDeviceToHost)
                    != hipSuccess) {
        (void)hipHostFree(host_ptr);
        return dnnl_runtime_error;
    }
    m->mapped = host_ptr;
    *mapped = host_ptr;
    return dnnl_success;
}

dnnl_status_t dnnl_memory_unmap_data(const_dnnl_memory_t memory, void *mapped) {
    if (!memory) return dnnl_invalid_arguments;
    dnnl_memory *m = const_cast<dnnl_memory *>(memory);
    if (!mapped && !m->mapped) return dnnl_success;
    if (mapped != m->mapped) return dnnl_invalid_arguments;
    if (!set_device(m->engine)) return dnnl_runtime_error;
    const size_t sz = md_size(m->md);
    const bool ok
            = hipMemcpy(m->handle, mapped, sz, hipMemcpyHostToDevice) == hipSuccess;
    (void)hipHostFree(mapped);
    m->mapped = nullptr;
    return ok ? dnnl_success : dnnl_runtime_error;
}

dnnl_status_t dnnl_memory_get_data_handle(
        const_dnnl_memory_t memory, void **handle) {
    if (!memory || !handle) return dnnl_invalid_arguments;
    *handle = memory->handle;
    return dnnl_success;
}

dnnl_status_t dnnl_memory_set_data_handle(dnnl_memory_t memory, void *handle) {
    if (!memory) return dnnl_invalid_arguments;
    if (memory->owns_handle && memory->handle && set_device(memory->engine))
        (void)hipFree(memory->handle);
    memory->handle = handle;
    memory->owns_handle = false;
    return dnnl_success;
}

dnnl_status_t dnnl_memory_destroy(dnnl_memory_t memory) {
    if (!memory) return dnnl_success;
    if (memory->mapped) (void)hipHostFree(memory->mapped);
    if (memory->owns_handle && memory->handle && set_device(memory->engine))
        (void)hipFree(memory->handle);
    dnnl_engine_destroy(memory->engine);
    delete memory;
    return dnnl_success;
}

// ======================= attributes =========================================
dnnl_status_t dnnl_primitive_attr_create(dnnl_primitive_attr_t *attr) {
    if (!attr) return dnnl_invalid_arguments;
    *attr = new (std::nothrow) dnnl_primitive_attr();
    if (!*attr) return dnnl_out_of_memory;
    (*attr)->fpmath_mode = g_default_fpmath;
    return dnnl_success;
}
dnnl_status_t dnnl_primitive_attr_clone(
        dnnl_primitive_attr_t *attr, const_dnnl_primitive_attr_t existing) {
    if (!attr || !existing) return dnnl_invalid_arguments;
    *attr = new (std::nothrow) dnnl_primitive_attr(*existing);
    return *attr ? dnnl_success : dnnl_out_of_memory;
}
dnnl_status_t dnnl_primitive_attr_destroy(dnnl_primitive_attr_t attr) {
    delete attr;
    return dnnl_success;
}
dnnl_status_t dnnl_primitive_attr_get_fpmath_mode(
        const_dnnl_primitive_attr_t attr, dnnl_fpmath_mode_t *mode) {
    if (!attr || !mode) return dnnl_invalid_arguments;
    *mode = attr->fpmath_mode;
    return dnnl_success;
}
dnnl_status_t dnnl_primitive_attr_set_fpmath_mode(
        dnnl_primitive_attr_t attr, dnnl_fpmath_mode_t mode) {
    return dnnl_primitive_attr_set_fpmath_mode_v2(attr, mode, 0);
}
dnnl_status_t dnnl_primitive_attr_get_fpmath_mode_v2(
        const_dnnl_primitive_attr_t attr, dnnl_fpmath_mode_t *mode,
        int *apply_to_int) {
    if (!attr) return dnnl_invalid_arguments;
    if (mode) *mode = attr->fpmath_mode;
    if (apply_to_int) *apply_to_int = attr->fpmath_apply_to_int;
    return dnnl_success;
}
dnnl_status_t dnnl_primitive_attr_set_fpmath_mode_v2(
        dnnl_primitive_attr_t attr, dnnl_fpmath_mode_t mode, int apply_to_int) {
    if (!attr) return dnnl_invalid_arguments;
    if ((int)mode < 0 || mode > dnnl_fpmath_mode_tf32)
        return dnnl_invalid_arguments;
    attr->fpmath_mode = mode;
    attr->fpmath_apply_to_int = apply_to_int != 0;
    return dnnl_success;
}
// src/common/primitive_attr.cpp:430-442, primitive_attr.hpp:351-356
dnnl_status_t dnnl_primitive_attr_get_dropout(const_dnnl_primitive_attr_t attr,
        const_dnnl_memory_desc_t *dropout_desc) {
    if (!attr) return dnnl_invalid_arguments;
    if (dropout_desc) *dropout_desc = &attr->dropout_desc;
    return dnnl_success;
}
dnnl_status_t dnnl_primitive_attr_set_dropout(
        dnnl_primitive_attr_t attr, const_dnnl_memory_desc_t dropout_desc) {
    if (!attr || !dropout_desc) return dnnl_invalid_arguments;
    attr->dropout_desc = *dropout_desc;
    return dnnl_success;
}
// src/common/primitive_attr.cpp:564-575, primitive_attr.hpp:207-238: only
// dst and the gradients may take a non-default mode; the default is not stored
dnnl_status_t dnnl_primitive_attr_get_rounding(
        dnnl_primitive_attr_t attr, int arg, dnnl_rounding_mode_t *mode) {
    if (!attr || !mode) return dnnl_invalid_arguments;
    auto it = attr->rounding.find(arg);
    *mode = it == attr->rounding.end() ? dnnl_rounding_mode_environment
                                       : it->second;
    return dnnl_success;
}
dnnl_status_t dnnl_primitive_attr_set_rounding(
        dnnl_primitive_attr_t attr, int arg, dnnl_rounding_mode_t mode) {
    if (!attr) return dnnl_invalid_arguments;
    if (mode != dnnl_rounding_mode_environment) {
        if (arg != DNNL_ARG_DST && arg != DNNL_ARG_DIFF_SRC
                && arg != DNNL_ARG_DIFF_WEIGHTS)
            return dnnl_invalid_arguments;
        attr->rounding[arg] = mode;
    }
    return dnnl_success;
}
dnnl_status_t dnnl_primitive_attr_get_deterministic(
        const_dnnl_primitive_attr_t attr, int *value) {
    if (!attr || !value) return dnnl_invalid_arguments;
    *value = attr->deterministic;
    return dnnl_success;
}
dnnl_status_t dnnl_primitive_attr_set_deterministic(
        dnnl_primitive_attr_t attr, int value) {
    if (!attr) return dnnl_invalid_arguments;
    attr->deterministic = value != 0;
    return dnnl_success;
}
dnnl_status_t dnnl_primitive_attr_get_accumulation_mode(
        const_dnnl_primitive_attr_t attr, dnnl_accumulation_mode_t *mode) {
    if (!attr || !mode) return dnnl_invalid_arguments;
    *mode = attr->acc_mode;
    return dnnl_success;
}
dnnl_status_t dnnl_primitive_attr_set_accumulation_mode(
        dnnl_primitive_attr_t attr, dnnl_accumulation_mode_t mode) {
    if (!attr) return dnnl_invalid_arguments;
    if ((int)mode < 0 || mode > dnnl_accumulation_mode_f16)
        return dnnl_invalid_arguments;
    attr->acc_mode = mode;
    return dnnl_success;
}
dnnl_status_t dnnl_primitive_attr_get_scratchpad_mode(
        const_dnnl_primitive_attr_t attr, dnnl_scratchpad_mode_t *mode) {
    if (!attr || !mode) return dnnl_invalid_arguments;
    *mode = attr->scratchpad_mode;
    return dnnl_success;
}
dnnl_status_t dnnl_primitive_attr_set_scratchpad_mode(
        dnnl_primitive_attr_t attr, dnnl_scratchpad_mode_t mode) {
    if (!attr) return dnnl_invalid_arguments;
    if (mode != dnnl_scratchpad_mode_library && mode != dnnl_scratchpad_mode_user)
        return dnnl_invalid_arguments;
    attr->scratchpad_mode = mode;
    return dnnl_success;
}

// src/common/primitive_attr.cpp:513-562 and the argument whitelists of
// src/common/primitive_attr_quant.hpp:235-324
static bool scales_arg_ok(int arg) {
    if (arg == DNNL_ARG_SRC || arg == DNNL_ARG_SRC_1 || arg == DNNL_ARG_SRC_2
            || arg == DNNL_ARG_WEIGHTS || arg == DNNL_ARG_DST)
        return true;
    if (arg & 1024) return true; // DNNL_ARG_MULTIPLE_SRC (concat)
    const int dw = 16384; // DNNL_ARG_ATTR_POST_OP_DW
    return arg == (dw | DNNL_ARG_SRC) || arg == (dw | DNNL_ARG_WEIGHTS)
            || arg == (dw | DNNL_ARG_DST);
}
static bool zp_arg_ok(int arg) {
    return arg == DNNL_ARG_SRC || arg == DNNL_ARG_WEIGHTS || arg == DNNL_ARG_DST
            || arg == DNNL_ARG_SRC_2;
}
static bool group_dims_ok(int ndims, const dnnl_dims_t g) {
    if (ndims == 0) return true;
    if (ndims < 0 || ndims > DNNL_MAX_NDIMS || !g) return false;
    for (int d = 0; d < ndims; d++)
        if (g[d] < 0) return false;
    return true;
}
static void quant_set(std::map<int, quant_entry_t> &m, int arg, int mask,
        dnnl_data_type_t dt, int ndims, const dnnl_dims_t g) {
    quant_entry_t e;
    e.mask = mask;
    e.dt = dt;
    e.group_ndims = ndims;
    for (int d = 0; d < ndims; d++)
        e.group_dims[d] = g[d];
    m[arg] = e;
}

dnnl_status_t dnnl_primitive_attr_set_scales_mask(
        dnnl_primitive_attr_t attr, int arg, int mask) {
    if (!attr || mask < 0 || arg < 0) return dnnl_invalid_arguments;
    if (!scales_arg_ok(arg)) return dnnl_invalid_arguments;
    quant_set(attr->scales, arg, mask, dnnl_f32, 0, nullptr);
    return dnnl_success;
}
dnnl_status_t dnnl_primitive_attr_set_scales(dnnl_primitive_attr_t attr,
        int arg, int mask, int ndims, const dnnl_dims_t group_dims,
        dnnl_data_type_t dt) {
    if (!attr || mask < 0 || arg < 0 || ndims < 0) return dnnl_invalid_arguments;
    if (dt != dnnl_f32 && dt != dnnl_bf16 && dt != dnnl_f16 && dt != dnnl_e8m0
            && dt != dnnl_f8_e5m2 && dt != dnnl_f8_e4m3)
        return dnnl_invalid_arguments;
    if (!group_dims_ok(ndims, group_dims)) return dnnl_invalid_arguments;
    if (!scales_arg_ok(arg)) return dnnl_invalid_arguments;
    quant_set(attr->scales, arg, mask, dt, ndims, group_dims);
    return dnnl_success;
}
dnnl_status_t dnnl_primitive_attr_set_zero_points_mask(
        dnnl_primitive_attr_t attr, int arg, int mask) {
    if (!attr || mask < 0) return dnnl_invalid_arguments;
    if (!zp_arg_ok(arg)) return dnnl_invalid_arguments;
    quant_set(attr->zero_points, arg, mask, dnnl_s32, 0, nullptr);
    return dnnl_success;
}
dnnl_status_t dnnl_primitive_attr_set_zero_points(dnnl_primitive_attr_t attr,
        int arg, int mask, int ndims, const dnnl_dims_t group_dims,
        dnnl_data_type_t dt) {
    if (!attr || mask < 0 || arg < 0 || ndims < 0) return dnnl_invalid_arguments;
    if (dt != dnnl_s32 && dt != dnnl_s8 && dt != dnnl_u8 && dt != dnnl_s4
            && dt != dnnl_u4)
        return dnnl_invalid_arguments;
    if ((dt == dnnl_s4 || dt == dnnl_u4) && mask <= 0)
        return dnnl_invalid_arguments;
    if (arg != DNNL_ARG_SRC && arg != DNNL_ARG_WEIGHTS
            && !(dt == dnnl_s32 && ndims == 0))
        return dnnl_invalid_arguments;
    if (!group_dims_ok(ndims, group_dims)) return dnnl_invalid_arguments;
    if (!zp_arg_ok(arg)) return dnnl_invalid_arguments;
    quant_set(attr->zero_points, arg, mask, dt, ndims, group_dims);
    return dnnl_success;
}

dnnl_status_t dnnl_primitive_attr_get_post_ops(
        const_dnnl_primitive_attr_t attr, const_dnnl_post_ops_t *post_ops) {
    if (!attr || !post_ops) return dnnl_invalid_arguments;
    *post_ops = &attr->post_ops;
    return dnnl_success;
}
dnnl_status_t dnnl_primitive_attr_set_post_ops(
        dnnl_primitive_attr_t attr, const_dnnl_post_ops_t post_ops) {
    if (!attr || !post_ops) return dnnl_invalid_arguments;
    if ((int)post_ops->entries.size() > dnnl_post_ops::limit)
        return dnnl_invalid_arguments;
    attr->post_ops = *post_ops;
    return dnnl_success;
}

// ======================= post-ops ===========================================
dnnl_status_t dnnl_post_ops_create(dnnl_post_ops_t *post_ops) {
    if (!post_ops) return dnnl_invalid_arguments;
    *post_ops = new (std::nothrow) dnnl_post_ops();
    return *post_ops ? dnnl_success : dnnl_out_of_memory;
}
dnnl_status_t dnnl_post_ops_clone(
        dnnl_post_ops_t *post_ops, const_dnnl_post_ops_t existing) {
    if (!post_ops || !existing) return dnnl_invalid_arguments;
    *post_ops = new (std::nothrow) dnnl_post_ops(*existing);
    return *post_ops ? dnnl_success : dnnl_out_of_memory;
}
dnnl_status_t dnnl_post_ops_destroy(dnnl_post_ops_t post_ops) {
    delete post_ops;
    return dnnl_success;
}
int dnnl_post_ops_len(const_dnnl_post_ops_t post_ops) {
    return post_ops ? (int)post_ops->entries.size() : 0;
}
dnnl_primitive_kind_t dnnl_post_ops_get_kind(
        const_dnnl_post_ops_t post_ops, int index) {
    if (!post_ops || index < 0 || index >= (int)post_ops->entries.size())
        return dnnl_undefined_primitive;
    return post_ops->entries[index].kind;
}

// src/common/primitive_attr.cpp:150-265
dnnl_status_t dnnl_post_ops_append_sum(dnnl_post_ops_t post_ops, float scale,
        int32_t zero_point, dnnl_data_type_t dt) {
    if (!post_ops) return dnnl_invalid_arguments;
    if ((int)post_ops->entries.size() == dnnl_post_ops::limit)
        return dnnl_out_of_memory;
    if (is_runtime_f32(scale)) return dnnl_invalid_arguments;
    post_op_entry_t e;
    e.kind = dnnl_sum;
    e.sum_scale = scale;
    e.sum_zero_point = zero_point;
    e.sum_dt = dt;
    post_ops->entries.push_back(e);
    return dnnl_success;
}
dnnl_status_t dnnl_post_ops_get_params_sum(const_dnnl_post_ops_t post_ops,
        int index, float *scale, int32_t *zero_point, dnnl_data_type_t *dt) {
    if (!post_ops || index < 0 || index >= (int)post_ops->entries.size()
            || post_ops->entries[index].kind != dnnl_sum)
        return dnnl_invalid_arguments;
    const post_op_entry_t &e = post_ops->entries[index];
    if (scale) *scale = e.sum_scale;
    if (zero_point) *zero_point = e.sum_zero_point;
    if (dt) *dt = e.sum_dt;
    return dnnl_success;
}
dnnl_status_t dnnl_post_ops_append_eltwise(dnnl_post_ops_t post_ops,
        dnnl_alg_kind_t alg, float alpha, float beta) {
    if (!post_ops) return dnnl_invalid_arguments;
    if ((int)post_ops->entries.size() == dnnl_post_ops::limit)
        return dnnl_out_of_memory;
    if (!eltwise_ok(alg, alpha, beta)) return dnnl_invalid_arguments;
    if (is_runtime_f32(alpha) || is_runtime_f32(beta))
        return dnnl_invalid_arguments;
    post_op_entry_t e;
    e.kind = dnnl_eltwise;
    e.alg = alg;
    e.alpha = alpha;
    e.beta = beta;
    e.eltwise_scale = 1.f;
    post_ops->entries.push_back(e);
    return dnnl_success;
}
dnnl_status_t dnnl_post_ops_get_params_eltwise(const_dnnl_post_ops_t post_ops,
        int index, dnnl_alg_kind_t *alg, float *alpha, float *beta) {
    if (!post_ops || index < 0 || index >= (int)post_ops->entries.size()
            || post_ops->entries[index].kind != dnnl_eltwise)
        return dnnl_invalid_arguments;
    const post_op_entry_t &e = post_ops->entries[index];
    if (alg) *alg = e.alg;
    if (alpha) *alpha = e.alpha;
    if (beta) *beta = e.beta;
    return dnnl_success;
}
dnnl_status_t dnnl_post_ops_append_binary(dnnl_post_ops_t post_ops,
        dnnl_alg_kind_t alg, const_dnnl_memory_desc_t src1_desc) {
    if (!post_ops || !src1_desc) return dnnl_invalid_arguments;
    if ((int)post_ops->entries.size() == dnnl_post_ops::limit)
        return dnnl_out_of_memory;
    if (alg < dnnl_binary_add || alg > dnnl_binary_ne)
        return dnnl_invalid_arguments;
    if (src1_desc->ndims == 0 || src1_desc->has_runtime_dims())
        return dnnl_invalid_arguments;
    post_op_entry_t e;
    e.kind = dnnl_binary;
    e.alg = alg;
    e.user_src1_desc = *src1_desc;
    e.src1_desc = *src1_desc;
    post_ops->entries.push_back(e);
    return dnnl_success;
}
dnnl_status_t dnnl_post_ops_get_params_binary(const_dnnl_post_ops_t post_ops,
        int index, dnnl_alg_kind_t *alg, const_dnnl_memory_desc_t *src1_desc) {
    if (!post_ops || index < 0 || index >= (int)post_ops->entries.size()
            || post_ops->entries[index].kind != dnnl_binary)
        return dnnl_invalid_arguments;
    const post_op_entry_t &e = post_ops->entries[index];
    if (alg) *alg = e.alg;
    if (src1_desc) *src1_desc = &e.user_src1_desc;
    return dnnl_success;
}
dnnl_status_t dnnl_post_ops_append_prelu(dnnl_post_ops_t post_ops, int mask) {
    if (!post_ops) return dnnl_invalid_arguments;
    if ((int)post_ops->entries.size() == dnnl_post_ops::limit)
        return dnnl_out_of_memory;
    post_op_entry_t e;
    e.kind = dnnl_prelu;
    e.prelu_mask = mask;
    post_ops->entries.push_back(e);
    return dnnl_success;
}
dnnl_status_t dnnl_post_ops_get_params_prelu(
        const_dnnl_post_ops_t post_ops, int index, int *mask) {
    if (!post_ops || index < 0 || index >= (int)post_ops->entries.size()
            || post_ops->entries[index].kind != dnnl_prelu)
        return dnnl_invalid_arguments;
    if (mask) *mask = post_ops->entries[index].prelu_mask;
    return dnnl_success;
}

} // extern "C"

// ---- enumerator names (include/oneapi/dnnl/dnnl_debug.h) --------------------
// One switch per enumeration of the public headers: the enumerator's name
// without its dnnl_ prefix, as the reference's generated
// src/common/dnnl_debug_autogenerated.cpp returns it.
extern "C" {
const char *dnnl_status2str(dnnl_status_t v) {
    switch ((int)v) {
        case dnnl_success: return "success";
        case dnnl_out_of_memory: return "out_of_memory";
        case dnnl_invalid_arguments: return "invalid_arguments";
        case dnnl_unimplemented: return "unimplemented";
        case dnnl_last_impl_reached: return "last_impl_reached";
        case dnnl_runtime_error: return "runtime_error";
        case dnnl_not_required: return "not_required";
        case dnnl_invalid_graph: return "invalid_graph";
        case dnnl_invalid_graph_op: return "invalid_graph_op";
        case dnnl_invalid_shape: return "invalid_shape";
        case dnnl_invalid_data_type: return "invalid_data_type";
        default: return "unknown status";
    }
}
const char *dnnl_dt2str(dnnl_data_type_t v) {
    switch ((int)v) {
        case dnnl_data_type_undef: return "undef";
        case dnnl_f16: return "f16";
        case dnnl_bf16: return "bf16";
        case dnnl_f32: return "f32";
        case dnnl_s32: return "s32";
        case dnnl_s8: return "s8";
        case dnnl_u8: return "u8";
        case dnnl_f64: return "f64";
        case dnnl_boolean: return "boolean";
        case dnnl_f8_e5m2: return "f8_e5m2";
        case dnnl_f8_e4m3: return "f8_e4m3";
        case dnnl_s4: return "s4";
        case dnnl_u4: return "u4";
        case dnnl_e8m0: return "e8m0";
        case dnnl_f4_e2m1: return "f4_e2m1";
        case dnnl_f4_e3m0: return "f4_e3m0";
        default: return "unknown dt";
    }
}
const char *dnnl_fpmath_mode2str(dnnl_fpmath_mode_t v) {
    switch ((int)v) {
        case dnnl_fpmath_mode_strict: return "strict";
        case dnnl_fpmath_mode_bf16: return "bf16";
        case dnnl_fpmath_mode_f16: return "f16";
        case dnnl_fpmath_mode_any: return "any";
        case dnnl_fpmath_mode_tf32: return "tf32";
        default: return "unknown fpmath_mode";
    }
}
const char *dnnl_accumulation_mode2str(dnnl_accumulation_mode_t v) {
    switch ((int)v) {
        case dnnl_accumulation_mode_strict: return "strict";
        case dnnl_accumulation_mode_relaxed: return "relaxed";
        case dnnl_accumulation_mode_any: return "any";
        case dnnl_accumulation_mode_s32: return "s32";
        case dnnl_accumulation_mode_f32: return "f32";
        case dnnl_accumulation_mode_f16: return "f16";
        default: return "unknown accumulation_mode";
    }
}
const char *dnnl_engine_kind2str(dnnl_engine_kind_t v) {
    switch ((int)v) {
        case dnnl_any_engine: return "any";
        case dnnl_cpu: return "cpu";
        case dnnl_gpu: return "gpu";
        default: return "unknown engine_kind";
    }
}
const char *dnnl_fmt_tag2str(dnnl_format_tag_t v) {
    switch ((int)v) {
        case dnnl_format_tag_undef: return "undef";
        case dnnl_format_tag_any: return "any";
        case dnnl_a: return "a";
        case dnnl_ab: return "ab";
        case dnnl_abc: return "abc";
        case dnnl_abcd: return "abcd";
        case dnnl_abcde: return "abcde";
        case dnnl_abcdef: return "abcdef";
        case dnnl_abcdefg: return "abcdefg";
        case dnnl_abcdefgh: return "abcdefgh";
        case dnnl_abcdefghi: return "abcdefghi";
        case dnnl_abcdefghij: return "abcdefghij";
        case dnnl_abcdefghijk: return "abcdefghijk";
        case dnnl_abcdefghijkl: return "abcdefghijkl";
        case dnnl_ba: return "ba";
        case dnnl_acb: return "acb";
        case dnnl_bac: return "bac";
        case dnnl_bca: return "bca";
        case dnnl_cab: return "cab";
        case dnnl_cba: return "cba";
        case dnnl_abdc: return "abdc";
        case dnnl_acbd: return "acbd";
        case dnnl_acdb: return "acdb";
        case dnnl_adbc: return "adbc";
        case dnnl_adcb: return "adcb";
        case dnnl_bacd: return "bacd";
        case dnnl_bcda: return "bcda";
        case dnnl_cdab: return "cdab";
        case dnnl_cdba: return "cdba";
        case dnnl_dcab: return "dcab";
        case dnnl_abced: return "abced";
        case dnnl_abdec: return "abdec";
        case dnnl_acbde: return "acbde";
        case dnnl_acdeb: return "acdeb";
        case dnnl_adecb: return "adecb";
        case dnnl_bacde: return "bacde";
        case dnnl_bcdea: return "bcdea";
        case dnnl_cdeab: return "cdeab";
        case dnnl_cdeba: return "cdeba";
        case dnnl_decab: return "decab";
        case dnnl_abcdfe: return "abcdfe";
        case dnnl_abdefc: return "abdefc";
        case dnnl_abdfce: return "abdfce";
        case dnnl_acbdef: return "acbdef";
        case dnnl_adefcb: return "adefcb";
        case dnnl_defcab: return "defcab";
        case dnnl_abcdegf: return "abcdegf";
        case dnnl_abcdefhg: return "abcdefhg";
        case dnnl_abcdefgih: return "abcdefgih";
        case dnnl_abcdefghji: return "abcdefghji";
        case dnnl_abcdefghikj: return "abcdefghikj";
        case dnnl_abcdefghijlk: return "abcdefghijlk";
        default: return "unknown fmt_tag";
    }
}
const char *dnnl_prop_kind2str(dnnl_prop_kind_t v) {
    switch ((int)v) {
        case dnnl_prop_kind_undef: return "undef";
        case dnnl_forward_training: return "forward_training";
        case dnnl_forward_inference: return "forward_inference";
        default: return "unknown prop_kind";
    }
}
const char *dnnl_prim_kind2str(dnnl_primitive_kind_t v) {
    switch ((int)v) {
        case dnnl_undefined_primitive: return "undef";
        case dnnl_reorder: return "reorder";
        case dnnl_shuffle: return "shuffle";
        case dnnl_concat: return "concat";
        case dnnl_sum: return "sum";
        case dnnl_convolution: return "convolution";
        case dnnl_deconvolution: return "deconvolution";
        case dnnl_eltwise: return "eltwise";
        case dnnl_lrn: return "lrn";
        case dnnl_batch_normalization: return "batch_normalization";
        case dnnl_inner_product: return "inner_product";
        case dnnl_rnn: return "rnn";
        case dnnl_gemm: return "gemm";
        case dnnl_binary: return "binary";
        case dnnl_matmul: return "matmul";
        case dnnl_resampling: return "resampling";
        case dnnl_pooling: return "pooling";
        case dnnl_reduction: return "reduction";
        case dnnl_prelu: return "prelu";
        case dnnl_softmax: return "softmax";
        case dnnl_layer_normalization: return "layer_normalization";
        case dnnl_group_normalization: return "group_normalization";
        default: return "unknown prim_kind";
    }
}
const char *dnnl_alg_kind2str(dnnl_alg_kind_t v) {
    switch ((int)v) {
        case dnnl_alg_kind_undef: return "undef";
        case dnnl_eltwise_relu: return "eltwise_relu";
        case dnnl_eltwise_tanh: return "eltwise_tanh";
        case dnnl_eltwise_elu: return "eltwise_elu";
        case dnnl_eltwise_square: return "eltwise_square";
        case dnnl_eltwise_abs: return "eltwise_abs";
        case dnnl_eltwise_sqrt: return "eltwise_sqrt";
        case dnnl_eltwise_linear: return "eltwise_linear";
        case dnnl_eltwise_soft_relu: return "eltwise_soft_relu";
        case dnnl_eltwise_hardsigmoid: return "eltwise_hardsigmoid";
        case dnnl_eltwise_logistic: return "eltwise_logistic";
        case dnnl_eltwise_exp: return "eltwise_exp";
        case dnnl_eltwise_gelu_tanh: return "eltwise_gelu_tanh";
        case dnnl_eltwise_swish: return "eltwise_swish";
        case dnnl_eltwise_log: return "eltwise_log";
        case dnnl_eltwise_clip: return "eltwise_clip";
        case dnnl_eltwise_clip_v2: return "eltwise_clip_v2";
        case dnnl_eltwise_pow: return "eltwise_pow";
        case dnnl_eltwise_gelu_erf: return "eltwise_gelu_erf";
        case dnnl_eltwise_round: return "eltwise_round";
        case dnnl_eltwise_mish: return "eltwise_mish";
        case dnnl_eltwise_hardswish: return "eltwise_hardswish";
        case dnnl_eltwise_relu_use_dst_for_bwd: return "eltwise_relu_use_dst_for_bwd";
        case dnnl_eltwise_tanh_use_dst_for_bwd: return "eltwise_tanh_use_dst_for_bwd";
        case dnnl_eltwise_elu_use_dst_for_bwd: return "eltwise_elu_use_dst_for_bwd";
        case dnnl_eltwise_sqrt_use_dst_for_bwd: return "eltwise_sqrt_use_dst_for_bwd";
        case dnnl_eltwise_logistic_use_dst_for_bwd: return "eltwise_logistic_use_dst_for_bwd";
        case dnnl_eltwise_exp_use_dst_for_bwd: return "eltwise_exp_use_dst_for_bwd";
        case dnnl_eltwise_clip_v2_use_dst_for_bwd: return "eltwise_clip_v2_use_dst_for_bwd";
        case dnnl_binary_add: return "binary_add";
        case dnnl_binary_mul: return "binary_mul";
        case dnnl_binary_max: return "binary_max";
        case dnnl_binary_min: return "binary_min";
        case dnnl_binary_div: return "binary_div";
        case dnnl_binary_sub: return "binary_sub";
        case dnnl_binary_ge: return "binary_ge";
        case dnnl_binary_gt: return "binary_gt";
        case dnnl_binary_le: return "binary_le";
        case dnnl_binary_lt: return "binary_lt";
        case dnnl_binary_eq: return "binary_eq";
        case dnnl_binary_ne: return "binary_ne";
        case dnnl_binary_select: return "binary_select";
        default: return "unknown alg_kind";
    }
}
const char *dnnl_scratchpad_mode2str(dnnl_scratchpad_mode_t v) {
    switch ((int)v) {
        case dnnl_scratchpad_mode_library: return "library";
        case dnnl_scratchpad_mode_user: return "user";
        default: return "unknown scratchpad_mode";
    }
}
const char *dnnl_rounding_mode2str(dnnl_rounding_mode_t v) {
    switch ((int)v) {
        case dnnl_rounding_mode_environment: return "environment";
        case dnnl_rounding_mode_stochastic: return "stochastic";
        default: return "unknown rounding_mode";
    }
}
const char *dnnl_fmt_kind2str(dnnl_format_kind_t v) {
    switch ((int)v) {
        case dnnl_format_kind_undef: return "undef";
        case dnnl_format_kind_any: return "any";
        case dnnl_blocked: return "blocked";
        case dnnl_format_kind_opaque: return "opaque";
        default: return "unknown fmt_kind";
    }
}
const char *dnnl_runtime2str(unsigned v) {
    switch (v) {
        case DNNL_RUNTIME_NONE: return "none";
        case DNNL_RUNTIME_SEQ: return "sequential";
        case DNNL_RUNTIME_OMP: return "OpenMP";
        case DNNL_RUNTIME_TBB: return "TBB";
        case DNNL_RUNTIME_THREADPOOL: return "threadpool";
        case DNNL_RUNTIME_OCL: return "OpenCL";
        case DNNL_RUNTIME_SYCL: return "DPC++";
        case DNNL_RUNTIME_HIP: return "HIP";
        default: return "unknown";
    }
}
} // extern "C"
