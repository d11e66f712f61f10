// Host objects behind the opaque dnnl_* handles of the quantized-matmul library
// (include/oneapi/dnnl/dnnl.h). This is host-only C++: descriptors, attribute
// bookkeeping and the HIP engine / stream / memory wrappers; all computation
// happens in the kernels reached through include/qmm_hip.h.
#pragma once

#include <atomic>
#include <climits>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "oneapi/dnnl/dnnl.h"
#include "qmm_hip.h"

// ---- memory descriptor -----------------------------------------------------
// Plain tensors carry strides (format kind "blocked" with no inner blocks, as
// the reference reports plain layouts); prepacked weights are an opaque
// descriptor that only records which MFMA layout and how many bytes.
struct dnnl_memory_desc {
    int ndims = 0;
    dnnl_dims_t dims = {};
    dnnl_data_type_t data_type = dnnl_data_type_undef;
    dnnl_format_kind_t format_kind = dnnl_format_kind_undef;
    dnnl_dims_t strides = {}; // format_kind == dnnl_blocked
    int64_t offset0 = 0;
    int packed_layout = QMM_LAYOUT_PLAIN; // format_kind == opaque
    size_t packed_bytes = 0;
    // opaque weights of an inner product: dims are [OC, IC, spatial...], the
    // packed image is that of the matmul weights [K = IC * spatial, N = OC]
    bool packed_transposed = false;

    bool is_zero() const { return ndims == 0; }
    bool is_any() const { return format_kind == dnnl_format_kind_any; }
    bool is_plain() const { return format_kind == dnnl_blocked; }
    bool is_packed() const { return format_kind == dnnl_format_kind_opaque; }
    bool has_zero_dim() const {
        for (int d = 0; d < ndims; d++)
            if (dims[d] == 0) return true;
        return false;
    }
    bool has_runtime_dims() const {
        for (int d = 0; d < ndims; d++)
            if (dims[d] == DNNL_RUNTIME_DIM_VAL) return true;
        return false;
    }
    int64_t nelems() const {
        int64_t n = 1;
        for (int d = 0; d < ndims; d++)
            n *= dims[d];
        return ndims ? n : 0;
    }
};

// ---- attributes -------------------------------------------------------------
// One scales / zero-points entry. A default entry has mask INT_MIN and no data
// type (src/common/primitive_attr_quant.hpp:45-119).
struct quant_entry_t {
    int mask = INT_MIN;
    dnnl_data_type_t dt = dnnl_data_type_undef;
    int group_ndims = 0;
    dnnl_dims_t group_dims = {};

    bool is_default() const {
        return mask == INT_MIN && dt == dnnl_data_type_undef && group_ndims == 0;
    }
    bool has_groups() const { return group_ndims > 0; }
    // 1 when no groups were requested; 0 for an out-of-range index
    int64_t group(int d) const {
        if (group_ndims == 0) return 1;
        if (d >= group_ndims) return 0;
        return group_dims[d];
    }
    bool operator==(const quant_entry_t &o) const {
        return mask == o.mask && dt == o.dt && group_ndims == o.group_ndims
                && (group_ndims == 0
                        || !std::memcmp(group_dims, o.group_dims,
                                sizeof(int64_t) * group_ndims));
    }
};

struct post_op_entry_t {
    dnnl_primitive_kind_t kind = dnnl_undefined_primitive;
    // sum
    float sum_scale = 1.f;
    int32_t sum_zero_point = 0;
    dnnl_data_type_t sum_dt = dnnl_data_type_undef;
    // eltwise
    dnnl_alg_kind_t alg = dnnl_alg_kind_undef;
    float alpha = 0.f, beta = 0.f, eltwise_scale = 1.f;
    // binary
    dnnl_memory_desc user_src1_desc, src1_desc;
    // prelu
    int prelu_mask = 0;
};

struct dnnl_post_ops {
    std::vector<post_op_entry_t> entries;
    static constexpr int limit = 32; // src/common/primitive_attr.hpp:510
    int find(dnnl_primitive_kind_t k, int start = 0) const {
        for (int i = start; i < (int)entries.size(); i++)
            if (entries[i].kind == k) return i;
        return -1;
    }
};

struct dnnl_primitive_attr {
    std::map<int, quant_entry_t> scales, zero_points;
    dnnl_fpmath_mode_t fpmath_mode = dnnl_fpmath_mode_strict;
    bool fpmath_apply_to_int = false;
    dnnl_accumulation_mode_t acc_mode = dnnl_accumulation_mode_strict;
    dnnl_scratchpad_mode_t scratchpad_mode = dnnl_scratchpad_mode_library;
    bool deterministic = false;
    dnnl_memory_desc dropout_desc; // zero descriptor: no dropout
    std::map<int, dnnl_rounding_mode_t> rounding; // non-default entries only
    dnnl_post_ops post_ops;

    const quant_entry_t &scale(int arg) const { return get(scales, arg); }
    const quant_entry_t &zp(int arg) const { return get(zero_points, arg); }
    bool has_default_scales() const { return all_default(scales); }
    bool has_default_zps() const { return all_default(zero_points); }

private:
    static const quant_entry_t &get(
            const std::map<int, quant_entry_t> &m, int arg) {
        static const quant_entry_t dflt;
        auto it = m.find(arg);
        return it == m.end() ? dflt : it->second;
    }
    static bool all_default(const std::map<int, quant_entry_t> &m) {
        for (auto &kv : m)
            if (!kv.second.is_default()) return false;
        return true;
    }
};

// ---- engine / stream / memory ----------------------------------------------
struct dnnl_engine {
    dnnl_engine_kind_t kind;
    int device; // HIP device ordinal; -1: no device behind it (descriptor-only)
    std::atomic<int> refs {1};
};

struct dnnl_stream {
    dnnl_engine_t engine;
    void *hip_stream; // hipStream_t
    bool owns_stream;
    unsigned flags;
};

struct dnnl_memory {
    dnnl_engine_t engine;
    dnnl_memory_desc md;
    void *handle; // device pointer
    bool owns_handle;
    void *mapped; // pinned staging buffer while mapped
};

// ---- primitive descriptor / primitive --------------------------------------
struct pd_impl_t {
    dnnl_primitive_kind_t kind = dnnl_undefined_primitive;
    dnnl_engine_t engine = nullptr;
    dnnl_primitive_attr attr;
    // descriptors as the user passed them and as the implementation resolved
    dnnl_memory_desc user_src, user_wei, user_bias, user_dst;
    dnnl_memory_desc src, wei, bias, dst;
    dnnl_memory_desc scratchpad;
    int impl = -1; // index into the implementation list
    std::string impl_name;
    // inner product lowered to matmul: src / wei / bias / dst above are the
    // matmul view ([MB, K] x [K, OC]); these are what the user sees
    bool ip = false;
    dnnl_memory_desc ip_src, ip_wei, ip_bias, ip_dst;
    dnnl_memory_desc ip_wei_user; // weights as passed (may be format any)
    qmm_matmul_desc_t mm; // kernel-level description (matmul)
    qmm_reorder_desc_t ro; // kernel-level description (reorder)
    qmm_softmax_desc_t sm; // kernel-level description (softmax)
    qmm_sdpa_desc_t sd; // kernel-level description (sdpa)
    dnnl_memory_desc sdpa_k, sdpa_v, sdpa_mask; // src = queries
    dnnl_prop_kind_t prop_kind = dnnl_forward_inference;
    size_t scratch_bytes = 0;
    // matmul whose descriptors hold DNNL_RUNTIME_DIM_VAL: no implementation is
    // chosen until execute sees the memory objects' own descriptors
    bool runtime = false;
};

// A library-owned scratchpad is one buffer per primitive (or per cached shape
// of a runtime-dims primitive), so launches of that primitive from different
// streams (host threads) must not overlap on the device. The guard orders them:
// under its mutex a launch on another stream than the previous one first waits
// for an event recorded behind the previous launch. Launches on one stream pay
// one event record each, and only when the primitive uses such a scratchpad.
struct scratch_guard_t {
    std::mutex mu;
    void *event = nullptr; // hipEvent_t, created on first use
    void *last_stream = nullptr;
    bool used = false;
    ~scratch_guard_t();
};

// One resolved shape of a runtime-dims matmul: the concrete descriptor, its
// plan and a library-owned scratchpad. Owned by the primitive's cache.
struct rt_entry_t {
    dnnl_memory_desc src, wei, bias, dst;
    std::shared_ptr<pd_impl_t> pd;
    qmm_plan_t *plan = nullptr;
    void *scratch = nullptr;
    scratch_guard_t guard; // orders launches that share `scratch`
    uint64_t stamp = 0;
    ~rt_entry_t();
};

struct dnnl_primitive_desc {
    std::shared_ptr<pd_impl_t> p;
};

struct dnnl_primitive {
    std::shared_ptr<pd_impl_t> pd;
    dnnl_primitive_desc pd_handle; // what dnnl_primitive_get_primitive_desc returns
    qmm_plan_t *plan = nullptr;
    void *lib_scratch = nullptr; // library-managed scratchpad
    mutable scratch_guard_t guard; // orders launches that share lib_scratch
    // runtime dims: the shapes seen so far, least recently used evicted
    std::mutex rt_mutex;
    std::vector<std::shared_ptr<rt_entry_t>> rt;
    uint64_t rt_clock = 0;
};

// helpers shared between translation units
namespace host {
size_t dt_bits(dnnl_data_type_t dt);
bool md_init_plain(dnnl_memory_desc &md, int ndims, const dnnl_dims_t dims,
        dnnl_data_type_t dt, const dnnl_dims_t strides_or_null);
bool md_equal(const dnnl_memory_desc &a, const dnnl_memory_desc &b);
size_t md_size(const dnnl_memory_desc &md);
void md_to_tensor(qmm_tensor_t &t, const dnnl_memory_desc &md);
dnnl_status_t from_qmm(int st);
} // namespace host
