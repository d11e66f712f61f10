// C++ layer over the dnnl C API subset of this library (oneapi/dnnl/dnnl.h):
// the classes, member names and enum spellings of the reference's dnnl.hpp
// (include/oneapi/dnnl/dnnl.hpp) for what the quantized-matmul path needs --
// engine, stream, memory and memory::desc, primitive_attr, post_ops, matmul,
// reorder, inner_product_forward -- so that application code written against
// the reference compiles and runs unchanged on this library. Header-only: every
// method is a call into the C API; objects are reference-counted handles with
// the C destroy functions as deleters.
#ifndef ONEAPI_DNNL_DNNL_HPP
#define ONEAPI_DNNL_DNNL_HPP

#include <cstdint>
#include <exception>
#include <memory>
#include <string>
#include <type_traits>
#include <unordered_map>
#include <vector>

#include "oneapi/dnnl/dnnl.h"

namespace dnnl {

/// Exception carrying the C status (dnnl.hpp: struct error).
struct error : public std::exception {
    dnnl_status_t status;
    const char *message;
    error(dnnl_status_t s, const char *m) : status(s), message(m) {}
    const char *what() const noexcept override { return message; }
    static void wrap_c_api(dnnl_status_t s, const char *m) {
        if (s != dnnl_success) throw error(s, m);
    }
};

template <typename T>
struct handle_traits {};
#define DNNL_HPP_TRAITS(T, DTOR) \
    template <> \
    struct handle_traits<T> { \
        static dnnl_status_t destructor(T p) { return DTOR(p); } \
    };
DNNL_HPP_TRAITS(dnnl_engine_t, dnnl_engine_destroy)
DNNL_HPP_TRAITS(dnnl_stream_t, dnnl_stream_destroy)
DNNL_HPP_TRAITS(dnnl_memory_desc_t, dnnl_memory_desc_destroy)
DNNL_HPP_TRAITS(dnnl_memory_t, dnnl_memory_destroy)
DNNL_HPP_TRAITS(dnnl_primitive_desc_t, dnnl_primitive_desc_destroy)
DNNL_HPP_TRAITS(dnnl_primitive_attr_t, dnnl_primitive_attr_destroy)
DNNL_HPP_TRAITS(dnnl_post_ops_t, dnnl_post_ops_destroy)
DNNL_HPP_TRAITS(dnnl_primitive_t, dnnl_primitive_destroy)
#undef DNNL_HPP_TRAITS

/// Shared ownership of a C handle; `weak` handles are not destroyed.
template <typename T, typename traits = handle_traits<T>>
struct handle {
private:
    static dnnl_status_t dummy_destructor(T) { return dnnl_success; }
    std::shared_ptr<typename std::remove_pointer<T>::type> data_ {nullptr};

public:
    handle() = default;
    explicit handle(T t, bool weak = false) { reset(t, weak); }
    void reset(T t, bool weak = false) {
        data_.reset(t, weak ? &dummy_destructor : traits::destructor);
    }
    T get(bool allow_empty = false) const {
        T r = data_.get();
        if (!allow_empty && r == nullptr)
            throw error(dnnl_invalid_arguments, "object is not initialized");
        return r;
    }
    explicit operator T() const { return get(true); }
    explicit operator bool() const { return get(true) != nullptr; }
    bool operator==(const handle &o) const { return o.data_.get() == data_.get(); }
    bool operator!=(const handle &o) const { return !(*this == o); }
};

enum class scratchpad_mode {
    library = dnnl_scratchpad_mode_library,
    user = dnnl_scratchpad_mode_user,
};
enum class rounding_mode {
    environment = dnnl_rounding_mode_environment,
    stochastic = dnnl_rounding_mode_stochastic,
};
inline dnnl_rounding_mode_t convert_to_c(rounding_mode mode) {
    return static_cast<dnnl_rounding_mode_t>(mode);
}
enum class fpmath_mode {
    strict = dnnl_fpmath_mode_strict,
    bf16 = dnnl_fpmath_mode_bf16,
    f16 = dnnl_fpmath_mode_f16,
    tf32 = dnnl_fpmath_mode_tf32,
    any = dnnl_fpmath_mode_any,
};
enum class prop_kind {
    undef = dnnl_prop_kind_undef,
    forward_training = dnnl_forward_training,
    forward_inference = dnnl_forward_inference,
    forward = dnnl_forward,
};
enum class algorithm {
    undef = dnnl_alg_kind_undef,
    eltwise_relu = dnnl_eltwise_relu,
    eltwise_tanh = dnnl_eltwise_tanh,
    eltwise_elu = dnnl_eltwise_elu,
    eltwise_square = dnnl_eltwise_square,
    eltwise_abs = dnnl_eltwise_abs,
    eltwise_sqrt = dnnl_eltwise_sqrt,
    eltwise_linear = dnnl_eltwise_linear,
    eltwise_soft_relu = dnnl_eltwise_soft_relu,
    eltwise_hardsigmoid = dnnl_eltwise_hardsigmoid,
    eltwise_logistic = dnnl_eltwise_logistic,
    eltwise_exp = dnnl_eltwise_exp,
    eltwise_gelu_tanh = dnnl_eltwise_gelu_tanh,
    eltwise_swish = dnnl_eltwise_swish,
    eltwise_log = dnnl_eltwise_log,
    eltwise_clip = dnnl_eltwise_clip,
    eltwise_clip_v2 = dnnl_eltwise_clip_v2,
    eltwise_pow = dnnl_eltwise_pow,
    eltwise_gelu_erf = dnnl_eltwise_gelu_erf,
    eltwise_round = dnnl_eltwise_round,
    eltwise_mish = dnnl_eltwise_mish,
    eltwise_hardswish = dnnl_eltwise_hardswish,
    binary_add = dnnl_binary_add,
    binary_mul = dnnl_binary_mul,
    binary_max = dnnl_binary_max,
    binary_min = dnnl_binary_min,
    binary_div = dnnl_binary_div,
    binary_sub = dnnl_binary_sub,
    binary_ge = dnnl_binary_ge,
    binary_gt = dnnl_binary_gt,
    binary_le = dnnl_binary_le,
    binary_lt = dnnl_binary_lt,
    binary_eq = dnnl_binary_eq,
    binary_ne = dnnl_binary_ne,
    softmax_accurate = dnnl_softmax_accurate,
    softmax_log = dnnl_softmax_log,
};
enum class query {
    undef = dnnl_query_undef,
    engine = dnnl_query_engine,
    primitive_kind = dnnl_query_primitive_kind,
    num_of_inputs_s32 = dnnl_query_num_of_inputs_s32,
    num_of_outputs_s32 = dnnl_query_num_of_outputs_s32,
    memory_consumption_s64 = dnnl_query_memory_consumption_s64,
    impl_info_str = dnnl_query_impl_info_str,
    prop_kind = dnnl_query_prop_kind,
    src_md = dnnl_query_src_md,
    weights_md = dnnl_query_weights_md,
    dst_md = dnnl_query_dst_md,
    scratchpad_md = dnnl_query_scratchpad_md,
    exec_arg_md = dnnl_query_exec_arg_md,
};
inline dnnl_alg_kind_t convert_to_c(algorithm a) { return (dnnl_alg_kind_t)a; }
inline dnnl_query_t convert_to_c(query q) { return (dnnl_query_t)q; }
inline dnnl_prop_kind_t convert_to_c(prop_kind k) { return (dnnl_prop_kind_t)k; }
inline dnnl_fpmath_mode_t convert_to_c(fpmath_mode m) {
    return (dnnl_fpmath_mode_t)m;
}
inline dnnl_scratchpad_mode_t convert_to_c(scratchpad_mode m) {
    return (dnnl_scratchpad_mode_t)m;
}

struct engine : public handle<dnnl_engine_t> {
    using handle::handle;
    enum class kind {
        any = dnnl_any_engine,
        cpu = dnnl_cpu,
        gpu = dnnl_gpu,
    };
    engine() = default;
    static size_t get_count(kind k) {
        return dnnl_engine_get_count((dnnl_engine_kind_t)k);
    }
    engine(kind k, size_t index) {
        dnnl_engine_t e;
        error::wrap_c_api(dnnl_engine_create(&e, (dnnl_engine_kind_t)k, index),
                "could not create an engine");
        reset(e);
    }
    kind get_kind() const {
        dnnl_engine_kind_t k;
        error::wrap_c_api(dnnl_engine_get_kind(get(), &k),
                "could not get kind of an engine");
        return (kind)k;
    }
};

struct stream : public handle<dnnl_stream_t> {
    using handle::handle;
    enum class flags : unsigned {
        in_order = dnnl_stream_in_order,
        out_of_order = dnnl_stream_out_of_order,
        default_flags = dnnl_stream_default_flags,
    };
    stream() = default;
    explicit stream(const engine &e, flags f = flags::default_flags) {
        dnnl_stream_t s;
        error::wrap_c_api(dnnl_stream_create(&s, e.get(), (unsigned)f),
                "could not create a stream");
        reset(s);
    }
    engine get_engine() const {
        dnnl_engine_t e;
        error::wrap_c_api(dnnl_stream_get_engine(get(), &e),
                "could not get an engine from a stream object");
        return engine(e, true);
    }
    stream &wait() {
        error::wrap_c_api(dnnl_stream_wait(get()), "could not wait on a stream");
        return *this;
    }
};

struct memory : public handle<dnnl_memory_t> {
    using handle::handle;
    typedef dnnl_dim_t dim;
    typedef std::vector<dim> dims;

    enum class data_type {
        undef = dnnl_data_type_undef,
        f16 = dnnl_f16,
        bf16 = dnnl_bf16,
        f32 = dnnl_f32,
        s32 = dnnl_s32,
        s8 = dnnl_s8,
        u8 = dnnl_u8,
        f64 = dnnl_f64,
        f8_e5m2 = dnnl_f8_e5m2,
        f8_e4m3 = dnnl_f8_e4m3,
        s4 = dnnl_s4,
        u4 = dnnl_u4,
    };
    enum class format_kind {
        undef = dnnl_format_kind_undef,
        any = dnnl_format_kind_any,
        blocked = dnnl_blocked,
        opaque = dnnl_format_kind_opaque,
    };
    enum class format_tag {
        undef = dnnl_format_tag_undef,
        any = dnnl_format_tag_any,
        a = dnnl_a,
        ab = dnnl_ab,
        ba = dnnl_ba,
        abc = dnnl_abc,
        acb = dnnl_acb,
        bac = dnnl_bac,
        abcd = dnnl_abcd,
        abdc = dnnl_abdc,
        acbd = dnnl_acbd,
        acdb = dnnl_acdb,
        abcde = dnnl_abcde,
        abced = dnnl_abced,
        x = a,
        nc = ab,
        cn = ba,
        tn = ab,
        nt = ba,
        oi = ab,
        io = ba,
        ncw = abc,
        nwc = acb,
        nchw = abcd,
        nhwc = acdb,
        ncdhw = abcde,
    };
    static dnnl_data_type_t convert_to_c(data_type t) {
        return (dnnl_data_type_t)t;
    }
    static dnnl_format_tag_t convert_to_c(format_tag t) {
        return (dnnl_format_tag_t)t;
    }
    static size_t data_type_size(data_type t) {
        return dnnl_data_type_size(convert_to_c(t));
    }

    struct desc : public handle<dnnl_memory_desc_t> {
        using handle::handle;
        desc() = default;
        desc(const dims &adims, data_type adt, format_tag atag,
                bool allow_empty = false) {
            dnnl_memory_desc_t md = nullptr;
            const dnnl_status_t st = dnnl_memory_desc_create_with_tag(&md,
                    (int)adims.size(), adims.data(), convert_to_c(adt),
                    convert_to_c(atag));
            if (!allow_empty)
                error::wrap_c_api(st,
                        "could not construct a memory descriptor using a "
                        "format tag");
            reset(md);
        }
        desc(const dims &adims, data_type adt, const dims &strides,
                bool allow_empty = false) {
            dnnl_memory_desc_t md = nullptr;
            const dnnl_status_t st = dnnl_memory_desc_create_with_strides(&md,
                    (int)adims.size(), adims.data(), convert_to_c(adt),
                    strides.empty() ? nullptr : strides.data());
            if (!allow_empty)
                error::wrap_c_api(st,
                        "could not construct a memory descriptor using "
                        "strides");
            reset(md);
        }
        /// Takes ownership of a C descriptor.
        explicit desc(dnnl_memory_desc_t md) : handle<dnnl_memory_desc_t>(md) {}

        desc reshape(const dims &adims, bool allow_empty = false) const {
            dnnl_memory_desc_t out = nullptr;
            const dnnl_status_t st = dnnl_memory_desc_reshape(
                    &out, get(), (int)adims.size(), adims.data());
            if (!allow_empty)
                error::wrap_c_api(st, "could not reshape a memory descriptor");
            return desc(out);
        }
        desc permute_axes(const std::vector<int> &perm,
                bool allow_empty = false) const {
            dnnl_memory_desc_t out = nullptr;
            const dnnl_status_t st
                    = dnnl_memory_desc_permute_axes(&out, get(), perm.data());
            if (!allow_empty)
                error::wrap_c_api(st,
                        "could not permute axes of a memory descriptor");
            return desc(out);
        }
        int get_ndims() const { return query_s32(dnnl_query_ndims_s32); }
        dims get_dims() const { return query_dims(dnnl_query_dims); }
        dims get_strides() const { return query_dims(dnnl_query_strides); }
        data_type get_data_type() const {
            dnnl_data_type_t t = dnnl_data_type_undef;
            if (get(true)) dnnl_memory_desc_query(get(), dnnl_query_data_type, &t);
            return (data_type)t;
        }
        memory::format_kind get_format_kind() const {
            dnnl_format_kind_t k = dnnl_format_kind_undef;
            if (get(true))
                dnnl_memory_desc_query(get(), dnnl_query_format_kind, &k);
            return (memory::format_kind)k;
        }
        size_t get_size() const {
            return get(true) ? dnnl_memory_desc_get_size(get()) : 0;
        }
        bool is_zero() const { return get_ndims() == 0; }
        bool operator==(const desc &o) const {
            return dnnl_memory_desc_equal(get(true), o.get(true)) != 0;
        }
        bool operator!=(const desc &o) const { return !operator==(o); }

    private:
        int query_s32(dnnl_query_t what) const {
            int v = 0;
            if (get(true)) dnnl_memory_desc_query(get(), what, &v);
            return v;
        }
        dims query_dims(dnnl_query_t what) const {
            const int nd = get_ndims();
            dnnl_dim_t *p = nullptr;
            if (nd == 0 || dnnl_memory_desc_query(get(), what, &p) != dnnl_success
                    || !p)
                return {};
            return dims(p, p + nd);
        }
    };

    memory() = default;
    /// handle: a device pointer, DNNL_MEMORY_ALLOCATE or DNNL_MEMORY_NONE.
    memory(const desc &md, const engine &e, void *ahandle) {
        dnnl_memory_t m;
        error::wrap_c_api(dnnl_memory_create(&m, md.get(), e.get(), ahandle),
                "could not create a memory object");
        reset(m);
    }
    memory(const desc &md, const engine &e)
        : memory(md, e, DNNL_MEMORY_ALLOCATE) {}

    desc get_desc() const {
        const_dnnl_memory_desc_t c;
        error::wrap_c_api(dnnl_memory_get_memory_desc(get(), &c),
                "could not get a memory descriptor from a memory object");
        dnnl_memory_desc_t copy = nullptr;
        error::wrap_c_api(dnnl_memory_desc_clone(&copy, c),
                "could not clone a memory descriptor");
        return desc(copy);
    }
    engine get_engine() const {
        dnnl_engine_t e;
        error::wrap_c_api(dnnl_memory_get_engine(get(), &e),
                "could not get an engine from a memory object");
        return engine(e, true);
    }
    void *get_data_handle() const {
        void *h;
        error::wrap_c_api(dnnl_memory_get_data_handle(get(), &h),
                "could not get a native handle from a memory object");
        return h;
    }
    void set_data_handle(void *h) const {
        error::wrap_c_api(dnnl_memory_set_data_handle(get(), h),
                "could not set native handle of a memory object");
    }
    template <typename T = void>
    T *map_data() const {
        void *p;
        error::wrap_c_api(dnnl_memory_map_data(get(), &p),
                "could not map memory object data");
        return static_cast<T *>(p);
    }
    void unmap_data(void *mapped_ptr) const {
        error::wrap_c_api(dnnl_memory_unmap_data(get(), mapped_ptr),
                "could not unmap memory object data");
    }
};

struct primitive : public handle<dnnl_primitive_t> {
    using handle::handle;
    enum class kind {
        undef = dnnl_undefined_primitive,
        reorder = dnnl_reorder,
        eltwise = dnnl_eltwise,
        inner_product = dnnl_inner_product,
        binary = dnnl_binary,
        matmul = dnnl_matmul,
        prelu = dnnl_prelu,
        sum = dnnl_sum,
    };
    primitive() = default;
    explicit primitive(const_dnnl_primitive_desc_t c_pd) {
        dnnl_primitive_t p;
        error::wrap_c_api(
                dnnl_primitive_create(&p, c_pd), "could not create a primitive");
        reset(p);
    }
    void execute(const stream &astream,
            const std::unordered_map<int, memory> &args) const {
        std::vector<dnnl_exec_arg_t> c_args;
        c_args.reserve(args.size());
        for (const auto &a : args)
            c_args.push_back({a.first, a.second.get(true)});
        error::wrap_c_api(dnnl_primitive_execute(get(), astream.get(),
                                  (int)c_args.size(), c_args.data()),
                "could not execute a primitive");
    }
};

struct post_ops : public handle<dnnl_post_ops_t> {
    using handle::handle;
    post_ops() {
        dnnl_post_ops_t p;
        error::wrap_c_api(
                dnnl_post_ops_create(&p), "could not create post-ops");
        reset(p);
    }
    int len() const { return dnnl_post_ops_len(get()); }
    primitive::kind kind(int index) const {
        error::wrap_c_api(index < len() ? dnnl_success : dnnl_invalid_arguments,
                "post-ops index is out of range");
        return (primitive::kind)dnnl_post_ops_get_kind(get(), index);
    }
    void append_sum(float scale = 1.f, int32_t zero_point = 0,
            memory::data_type dt = memory::data_type::undef) {
        error::wrap_c_api(dnnl_post_ops_append_sum(get(), scale, zero_point,
                                  memory::convert_to_c(dt)),
                "could not append a sum post-op");
    }
    void get_params_sum(int index, float &scale, int32_t &zero_point,
            memory::data_type &dt) const {
        dnnl_data_type_t c_dt;
        error::wrap_c_api(dnnl_post_ops_get_params_sum(
                                  get(), index, &scale, &zero_point, &c_dt),
                "could not get parameters of a sum post-op");
        dt = (memory::data_type)c_dt;
    }
    void append_eltwise(algorithm alg, float alpha, float beta) {
        error::wrap_c_api(dnnl_post_ops_append_eltwise(
                                  get(), convert_to_c(alg), alpha, beta),
                "could not append an elementwise post-op");
    }
    void get_params_eltwise(
            int index, algorithm &alg, float &alpha, float &beta) const {
        dnnl_alg_kind_t c_alg;
        error::wrap_c_api(dnnl_post_ops_get_params_eltwise(
                                  get(), index, &c_alg, &alpha, &beta),
                "could not get parameters of an elementwise post-op");
        alg = (algorithm)c_alg;
    }
    void append_binary(algorithm alg, const memory::desc &src1_desc) {
        error::wrap_c_api(dnnl_post_ops_append_binary(get(), convert_to_c(alg),
                                  src1_desc.get()),
                "could not append a binary post-op");
    }
    void get_params_binary(
            int index, algorithm &alg, memory::desc &src1_desc) const {
        dnnl_alg_kind_t c_alg;
        const_dnnl_memory_desc_t c;
        error::wrap_c_api(
                dnnl_post_ops_get_params_binary(get(), index, &c_alg, &c),
                "could not get parameters of a binary post-op");
        alg = (algorithm)c_alg;
        dnnl_memory_desc_t copy = nullptr;
        error::wrap_c_api(dnnl_memory_desc_clone(&copy, c),
                "could not clone a memory descriptor");
        src1_desc = memory::desc(copy);
    }
    void append_prelu(int mask) {
        error::wrap_c_api(dnnl_post_ops_append_prelu(get(), mask),
                "could not append a prelu post-op");
    }
    void get_params_prelu(int index, int &mask) const {
        error::wrap_c_api(dnnl_post_ops_get_params_prelu(get(), index, &mask),
                "could not get parameters of a prelu post-op");
    }
};

struct primitive_attr : public handle<dnnl_primitive_attr_t> {
    using handle::handle;
    primitive_attr() {
        dnnl_primitive_attr_t a;
        error::wrap_c_api(dnnl_primitive_attr_create(&a),
                "could not create primitive attribute");
        reset(a);
    }
    /// Takes ownership of a C attribute object.
    explicit primitive_attr(dnnl_primitive_attr_t a)
        : handle<dnnl_primitive_attr_t>(a) {}

    fpmath_mode get_fpmath_mode() const {
        dnnl_fpmath_mode_t m;
        error::wrap_c_api(dnnl_primitive_attr_get_fpmath_mode(get(), &m),
                "could not get fpmath mode primitive attribute");
        return (fpmath_mode)m;
    }
    void get_fpmath_mode(fpmath_mode &mode, bool &apply_to_int) const {
        dnnl_fpmath_mode_t m;
        int a = 0;
        error::wrap_c_api(dnnl_primitive_attr_get_fpmath_mode_v2(get(), &m, &a),
                "could not get fpmath mode primitive attribute");
        mode = (fpmath_mode)m;
        apply_to_int = a != 0;
    }
    void set_fpmath_mode(fpmath_mode mode, bool apply_to_int = false) {
        error::wrap_c_api(dnnl_primitive_attr_set_fpmath_mode_v2(
                                  get(), convert_to_c(mode), apply_to_int),
                "could not set fpmath mode primitive attribute");
    }
    scratchpad_mode get_scratchpad_mode() const {
        dnnl_scratchpad_mode_t m;
        error::wrap_c_api(dnnl_primitive_attr_get_scratchpad_mode(get(), &m),
                "could not get scratchpad mode primitive attribute");
        return (scratchpad_mode)m;
    }
    void set_scratchpad_mode(scratchpad_mode mode) {
        error::wrap_c_api(
                dnnl_primitive_attr_set_scratchpad_mode(get(), convert_to_c(mode)),
                "could not set scratchpad mode primitive attribute");
    }
    void get_dropout(memory::desc &mask_desc) const {
        const_dnnl_memory_desc_t cdesc;
        error::wrap_c_api(dnnl_primitive_attr_get_dropout(get(), &cdesc),
                "could not get parameters of a dropout attribute");
        dnnl_memory_desc_t cloned;
        error::wrap_c_api(dnnl_memory_desc_clone(&cloned, cdesc),
                "could not clone a memory descriptor");
        mask_desc = memory::desc(cloned);
    }
    void set_dropout(const memory::desc &mask_desc) {
        error::wrap_c_api(
                dnnl_primitive_attr_set_dropout(get(), mask_desc.get()),
                "could not set dropout primitive attribute");
    }
    rounding_mode get_rounding_mode(int arg) const {
        dnnl_rounding_mode_t result;
        error::wrap_c_api(dnnl_primitive_attr_get_rounding(get(), arg, &result),
                "could not get rounding mode primitive attribute");
        return rounding_mode(result);
    }
    void set_rounding_mode(int arg, rounding_mode mode) {
        error::wrap_c_api(dnnl_primitive_attr_set_rounding(
                                  get(), arg, convert_to_c(mode)),
                "could not set rounding mode primitive attribute");
    }
    void set_scales_mask(int arg, int mask) {
        error::wrap_c_api(dnnl_primitive_attr_set_scales_mask(get(), arg, mask),
                "could not set scales primitive attribute");
    }
    void set_scales(int arg, int mask, const memory::dims &groups,
            memory::data_type dt = memory::data_type::f32) {
        error::wrap_c_api(dnnl_primitive_attr_set_scales(get(), arg, mask,
                                  (int)groups.size(), groups.data(),
                                  memory::convert_to_c(dt)),
                "could not set scales primitive attribute");
    }
    void set_zero_points_mask(int arg, int mask) {
        error::wrap_c_api(
                dnnl_primitive_attr_set_zero_points_mask(get(), arg, mask),
                "could not set zero points primitive attribute");
    }
    void set_zero_points(int arg, int mask, const memory::dims &groups,
            memory::data_type dt = memory::data_type::s32) {
        error::wrap_c_api(dnnl_primitive_attr_set_zero_points(get(), arg, mask,
                                  (int)groups.size(), groups.data(),
                                  memory::convert_to_c(dt)),
                "could not set zero points primitive attribute");
    }
    post_ops get_post_ops() const {
        const_dnnl_post_ops_t c;
        error::wrap_c_api(dnnl_primitive_attr_get_post_ops(get(), &c),
                "could not get post-ops primitive attribute");
        dnnl_post_ops_t copy;
        error::wrap_c_api(
                dnnl_post_ops_clone(&copy, c), "could not clone post-ops");
        post_ops r;
        r.reset(copy);
        return r;
    }
    void set_post_ops(const post_ops &ops) {
        error::wrap_c_api(dnnl_primitive_attr_set_post_ops(get(), ops.get()),
                "could not set post-ops primitive attribute");
    }
};

/// Base of the primitive descriptors: queries and implementation iteration.
struct primitive_desc_base : public handle<dnnl_primitive_desc_t> {
    using handle::handle;
    primitive_desc_base() = default;

    engine get_engine() const {
        dnnl_engine_t e;
        error::wrap_c_api(
                dnnl_primitive_desc_query(get(), dnnl_query_engine, 0, &e),
                "could not retrieve engine from a primitive descriptor");
        return engine(e, true);
    }
    const char *impl_info_str() const {
        const char *s;
        error::wrap_c_api(dnnl_primitive_desc_query(
                                  get(), dnnl_query_impl_info_str, 0, &s),
                "could not retrieve implementation info string from a "
                "primitive descriptor");
        return s;
    }
    memory::dim query_s64(query what) const {
        memory::dim v = 0;
        dnnl_primitive_desc_query(get(), convert_to_c(what), 0, &v);
        return v;
    }
    memory::desc query_md(query what, int idx = 0) const {
        const_dnnl_memory_desc_t c
                = dnnl_primitive_desc_query_md(get(), convert_to_c(what), idx);
        if (!c) return memory::desc();
        dnnl_memory_desc_t copy = nullptr;
        error::wrap_c_api(dnnl_memory_desc_clone(&copy, c),
                "could not clone a memory descriptor");
        return memory::desc(copy);
    }
    memory::desc src_desc(int idx) const { return query_md(query::src_md, idx); }
    memory::desc weights_desc(int idx) const {
        return query_md(query::weights_md, idx);
    }
    memory::desc dst_desc(int idx) const { return query_md(query::dst_md, idx); }
    memory::desc src_desc() const { return src_desc(0); }
    memory::desc weights_desc() const { return weights_desc(0); }
    memory::desc dst_desc() const { return dst_desc(0); }
    memory::desc scratchpad_desc() const {
        return query_md(query::scratchpad_md, 0);
    }
    primitive_attr get_primitive_attr() const {
        const_dnnl_primitive_attr_t c;
        error::wrap_c_api(dnnl_primitive_desc_get_attr(get(), &c),
                "could not get attributes from a primitive descriptor");
        dnnl_primitive_attr_t copy;
        error::wrap_c_api(dnnl_primitive_attr_clone(&copy, c),
                "could not clone primitive attributes");
        return primitive_attr(copy);
    }
    dnnl::primitive::kind get_kind() const {
        dnnl_primitive_kind_t k;
        error::wrap_c_api(dnnl_primitive_desc_query(get(),
                                  dnnl_query_primitive_kind, 0, (void *)&k),
                "could not get primitive kind from a primitive descriptor");
        return (dnnl::primitive::kind)k;
    }
    /// Advances to the next implementation; false when there is none.
    bool next_impl() {
        const dnnl_status_t st = dnnl_primitive_desc_next_impl(get());
        if (st == dnnl_last_impl_reached) return false;
        error::wrap_c_api(st, "last available implementation is reached");
        return true;
    }
};

struct reorder : public primitive {
    struct primitive_desc : public primitive_desc_base {
        using primitive_desc_base::primitive_desc_base;
        primitive_desc() = default;
        primitive_desc(const engine &src_engine, const memory::desc &src_md,
                const engine &dst_engine, const memory::desc &dst_md,
                const primitive_attr &attr = primitive_attr(),
                bool allow_empty = false) {
            dnnl_primitive_desc_t pd = nullptr;
            const dnnl_status_t st = dnnl_reorder_primitive_desc_create(&pd,
                    src_md.get(), src_engine.get(), dst_md.get(),
                    dst_engine.get(), attr.get());
            if (!allow_empty)
                error::wrap_c_api(st,
                        "could not create a primitive descriptor for a "
                        "reorder primitive");
            reset(pd);
        }
        primitive_desc(const memory &src, const memory &dst,
                const primitive_attr &attr = primitive_attr(),
                bool allow_empty = false)
            : primitive_desc(src.get_engine(), src.get_desc(), dst.get_engine(),
                    dst.get_desc(), attr, allow_empty) {}
    };
    reorder() = default;
    explicit reorder(const primitive_desc &pd) : primitive(pd.get()) {}
    reorder(const memory &src, const memory &dst,
            const primitive_attr &attr = primitive_attr())
        : primitive(primitive_desc(src, dst, attr).get()) {}
    using primitive::execute;
    void execute(const stream &astream, memory &src, memory &dst) const {
        primitive::execute(astream, {{DNNL_ARG_FROM, src}, {DNNL_ARG_TO, dst}});
    }
};

struct matmul : public primitive {
    struct primitive_desc : public primitive_desc_base {
        using primitive_desc_base::primitive_desc_base;
        primitive_desc() = default;
        primitive_desc(const engine &aengine, const memory::desc &src_desc,
                const memory::desc &weights_desc, const memory::desc &dst_desc,
                const primitive_attr &attr = primitive_attr(),
                bool allow_empty = false)
            : primitive_desc(aengine, src_desc, weights_desc, nullptr, dst_desc,
                    attr, allow_empty) {}
        primitive_desc(const engine &aengine, const memory::desc &src_desc,
                const memory::desc &weights_desc, const memory::desc &bias_desc,
                const memory::desc &dst_desc,
                const primitive_attr &attr = primitive_attr(),
                bool allow_empty = false)
            : primitive_desc(aengine, src_desc, weights_desc, &bias_desc,
                    dst_desc, attr, allow_empty) {}
        memory::desc bias_desc() const { return weights_desc(1); }

    private:
        primitive_desc(const engine &aengine, const memory::desc &src_desc,
                const memory::desc &weights_desc, const memory::desc *bias_desc,
                const memory::desc &dst_desc, const primitive_attr &attr,
                bool allow_empty) {
            dnnl_primitive_desc_t pd = nullptr;
            const dnnl_status_t st = dnnl_matmul_primitive_desc_create(&pd,
                    aengine.get(), src_desc.get(), weights_desc.get(),
                    bias_desc ? bias_desc->get(true) : nullptr, dst_desc.get(),
                    attr.get());
            if (!allow_empty)
                error::wrap_c_api(st,
                        "could not create a primitive descriptor for a matmul "
                        "primitive");
            reset(pd);
        }
    };
    matmul() = default;
    explicit matmul(const primitive_desc &pd) : primitive(pd.get()) {}
};

struct inner_product_forward : public primitive {
    struct primitive_desc : public primitive_desc_base {
        using primitive_desc_base::primitive_desc_base;
        primitive_desc() = default;
        primitive_desc(const engine &aengine, prop_kind aprop_kind,
                const memory::desc &src_desc, const memory::desc &weights_desc,
                const memory::desc &bias_desc, const memory::desc &dst_desc,
                const primitive_attr &attr = primitive_attr(),
                bool allow_empty = false)
            : primitive_desc(aengine, aprop_kind, src_desc, weights_desc,
                    &bias_desc, dst_desc, attr, allow_empty) {}
        primitive_desc(const engine &aengine, prop_kind aprop_kind,
                const memory::desc &src_desc, const memory::desc &weights_desc,
                const memory::desc &dst_desc,
                const primitive_attr &attr = primitive_attr(),
                bool allow_empty = false)
            : primitive_desc(aengine, aprop_kind, src_desc, weights_desc,
                    nullptr, dst_desc, attr, allow_empty) {}
        memory::desc bias_desc() const { return weights_desc(1); }

    private:
        primitive_desc(const engine &aengine, prop_kind aprop_kind,
                const memory::desc &src_desc, const memory::desc &weights_desc,
                const memory::desc *bias_desc, const memory::desc &dst_desc,
                const primitive_attr &attr, bool allow_empty) {
            dnnl_primitive_desc_t pd = nullptr;
            const dnnl_status_t st
                    = dnnl_inner_product_forward_primitive_desc_create(&pd,
                            aengine.get(), convert_to_c(aprop_kind),
                            src_desc.get(), weights_desc.get(),
                            bias_desc ? bias_desc->get(true) : nullptr,
                            dst_desc.get(), attr.get());
            if (!allow_empty)
                error::wrap_c_api(st,
                        "could not create a primitive descriptor for an inner "
                        "product forward propagation primitive");
            reset(pd);
        }
    };
    inner_product_forward() = default;
    explicit inner_product_forward(const primitive_desc &pd)
        : primitive(pd.get()) {}
};

// Softmax forward (reference include/oneapi/dnnl/dnnl.hpp softmax_forward):
// the step between the score and the value matmul of an attention block.
struct softmax_forward : public primitive {
    struct primitive_desc : public primitive_desc_base {
        using primitive_desc_base::primitive_desc_base;
        primitive_desc() = default;
        primitive_desc(const engine &aengine, prop_kind aprop_kind,
                algorithm aalgorithm, const memory::desc &src_desc,
                const memory::desc &dst_desc, int axis,
                const primitive_attr &attr = primitive_attr(),
                bool allow_empty = false) {
            dnnl_primitive_desc_t pd = nullptr;
            const dnnl_status_t st = dnnl_softmax_forward_primitive_desc_create(
                    &pd, aengine.get(), convert_to_c(aprop_kind),
                    convert_to_c(aalgorithm), src_desc.get(), dst_desc.get(),
                    axis, attr.get());
            if (!allow_empty)
                error::wrap_c_api(st,
                        "could not create a primitive descriptor for a softmax "
                        "forward propagation primitive");
            reset(pd);
        }
        algorithm get_algorithm() const {
            dnnl_alg_kind_t a = dnnl_alg_kind_undef;
            error::wrap_c_api(dnnl_primitive_desc_query(
                                      get(), dnnl_query_alg_kind, 0, &a),
                    "could not query the algorithm");
            return (algorithm)a;
        }
        int get_axis() const {
            int a = -1;
            error::wrap_c_api(dnnl_primitive_desc_query(
                                      get(), dnnl_query_axis_s32, 0, &a),
                    "could not query the axis");
            return a;
        }
    };
    softmax_forward() = default;
    explicit softmax_forward(const primitive_desc &pd) : primitive(pd.get()) {}
};

} // namespace dnnl

#endif
