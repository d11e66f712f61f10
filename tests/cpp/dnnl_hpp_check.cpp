// Exercises the C++ layer (oneapi/dnnl/dnnl.hpp) the way an application written
// against the reference's C++ API would: the flow of the reference's int8
// matmul example (examples/matmul/inference_int8_matmul.cpp) -- descriptors,
// attributes with run-time scales / zero points and a post-op, weights in
// format `any` prepacked by a reorder, execute -- and an inner product over the
// same weights. `host` needs no GPU (descriptor-level checks only); `gpu` runs
// the primitives and compares them with a scalar loop over the same numbers.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <stdexcept>
#include <vector>

#include "oneapi/dnnl/dnnl.hpp"

using namespace dnnl;
using dt = memory::data_type;
using tag = memory::format_tag;

#define CHECK(cond) \
    do { \
        if (!(cond)) { \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); \
            return 1; \
        } \
    } while (0)

static uint32_t lcg(uint32_t &s) {
    s = s * 1664525u + 1013904223u;
    return s >> 8;
}

template <typename T>
static void upload(const memory &m, const std::vector<T> &v) {
    T *p = m.map_data<T>();
    std::memcpy(p, v.data(), v.size() * sizeof(T));
    m.unmap_data(p);
}
template <typename T>
static std::vector<T> download(const memory &m, size_t n) {
    std::vector<T> v(n);
    T *p = m.map_data<T>();
    std::memcpy(v.data(), p, n * sizeof(T));
    m.unmap_data(p);
    return v;
}

static primitive_attr linear_attr() {
    primitive_attr attr;
    attr.set_scales_mask(DNNL_ARG_SRC, 0);
    attr.set_scales_mask(DNNL_ARG_WEIGHTS, 1 << 1);
    attr.set_zero_points_mask(DNNL_ARG_SRC, 0);
    post_ops po;
    po.append_eltwise(algorithm::eltwise_relu, 0.f, 0.f);
    attr.set_post_ops(po);
    return attr;
}

static int host_checks() {
    // descriptors
    memory::desc a({6, 10}, dt::u8, tag::ab);
    CHECK(a.get_ndims() == 2);
    CHECK(a.get_dims() == memory::dims({6, 10}));
    CHECK(a.get_strides() == memory::dims({10, 1}));
    CHECK(a.get_size() == 60);
    CHECK(a.get_data_type() == dt::u8);
    CHECK(a.get_format_kind() == memory::format_kind::blocked);
    memory::desc at({6, 10}, dt::u8, tag::ba);
    CHECK(at.get_strides() == memory::dims({1, 6}));
    CHECK(a != at);
    CHECK(a == memory::desc({6, 10}, dt::u8, memory::dims({10, 1})));
    CHECK(a.reshape({3, 2, 10}).get_dims() == memory::dims({3, 2, 10}));
    CHECK(a.permute_axes({1, 0}).get_dims() == memory::dims({10, 6}));
    CHECK(memory::desc().is_zero());
    CHECK(memory::data_type_size(dt::bf16) == 2);

    // an invalid descriptor throws, or stays empty when asked to
    bool thrown = false;
    try {
        memory::desc bad({2, -3}, dt::f32, tag::ab);
    } catch (const error &e) {
        thrown = e.status == dnnl_invalid_arguments;
    }
    CHECK(thrown);
    CHECK(!memory::desc({2, -3}, dt::f32, tag::ab, true));

    // attributes and post-ops round trip
    primitive_attr attr = linear_attr();
    post_ops po = attr.get_post_ops();
    CHECK(po.len() == 1 && po.kind(0) == primitive::kind::eltwise);
    algorithm alg;
    float alpha, beta;
    po.get_params_eltwise(0, alg, alpha, beta);
    CHECK(alg == algorithm::eltwise_relu && alpha == 0.f);
    attr.set_scratchpad_mode(scratchpad_mode::user);
    CHECK(attr.get_scratchpad_mode() == scratchpad_mode::user);
    attr.set_scratchpad_mode(scratchpad_mode::library);
    attr.set_fpmath_mode(fpmath_mode::bf16, true);
    fpmath_mode fm;
    bool to_int;
    attr.get_fpmath_mode(fm, to_int);
    CHECK(fm == fpmath_mode::bf16 && to_int);
    attr.set_fpmath_mode(fpmath_mode::strict);

    // a primitive descriptor on an engine without a device behind it:
    // creation, the implementation name and the opaque weights layout
    // (index 0 with DNNL_AMD_DESCRIPTOR_ONLY=1 set where there is no GPU)
    engine eng(engine::kind::gpu, 0);
    CHECK(eng.get_kind() == engine::kind::gpu);
    const memory::dim M = 256, K = 512, N = 384;
    memory::desc src_md({M, K}, dt::u8, tag::ab);
    memory::desc wei_any({K, N}, dt::s8, tag::any);
    memory::desc dst_md({M, N}, dt::f32, tag::ab);
    matmul::primitive_desc pd(eng, src_md, wei_any, dst_md, attr);
    CHECK(std::strstr(pd.impl_info_str(), "hip:gfx950") != nullptr);
    CHECK(pd.get_kind() == primitive::kind::matmul);
    CHECK(pd.weights_desc().get_format_kind() == memory::format_kind::opaque);
    CHECK(pd.src_desc() == src_md && pd.dst_desc() == dst_md);
    CHECK(pd.weights_desc() != memory::desc({K, N}, dt::s8, tag::ab));
    CHECK(pd.get_primitive_attr().get_post_ops().len() == 1);
    int n_impl = 1;
    while (pd.next_impl()) ++n_impl;
    CHECK(n_impl >= 1);

    // an unsupported combination is an error, or an empty object on request
    memory::desc bad_dst({M, N + 1}, dt::f32, tag::ab);
    thrown = false;
    try {
        matmul::primitive_desc p2(eng, src_md, wei_any, bad_dst, attr);
    } catch (const error &) { thrown = true; }
    CHECK(thrown);
    CHECK(!matmul::primitive_desc(eng, src_md, wei_any, bad_dst, attr, true));

    // the reorder that prepacks the weights, and the inner product descriptor
    memory::desc wei_user({K, N}, dt::s8, tag::ab);
    matmul::primitive_desc pd_w(eng, src_md, wei_any, dst_md, attr);
    reorder::primitive_desc rpd(eng, wei_user, eng, pd_w.weights_desc());
    CHECK(rpd.get_kind() == primitive::kind::reorder);
    memory::desc ip_wei({N, K}, dt::s8, tag::any);
    memory::desc ip_bias({N}, dt::f32, tag::a);
    inner_product_forward::primitive_desc ipd(eng, prop_kind::forward_inference,
            src_md, ip_wei, ip_bias, dst_md);
    CHECK(ipd.get_kind() == primitive::kind::inner_product);
    CHECK(ipd.bias_desc() == ip_bias);

    // softmax forward descriptor: axis, algorithm, destination layout from any
    memory::desc sm_src({4, 6, 32}, dt::f32, tag::abc);
    softmax_forward::primitive_desc spd(eng, prop_kind::forward_inference,
            algorithm::softmax_accurate, sm_src,
            memory::desc({4, 6, 32}, dt::f16, tag::any), 2);
    CHECK(spd.get_axis() == 2);
    CHECK(spd.get_algorithm() == algorithm::softmax_accurate);
    CHECK(spd.dst_desc() == memory::desc({4, 6, 32}, dt::f16, tag::abc));
    thrown = false;
    try {
        softmax_forward::primitive_desc bad(eng, prop_kind::forward_inference,
                algorithm::softmax_accurate, sm_src, sm_src, 3);
    } catch (const error &e) { thrown = e.status == dnnl_invalid_arguments; }
    CHECK(thrown);
    std::printf("host ok\n");
    return 0;
}

static int gpu_checks() {
    CHECK(engine::get_count(engine::kind::gpu) >= 1);
    engine eng(engine::kind::gpu, 0);
    stream strm(eng);
    const memory::dim M = 200, K = 320, N = 448;

    uint32_t seed = 2024;
    std::vector<uint8_t> src(M * K);
    std::vector<int8_t> wei(K * N);
    std::vector<float> wscale(N), bias(N);
    for (auto &v : src) v = (uint8_t)(lcg(seed) % 256);
    for (auto &v : wei) v = (int8_t)((int)(lcg(seed) % 255) - 127);
    for (auto &v : wscale) v = 0.001f + (float)(lcg(seed) % 1000) * 1e-5f;
    for (auto &v : bias) v = (float)((int)(lcg(seed) % 200) - 100) * 0.25f;
    const float sscale = 0.0375f;
    const int32_t szp = 117;

    memory::desc src_md({M, K}, dt::u8, tag::ab);
    memory::desc wei_user_md({K, N}, dt::s8, tag::ab);
    memory::desc bias_md({1, N}, dt::f32, tag::ab);
    memory::desc dst_md({M, N}, dt::f32, tag::ab);
    primitive_attr attr = linear_attr();
    matmul::primitive_desc pd(eng, src_md, memory::desc({K, N}, dt::s8, tag::any),
            bias_md, dst_md, attr);
    std::printf("matmul impl: %s\n", pd.impl_info_str());

    memory src_m(src_md, eng), wei_user_m(wei_user_md, eng);
    memory wei_m(pd.weights_desc(), eng), bias_m(bias_md, eng), dst_m(dst_md, eng);
    memory ss_m({{1}, dt::f32, tag::x}, eng), ws_m({{N}, dt::f32, tag::x}, eng);
    memory zp_m({{1}, dt::s32, tag::x}, eng);
    upload(src_m, src);
    upload(wei_user_m, wei);
    upload(bias_m, bias);
    upload(ss_m, std::vector<float> {sscale});
    upload(ws_m, wscale);
    upload(zp_m, std::vector<int32_t> {szp});

    reorder(wei_user_m, wei_m).execute(strm, wei_user_m, wei_m);
    matmul mm(pd);
    mm.execute(strm,
            {{DNNL_ARG_SRC, src_m}, {DNNL_ARG_WEIGHTS, wei_m},
                    {DNNL_ARG_BIAS, bias_m}, {DNNL_ARG_DST, dst_m},
                    {DNNL_ARG_ATTR_SCALES | DNNL_ARG_SRC, ss_m},
                    {DNNL_ARG_ATTR_SCALES | DNNL_ARG_WEIGHTS, ws_m},
                    {DNNL_ARG_ATTR_ZERO_POINTS | DNNL_ARG_SRC, zp_m}});
    strm.wait();
    std::vector<float> got = download<float>(dst_m, M * N);

    double worst = 0;
    for (memory::dim m = 0; m < M; ++m)
        for (memory::dim n = 0; n < N; ++n) {
            int32_t acc = 0;
            for (memory::dim k = 0; k < K; ++k)
                acc += ((int32_t)src[m * K + k] - szp) * (int32_t)wei[k * N + n];
            float v = (float)acc * sscale * wscale[n] + bias[n];
            v = v > 0.f ? v : 0.f;
            const double err = std::fabs((double)got[m * N + n] - v)
                    / (std::fabs((double)v) + 1e-3);
            if (err > worst) worst = err;
        }
    std::printf("matmul worst relative error %.3g\n", worst);
    CHECK(worst < 1e-5);

    // inner product: dst[m][n] = sum_k src[m][k] * wei[n][k] + bias[n]
    std::vector<int8_t> src8(M * K), wei_oi(N * K);
    for (auto &v : src8) v = (int8_t)((int)(lcg(seed) % 255) - 127);
    for (memory::dim n = 0; n < N; ++n)
        for (memory::dim k = 0; k < K; ++k) wei_oi[n * K + k] = wei[k * N + n];
    memory::desc ip_src_md({M, K}, dt::s8, tag::nc);
    memory::desc ip_wei_user_md({N, K}, dt::s8, tag::oi);
    memory::desc ip_bias_md({N}, dt::f32, tag::x);
    memory::desc ip_dst_md({M, N}, dt::s32, tag::nc);
    inner_product_forward::primitive_desc ipd(eng, prop_kind::forward_inference,
            ip_src_md, memory::desc({N, K}, dt::s8, tag::any), ip_bias_md,
            ip_dst_md);
    std::printf("inner product impl: %s\n", ipd.impl_info_str());
    memory ip_src_m(ip_src_md, eng), ip_wei_user_m(ip_wei_user_md, eng);
    memory ip_wei_m(ipd.weights_desc(), eng), ip_bias_m(ip_bias_md, eng);
    memory ip_dst_m(ip_dst_md, eng);
    upload(ip_src_m, src8);
    upload(ip_wei_user_m, wei_oi);
    upload(ip_bias_m, bias);
    reorder(ip_wei_user_m, ip_wei_m).execute(strm, ip_wei_user_m, ip_wei_m);
    inner_product_forward(ipd).execute(strm,
            {{DNNL_ARG_SRC, ip_src_m}, {DNNL_ARG_WEIGHTS, ip_wei_m},
                    {DNNL_ARG_BIAS, ip_bias_m}, {DNNL_ARG_DST, ip_dst_m}});
    strm.wait();
    std::vector<int32_t> got32 = download<int32_t>(ip_dst_m, M * N);
    for (memory::dim m = 0; m < M; ++m)
        for (memory::dim n = 0; n < N; ++n) {
            int32_t acc = 0;
            for (memory::dim k = 0; k < K; ++k)
                acc += (int32_t)src8[m * K + k] * (int32_t)wei_oi[n * K + k];
            // bias is added in f32, the result rounds to nearest even into s32
            const int32_t want = (int32_t)std::nearbyintf((float)acc + bias[n]);
            if (got32[m * N + n] != want) {
                std::printf("inner product mismatch at (%ld, %ld): %d vs %d\n",
                        (long)m, (long)n, got32[m * N + n], want);
                return 1;
            }
        }
    // softmax over rows of equal values: every probability is exactly 1 / 64
    memory::desc sm_md({8, 64}, dt::f32, tag::ab);
    softmax_forward::primitive_desc spd(eng, prop_kind::forward_inference,
            algorithm::softmax_accurate, sm_md, sm_md, 1);
    memory sm_src(sm_md, eng), sm_dst(sm_md, eng);
    std::vector<float> ones(8 * 64, 3.25f);
    upload(sm_src, ones);
    softmax_forward(spd).execute(
            strm, {{DNNL_ARG_SRC, sm_src}, {DNNL_ARG_DST, sm_dst}});
    strm.wait();
    for (float v : download<float>(sm_dst, 8 * 64))
        if (v != 1.f / 64.f) {
            std::printf("softmax mismatch: %g\n", v);
            return 1;
        }
    std::printf("gpu ok\n");
    return 0;
}

int main(int argc, char **argv) {
    const bool gpu = argc > 1 && std::strcmp(argv[1], "gpu") == 0;
    try {
        return gpu ? gpu_checks() : host_checks();
    } catch (const error &e) {
        std::printf("dnnl::error status %d: %s\n", (int)e.status, e.message);
        return 2;
    }
}
