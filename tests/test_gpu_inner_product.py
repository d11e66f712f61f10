"""Inner product (forward) lowered onto the matmul implementations: parity
against the CPU oracle's matmul on the equivalent [MB, K] x [K, OC] problem,
through the C ABI (dnnl_inner_product_forward_primitive_desc_create)."""
import sys

import numpy as np
import pytest

import onednn_amd as dnnl
import oracle as O
from onednn_amd import memory
from qmm_harness import Problem, T, TensorSpec, assert_bit_exact, dt, tag

pytestmark = pytest.mark.gpu
A = dnnl.algorithm


def say(msg):
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def ctx():
    eng = dnnl.engine(dnnl.engine.kind.gpu, 0)
    return eng, dnnl.stream(eng)


def run_ip(eng, strm, src_dims, OC, seed, wei_mode="plain", dst_dt=dt.f32, relu=True):
    """int8 inner product with a common src scale, per-OC weights scales, f32
    bias and an optional relu; returns (result, oracle result, pd)."""
    r = np.random.default_rng(seed)
    MB = src_dims[0]
    K = int(np.prod(src_dims[1:]))
    nd = len(src_dims)
    letters = "abcde"[:nd]
    s = np.clip(np.rint(r.standard_normal(src_dims) * 30), -127, 127).astype(np.int8)
    w = r.integers(-127, 128, [OC] + list(src_dims[1:])).astype(np.int8)
    bias = r.standard_normal(OC).astype(np.float32)
    wsc = r.uniform(0.001, 0.01, OC).astype(np.float32)
    attr = dnnl.primitive_attr()
    attr.set_scales_mask(dnnl.DNNL_ARG_SRC, 0)
    attr.set_scales_mask(dnnl.DNNL_ARG_WEIGHTS, 1)  # per output channel: dim 0 of [OC, IC, ...]
    po = []
    if relu:
        p_ = dnnl.post_ops()
        p_.append_eltwise(A.eltwise_relu, 0.0, 0.0)
        attr.set_post_ops(p_)
        po = [{"kind": "eltwise", "alg": A.eltwise_relu, "alpha": 0.0}]
    src_md = memory.desc(list(src_dims), dt.s8, T(letters))
    wdims = [OC] + list(src_dims[1:])
    plain_w_md = memory.desc(wdims, dt.s8, T(letters))
    w_md = memory.desc(wdims, dt.s8, tag.any) if wei_mode == "any" else plain_w_md
    dst_md = memory.desc([MB, OC], dst_dt, T("ab"))
    pd = dnnl.inner_product_forward.primitive_desc(eng, dnnl.prop_kind.forward_inference, src_md, w_md, dst_md,
                                                   bias_md=memory.desc([OC], dt.f32, T("a")), attr=attr)
    assert pd.src_desc().get_dims() == list(src_dims)
    assert pd.weights_desc().get_dims() == wdims
    prim = dnnl.inner_product_forward(pd)
    m_plain_w = memory(plain_w_md, eng).write(w)
    m_w = m_plain_w
    if wei_mode == "any":
        assert pd.weights_desc().get_format_kind() == memory.format_kind.opaque
        m_w = memory(pd.weights_desc(), eng)
        dnnl.reorder(m_plain_w, m_w).execute(strm, m_plain_w, m_w)
    m_dst = memory(pd.dst_desc(), eng)
    prim.execute(strm, {dnnl.DNNL_ARG_SRC: memory(src_md, eng).write(s), dnnl.DNNL_ARG_WEIGHTS: m_w,
                        dnnl.DNNL_ARG_BIAS: memory(memory.desc([OC], dt.f32, T("a")), eng).write(bias),
                        dnnl.DNNL_ARG_DST: m_dst,
                        dnnl.DNNL_ARG_ATTR_SCALES | dnnl.DNNL_ARG_SRC: memory(memory.desc([1], dt.f32, T("a")), eng).write(
                            np.array([0.05], np.float32)),
                        dnnl.DNNL_ARG_ATTR_SCALES | dnnl.DNNL_ARG_WEIGHTS: memory(memory.desc([OC], dt.f32, T("a")), eng).write(wsc)})
    strm.wait()
    # the same numbers as a matmul for the oracle
    p = Problem(TensorSpec(dt.s8, [MB, K], None, s.reshape(MB, K)),
                TensorSpec(dt.s8, [K, OC], None, w.reshape(OC, K).T.copy()),
                TensorSpec(dst_dt, [MB, OC]),
                bias=TensorSpec(dt.f32, [1, OC], None, bias),
                scales={"src": (0, dt.f32, None, [0.05]), "wei": (2, dt.f32, None, wsc)}, post_ops=po)
    return m_dst.read(p.dst.raw.dtype), p.run_oracle(), pd


@pytest.mark.parametrize("wei_mode", ["plain", "any"])
def test_inner_product_int8_2d(ctx, wei_mode):
    eng, strm = ctx
    say("inner product s8 [70, 256] x [96, 256], weights %s" % wei_mode)
    got, want, pd = run_ip(eng, strm, (70, 256), 96, 1, wei_mode)
    assert pd.impl_info_str() == "hip:gfx950:mfma_b8"
    assert_bit_exact(got, want, "ip 2d %s" % wei_mode)


@pytest.mark.parametrize("wei_mode", ["plain", "any"])
def test_inner_product_int8_4d_source(ctx, wei_mode):
    eng, strm = ctx
    say("inner product s8 [33, 16, 4, 4] x [80, 16, 4, 4], weights %s" % wei_mode)
    got, want, pd = run_ip(eng, strm, (33, 16, 4, 4), 80, 2, wei_mode, relu=False)
    assert pd.impl_info_str() == "hip:gfx950:mfma_b8"
    assert_bit_exact(got, want, "ip 4d %s" % wei_mode)


def test_inner_product_large_takes_the_256_tile_kernel(ctx):
    eng, strm = ctx
    say("inner product s8 [4096, 1024] x [3072, 1024] -> s8-like f32 epilogue")
    got, want, pd = run_ip(eng, strm, (4096, 1024), 3072, 3, "any")
    assert_bit_exact(got, want, "ip large")
