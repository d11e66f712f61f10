"""Matmul primitives created with DNNL_RUNTIME_DIM_VAL: one primitive serves
every shape, each execution resolving the memory objects' own descriptors to
the implementation a concrete primitive of that shape would get. Results are
held to the same bar as the concrete primitives (bit-exact for integer
arithmetic, 1 bf16 ulp for bf16 results)."""
import numpy as np
import pytest

import onednn_amd as dnnl
from onednn_amd import memory, status
from qmm_harness import T, assert_bf16_within_1ulp, assert_bit_exact, dt
import test_gpu_parity as cases

pytestmark = pytest.mark.gpu
A = dnnl.algorithm


@pytest.fixture(scope="module")
def ctx():
    eng = dnnl.engine(dnnl.engine.kind.gpu, 0)
    return eng, dnnl.stream(eng)


def test_runtime_m_one_primitive_many_batch_sizes(ctx):
    eng, strm = ctx
    K, N = 256, 384
    mk = lambda M, seed: cases.int8_linear(M, K, N, seed, bias_dt=dt.f32)
    prim = dnnl.matmul(mk(8, 1).runtime_primitive_desc(eng, {"src": [0], "dst": [0]}))
    for i, M in enumerate([5, 64, 300, 5, 1024, 64, 1]):
        cases.say("runtime M = %d" % M)
        p = mk(M, 100 + i)
        assert_bit_exact(p.run_gpu(eng, strm, prim=prim), p.run_oracle(), "M=%d" % M)


def test_runtime_m_with_prepacked_weights(ctx):
    """The reference's int8 inference tutorial
    (examples/tutorials/matmul/inference_int8_matmul.cpp:104-125): M open, weights
    format_tag::any, u8 source and dst with run-time zero points and scales, relu."""
    eng, strm = ctx
    K, N = 256, 384
    mk = lambda M, seed: cases.int8_linear(M, K, N, seed, dst_dt=dt.u8, src_zp=7, dst_scale=0.25, dst_zp=[3],
                                           post_ops=[{"kind": "eltwise", "alg": A.eltwise_relu, "alpha": 0.0}])
    pd = mk(8, 1).runtime_primitive_desc(eng, {"src": [0], "dst": [0]}, weights_any=True)
    assert pd.weights_desc().get_format_kind() == memory.format_kind.opaque
    prim = dnnl.matmul(pd)
    for i, M in enumerate([5, 300, 64, 1024, 1]):
        cases.say("runtime M = %d, prepacked weights" % M)
        p = mk(M, 150 + i)
        assert_bit_exact(p.run_gpu(eng, strm, prim=prim, prim_wei_md=pd.weights_desc()), p.run_oracle(), "M=%d" % M)


def test_runtime_everything_and_post_ops(ctx):
    eng, strm = ctx
    po = [{"kind": "eltwise", "alg": A.eltwise_swish, "alpha": 1.0}]

    def mk(M, K, N, seed):
        # common src scale, per-N weights scales: nothing in the attributes depends on the dims
        return cases.int8_linear(M, K, N, seed, src_dt=dt.s8, dst_dt=dt.bf16, src_zp=None, post_ops=po)
    every = {"src": [0, 1], "wei": [0, 1], "dst": [0, 1]}
    prim = dnnl.matmul(mk(8, 64, 8, 1).runtime_primitive_desc(eng, every))
    for i, (M, K, N) in enumerate([(33, 128, 70), (256, 512, 256), (1, 64, 2), (1024, 256, 1024)]):
        cases.say("runtime M K N = %d %d %d" % (M, K, N))
        p = mk(M, K, N, 200 + i)
        assert_bf16_within_1ulp(p.run_gpu(eng, strm, prim=prim), p.run_oracle(), "%d %d %d" % (M, K, N))


def test_runtime_batch_and_decode_weights(ctx):
    eng, strm = ctx
    mk = lambda B, M, seed: cases.int8_linear(M, 128, 96, seed, src_dt=dt.s8, src_zp=None, batch=(B,))
    prim = dnnl.matmul(mk(2, 8, 1).runtime_primitive_desc(
        eng, {"src": [0, 1], "wei": [0], "dst": [0, 1]}))
    for i, (B, M) in enumerate([(3, 40), (1, 7), (6, 128)]):
        cases.say("runtime batch %d M %d" % (B, M))
        p = mk(B, M, 300 + i)
        assert_bit_exact(p.run_gpu(eng, strm, prim=prim), p.run_oracle(), "B=%d M=%d" % (B, M))
    # 4-bit weights, grouped scales and zero points: M open, the decode kernel per shape
    mk = lambda M, seed: cases.decode_w4(M, 512, 256, seed)
    prim = dnnl.matmul(mk(1, 1).runtime_primitive_desc(eng, {"src": [0], "dst": [0]}))
    for i, M in enumerate([1, 16, 3]):
        cases.say("runtime decode M %d" % M)
        p = mk(M, 400 + i)
        assert_bf16_within_1ulp(p.run_gpu(eng, strm, prim=prim), p.run_oracle(), "decode M=%d" % M)


def test_runtime_shape_cache_evicts_and_keeps_working(ctx):
    eng, strm = ctx
    mk = lambda M, seed: cases.int8_linear(M, 64, 64, seed)
    prim = dnnl.matmul(mk(8, 1).runtime_primitive_desc(eng, {"src": [0], "dst": [0]}))
    for rep in range(2):
        for M in range(1, 41):  # more shapes than the primitive remembers
            p = mk(M, 500 + M)
            assert_bit_exact(p.run_gpu(eng, strm, prim=prim), p.run_oracle(), "M=%d" % M)


def test_runtime_mismatching_memory_is_refused(ctx):
    eng, strm = ctx
    p = cases.int8_linear(16, 64, 32, 600)
    prim = dnnl.matmul(p.runtime_primitive_desc(eng, {"src": [0], "dst": [0]}))
    q = cases.int8_linear(16, 128, 32, 601)  # K differs from the descriptor's
    with pytest.raises(dnnl.error) as e:
        q.run_gpu(eng, strm, prim=prim)
    assert e.value.status == status.invalid_arguments
    q = cases.int8_linear(16, 64, 32, 602)
    q.dst = type(q.dst)(dt.f32, [17, 32])  # M of dst differs from M of src
    with pytest.raises(dnnl.error) as e:
        q.run_gpu(eng, strm, prim=prim)
    assert e.value.status == status.invalid_arguments
