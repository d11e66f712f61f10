"""Parity at the full sizes of the benchmark configurations.

The oracle cannot run these shapes whole in seconds, so each test uses a
property of the problem that is independent of the size: output rows of a
matmul depend only on their own source row, hence an evenly spaced sample of
rows, recomputed by the oracle from the same operands, pins the full-size
launch (tile scheduling, XCD mapping, tails, large strides)."""
import sys

import numpy as np
import pytest

import onednn_amd as dnnl
import oracle as O
from onednn_amd import memory
from qmm_harness import T, assert_bf16_within_1ulp, assert_bit_exact, assert_f32_close, dt, tag

pytestmark = pytest.mark.gpu
A = dnnl


def say(msg):
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def ctx():
    eng = dnnl.engine(dnnl.engine.kind.gpu, 0)
    return eng, dnnl.stream(eng)


def prepack(eng, strm, pd, plain_md, raw):
    plain = memory(plain_md, eng).write(raw)
    packed = memory(pd.weights_desc(), eng)
    dnnl.reorder(plain, packed).execute(strm, plain, packed)
    strm.wait()
    return packed


def test_config2_w8a8_linear_full(ctx):
    eng, strm = ctx
    say("config 2 full size 4096x4096x14336, sampled rows vs oracle")
    M, K, N = 4096, 4096, 14336
    r = np.random.default_rng(2)
    src = np.clip(np.rint(r.standard_normal((M, K)) * 32), -127, 127).astype(np.int8)
    wei = r.integers(-127, 128, (K, N), dtype=np.int8)
    ss = r.uniform(0.005, 0.05, M).astype(np.float32)
    ws = r.uniform(0.0005, 0.005, N).astype(np.float32)
    sel = np.linspace(0, M - 1, 24).astype(np.int64)
    for alg, exact in ((None, True), (A.algorithm.eltwise_swish, False)):
        attr = A.primitive_attr()
        attr.set_scales(A.DNNL_ARG_SRC, 3, [1, K], dt.f32)
        attr.set_scales_mask(A.DNNL_ARG_WEIGHTS, 2)
        pos = []
        if alg is not None:
            po = A.post_ops()
            po.append_eltwise(alg, 1.0, 0.0)
            attr.set_post_ops(po)
            pos = [{"kind": "eltwise", "alg": alg, "alpha": 1.0}]
        pd = A.matmul.primitive_desc(eng, memory.desc([M, K], dt.s8, T("ab")), memory.desc([K, N], dt.s8, tag.any),
                                     memory.desc([M, N], dt.bf16, T("ab")), attr=attr)
        assert pd.impl_info_str() == "hip:gfx950:mfma_b8"
        m_wei = prepack(eng, strm, pd, memory.desc([K, N], dt.s8, T("ab")), wei)
        m_dst = memory(pd.dst_desc(), eng)
        A.matmul(pd).execute(strm, {
            A.DNNL_ARG_SRC: memory(pd.src_desc(), eng).write(src), A.DNNL_ARG_WEIGHTS: m_wei, A.DNNL_ARG_DST: m_dst,
            A.DNNL_ARG_ATTR_SCALES | A.DNNL_ARG_SRC: memory(memory.desc([M], dt.f32, T("a")), eng).write(ss),
            A.DNNL_ARG_ATTR_SCALES | A.DNNL_ARG_WEIGHTS: memory(memory.desc([N], dt.f32, T("a")), eng).write(ws)})
        strm.wait()
        got = m_dst.read(np.uint16, (M, N))[sel]
        want = np.zeros((len(sel), N), np.uint16)
        O.matmul(O.Tensor(O.S8, [len(sel), K], np.ascontiguousarray(src[sel])), O.Tensor(O.S8, [K, N], wei),
                 O.Tensor(O.BF16, [len(sel), N], want),
                 scales={O.Q_SRC: O.Quant(3, O.F32, np.ascontiguousarray(ss[sel]), (1, K)), O.Q_WEI: O.Quant(2, O.F32, ws)},
                 post_ops=pos)
        if exact:
            assert_bit_exact(got, want, "config 2 without swish")  # bf16 of exact arithmetic: bit-exact
        else:
            # 1 bf16 ulp (the exp implementation differs from libm); swish results
            # below 1e-30 in magnitude may flush to zero (hardware rcp has no denormals)
            off = assert_bf16_within_1ulp(got, want, "config 2", abs_slack=1e-30)
            assert off < 0.01


def test_config3_decode_full(ctx):
    eng, strm = ctx
    K = N = 4096
    G = 128
    r = np.random.default_rng(3)
    w = r.integers(0, 16, (K, N))
    sc = O.from_f32(O.F16, r.uniform(0.005, 0.02, (K // G, N)).astype(np.float32))
    zp = r.integers(6, 10, (K // G, N))
    for M in (1, 16):
        say("config 3 full size M=%d K=N=4096" % M)
        a = O.from_f32(O.BF16, r.standard_normal((M, K)).astype(np.float32))
        attr = A.primitive_attr()
        attr.set_fpmath_mode(A.fpmath_mode.bf16, True)
        attr.set_scales(A.DNNL_ARG_WEIGHTS, 3, [G, 1], dt.f16)
        attr.set_zero_points(A.DNNL_ARG_WEIGHTS, 3, [G, 1], dt.u4)
        pd = A.matmul.primitive_desc(eng, memory.desc([M, K], dt.bf16, T("ab")), memory.desc([K, N], dt.u4, tag.any),
                                     memory.desc([M, N], dt.bf16, T("ab")), attr=attr)
        assert pd.impl_info_str() == "hip:gfx950:decode_w4"
        m_wei = prepack(eng, strm, pd, memory.desc([K, N], dt.u4, T("ab")), O.pack4(w))
        m_dst = memory(pd.dst_desc(), eng)
        A.matmul(pd).execute(strm, {
            A.DNNL_ARG_SRC: memory(pd.src_desc(), eng).write(a), A.DNNL_ARG_WEIGHTS: m_wei, A.DNNL_ARG_DST: m_dst,
            A.DNNL_ARG_ATTR_SCALES | A.DNNL_ARG_WEIGHTS: memory(memory.desc([sc.nbytes], dt.u8, T("a")), eng).write(sc),
            A.DNNL_ARG_ATTR_ZERO_POINTS | A.DNNL_ARG_WEIGHTS:
                memory(memory.desc([K // G * N // 2], dt.u8, T("a")), eng).write(O.pack4(zp))})
        strm.wait()
        got = m_dst.read(np.uint16, (M, N))
        want = np.zeros((M, N), np.uint16)
        O.matmul(O.Tensor(O.BF16, [M, K], a), O.Tensor(O.U4, [K, N], O.pack4(w)), O.Tensor(O.BF16, [M, N], want),
                 scales={O.Q_WEI: O.Quant(3, O.F16, sc, (G, 1))}, zps={O.Q_WEI: O.Quant(3, O.U4, O.pack4(zp), (G, 1))},
                 apply_to_int=True)
        g, wv = O.to_f32(O.BF16, got), O.to_f32(O.BF16, want)
        scf = np.repeat(O.to_f32(O.F16, sc).astype(np.float64), G, 0)
        terms = np.abs(O.to_f32(O.BF16, a).astype(np.float64)) @ (np.abs(w - np.repeat(zp, G, 0)) * scf)
        assert_f32_close(g, wv, rel=1e-2, scale=np.abs(wv).mean(), what="config 3")  # the bar: rel 1e-2
        assert_bf16_within_1ulp(got, want, "config 3 bf16", abs_slack=2e-5 * terms)  # what it achieves


def test_config4_batched_scores_full(ctx):
    eng, strm = ctx
    say("config 4 full size 32x2048x128x2048 + causal mask, sampled rows vs oracle")
    B, S, D = 32, 2048, 128
    r = np.random.default_rng(4)
    q = np.clip(np.rint(r.standard_normal((B, S, D)) * 40), -127, 127).astype(np.int8)
    k = np.clip(np.rint(r.standard_normal((B, S, D)) * 40), -127, 127).astype(np.int8)  # K, used as K^T
    mask = np.where(np.arange(S)[None, :] > np.arange(S)[:, None], -1e4, 0).astype(np.float32)[None]
    attr = A.primitive_attr()
    attr.set_scales_mask(A.DNNL_ARG_SRC, 0)
    attr.set_scales_mask(A.DNNL_ARG_WEIGHTS, 0)
    po = A.post_ops()
    po.append_binary(A.algorithm.binary_add, memory.desc([1, S, S], dt.f32, T("abc")))
    attr.set_post_ops(po)
    kt_md = memory.desc([B, D, S], dt.s8, T("acb"))  # K^T as a strided view of K
    pd = A.matmul.primitive_desc(eng, memory.desc([B, S, D], dt.s8, T("abc")), kt_md,
                                 memory.desc([B, S, S], dt.f32, T("abc")), attr=attr)
    assert pd.impl_info_str() == "hip:gfx950:mfma_b8"
    m_dst = memory(pd.dst_desc(), eng)
    A.matmul(pd).execute(strm, {
        A.DNNL_ARG_SRC: memory(pd.src_desc(), eng).write(q), A.DNNL_ARG_WEIGHTS: memory(kt_md, eng).write(k),
        A.DNNL_ARG_DST: m_dst,
        A.DNNL_ARG_ATTR_SCALES | A.DNNL_ARG_SRC: memory(memory.desc([1], dt.f32, T("a")), eng).write(np.array([0.01], np.float32)),
        A.DNNL_ARG_ATTR_SCALES | A.DNNL_ARG_WEIGHTS: memory(memory.desc([1], dt.f32, T("a")), eng).write(np.array([0.012], np.float32)),
        A.DNNL_ARG_ATTR_MULTIPLE_POST_OP(0) | A.DNNL_ARG_SRC_1: memory(memory.desc([1, S, S], dt.f32, T("abc")), eng).write(mask)})
    strm.wait()
    got = m_dst.read(np.float32, (B, S, S))
    bsel, msel = [0, 13, 31], np.linspace(0, S - 1, 16).astype(np.int64)
    for b in bsel:
        want = np.zeros((1, len(msel), S), np.float32)
        O.matmul(O.Tensor(O.S8, [1, len(msel), D], np.ascontiguousarray(q[b][msel])),
                 O.Tensor(O.S8, [1, D, S], k[b], (D * S, 1, D)), O.Tensor(O.F32, [1, len(msel), S], want),
                 scales={O.Q_SRC: O.Quant(0, O.F32, np.array([0.01], np.float32)),
                         O.Q_WEI: O.Quant(0, O.F32, np.array([0.012], np.float32))},
                 post_ops=[{"kind": "binary", "alg": A.algorithm.binary_add,
                            "src1": O.Tensor(O.F32, [1, len(msel), S], np.ascontiguousarray(mask[:, msel]))}])
        assert_bit_exact(got[b][msel], want[0], "config 4 head %d" % b)  # exact ops: f32 bit-exact


def test_config5_fp8_full(ctx):
    eng, strm = ctx
    say("config 5 full size 8192^3 fp8 + sum, sampled rows vs oracle")
    n = 8192
    r = np.random.default_rng(5)
    base = O.from_f32(O.F8_E4M3, np.clip(r.standard_normal(1 << 20) * 4, -448, 448).astype(np.float32))
    a = np.resize(base, (n, n))
    b = np.resize(np.roll(base, 12345), (n, n))
    old = O.from_f32(O.BF16, np.resize(r.standard_normal(1 << 20).astype(np.float32), (n, n)))
    attr = A.primitive_attr()
    attr.set_scales_mask(A.DNNL_ARG_SRC, 0)
    attr.set_scales_mask(A.DNNL_ARG_WEIGHTS, 0)
    po = A.post_ops()
    po.append_sum(1.0)
    attr.set_post_ops(po)
    pd = A.matmul.primitive_desc(eng, memory.desc([n, n], dt.f8_e4m3, T("ab")), memory.desc([n, n], dt.f8_e4m3, tag.any),
                                 memory.desc([n, n], dt.bf16, T("ab")), attr=attr)
    assert pd.impl_info_str() == "hip:gfx950:mfma_b8"
    m_wei = prepack(eng, strm, pd, memory.desc([n, n], dt.f8_e4m3, T("ab")), b)
    m_dst = memory(pd.dst_desc(), eng).write(old)
    A.matmul(pd).execute(strm, {
        A.DNNL_ARG_SRC: memory(pd.src_desc(), eng).write(a), A.DNNL_ARG_WEIGHTS: m_wei, A.DNNL_ARG_DST: m_dst,
        A.DNNL_ARG_ATTR_SCALES | A.DNNL_ARG_SRC: memory(memory.desc([1], dt.f32, T("a")), eng).write(np.array([0.5], np.float32)),
        A.DNNL_ARG_ATTR_SCALES | A.DNNL_ARG_WEIGHTS: memory(memory.desc([1], dt.f32, T("a")), eng).write(np.array([0.25], np.float32))})
    strm.wait()
    sel = np.array([0, 1777, 4096, 8191])
    got = m_dst.read(np.uint16, (n, n))[sel]
    want = np.ascontiguousarray(old[sel])
    O.matmul(O.Tensor(O.F8_E4M3, [len(sel), n], np.ascontiguousarray(a[sel])), O.Tensor(O.F8_E4M3, [n, n], b),
             O.Tensor(O.BF16, [len(sel), n], want),
             scales={O.Q_SRC: O.Quant(0, O.F32, np.array([0.5], np.float32)), O.Q_WEI: O.Quant(0, O.F32, np.array([0.25], np.float32))},
             post_ops=[{"kind": "sum", "scale": 1.0}])
    terms = np.abs(O.to_f32(O.F8_E4M3, a[sel]).astype(np.float64)) @ np.abs(O.to_f32(O.F8_E4M3, b).astype(np.float64)) * 0.125
    # f32 accumulation in MFMA order vs the reference's k loop: 1 bf16 ulp, or 1e-5 of the
    # summed magnitudes where the result cancels
    assert_bf16_within_1ulp(got, want, "config 5", abs_slack=1e-5 * terms)
