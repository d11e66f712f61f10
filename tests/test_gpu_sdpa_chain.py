"""The attention block as the chain of primitives the reference's own SDPA test uses as its gold path
(tests/gtests/internals/test_sdpa.cpp:893-1043 `prim_sdpa_quant`): dequantizing reorders of a quantized K / V cache,
score matmul with the scale and the mask as binary post-ops, softmax over the keys, value matmul.

Two chains:
 * the f16 chain of that test (K, V s8 with per-token f16 scales and s8 zero points), every stage on the device,
   checked stage by stage against the oracle on the device's own previous stage (so a stage's bar is its own),
   and end to end against float64 attention with the reference test's rule (abs 0.001466 for |gold| <= 1, relative
   above; at most 0.06 % of the elements outside);
 * the int8 chain on the MFMA kernels: s8 Q x s8 K^T -> f32 scores + causal mask (the batched attention-scores
   configuration), softmax -> u8 probabilities (dst scale 1/255), u8 P x s8 V -> f32.
"""
import sys

import numpy as np
import pytest

import onednn_amd as dnnl
import oracle as O
from onednn_amd import memory
from qmm_harness import T, dt

pytestmark = pytest.mark.gpu
A = dnnl.algorithm
FWD = dnnl.prop_kind.forward_inference


def say(msg):
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def ctx():
    eng = dnnl.engine(dnnl.engine.kind.gpu, 0)
    return eng, dnnl.stream(eng)


def mem(eng, dims, code, tagname, array=None):
    m = memory(memory.desc(list(dims), code, T(tagname)), eng)
    if array is not None:
        m.write(np.ascontiguousarray(array))
    return m


def reference_rule(test, gold, thr=0.001466):
    """check_memory of the reference test (test_sdpa.cpp:1043-1106)."""
    t, g = test.astype(np.float64).reshape(-1), gold.astype(np.float64).reshape(-1)
    diff = np.abs(t - g)
    bad = np.where(np.abs(g) > 1.0, diff > np.abs(g) * thr, diff > thr) | np.isnan(t) | np.isnan(g)
    return int(bad.sum()), t.size, float(diff.max())


@pytest.mark.parametrize("Qn", [1, 48], ids=["decode", "prefill"])
def test_f16_chain_with_quantized_kv_cache(ctx, Qn):
    eng, strm = ctx
    MB, H, S, D = 2, 3, 160, 64
    say("sdpa chain f16, K/V s8 per-token scales + zero points, queries %d keys %d head %d" % (Qn, S, D))
    r = np.random.default_rng(20 + Qn)
    q = O.from_f32(dt.f16, r.standard_normal((MB, H, Qn, D)).astype(np.float32)).reshape(MB, H, Qn, D)
    kq = r.integers(-128, 128, (MB, H, D, S)).astype(np.int8)       # K^T view: [mb, h, d, keys]
    vq = r.integers(-128, 128, (MB, H, S, D)).astype(np.int8)
    # one scale / zero point per (head, key): mask over dims 1..3, the head-size dim covered by one group
    k_sc = O.from_f32(dt.f16, r.uniform(0.005, 0.02, (MB * 0 + 1, H, 1, S)).astype(np.float32)).reshape(H, S)
    k_zp = r.integers(-6, 7, (H, S)).astype(np.int8)
    v_sc = O.from_f32(dt.f16, r.uniform(0.005, 0.02, (H, S)).astype(np.float32)).reshape(H, S)
    v_zp = r.integers(-6, 7, (H, S)).astype(np.int8)
    scale = np.array([1.0 / np.sqrt(D)], np.float32)
    mask = np.zeros((1, 1, Qn, S), np.float32)
    if Qn > 1:
        mask[0, 0] = np.triu(np.full((Qn, S), -1e4, np.float32), S - Qn + 1)  # causal over the last Qn keys

    # ---- stage 0: dequantize the cache (reorder with source scales and zero points)
    def dequantize(raw, dims, sc, zp, qmask, groups, what):
        attr = dnnl.primitive_attr()
        attr.set_scales(dnnl.DNNL_ARG_FROM, qmask, list(groups), dt.f16)
        attr.set_zero_points(dnnl.DNNL_ARG_SRC, qmask, list(groups), dt.s8)
        src_md = memory.desc(list(dims), dt.s8, T("abcd"))
        dst_md = memory.desc(list(dims), dt.f16, T("abcd"))
        pd = dnnl.reorder.primitive_desc(eng, src_md, eng, dst_md, attr=attr)
        s_mem, d_mem = memory(src_md, eng).write(raw), memory(dst_md, eng)
        sc_m = mem(eng, [sc.size], dt.f16, "a", sc)
        zp_m = mem(eng, [zp.size], dt.s8, "a", zp)
        dnnl.reorder(pd).execute(strm, {dnnl.DNNL_ARG_FROM: s_mem, dnnl.DNNL_ARG_TO: d_mem,
                                        dnnl.DNNL_ARG_ATTR_SCALES | dnnl.DNNL_ARG_FROM: sc_m,
                                        dnnl.DNNL_ARG_ATTR_ZERO_POINTS | dnnl.DNNL_ARG_FROM: zp_m})
        strm.wait()
        got = d_mem.read(np.uint16, dims)
        want = np.zeros(dims, np.uint16)
        O.reorder(O.Tensor(dt.s8, list(dims), raw), O.Tensor(dt.f16, list(dims), want),
                  src_scale=O.Quant(qmask, dt.f16, sc, groups), src_zp=O.Quant(qmask, dt.s8, zp, groups))
        assert np.array_equal(got, want), what
        return d_mem, got

    k_mem, k_deq = dequantize(kq, (MB, H, D, S), k_sc, k_zp, 0b1110, (D, 1), "K dequantization")  # [h, keys]
    v_mem, v_deq = dequantize(vq, (MB, H, S, D), v_sc, v_zp, 0b1110, (1, D), "V dequantization")  # [h, keys]

    # ---- stage 1: scores = (Q x K) * scale + mask, f32
    attr = dnnl.primitive_attr()
    po = dnnl.post_ops()
    po.append_binary(A.binary_mul, memory.desc([1, 1, 1, 1], dt.f32, T("abcd")))
    po.append_binary(A.binary_add, memory.desc([1, 1, Qn, S], dt.f32, T("abcd")))
    attr.set_post_ops(po)
    q_md = memory.desc([MB, H, Qn, D], dt.f16, T("abcd"))
    s_md = memory.desc([MB, H, Qn, S], dt.f32, T("abcd"))
    pd1 = dnnl.matmul.primitive_desc(eng, q_md, k_mem.get_desc(), s_md, attr=attr)
    q_mem, score = memory(q_md, eng).write(q), memory(s_md, eng)
    sc_mem = mem(eng, [1, 1, 1, 1], dt.f32, "abcd", scale)
    mk_mem = mem(eng, [1, 1, Qn, S], dt.f32, "abcd", mask)
    dnnl.matmul(pd1).execute(strm, {dnnl.DNNL_ARG_SRC: q_mem, dnnl.DNNL_ARG_WEIGHTS: k_mem, dnnl.DNNL_ARG_DST: score,
                                    dnnl.DNNL_ARG_ATTR_MULTIPLE_POST_OP(0) | dnnl.DNNL_ARG_SRC_1: sc_mem,
                                    dnnl.DNNL_ARG_ATTR_MULTIPLE_POST_OP(1) | dnnl.DNNL_ARG_SRC_1: mk_mem})
    strm.wait()
    got_s = score.read(np.float32, (MB, H, Qn, S))
    want_s = np.zeros((MB, H, Qn, S), np.float32)
    O.matmul(O.Tensor(dt.f16, [MB, H, Qn, D], q), O.Tensor(dt.f16, [MB, H, D, S], k_deq),
             O.Tensor(dt.f32, [MB, H, Qn, S], want_s),
             post_ops=[{"kind": "binary", "alg": A.binary_mul, "src1": O.Tensor(dt.f32, [1, 1, 1, 1], scale)},
                       {"kind": "binary", "alg": A.binary_add, "src1": O.Tensor(dt.f32, [1, 1, Qn, S], mask)}])
    # the 16-bit MFMA matmul sums in another order than the oracle's k loop: 1e-5 of the magnitude of the summed terms
    err_s = np.abs(got_s.astype(np.float64) - want_s)
    tol_s = 1e-5 * np.maximum(np.abs(want_s), np.sqrt(D) * np.abs(float(scale[0])))
    assert np.all((err_s <= tol_s) | np.isinf(want_s)), ("scores", float(err_s[np.isfinite(want_s)].max()))

    # ---- stage 2: softmax over the keys, f32 -> f16
    p_md = memory.desc([MB, H, Qn, S], dt.f16, T("abcd"))
    pd2 = dnnl.softmax_forward.primitive_desc(eng, FWD, A.softmax_accurate, s_md, p_md, 3)
    prob = memory(p_md, eng)
    dnnl.softmax_forward(pd2).execute(strm, score, prob)
    strm.wait()
    got_p = prob.read(np.uint16, (MB, H, Qn, S))
    want_p = np.zeros((MB, H, Qn, S), np.uint16)
    O.softmax(O.Tensor(dt.f32, [MB, H, Qn, S], got_s), O.Tensor(dt.f16, [MB, H, Qn, S], want_p), 3)
    d = np.abs(got_p.astype(np.int32) - want_p.astype(np.int32))
    assert d.max() <= 1 and (d != 0).mean() < 0.02, ("probabilities", int(d.max()), float((d != 0).mean()))

    # ---- stage 3: out = P x V, f16
    o_md = memory.desc([MB, H, Qn, D], dt.f16, T("abcd"))
    pd3 = dnnl.matmul.primitive_desc(eng, p_md, v_mem.get_desc(), o_md)
    out = memory(o_md, eng)
    dnnl.matmul(pd3).execute(strm, {dnnl.DNNL_ARG_SRC: prob, dnnl.DNNL_ARG_WEIGHTS: v_mem, dnnl.DNNL_ARG_DST: out})
    strm.wait()
    got_o = out.read(np.uint16, (MB, H, Qn, D))
    want_o = np.zeros((MB, H, Qn, D), np.uint16)
    O.matmul(O.Tensor(dt.f16, [MB, H, Qn, S], got_p), O.Tensor(dt.f16, [MB, H, S, D], v_deq),
             O.Tensor(dt.f16, [MB, H, Qn, D], want_o))
    d_o = np.abs(got_o.astype(np.int32) - want_o.astype(np.int32))  # f16 codes: at most one step apart
    near_zero = np.abs(O.to_f32(dt.f16, want_o).reshape(want_o.shape)) < 2.0 ** -10
    assert np.all((d_o <= 1) | near_zero) and (d_o != 0).mean() < 0.05, ("output", int(d_o.max()), float((d_o != 0).mean()))

    # ---- end to end against float64 attention on the dequantized operands, the reference test's rule
    kf = O.to_f32(dt.f16, k_deq).reshape(MB, H, D, S).astype(np.float64)
    vf = O.to_f32(dt.f16, v_deq).reshape(MB, H, S, D).astype(np.float64)
    qf = O.to_f32(dt.f16, q).reshape(MB, H, Qn, D).astype(np.float64)
    s64 = qf @ kf * float(scale[0]) + mask
    p64 = np.exp(s64 - s64.max(axis=-1, keepdims=True))
    p64 /= p64.sum(axis=-1, keepdims=True)
    gold = p64 @ vf
    bad, total, worst = reference_rule(O.to_f32(dt.f16, got_o), gold)
    print("[sdpa chain] %d of %d outside the reference test's threshold, max diff %.2e" % (bad, total, worst))
    assert bad <= total * 0.0006


def test_int8_chain_on_the_mfma_kernels(ctx):
    """s8 Q x s8 K^T (+ causal mask) -> softmax -> u8 P x s8 V: both matmuls on the int8 MFMA kernels, the
    probabilities quantized by the softmax's destination scale. Stage by stage against the oracle on the device's
    previous stage; end to end against float64 attention on the dequantized operands (u8 probabilities: the error
    budget is 1 / 255 / 2 per probability, far below it after the sum over keys)."""
    eng, strm = ctx
    B, S, D = 4, 512, 128
    say("int8 attention chain, %d heads x %d x %d" % (B, S, D))
    r = np.random.default_rng(31)
    q = np.clip(np.rint(r.standard_normal((B, S, D)) * 40), -127, 127).astype(np.int8)
    k = np.clip(np.rint(r.standard_normal((B, S, D)) * 40), -127, 127).astype(np.int8)   # [heads, keys, d]
    v = np.clip(np.rint(r.standard_normal((B, S, D)) * 40), -127, 127).astype(np.int8)
    q_scale, k_scale, v_scale = 0.01, 0.012, 0.02
    mask = np.triu(np.full((S, S), -1e4, np.float32), 1)[None]
    # ---- scores: weights are the K^T view (tag acb) of the [heads, keys, d] cache
    attr = dnnl.primitive_attr()
    attr.set_scales_mask(dnnl.DNNL_ARG_SRC, 0)
    attr.set_scales_mask(dnnl.DNNL_ARG_WEIGHTS, 0)
    po = dnnl.post_ops()
    po.append_binary(A.binary_add, memory.desc([1, S, S], dt.f32, T("abc")))
    attr.set_post_ops(po)
    q_md = memory.desc([B, S, D], dt.s8, T("abc"))
    kt_md = memory.desc([B, D, S], dt.s8, T("acb"))
    s_md = memory.desc([B, S, S], dt.f32, T("abc"))
    pd1 = dnnl.matmul.primitive_desc(eng, q_md, kt_md, s_md, attr=attr)
    assert pd1.impl_info_str() == "hip:gfx950:mfma_b8"
    score = memory(s_md, eng)
    one = lambda val: mem(eng, [1], dt.f32, "a", np.array([val], np.float32))
    dnnl.matmul(pd1).execute(strm, {dnnl.DNNL_ARG_SRC: memory(q_md, eng).write(q), dnnl.DNNL_ARG_WEIGHTS: memory(kt_md, eng).write(k),
                                    dnnl.DNNL_ARG_DST: score,
                                    dnnl.DNNL_ARG_ATTR_SCALES | dnnl.DNNL_ARG_SRC: one(q_scale),
                                    dnnl.DNNL_ARG_ATTR_SCALES | dnnl.DNNL_ARG_WEIGHTS: one(k_scale),
                                    dnnl.DNNL_ARG_ATTR_MULTIPLE_POST_OP(0) | dnnl.DNNL_ARG_SRC_1: mem(eng, [1, S, S], dt.f32, "abc", mask)})
    strm.wait()
    got_s = score.read(np.float32, (B, S, S))
    want_s = np.zeros((B, S, S), np.float32)
    O.matmul(O.Tensor(dt.s8, [B, S, D], q), O.Tensor(dt.s8, [B, D, S], k, [S * D, 1, D]), O.Tensor(dt.f32, [B, S, S], want_s),
             scales={O.Q_SRC: O.Quant(0, dt.f32, np.array([q_scale], np.float32)),
                     O.Q_WEI: O.Quant(0, dt.f32, np.array([k_scale], np.float32))},
             post_ops=[{"kind": "binary", "alg": A.binary_add, "src1": O.Tensor(dt.f32, [1, S, S], mask)}],
             k_group_mode=O.KGROUP_WHOLE)
    assert np.array_equal(got_s, want_s), "scores"
    # ---- probabilities as u8 with scale 1/255
    p_md = memory.desc([B, S, S], dt.u8, T("abc"))
    attr2 = dnnl.primitive_attr()
    attr2.set_scales_mask(dnnl.DNNL_ARG_DST, 0)
    pd2 = dnnl.softmax_forward.primitive_desc(eng, FWD, A.softmax_accurate, s_md, p_md, 2, attr2)
    prob = memory(p_md, eng)
    p_scale = np.array([1.0 / 255.0], np.float32)
    dnnl.softmax_forward(pd2).execute(strm, {dnnl.DNNL_ARG_SRC: score, dnnl.DNNL_ARG_DST: prob,
                                             dnnl.DNNL_ARG_ATTR_SCALES | dnnl.DNNL_ARG_DST: one(p_scale[0])})
    strm.wait()
    got_p = prob.read(np.uint8, (B, S, S))
    want_p = np.zeros((B, S, S), np.uint8)
    O.softmax(O.Tensor(dt.f32, [B, S, S], got_s), O.Tensor(dt.u8, [B, S, S], want_p), 2, dst_scale=O.Quant(0, dt.f32, p_scale))
    dd = np.abs(got_p.astype(np.int32) - want_p.astype(np.int32))
    assert dd.max() <= 1 and (dd != 0).mean() < 1e-3, ("probabilities", int(dd.max()), float((dd != 0).mean()))
    # ---- out = P x V on the int8 kernels
    attr3 = dnnl.primitive_attr()
    attr3.set_scales_mask(dnnl.DNNL_ARG_SRC, 0)
    attr3.set_scales_mask(dnnl.DNNL_ARG_WEIGHTS, 0)
    v_md = memory.desc([B, S, D], dt.s8, T("abc"))
    o_md = memory.desc([B, S, D], dt.f32, T("abc"))
    pd3 = dnnl.matmul.primitive_desc(eng, p_md, v_md, o_md, attr=attr3)
    assert pd3.impl_info_str() == "hip:gfx950:mfma_b8"
    out = memory(o_md, eng)
    dnnl.matmul(pd3).execute(strm, {dnnl.DNNL_ARG_SRC: prob, dnnl.DNNL_ARG_WEIGHTS: memory(v_md, eng).write(v), dnnl.DNNL_ARG_DST: out,
                                    dnnl.DNNL_ARG_ATTR_SCALES | dnnl.DNNL_ARG_SRC: one(p_scale[0]),
                                    dnnl.DNNL_ARG_ATTR_SCALES | dnnl.DNNL_ARG_WEIGHTS: one(v_scale)})
    strm.wait()
    got_o = out.read(np.float32, (B, S, D))
    want_o = np.zeros((B, S, D), np.float32)
    O.matmul(O.Tensor(dt.u8, [B, S, S], got_p), O.Tensor(dt.s8, [B, S, D], v), O.Tensor(dt.f32, [B, S, D], want_o),
             scales={O.Q_SRC: O.Quant(0, dt.f32, p_scale), O.Q_WEI: O.Quant(0, dt.f32, np.array([v_scale], np.float32))},
             k_group_mode=O.KGROUP_WHOLE)
    assert np.array_equal(got_o, want_o), "output"
    # ---- end to end
    s64 = (q.astype(np.float64) * q_scale) @ np.transpose(k.astype(np.float64) * k_scale, (0, 2, 1)) + mask
    p64 = np.exp(s64 - s64.max(axis=-1, keepdims=True))
    p64 /= p64.sum(axis=-1, keepdims=True)
    gold = p64 @ (v.astype(np.float64) * v_scale)
    err = np.abs(got_o - gold)
    bound = 0.5 / 255.0 * np.abs(v.astype(np.float64) * v_scale).sum(axis=1, keepdims=True)  # every probability off by half a step
    print("[int8 chain] max error %.3e, a priori bound %.3e" % (err.max(), bound.max()))
    assert np.all(err <= bound + 1e-6)
    assert err.mean() < 0.05 * np.abs(gold).mean() + 1e-3
