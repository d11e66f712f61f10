"""The fused attention kernel (hip:gfx950:sdpa_f16 / sdpa_bf16) behind the reference's internal sdpa entry point, against
float64 attention on the operands the kernel sees (for a quantized cache: the f16 values the chain's dequantizing
reorder produces, taken from the oracle), with the comparison rule of the reference's own SDPA test
(tests/gtests/internals/test_sdpa.cpp:1043-1106: abs 0.001466 (f16; 0.0079 for bf16) up to |gold| = 1, relative
above; at most 0.06 % of the elements outside), and against the primitive chain of that test run on the device."""
import sys

import numpy as np
import pytest

import onednn_amd as dnnl
import oracle as O
from onednn_amd import memory
from qmm_harness import T, dt

pytestmark = pytest.mark.gpu
A = dnnl.algorithm


def say(msg):
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def ctx():
    eng = dnnl.engine(dnnl.engine.kind.gpu, 0)
    return eng, dnnl.stream(eng)


def f16(x, code=dt.f16):
    return O.from_f32(code, np.ascontiguousarray(x, np.float32)).reshape(np.shape(x))


def f16_to_f64(raw, code=dt.f16):
    return O.to_f32(code, np.ascontiguousarray(raw)).reshape(raw.shape).astype(np.float64)


def reference_rule(test, gold, thr=0.001466):
    t, g = test.astype(np.float64).reshape(-1), gold.astype(np.float64).reshape(-1)
    diff = np.abs(t - g)
    bad = np.where(np.abs(g) > 1.0, diff > np.abs(g) * thr, diff > thr) | np.isnan(t) | np.isnan(g)
    return int(bad.sum()), t.size, float(diff.max())


def attention64(q, kt, v, scale, mask, causal, kv_rep):
    """q [.., Q, D], kt [.., D, S], v [.., S, D] as float64; kv_rep: how many query heads share a kv head."""
    if kv_rep > 1:
        kt = np.repeat(kt, kv_rep, axis=-3)
        v = np.repeat(v, kv_rep, axis=-3)
    s = q @ kt * scale
    if mask is not None:
        s = s + mask
    if causal:
        Qn, S = s.shape[-2:]
        s = s + np.triu(np.full((Qn, S), -np.inf), 1)
    p = np.exp(s - s.max(axis=-1, keepdims=True))
    p /= p.sum(axis=-1, keepdims=True)
    return p @ v


def run_sdpa(ctx, q, k_store, v, *, scale=None, invert=False, mask=None, mask_dt=dt.f32, causal=False, kv_heads=0,
             kv_dt=None, k_q=None, v_q=None, qdt=dt.f16):
    """q [.., Q, D] raw 16-bit values of type qdt; k_store [.., S, D] (the cache as stored: keys major), passed as its transposed view;
    v [.., S, D]. k_q / v_q: (mask, groups, scale_dt, scales, zp_dt, zps) for a quantized cache."""
    eng, strm = ctx
    nd = q.ndim
    letters = "abcd"[:nd]
    kv_dt = qdt if kv_dt is None else kv_dt
    q_md = memory.desc(list(q.shape), qdt, T(letters))
    kdims = list(k_store.shape[:-2]) + [k_store.shape[-1], k_store.shape[-2]]
    kt_md = memory.desc(kdims, kv_dt, T(letters[:-2] + letters[-1] + letters[-2]))  # D contiguous: the transposed view
    v_md = memory.desc(list(v.shape), kv_dt, T(letters))
    o_md = memory.desc(list(q.shape), qdt, T(letters))
    args = {dnnl.DNNL_ARG_QUERIES: memory(q_md, eng).write(q), dnnl.DNNL_ARG_KEYS: memory(kt_md, eng).write(k_store),
            dnnl.DNNL_ARG_VALUES: memory(v_md, eng).write(v)}
    m_md = None
    if mask is not None:
        m_md = memory.desc(list(mask.shape), mask_dt, T(letters))
        args[dnnl.DNNL_ARG_ATTN_MASK] = memory(m_md, eng).write(mask if mask_dt == dt.f32 else f16(mask, mask_dt))
    scale_dt = dt.undef
    if scale is not None:
        scale_dt = qdt
        args[dnnl.DNNL_ARG_SCALE] = memory(memory.desc([1], qdt, T("a")), eng).write(f16(np.array([scale]), qdt))
    attrs = []
    for which, qq in ((dnnl.DNNL_ARG_KEYS, k_q), (dnnl.DNNL_ARG_VALUES, v_q)):
        a = None
        if qq is not None:
            qmask, groups, sdt, sc, zdt, zp = qq
            a = dnnl.primitive_attr()
            a.set_scales(dnnl.DNNL_ARG_WEIGHTS, qmask, list(groups), sdt)
            args[dnnl.DNNL_ARG_ATTR_SCALES | which] = memory(memory.desc([sc.nbytes], dt.u8, T("a")), eng).write(sc)
            if zp is not None:
                a.set_zero_points(dnnl.DNNL_ARG_WEIGHTS, qmask, list(groups), zdt)
                args[dnnl.DNNL_ARG_ATTR_ZERO_POINTS | which] = memory(memory.desc([zp.nbytes], dt.u8, T("a")), eng).write(zp)
        attrs.append(a)
    pd = dnnl.sdpa.primitive_desc(eng, q_md, kt_md, v_md, m_md, scale_dt, o_md, invert, kv_heads, causal,
                                  None, attrs[0], attrs[1])
    assert pd.impl_info_str() == ("hip:gfx950:sdpa_bf16" if qdt == dt.bf16 else "hip:gfx950:sdpa_f16")
    out = memory(o_md, eng)
    args[dnnl.DNNL_ARG_DST] = out
    dnnl.sdpa(pd).execute(strm, args)
    strm.wait()
    return out.read(np.uint16, q.shape)


CASES = [
    # (batch dims, kv heads or 0, Qn, S, D, mask kind, scale mode)
    ((2, 3), 0, 48, 160, 64, "none", "mul"),
    ((1, 4), 0, 200, 385, 128, "2d", "div"),
    ((2, 2), 0, 1, 513, 128, "1d", "mul"),
    ((1, 8), 2, 130, 300, 128, "causal", "mul"),
    ((4,), 0, 128, 128, 64, "causal", "none"),
    ((), 0, 77, 1000, 128, "2d", "mul"),
    ((1, 2), 0, 16, 33, 64, "none", "mul"),
    # head sizes 32 and 256 (K / V in the queries' type): many queries, the few-queries form split over the keys, masks
    ((1, 4), 0, 150, 200, 32, "2d", "mul"),
    ((1, 2), 0, 384, 384, 96, "2d", "mul"),
    ((1, 2), 0, 1, 385, 96, "2d", "mul"),
    ((2, 3), 0, 33, 259, 96, "causal", "div"),
    ((1, 4), 2, 9, 129, 96, "none", "mul"),
    ((2, 2), 0, 8, 300, 32, "causal", "mul"),
    ((3,), 0, 1, 1000, 32, "1d", "div"),
    ((1, 2), 0, 130, 170, 256, "causal", "div"),
    ((1, 3), 0, 1, 513, 256, "1d", "mul"),
    ((1, 4), 2, 16, 700, 256, "none", "mul"),
    ((2,), 0, 70, 96, 256, "2d", "none"),
]


@pytest.mark.parametrize("qdt", [dt.f16, dt.bf16], ids=["f16", "bf16"])
@pytest.mark.parametrize("case", CASES, ids=str)
def test_f16_attention(ctx, case, qdt):
    bdims, kvh, Qn, S, D, mkind, smode = case
    say("sdpa %s %r" % (qdt, case))
    r = np.random.default_rng(Qn + S + D)
    kb = tuple(bdims[:-1]) + ((kvh,) if kvh else tuple(bdims[-1:])) if bdims else ()
    q = f16(r.standard_normal(bdims + (Qn, D)), qdt)
    k = f16(r.standard_normal(kb + (S, D)), qdt)
    v = f16(r.standard_normal(kb + (S, D)), qdt)
    scale = None if smode == "none" else (1.0 / np.sqrt(D) if smode == "mul" else np.sqrt(D))
    mask = None
    nb = len(bdims)
    if mkind == "2d":
        mask = (r.standard_normal((1,) * nb + (Qn, S)) * 2).astype(np.float32)
        mask[..., ::5] = -np.inf
        mask[..., 0] = 0  # no row fully masked
    elif mkind == "1d":
        mask = (r.standard_normal((1,) * nb + (1, S)) * 2).astype(np.float32)
    got = run_sdpa(ctx, q, k, v, scale=scale, invert=(smode == "div"), mask=mask,
                   mask_dt=qdt if mkind == "1d" else dt.f32, causal=(mkind == "causal"), kv_heads=kvh, qdt=qdt)
    s_eff = 1.0 if scale is None else float(f16_to_f64(f16(np.array([scale]), qdt), qdt)[0])
    if smode == "div":
        s_eff = 1.0 / s_eff
    m_eff = None if mask is None else (mask.astype(np.float64) if mkind != "1d" else f16_to_f64(f16(mask, qdt), qdt))
    gold = attention64(f16_to_f64(q, qdt), np.swapaxes(f16_to_f64(k, qdt), -1, -2), f16_to_f64(v, qdt), s_eff, m_eff,
                       mkind == "causal", (bdims[-1] // kvh) if kvh else 1)
    bad, total, worst = reference_rule(f16_to_f64(got, qdt), gold, 0.001466 if qdt == dt.f16 else 0.0079)
    print("[sdpa] %d of %d outside the reference test's threshold, max diff %.2e" % (bad, total, worst))
    assert bad <= total * 0.0006


@pytest.mark.parametrize("kv_dt,with_zp", [(dt.s8, True), (dt.u8, True), (dt.s8, False)], ids=str)
@pytest.mark.parametrize("Qn", [1, 96])
@pytest.mark.parametrize("D,qdt", [(128, dt.f16), (32, dt.f16), (96, dt.f16), (256, dt.f16), (128, dt.bf16), (64, dt.bf16),
                                   (256, dt.bf16)], ids=str)
def test_quantized_cache(ctx, kv_dt, with_zp, Qn, D, qdt):
    """K / V as an 8-bit cache with one f16 scale (and zero point) per head and key: the kernel dequantizes while
    staging, to the same values of the queries' type (f16 or bf16) as the chain's reorder (checked through the
    oracle's reorder)."""
    MB, H, S = 2, 4, 257
    say("sdpa quantized cache %s zp=%s queries %d head size %d %s" % (kv_dt, with_zp, Qn, D, qdt))
    r = np.random.default_rng(40 + Qn)
    q = f16(r.standard_normal((MB, H, Qn, D)), qdt)
    lo, hi, npdt = (-128, 128, np.int8) if kv_dt == dt.s8 else (0, 256, np.uint8)
    kq = r.integers(lo, hi, (MB, H, S, D)).astype(npdt)
    vq = r.integers(lo, hi, (MB, H, S, D)).astype(npdt)
    ksc, vsc = f16(r.uniform(0.005, 0.02, (H, S))), f16(r.uniform(0.005, 0.02, (H, S)))
    zdt = kv_dt
    kzp = r.integers(lo // 16 + (100 if kv_dt == dt.u8 else 0), hi // 16 + (100 if kv_dt == dt.u8 else 0), (H, S)).astype(npdt)
    vzp = r.integers(lo // 16 + (100 if kv_dt == dt.u8 else 0), hi // 16 + (100 if kv_dt == dt.u8 else 0), (H, S)).astype(npdt)
    kqa = (0b1110, (D, 1), dt.f16, ksc, zdt, kzp if with_zp else None)
    vqa = (0b1110, (1, D), dt.f16, vsc, zdt, vzp if with_zp else None)
    got = run_sdpa(ctx, q, kq, vq, scale=1.0 / np.sqrt(D), causal=(Qn > 1), kv_dt=kv_dt, k_q=kqa, v_q=vqa, qdt=qdt)
    # the dequantized cache as the reference chain's reorder produces it (oracle reorder, to the queries' type)
    kd, vd = np.zeros((MB, H, S, D), np.uint16), np.zeros((MB, H, S, D), np.uint16)
    for raw, sc, zp, outd in ((kq, ksc, kzp, kd), (vq, vsc, vzp, vd)):
        O.reorder(O.Tensor(kv_dt, [MB, H, S, D], raw), O.Tensor(qdt, [MB, H, S, D], outd),
                  src_scale=O.Quant(0b1110, dt.f16, sc, (1, D)),
                  src_zp=O.Quant(0b1110, zdt, zp, (1, D)) if with_zp else None)
    s_eff = float(f16_to_f64(f16(np.array([1.0 / np.sqrt(D)]), qdt), qdt)[0])
    gold = attention64(f16_to_f64(q, qdt), np.swapaxes(f16_to_f64(kd, qdt), -1, -2), f16_to_f64(vd, qdt), s_eff, None,
                       Qn > 1, 1)
    bad, total, worst = reference_rule(f16_to_f64(got, qdt), gold, 0.0079 if qdt == dt.bf16 else 0.001466)
    print("[sdpa quantized] %d of %d outside the threshold, max diff %.2e" % (bad, total, worst))
    assert bad <= total * 0.0006


@pytest.mark.parametrize("Qn,S,D,heads,kvh,mkind,quant", [
    (1, 4096, 128, 8, 0, "none", False), (1, 2049, 128, 32, 8, "none", True), (5, 1500, 64, 4, 0, "2d", False),
    (16, 3000, 128, 6, 2, "causal", False), (2, 640, 64, 40, 0, "1d", True), (1, 96, 128, 2, 0, "none", False),
    (1, 5000, 128, 8, 2, "none", "bf16"), (7, 1111, 64, 3, 0, "2d", "bf16"),
], ids=str)
def test_few_queries_split_over_the_keys(ctx, Qn, S, D, heads, kvh, mkind, quant):
    """At most 16 queries per head (the decode step): the keys are cut into ranges, one workgroup each, the ranges'
    running maxima, sums and accumulators merged afterwards (in the scratchpad when there are several ranges)."""
    say("sdpa decode Qn=%d S=%d D=%d heads=%d kv=%d mask=%s quant=%s" % (Qn, S, D, heads, kvh, mkind, quant))
    r = np.random.default_rng(Qn * 7 + S)
    kh = kvh or heads
    qdt = dt.bf16 if quant == "bf16" else dt.f16
    quant = quant is True
    q = f16(r.standard_normal((1, heads, Qn, D)), qdt)
    scale = 1.0 / np.sqrt(D)
    mask = None
    if mkind == "2d":
        mask = (r.standard_normal((1, 1, Qn, S)) * 2).astype(np.float32)
        mask[..., 3::7] = -np.inf
    elif mkind == "1d":
        mask = (r.standard_normal((1, 1, 1, S)) * 2).astype(np.float32)
    if quant:
        kq = r.integers(-128, 128, (1, kh, S, D)).astype(np.int8)
        vq = r.integers(-128, 128, (1, kh, S, D)).astype(np.int8)
        ksc, vsc = f16(r.uniform(0.005, 0.02, (kh, S))), f16(r.uniform(0.005, 0.02, (kh, S)))
        kzp, vzp = r.integers(-6, 7, (kh, S)).astype(np.int8), r.integers(-6, 7, (kh, S)).astype(np.int8)
        got = run_sdpa(ctx, q, kq, vq, scale=scale, mask=mask, causal=(mkind == "causal"), kv_heads=kvh, kv_dt=dt.s8,
                       k_q=(0b1110, (D, 1), dt.f16, ksc, dt.s8, kzp), v_q=(0b1110, (1, D), dt.f16, vsc, dt.s8, vzp))
        kd, vd = np.zeros((1, kh, S, D), np.uint16), np.zeros((1, kh, S, D), np.uint16)
        for raw, sc, zp, outd in ((kq, ksc, kzp, kd), (vq, vsc, vzp, vd)):
            O.reorder(O.Tensor(dt.s8, [1, kh, S, D], raw), O.Tensor(dt.f16, [1, kh, S, D], outd),
                      src_scale=O.Quant(0b1110, dt.f16, sc, (1, D)), src_zp=O.Quant(0b1110, dt.s8, zp, (1, D)))
        k64, v64 = f16_to_f64(kd), f16_to_f64(vd)
    else:
        k, v = f16(r.standard_normal((1, kh, S, D)), qdt), f16(r.standard_normal((1, kh, S, D)), qdt)
        got = run_sdpa(ctx, q, k, v, scale=scale, mask=mask, causal=(mkind == "causal"), kv_heads=kvh, qdt=qdt)
        k64, v64 = f16_to_f64(k, qdt), f16_to_f64(v, qdt)
    s_eff = float(f16_to_f64(f16(np.array([scale]), qdt), qdt)[0])
    gold = attention64(f16_to_f64(q, qdt), np.swapaxes(k64, -1, -2), v64, s_eff,
                       None if mask is None else mask.astype(np.float64), mkind == "causal", heads // kh)
    bad, total, worst = reference_rule(f16_to_f64(got, qdt), gold, 0.001466 if qdt == dt.f16 else 0.0079)
    print("[sdpa decode] %d of %d outside the threshold, max diff %.2e" % (bad, total, worst))
    assert bad <= total * 0.0006


def test_few_queries_with_a_user_scratchpad(ctx):
    """The ranges' partial results live in the primitive's scratchpad: library-owned by default, the user's in
    scratchpad_mode::user (filled with NaN patterns here, to show that nothing of it is read before it is written)."""
    eng, strm = ctx
    H, S, D = 16, 4096, 128
    r = np.random.default_rng(5)
    q, k, v = f16(r.standard_normal((1, H, 1, D))), f16(r.standard_normal((1, H, S, D))), f16(r.standard_normal((1, H, S, D)))
    attr = dnnl.primitive_attr()
    attr.set_scratchpad_mode(dnnl.scratchpad_mode.user)
    q_md = memory.desc([1, H, 1, D], dt.f16, T("abcd"))
    kt_md = memory.desc([1, H, D, S], dt.f16, T("abdc"))
    v_md = memory.desc([1, H, S, D], dt.f16, T("abcd"))
    pd = dnnl.sdpa.primitive_desc(eng, q_md, kt_md, v_md, None, dt.undef, q_md, False, 0, False, attr)
    smd = pd.scratchpad_desc()
    assert smd.get_size() > 0
    scratch = memory(smd, eng).write(np.full(smd.get_size(), 0xFF, np.uint8))
    out = memory(q_md, eng)
    dnnl.sdpa(pd).execute(strm, {dnnl.DNNL_ARG_QUERIES: memory(q_md, eng).write(q), dnnl.DNNL_ARG_KEYS: memory(kt_md, eng).write(k),
                                 dnnl.DNNL_ARG_VALUES: memory(v_md, eng).write(v), dnnl.DNNL_ARG_DST: out,
                                 dnnl.DNNL_ARG_SCRATCHPAD: scratch})
    strm.wait()
    gold = attention64(f16_to_f64(q), np.swapaxes(f16_to_f64(k), -1, -2), f16_to_f64(v), 1.0, None, False, 1)
    bad, total, worst = reference_rule(f16_to_f64(out.read(np.uint16, (1, H, 1, D))), gold)
    assert bad <= total * 0.0006, (bad, worst)


def test_fused_kernel_against_the_primitive_chain_on_the_device(ctx):
    """Same operands through matmul -> softmax -> matmul (generic kernels, f32 scores in memory) and through the
    fused kernel: the two device results agree under the reference test's rule."""
    eng, strm = ctx
    B, H, Qn, S, D = 1, 4, 64, 192, 64
    r = np.random.default_rng(77)
    q, k, v = (f16(r.standard_normal((B, H, n, D))) for n in (Qn, S, S))
    scale = 1.0 / np.sqrt(D)
    fused = run_sdpa(ctx, q, k, v, scale=scale, causal=True)
    # chain
    mask = np.triu(np.full((Qn, S), -np.inf, np.float32), 1).reshape(1, 1, Qn, S)
    q_md = memory.desc([B, H, Qn, D], dt.f16, T("abcd"))
    kt_md = memory.desc([B, H, D, S], dt.f16, T("abdc"))
    s_md = memory.desc([B, H, Qn, S], dt.f32, T("abcd"))
    p_md = memory.desc([B, H, Qn, S], dt.f16, T("abcd"))
    v_md = memory.desc([B, H, S, D], dt.f16, T("abcd"))
    o_md = memory.desc([B, H, Qn, D], dt.f16, T("abcd"))
    attr = dnnl.primitive_attr()
    po = dnnl.post_ops()
    po.append_binary(A.binary_mul, memory.desc([1, 1, 1, 1], dt.f32, T("abcd")))
    po.append_binary(A.binary_add, memory.desc([1, 1, Qn, S], dt.f32, T("abcd")))
    attr.set_post_ops(po)
    score, prob, out = memory(s_md, eng), memory(p_md, eng), memory(o_md, eng)
    s16 = O.to_f32(dt.f16, f16(np.array([scale]))).astype(np.float32)
    dnnl.matmul(dnnl.matmul.primitive_desc(eng, q_md, kt_md, s_md, attr=attr)).execute(strm, {
        dnnl.DNNL_ARG_SRC: memory(q_md, eng).write(q), dnnl.DNNL_ARG_WEIGHTS: memory(kt_md, eng).write(k),
        dnnl.DNNL_ARG_DST: score,
        dnnl.DNNL_ARG_ATTR_MULTIPLE_POST_OP(0) | dnnl.DNNL_ARG_SRC_1: memory(memory.desc([1, 1, 1, 1], dt.f32, T("abcd")), eng).write(s16),
        dnnl.DNNL_ARG_ATTR_MULTIPLE_POST_OP(1) | dnnl.DNNL_ARG_SRC_1: memory(memory.desc([1, 1, Qn, S], dt.f32, T("abcd")), eng).write(mask)})
    dnnl.softmax_forward(dnnl.softmax_forward.primitive_desc(eng, dnnl.prop_kind.forward_inference, A.softmax_accurate,
                                                             s_md, p_md, 3)).execute(strm, score, prob)
    dnnl.matmul(dnnl.matmul.primitive_desc(eng, p_md, v_md, o_md)).execute(strm, {
        dnnl.DNNL_ARG_SRC: prob, dnnl.DNNL_ARG_WEIGHTS: memory(v_md, eng).write(v), dnnl.DNNL_ARG_DST: out})
    strm.wait()
    chain = out.read(np.uint16, (B, H, Qn, D))
    bad, total, worst = reference_rule(f16_to_f64(fused), f16_to_f64(chain))
    print("[sdpa vs chain] %d of %d outside the threshold, max diff %.2e" % (bad, total, worst))
    assert bad <= total * 0.0006


def test_what_the_kernel_does_not_take_is_unimplemented(ctx):
    eng, _ = ctx
    md = lambda dims, code=dt.f16, t="abcd": memory.desc(dims, code, T(t))
    ok = dict(q=md([1, 2, 16, 64]), k=md([1, 2, 64, 32], t="abdc"), v=md([1, 2, 32, 64]), o=md([1, 2, 16, 64]))

    def make(**kw):
        a = dict(ok)
        a.update(kw)
        return dnnl.sdpa.primitive_desc(eng, a["q"], a["k"], a["v"], None, dt.undef, a["o"])

    make()
    for bad in (dict(q=md([1, 2, 16, 80]), k=md([1, 2, 80, 32], t="abdc"), v=md([1, 2, 32, 80]), o=md([1, 2, 16, 80])),  # head size
                dict(k=md([1, 2, 64, 32])),                                    # keys contiguous instead of head size
                dict(q=md([1, 2, 16, 64], dt.bf16), o=md([1, 2, 16, 64], dt.bf16)),  # bf16 queries on f16 keys
                dict(k=md([1, 2, 64, 32], dt.s32, t="abdc"), v=md([1, 2, 32, 64], dt.s32))):  # a 32-bit cache
        with pytest.raises(dnnl.error) as e:
            make(**bad)
        assert e.value.status == dnnl.status.unimplemented
    with pytest.raises(dnnl.error) as e:
        make(v=md([1, 2, 40, 64]))  # keys of K and V differ
    assert e.value.status == dnnl.status.invalid_arguments
