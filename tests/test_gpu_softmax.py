"""GPU parity of the softmax primitive (hip:gfx950:softmax_rows / softmax_generic) against the oracle
(src/cpu/ref_softmax.cpp), through the C ABI.

Bars: the device's expf and the order of the row sum differ from the host's, so f32 results are compared at
rel 4e-6 of the value plus the oracle's own worst-case summation error (channels x 2^-24: it adds the exponentials
one after the other), and f32 -> f32 rows also at rel 4e-6 against the exact float64 result; f16 / bf16 results within one unit of
the last place and mostly equal; u8 / s8 within one step and mostly equal. Masked positions (-1e4) are exactly 0."""
import sys

import numpy as np
import pytest

import onednn_amd as dnnl
import oracle as O
from onednn_amd import memory
from qmm_harness import T, dt

pytestmark = pytest.mark.gpu
A = dnnl.algorithm
ROWS, GENERIC = "hip:gfx950:softmax_rows", "hip:gfx950:softmax_generic"
NP = {dt.f32: np.float32, dt.bf16: np.uint16, dt.f16: np.uint16, dt.s8: np.int8, dt.u8: np.uint8}


def say(msg):
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def ctx():
    eng = dnnl.engine(dnnl.engine.kind.gpu, 0)
    return eng, dnnl.stream(eng)


def encode(code, x):
    if code == dt.f32:
        return np.ascontiguousarray(x, np.float32)
    if code in (dt.bf16, dt.f16):
        return O.from_f32(code, np.ascontiguousarray(x, np.float32)).reshape(x.shape)
    return np.clip(np.rint(x), -128 if code == dt.s8 else 0, 127 if code == dt.s8 else 255).astype(NP[code])


def run_both(ctx, x, src_dt, dst_dt, axis, alg=A.softmax_accurate, layout=None, src_scale=None, dst_scale=None):
    """x: logical values. layout: tag letters for src and dst (default row-major). Returns (got, want, impl) as raw
    storage arrays in logical order."""
    eng, strm = ctx
    dims = list(x.shape)
    tagname = layout or "abcdef"[:len(dims)]
    smd = memory.desc(dims, src_dt, T(tagname))
    dmd = memory.desc(dims, dst_dt, T(tagname))
    strides = smd.get_strides()
    # physical buffer: logical -> storage by the strides
    perm = np.argsort([-s for s in strides], kind="stable")
    phys = np.ascontiguousarray(np.transpose(encode(src_dt, x), perm))
    attr = dnnl.primitive_attr()
    args_extra = {}
    oq = {}
    for name, arg, val in (("src_scale", dnnl.DNNL_ARG_SRC, src_scale), ("dst_scale", dnnl.DNNL_ARG_DST, dst_scale)):
        if val is not None:
            attr.set_scales_mask(arg, 0)
            buf = np.array([val], np.float32)
            args_extra[dnnl.DNNL_ARG_ATTR_SCALES | arg] = memory(memory.desc([1], dt.f32, T("a")), eng).write(buf)
            oq[name] = O.Quant(0, O.F32, buf)
    pd = dnnl.softmax_forward.primitive_desc(eng, dnnl.prop_kind.forward_inference, alg, smd, dmd, axis, attr)
    prim = dnnl.softmax_forward(pd)
    src = memory(pd.src_desc(), eng).write(phys)
    dst = memory(pd.dst_desc(), eng)
    args = {dnnl.DNNL_ARG_SRC: src, dnnl.DNNL_ARG_DST: dst}
    args.update(args_extra)
    prim.execute(strm, args)
    strm.wait()
    got_phys = dst.read(NP[dst_dt], phys.shape)
    want_phys = np.zeros(phys.shape, NP[dst_dt])
    O.softmax(O.Tensor(src_dt, dims, phys, strides), O.Tensor(dst_dt, dims, want_phys, strides), axis,
              log=(alg == A.softmax_log), **oq)
    inv = np.argsort(perm)
    return np.transpose(got_phys, inv), np.transpose(want_phys, inv), pd.impl_info_str()


def compare(code, got, want, what, channels=0):
    if code == dt.f32:
        g, w = got.astype(np.float64), want.astype(np.float64)
        err = np.abs(g - w)
        # the oracle adds the row's exponentials one after the other in f32 (worst case channels x 2^-24 of the sum,
        # the same factor on every element of the row); the kernel adds per-lane partial sums pairwise
        tol = (4e-6 + channels * 2.0 ** -24) * np.abs(w) + 1e-37
        assert np.all(err <= tol), "%s: worst %.3g of the value" % (what, float(np.max(err / (np.abs(w) + 1e-37))))
        return
    if code in (dt.bf16, dt.f16):
        d = np.abs(got.astype(np.int32) - want.astype(np.int32))  # same sign: positive results or equal codes
    else:
        d = np.abs(got.astype(np.int32) - want.astype(np.int32))
    frac = float((d != 0).mean())
    print("[softmax] %s: %.4f %% of the elements one step off, max distance %d" % (what, 100 * frac, int(d.max())))
    assert d.max() <= 1 and frac < 0.02, (what, int(d.max()), frac)


@pytest.mark.parametrize("src_dt,dst_dt", [(dt.f32, dt.f32), (dt.f32, dt.f16), (dt.f32, dt.bf16), (dt.bf16, dt.bf16),
                                           (dt.f16, dt.f32), (dt.f16, dt.f16)], ids=str)
@pytest.mark.parametrize("dims,axis", [((6, 2048), 1), ((2, 3, 40, 256), 3), ((5, 4100), 1), ((3, 20000), 1),
                                       ((1, 77), 1)], ids=str)
def test_rows_kernel(ctx, src_dt, dst_dt, dims, axis):
    say("softmax rows %s -> %s dims %s" % (src_dt, dst_dt, dims))
    r = np.random.default_rng(sum(dims))
    x = (r.standard_normal(dims) * 4).astype(np.float32)
    x[..., ::7] = -1e4 if src_dt == dt.f32 else -3e4 if src_dt == dt.bf16 else -6e4  # masked positions
    got, want, impl = run_both(ctx, x, src_dt, dst_dt, axis)
    assert impl == ROWS
    compare(dst_dt, got, want, "rows", channels=dims[axis])
    if src_dt == dt.f32 and dst_dt == dt.f32:
        # against the exact result: the kernel's own error, without the oracle's summation error
        exact = __import__("scipy.special").special.softmax(x.astype(np.float64), axis=axis)
        assert np.max(np.abs(got - exact) / (exact + 1e-300)) < 4e-6
    masked = got[..., ::7]
    assert np.all(masked == 0)
    if dst_dt == dt.f32:
        assert np.allclose(got.sum(axis=axis), 1.0, atol=1e-5)


@pytest.mark.parametrize("alg", [A.softmax_accurate, A.softmax_log], ids=["softmax", "log"])
@pytest.mark.parametrize("dims,axis,layout", [((4, 6, 50), 1, None), ((4, 6, 50), 0, None), ((8, 64), 1, "ba"),
                                              ((3, 5, 7, 9), 2, "acdb"), ((6, 30), 1, None)], ids=str)
def test_generic_kernel_and_log_softmax(ctx, alg, dims, axis, layout):
    say("softmax alg %x dims %s axis %d layout %s" % (alg, dims, axis, layout))
    r = np.random.default_rng(sum(dims) + axis)
    x = (r.standard_normal(dims) * 3).astype(np.float32)
    got, want, impl = run_both(ctx, x, dt.f32, dt.f32, axis, alg=alg, layout=layout)
    if alg == A.softmax_log:
        g, w = got.astype(np.float64), want.astype(np.float64)
        assert np.all(np.abs(g - w) <= 4e-6 * np.max(np.abs(w)))
    else:
        compare(dt.f32, got, want, "generic", channels=dims[axis])


@pytest.mark.parametrize("dst_dt", [dt.u8, dt.s8], ids=str)
def test_quantized_probabilities(ctx, dst_dt):
    """f32 scores -> u8 / s8 probabilities with a destination scale: what feeds an int8 P x V matmul."""
    say("softmax f32 -> %s with dst scale" % dst_dt)
    r = np.random.default_rng(9)
    x = (r.standard_normal((64, 512)) * 2).astype(np.float32)
    peak = 255.0 if dst_dt == dt.u8 else 127.0
    got, want, impl = run_both(ctx, x, dt.f32, dst_dt, 1, dst_scale=0.05 / peak)  # probabilities above 0.05 saturate
    assert impl == ROWS
    assert want.max() == peak and len(np.unique(want)) > 30
    compare(dst_dt, got, want, "quantized")
    # s8 source with a source scale: the dequantised values are the scores
    xs = np.clip(np.rint(x * 20), -128, 127).astype(np.float32)
    got, want, impl = run_both(ctx, xs, dt.s8, dt.f32, 1, src_scale=1.0)
    compare(dt.f32, got, want, "s8 source", channels=512)


def test_minus_infinity_mask(ctx):
    """Masked scores given as -inf (what the reference's SDPA test fills its causal mask with): exactly 0, the rest
    of the row unaffected."""
    r = np.random.default_rng(12)
    x = (r.standard_normal((9, 300)) * 2).astype(np.float32)
    x[:, 1::3] = -np.inf
    got, want, impl = run_both(ctx, x, dt.f32, dt.f32, 1)
    assert impl == ROWS and not np.isnan(got).any()
    assert np.all(got[:, 1::3] == 0)
    compare(dt.f32, got, want, "-inf mask", channels=300)


def test_creation_rules(ctx):
    """src/common/softmax.cpp:42-140: axis range, algorithm, equal dims; scales only with an int8 side; post-ops
    are not implemented here."""
    eng, _ = ctx
    md = memory.desc([4, 8], dt.f32, T("ab"))
    fwd = dnnl.prop_kind.forward_inference

    def make(**kw):
        a = dict(eng=eng, p=fwd, alg=A.softmax_accurate, s=md, d=md, axis=1, attr=None)
        a.update(kw)
        return dnnl.softmax_forward.primitive_desc(a["eng"], a["p"], a["alg"], a["s"], a["d"], a["axis"], a["attr"])

    make()
    for bad in (dict(axis=2), dict(axis=-1), dict(alg=A.eltwise_relu), dict(d=memory.desc([4, 9], dt.f32, T("ab")))):
        with pytest.raises(dnnl.error) as e:
            make(**bad)
        assert e.value.status == dnnl.status.invalid_arguments
    attr = dnnl.primitive_attr()
    attr.set_scales_mask(dnnl.DNNL_ARG_DST, 0)
    with pytest.raises(dnnl.error) as e:
        make(attr=attr)  # no int8 side
    assert e.value.status == dnnl.status.unimplemented
    make(attr=attr, d=memory.desc([4, 8], dt.u8, T("ab")))
    po = dnnl.post_ops()
    po.append_eltwise(A.eltwise_relu, 0.0, 0.0)
    attr2 = dnnl.primitive_attr()
    attr2.set_post_ops(po)
    with pytest.raises(dnnl.error) as e:
        make(attr=attr2)
    assert e.value.status == dnnl.status.unimplemented
    # format any on dst takes the source's layout
    pd = make(s=memory.desc([4, 8], dt.f32, T("ba")), d=memory.desc([4, 8], dt.f16, memory.format_tag.any))
    assert pd.dst_desc().get_strides() == [1, 4]
    assert pd.impl_info_str() == GENERIC


def test_attention_scores_shape_full_size(ctx):
    """The scores tensor of the batched attention configuration (32 x 2048 x 2048 f32, causal mask already added):
    every row sums to 1, masked positions are exactly 0, a sample of rows matches the oracle."""
    eng, strm = ctx
    B, S = 32, 2048
    say("softmax 32 x 2048 x 2048 f32 -> f32")
    r = np.random.default_rng(11)
    x = (r.standard_normal((B, S, S)) * 3).astype(np.float32)
    x += np.triu(np.full((S, S), -1e4, np.float32), 1)[None]
    md = memory.desc([B, S, S], dt.f32, T("abc"))
    pd = dnnl.softmax_forward.primitive_desc(eng, dnnl.prop_kind.forward_inference, A.softmax_accurate, md, md, 2)
    assert pd.impl_info_str() == ROWS
    src, dst = memory(md, eng).write(x), memory(md, eng)
    dnnl.softmax_forward(pd).execute(strm, src, dst)
    strm.wait()
    got = dst.read(np.float32, (B, S, S))
    assert np.allclose(got.sum(axis=2), 1.0, atol=2e-5)
    assert np.all(got[:, np.triu_indices(S, 1)[0], np.triu_indices(S, 1)[1]] == 0)
    rows = np.ascontiguousarray(x[::5, 100::211])
    want = np.zeros_like(rows)
    O.softmax(O.Tensor(O.F32, list(rows.shape), rows), O.Tensor(O.F32, list(rows.shape), want), 2)
    compare(dt.f32, got[::5, 100::211], want, "full-size sample", channels=S)
