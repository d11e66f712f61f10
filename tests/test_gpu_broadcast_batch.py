"""Weights that are one matrix for every batch entry ([1, .., 1, K, N]) under a source whose batch dims nest densely
over its rows: the library runs the problem as the 2-D product [batch x M, K] x [K, N], so it reaches the kernels that
take two dims only (weights decompression, int8 x int4, f16 x 8-bit weights) instead of the per-element kernel
(src/cpu/matmul/ref_matmul.cpp:130-175 and ref_matmul_int8.cpp take any number of dims).

Every case is built from a 2-D problem of the other test files, given batch dims, and must produce, bit for bit, what
the same library produces for the 2-D problem itself (the kernels see the same description either way) and agree with
the oracle run on the batched tensors under the 2-D problem's own bar."""
import sys

import numpy as np
import pytest

import onednn_amd as dnnl
from qmm_harness import Problem, TensorSpec, assert_bf16_within_1ulp, assert_bit_exact, dt
import test_gpu_parity as cases

pytestmark = pytest.mark.gpu

A = dnnl.algorithm


def say(msg):
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def ctx():
    eng = dnnl.engine(dnnl.engine.kind.gpu, 0)
    return eng, dnnl.stream(eng)


def batched(p, bdims, src_pad=0):
    """The 2-D problem p as [bdims.., M / prod(bdims), K] x [1, .., 1, K, N]; src_pad: extra elements between batch
    entries of the source (then the batch does not nest and the problem must stay as it is)."""
    B = int(np.prod(bdims))
    nb = len(bdims)
    M, K = p.src.dims
    N = p.wei.dims[1]
    assert M % B == 0
    m = M // B
    sdims, wdims, ddims = list(bdims) + [m, K], [1] * nb + [K, N], list(bdims) + [m, N]
    layout = None
    if src_pad:
        st = [0] * (nb + 2)
        st[-1], st[-2] = 1, K
        run = m * K + src_pad
        for d in range(nb - 1, -1, -1):
            st[d] = run
            run *= sdims[d]
        layout = st
    src = TensorSpec(p.src.dt, sdims, layout, p.src.logical().reshape(sdims))
    wl = p.wei.layout if isinstance(p.wei.layout, str) else "ab"
    letters = "abcdefgh"[:nb]
    wei = TensorSpec(p.wei.dt, wdims, letters + "".join(chr(ord(c) + nb) for c in wl), p.wei.logical().reshape(wdims))
    dst = TensorSpec(p.dst.dt, ddims, None, p.dst.logical().reshape(ddims))
    rows = (1 << (nb + 1)) - 1

    def remap(name, q):
        mask, code, groups, values = q
        if name == "wei":
            return ((mask & 3) << nb, code, groups, values)
        return ((rows if mask & 1 else 0) | ((1 << (nb + 1)) if mask & 2 else 0), code, groups, values)

    scales = {k: remap(k, v) for k, v in p.scales.items()}
    zps = {k: remap(k, v) for k, v in p.zps.items()}
    bias = None
    if p.bias is not None:
        bias = TensorSpec(p.bias.dt, [1] * nb + list(p.bias.dims), None, p.bias.logical().reshape([1] * nb + list(p.bias.dims)))
    pos = []
    for po in p.post_ops:
        po = dict(po)
        if po.get("kind") == "binary":
            s1 = po["src1"]
            d1 = (list(bdims) + [m, s1.dims[1]]) if s1.dims[0] == M else ([1] * nb + list(s1.dims))
            po["src1"] = TensorSpec(s1.dt, d1, None, s1.logical().reshape(d1))
        pos.append(po)
    return Problem(src, wei, dst, bias=bias, scales=scales, zps=zps, post_ops=pos, apply_to_int=p.apply_to_int,
                   fpmath=p.fpmath)


def _add(M, N, seed, full):
    r = np.random.default_rng(seed)
    dims = [M, N] if full else [1, N]
    return {"kind": "binary", "alg": A.binary_add, "src1": TensorSpec(dt.f32, dims, None, r.integers(-8, 9, dims).astype(np.float32))}


CASES = {
    # config 3's format, 3 x 5 rows: the decode kernel
    "decode_bf16_u4_3d": (lambda: cases.decode_w4(15, 512, 256, 401), (3,), cases.DECODE),
    # f16 x u8 weights with a scale and a zero point per column, 4-D
    "decode_f16_u8_4d": (lambda: cases.decode_w4(12, 512, 256, 402, act_dt=dt.f16, wei_dt=dt.u8, zp_dt=dt.u8, per_column=True),
                         (2, 3), cases.DECODE),
    # the same at 2 x 160 rows: the 256-row kernel for 8-bit weights
    "prefill_f16_u8_3d": (lambda: cases.decode_w4(320, 512, 512, 403, act_dt=dt.f16, wei_dt=dt.u8, zp_dt=dt.u8, per_column=True),
                          (2,), "hip:gfx950:mfma_f16w8"),
    # int8 with per-column weights scales, swish into bf16; then bias, a per-column and a full binary operand
    "int8_swish_bf16_3d": (lambda: cases.int8_linear(384, 512, 320, 404, src_dt=dt.s8, dst_dt=dt.bf16, src_zp=None,
                                                           post_ops=[
                                                               {"kind": "eltwise", "alg": A.eltwise_swish, "alpha": 1.0}]),
                                (4,), cases.MFMA),
    "int8_binary_operands_3d": (lambda: cases.int8_linear(192, 256, 200, 405, src_dt=dt.u8, dst_dt=dt.f32, post_ops=[
        _add(192, 200, 1, True), _add(192, 200, 2, False)], bias_dt=dt.f32), (2, 3), cases.MFMA),
}


@pytest.mark.parametrize("name", sorted(CASES))
def test_broadcast_weights_run_as_two_dims(ctx, name):
    eng, strm = ctx
    make, bdims, impl = CASES[name]
    say("broadcast weights over batch %s: %s" % (bdims, name))
    p2 = make()
    p = batched(p2, bdims)
    got, pd = p.run_gpu(eng, strm, weights_any=True, return_pd=True)
    assert pd.impl_info_str() == impl, pd.impl_info_str()
    flat, pd2 = p2.run_gpu(eng, strm, weights_any=True, return_pd=True)
    assert pd2.impl_info_str() == impl
    assert_bit_exact(got, flat, name + " (batched against the 2-D problem)")
    if p.dst.dt == dt.f16:
        return  # the 2-D problem's own parity with the oracle is the other files' subject
    want = p.run_oracle()
    if p.dst.dt == dt.bf16 and "decode" in name:
        assert_bf16_within_1ulp(got, want, name, abs_slack=2e-5 * cases.decode_term_scale(p2))
    elif p.dst.dt == dt.bf16:
        assert_bf16_within_1ulp(got, want, name, abs_slack=1e-30)
    else:
        assert_bit_exact(got, want, name)


def test_a_batch_that_does_not_nest_stays_batched(ctx):
    """Padding between the batch entries of the source: no single row index exists, the problem keeps its batch dims
    (and the decompression kernels, which take two dims, leave it to the per-element kernel)."""
    eng, strm = ctx
    say("source batch entries 64 elements apart: not collapsed")
    p = batched(cases.decode_w4(15, 512, 256, 406), (3,), src_pad=64)
    got, pd = p.run_gpu(eng, strm, weights_any=True, return_pd=True)
    assert pd.impl_info_str() == cases.GENERIC, pd.impl_info_str()
    assert_bf16_within_1ulp(got, p.run_oracle(), "padded batch", abs_slack=2e-5 * cases.decode_term_scale(cases.decode_w4(15, 512, 256, 406)))
