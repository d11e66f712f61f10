"""GPU parity of hip:gfx950:mfma_b8 with u8 weights and weights zero points (one for the tensor or per column) against
the CPU oracle: the layout of the W8A8 entries of tests/benchdnn/inputs/matmul/option_set_fwks_llm_gpu
(--dt=s8:u8:f16, source scales per row, weights scales and u8 zero points per column). Arithmetic:
src/cpu/matmul/ref_matmul_int8.cpp:165-219 -- the s32 sum of (s - z_s)(w - z_w) over K, exact, so integer results
and results on exact-arithmetic scales are compared bit for bit."""
import sys

import numpy as np
import pytest

import onednn_amd as dnnl
import oracle as O
from onednn_amd import memory
from qmm_harness import Problem, T, TensorSpec, assert_bf16_within_1ulp, assert_bit_exact, assert_f32_close, dt, tag

pytestmark = pytest.mark.gpu
MFMA, GENERIC = "hip:gfx950:mfma_b8", "hip:gfx950:generic"


def say(msg):
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def ctx():
    eng = dnnl.engine(dnnl.engine.kind.gpu, 0)
    return eng, dnnl.stream(eng)


def w8a8(M, K, N, seed, src_dt=dt.s8, wei_dt=dt.u8, dst_dt=dt.f32, wei_zp="n", wei_zp_dt=dt.u8, src_zp=None,
         exact=True, wei_layout="ba", batch=(), post_ops=None, bias_dt=None):
    r = np.random.default_rng(seed)
    b = list(batch)
    nd = len(b) + 2
    s = r.integers(0, 256, b + [M, K]) if src_dt == dt.u8 else r.integers(-128, 128, b + [M, K])
    w = r.integers(0, 256, b + [K, N]) if wei_dt == dt.u8 else r.integers(-128, 128, b + [K, N])
    letters = list("abcd"[:nd])
    if wei_layout == "ba":
        letters[-2], letters[-1] = letters[-1], letters[-2]
    src = TensorSpec(src_dt, b + [M, K], None, s)
    wei = TensorSpec(wei_dt, b + [K, N], "".join(letters), w)
    dst = TensorSpec(dst_dt, b + [M, N])
    last, prev = 1 << (nd - 1), 1 << (nd - 2)
    scales = {}
    if dst_dt != dt.s32:
        ss = 2.0 ** r.integers(-9, -6, M) if exact else r.uniform(0.002, 0.01, M)
        sw = 2.0 ** r.integers(-8, -5, N) if exact else r.uniform(0.002, 0.01, N)
        if not b:
            scales["src"] = (last | prev, dt.f16 if exact else dt.f32, (1, K), ss)
        scales["wei"] = (last, dt.f16 if exact else dt.f32, None, sw)
    zps = {}
    lo, hi = (100, 156) if wei_zp_dt == dt.u8 else (-30, 31)
    if wei_zp == "n":
        zps["wei"] = (last, wei_zp_dt, None, r.integers(lo, hi, N))
    elif wei_zp == "common":
        zps["wei"] = (0, wei_zp_dt, None, r.integers(lo, hi, 1))
    if src_zp is not None:
        zps["src"] = (0, dt.s32, None, [src_zp])
    bias = None
    if bias_dt is not None:
        bias = TensorSpec(bias_dt, [1] * (nd - 1) + [N], None, r.integers(-20, 20, N))
    p = Problem(src, wei, dst, bias=bias, scales=scales, zps=zps, post_ops=post_ops)
    p.term_scale = 74.0 * 74.0 * np.sqrt(K) * 0.006 * 0.006
    return p


CASES = {
    "s8_u8_zp_per_column": dict(M=70, K=256, N=100),
    "s8_u8_zp_common_s32_dst": dict(M=33, K=512, N=72, wei_zp="common", dst_dt=dt.s32),
    "s8_u8_no_zp": dict(M=130, K=192, N=96, wei_zp=None),
    "s8_s8_zp_s8_per_column": dict(M=40, K=384, N=160, wei_dt=dt.s8, wei_zp_dt=dt.s8),
    "s8_s8_zp_s32_common": dict(M=17, K=128, N=48, wei_dt=dt.s8, wei_zp="common", wei_zp_dt=dt.s32),
    "u8_u8_both_zero_points": dict(M=200, K=320, N=130, src_dt=dt.u8, src_zp=121),
    "u8_src_s8_wei_zp": dict(M=64, K=256, N=64, src_dt=dt.u8, wei_dt=dt.s8, wei_zp_dt=dt.s8, src_zp=7),
    "m1_decode": dict(M=1, K=4096, N=200),
    "m300_k3072": dict(M=300, K=3072, N=520),
    # at most 4 rows: the single-token kernel
    "m3_u8_src_zp_s8_weights_no_wzp": dict(M=3, K=1024, N=100, src_dt=dt.u8, wei_dt=dt.s8, wei_zp=None, src_zp=77),
    "m4_k208_half_fragment": dict(M=4, K=208, N=72, src_dt=dt.u8, src_zp=130, dst_dt=dt.s32),
    "m2_u8_u8_common_zp_s32_dst": dict(M=2, K=14336, N=64, src_dt=dt.u8, wei_zp="common", dst_dt=dt.s32, src_zp=3),
    # 5 ... 64 rows of one matrix: the streaming kernel keeps all rows of one or two 32-row MFMA blocks
    "m32_k4096_zp_per_column": dict(M=32, K=4096, N=200),
    "m17_u8_src_both_zero_points_s32_dst": dict(M=17, K=1040, N=72, src_dt=dt.u8, src_zp=99, dst_dt=dt.s32),
    "m9_s8_s8_plain_k_tail_s32_dst": dict(M=9, K=208, N=130, wei_dt=dt.s8, wei_zp=None, dst_dt=dt.s32),
    "m31_s8_s8_zp_s8_bias": dict(M=31, K=512, N=96, wei_dt=dt.s8, wei_zp_dt=dt.s8, bias_dt=dt.f32),
    "m33_k2048_zp_per_column": dict(M=33, K=2048, N=130),
    "m64_u8_src_zp_s8_weights_zp": dict(M=64, K=1040, N=96, src_dt=dt.u8, wei_dt=dt.s8, wei_zp_dt=dt.s8, src_zp=131,
                                        dst_dt=dt.s32),
    "m48_s8_s8_plain_bias": dict(M=48, K=512, N=200, wei_dt=dt.s8, wei_zp=None, bias_dt=dt.f32),
    "m1_s8_s8_plain": dict(M=1, K=512, N=1000, wei_dt=dt.s8, wei_zp=None),
    "ab_weights_bias_s8_dst": dict(M=50, K=256, N=80, wei_layout="ab", bias_dt=dt.f32, dst_dt=dt.s8),
    "batched_broadcast_zp": dict(M=20, K=128, N=64, batch=(3,), dst_dt=dt.s32),
}


@pytest.mark.parametrize("name", sorted(CASES))
@pytest.mark.parametrize("weights_any", [True, False])
def test_weights_zero_points_exact(ctx, name, weights_any):
    eng, strm = ctx
    say("mfma_b8 weights zero points %s any=%s" % (name, weights_any))
    p = w8a8(seed=500 + len(name), **CASES[name])
    got, pd = p.run_gpu(eng, strm, weights_any=weights_any, return_pd=True)
    assert pd.impl_info_str() == MFMA
    assert_bit_exact(got, p.run_oracle(), name)


TILE256_CASES = {
    "s8_u8_zp_per_column_ragged": dict(M=300, K=320, N=200),
    "s8_u8_zp_per_column_k3072": dict(M=300, K=3072, N=520),
    "s8_u8_no_zp_s32_dst": dict(M=257, K=512, N=130, wei_zp=None, dst_dt=dt.s32),
    "s8_s8_zp_s32_common_bias": dict(M=130, K=384, N=260, wei_dt=dt.s8, wei_zp="common", wei_zp_dt=dt.s32,
                                     bias_dt=dt.f32),
    "s8_u8_src_zp_f16_dst": dict(M=512, K=1024, N=256, src_zp=-5, dst_dt=dt.f16),
    "s8_u8_batched_s32_dst": dict(M=140, K=320, N=136, batch=(2,), dst_dt=dt.s32),
    # u8 sources: only the 256 x 128 kernel reads them as they are
    "u8_u8_both_zero_points": dict(M=200, K=320, N=130, src_dt=dt.u8, src_zp=121),
    "u8_s8_zp_s8_per_column_s32_dst": dict(M=384, K=576, N=128, src_dt=dt.u8, wei_dt=dt.s8, wei_zp_dt=dt.s8,
                                           src_zp=7, dst_dt=dt.s32),
}


@pytest.mark.parametrize("name", sorted(TILE256_CASES))
@pytest.mark.parametrize("tiling", ["two_per_cu", "one_per_cu"])
def test_weights_zero_points_on_the_256_row_kernels(ctx, name, tiling):
    """Forced onto the 256 x 128 and 256 x 256 tilings, whose epilogue takes z_w'[n] x rowsum[m] off the s32 sums in
    its row path; a u8 source reaches the 256 x 256 kernels only as an s8 copy, which these problems do not make, so
    there the general kernel answers (still bit-exact)."""
    from onednn_amd import _capi
    eng, strm = ctx
    say("mfma_b8 weights zero points, 256-row kernels: %s %s" % (name, tiling))
    p = w8a8(seed=900 + len(name), **TILE256_CASES[name])
    with _capi.kernel_variants(gemm=6, b8x=2 if tiling == "two_per_cu" else 3):
        got, pd = p.run_gpu(eng, strm, weights_any=True, return_pd=True)
    assert pd.impl_info_str() == MFMA
    assert_bit_exact(got, p.run_oracle(), name)


def test_matches_the_per_element_kernel(ctx):
    eng, strm = ctx
    say("mfma_b8 weights zero points vs generic")
    p = w8a8(37, 256, 72, 7, src_dt=dt.u8, src_zp=100)
    assert_bit_exact(p.run_gpu(eng, strm, impl=MFMA), p.run_gpu(eng, strm, impl=GENERIC), "vs generic")


@pytest.mark.parametrize("dst_dt", [dt.f32, dt.f16])
def test_llm_list_shape_arbitrary_scales(ctx, dst_dt):
    """32 x 4096 x 14336-like entry (here 4096 x 1536), f16 / f32 dst, scales that are not powers of two."""
    eng, strm = ctx
    say("mfma_b8 s8:u8 llm entry dst=%d" % dst_dt)
    p = w8a8(32, 4096, 1536, 9, dst_dt=dst_dt, exact=False)
    got, pd = p.run_gpu(eng, strm, weights_any=True, return_pd=True)
    assert pd.impl_info_str() == MFMA
    want = p.run_oracle()
    g, w = O.to_f32(dst_dt, got), O.to_f32(dst_dt, want)
    if dst_dt == dt.f32:
        assert_f32_close(g, w, rel=1e-5, scale=p.term_scale, what="f32")
    else:
        assert_f32_close(g, w, rel=2.0 ** -10, scale=p.term_scale, what="f16")


def test_prepacked_u8_weights_round_trip(ctx):
    eng, strm = ctx
    say("u8 weights prepack round trip")
    r = np.random.default_rng(3)
    dims = [208, 72]
    t = TensorSpec(dt.u8, dims, "ab", r.integers(0, 256, dims))
    pd = dnnl.matmul.primitive_desc(eng, memory.desc([4, dims[0]], dt.s8, T("ab")), memory.desc(dims, dt.u8, tag.any),
                                    memory.desc([4, dims[1]], dt.s32, T("ab")))
    assert pd.impl_info_str() == MFMA
    plain = memory(t.md(), eng).write(t.raw)
    packed = memory(pd.weights_desc(), eng)
    back = memory(t.md(), eng).write(np.zeros_like(t.raw))
    dnnl.reorder(plain, packed).execute(strm, plain, packed)
    dnnl.reorder(packed, back).execute(strm, packed, back)
    strm.wait()
    assert_bit_exact(back.read(t.raw.dtype), t.raw, "round trip")
