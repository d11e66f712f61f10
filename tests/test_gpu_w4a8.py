"""GPU parity of hip:gfx950:mfma_w4a8 (s8 activations x 4-bit weights, scales
grouped along K on both operands) against the CPU oracle, through the C ABI.

Bars: with integer data and power-of-two scales every order of operations gives
the same bits, so those cases are compared bit for bit; with arbitrary scales
the f32 result is within 1e-5 of the magnitude of the summed terms, bf16 / f16
results within one representable value of the rounded oracle value.
"""
import sys

import numpy as np
import pytest

import onednn_amd as dnnl
import oracle as O
from onednn_amd import _capi, memory
from qmm_harness import (Problem, T, TensorSpec, assert_bf16_within_1ulp, assert_bit_exact,
                         assert_f32_close, dt, tag)

pytestmark = pytest.mark.gpu

A = dnnl.algorithm
W4A8, GENERIC = "hip:gfx950:mfma_w4a8", "hip:gfx950:generic"


def say(msg):
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def ctx():
    eng = dnnl.engine(dnnl.engine.kind.gpu, 0)
    return eng, dnnl.stream(eng)


@pytest.fixture(params=[0, 1, 2, 3, 4, 5])
def variant(request):
    with _capi.kernel_variants(w4a8=request.param):
        yield request.param


def dynamic_quant(M, K, N, seed, wei_dt=dt.s4, gs=128, gw=128, gz=None, zp_dt=dt.u8, exact=False,
                  dst_dt=dt.f32, scale_dt=dt.f16, post_ops=None, wei_layout="ab", dst_init=None,
                  src_dt=dt.s8, src_zp=None, src_zp_dt=dt.u8):
    """s8 src with per-row K-grouped scales (1 x gs), int4 weights with K-grouped
    scales (gw x 1) and optional zero points (gz x 1): the layout of
    tests/benchdnn/inputs/matmul/option_set_fwks_llm_gpu:32-117."""
    r = np.random.default_rng(seed)
    s = np.clip(np.rint(r.standard_normal((M, K)) * 40), -128, 127)
    if src_dt == dt.u8:
        s = s + 128
    lo, hi = (0, 16) if wei_dt == dt.u4 else (-8, 8)
    w = r.integers(lo, hi, (K, N))
    src = TensorSpec(src_dt, [M, K], None, s)
    wei = TensorSpec(wei_dt, [K, N], wei_layout, w)
    dst = TensorSpec(dst_dt, [M, N], None, dst_init)
    if exact:
        ss = 2.0 ** r.integers(-5, -2, (M, K // gs))
        sw = 2.0 ** r.integers(-5, -2, (K // gw, N))
    else:
        ss = r.uniform(0.005, 0.05, (M, K // gs))
        sw = r.uniform(0.002, 0.02, (K // gw, N))
    scales = {"src": (3, scale_dt, (1, gs), ss), "wei": (3, scale_dt, (gw, 1), sw)}
    zps = {}
    if gz is not None:
        if zp_dt in (dt.s4, dt.s8):
            z = r.integers(-3, 4, (K // gz, N))
        else:
            z = r.integers(5, 12, (K // gz, N))
        zps["wei"] = (3, zp_dt, (gz, 1), z)
    # source zero points: "common" (one value), "k" (per K group of src_zp[1]), "mk" (per row and K group)
    if src_zp is not None:
        kind, g = src_zp
        zlo, zhi = (100, 156) if src_zp_dt == dt.u8 else (-20, 21)
        if kind == "common":
            zps["src"] = (0, src_zp_dt, None, r.integers(zlo, zhi, (1,)))
        elif kind == "k":
            zps["src"] = (2, src_zp_dt, (1, g), r.integers(zlo, zhi, (K // g,)))
        else:
            zps["src"] = (3, src_zp_dt, (1, g), r.integers(zlo, zhi, (M, K // g)))
    p = Problem(src, wei, dst, scales=scales, zps=zps, post_ops=post_ops)
    # magnitude of one group's term, for the relative bar
    p.term_scale = float(np.abs(s).mean() * 4 * np.sqrt(min(gs, gw)) * ss.mean() * sw.mean())
    return p


EXACT_CASES = {
    "s4_g128": dict(M=70, K=256, N=100),
    "s4_g64": dict(M=33, K=256, N=64, gs=64, gw=64),
    "s4_src256_wei128": dict(M=6, K=256, N=100, gs=256, gw=128),
    "u4_no_zp": dict(M=40, K=384, N=96, wei_dt=dt.u4),
    "u4_zp_u8_g128": dict(M=130, K=256, N=130, wei_dt=dt.u4, gz=128),
    "s4_zp_s4_g64_scales_g128": dict(M=17, K=256, N=48, gz=64, zp_dt=dt.s4),
    "u4_zp_u4_g192": dict(M=12, K=576, N=192, wei_dt=dt.u4, gs=192, gw=192, gz=192, zp_dt=dt.u4),
    "s4_ba_weights": dict(M=64, K=128, N=64, wei_layout="ba"),
    "m1": dict(M=1, K=512, N=160),
    "m48_u4_zp": dict(M=48, K=512, N=200, wei_dt=dt.u4, gz=128),
    "m64_many_groups": dict(M=64, K=2560, N=96, gs=64, gw=64, gz=64, zp_dt=dt.s8),
    "m5_k4096": dict(M=5, K=4096, N=130, wei_dt=dt.u4),
    "m1_k4096_zp": dict(M=1, K=4096, N=200, wei_dt=dt.u4, gz=128),
    "m3_k2048_g64": dict(M=3, K=2048, N=70, gs=64, gw=64, gz=64, zp_dt=dt.s4),
    "m4_k8192": dict(M=4, K=8192, N=96),
    "edges": dict(M=129, K=320, N=162, gs=64, gw=64),
    # source zero points / u8 sources: the tiled kernel's third mode at every M
    "u8_src_no_zp": dict(M=70, K=256, N=100, src_dt=dt.u8),
    "u8_src_common_zp": dict(M=130, K=384, N=96, src_dt=dt.u8, src_zp=("common", 0), wei_dt=dt.u4),
    "u8_src_zp_per_row_group": dict(M=200, K=512, N=130, src_dt=dt.u8, src_zp=("mk", 128), wei_dt=dt.u4, gz=128),
    "s8_src_zp_s8_per_row_group64": dict(M=33, K=256, N=64, gs=64, gw=64, gz=64, zp_dt=dt.s4, src_zp=("mk", 64),
                                         src_zp_dt=dt.s8),
    "s8_src_zp_per_group_wider_than_scales": dict(M=17, K=512, N=48, gs=128, gw=128, src_zp=("k", 256),
                                                  src_zp_dt=dt.s8, gz=128, zp_dt=dt.u8, wei_dt=dt.u4),
    "u8_src_zp_m1": dict(M=1, K=512, N=160, src_dt=dt.u8, src_zp=("mk", 128)),
    # source scales per 32 k (--attr-scales=src0:per_ocic:f16:1x32+wei:per_ocic:f16:128x1 in the reference's list):
    # groups of half a tile, the tiled kernel at every M
    "src_g32_wei_g128_u4_zp": dict(M=70, K=256, N=100, gs=32, gw=128, wei_dt=dt.u4, gz=128),
    "src_g32_wei_g64_s4": dict(M=33, K=512, N=64, gs=32, gw=64),
    "src_g32_wei_g32_zp_s4_g32": dict(M=130, K=128, N=130, gs=32, gw=32, gz=32, zp_dt=dt.s4),
    "src_g32_m1_k4096": dict(M=1, K=4096, N=96, gs=32, gw=128, wei_dt=dt.u4, gz=128),
    "src_g32_m300_k1536": dict(M=300, K=1536, N=264, gs=32, gw=128, wei_dt=dt.u4, gz=128),
    "src_g32_m4_zp_s4_g32": dict(M=4, K=1024, N=70, gs=32, gw=32, gz=32, zp_dt=dt.s4),
    "src_g32_m2_k8192": dict(M=2, K=8192, N=64, gs=32, gw=128),
    "src_g32_m1_k14336_tiled": dict(M=1, K=14336, N=64, gs=32, gw=128, wei_dt=dt.u4, gz=128),
    "u8_src_no_zp_m3": dict(M=3, K=1024, N=100, src_dt=dt.u8, wei_dt=dt.u4),
    "s8_src_zp_s8_m2_k4096": dict(M=2, K=4096, N=96, src_zp=("k", 256), src_zp_dt=dt.s8, gz=128, zp_dt=dt.u8,
                                  wei_dt=dt.u4),
    "u8_src_zp_common_m1": dict(M=1, K=2048, N=160, src_dt=dt.u8, src_zp=("common", 0), gz=64, gs=64, gw=64,
                                zp_dt=dt.s4),
    # 5 ... 64 rows with groups of 32 k / source zero points: the split-K kernel's second and third mode
    "src_g32_m64_k4096_zp": dict(M=64, K=4096, N=200, gs=32, gw=128, wei_dt=dt.u4, gz=128),
    "src_g32_m5_k2048_g32_everything": dict(M=5, K=2048, N=130, gs=32, gw=32, gz=32, zp_dt=dt.s4),
    "src_g32_m24_k14336": dict(M=24, K=14336, N=64, gs=32, gw=128),
    "u8_src_zp_m40_k2048": dict(M=40, K=2048, N=264, src_dt=dt.u8, src_zp=("mk", 128), wei_dt=dt.u4, gz=128,
                                zp_dt=dt.u4),
    "s8_src_zp_m64_k4096_common": dict(M=64, K=4096, N=96, src_zp=("common", 0), src_zp_dt=dt.s8, gs=4096, gw=64,
                                       gz=64, zp_dt=dt.s8),
    "u8_src_no_zp_m9_k512": dict(M=9, K=512, N=100, src_dt=dt.u8),
    # 5 ... 32 rows, whole tiles per group (the decode batches of the LLM list: 31, 32 rows)
    "m32_k4096_u4_zp_g128": dict(M=32, K=4096, N=200, wei_dt=dt.u4, gz=128),
    "m31_k4096_s4_g64_everything": dict(M=31, K=4096, N=130, gs=64, gw=64, gz=64, zp_dt=dt.s8),
    "m9_k1024_src_per_row_only": dict(M=9, K=1024, N=96, gs=1024, gw=128),
    "m17_k512_u4_zp_u4_g256": dict(M=17, K=512, N=70, wei_dt=dt.u4, gs=256, gw=256, gz=256, zp_dt=dt.u4),
    "u8_src_zp_m300_k2048": dict(M=300, K=2048, N=264, src_dt=dt.u8, src_zp=("mk", 128), wei_dt=dt.u4, gz=128,
                                 zp_dt=dt.u4),
}


@pytest.mark.parametrize("name", sorted(EXACT_CASES))
@pytest.mark.parametrize("weights_any", [True, False])
def test_w4a8_exact(ctx, variant, name, weights_any):
    eng, strm = ctx
    say("mfma_w4a8 exact %s any=%s variant=%d" % (name, weights_any, variant))
    p = dynamic_quant(seed=300 + len(name), exact=True, **EXACT_CASES[name])
    got, pd = p.run_gpu(eng, strm, weights_any=weights_any, return_pd=True)
    assert pd.impl_info_str() == W4A8
    assert_bit_exact(got, p.run_oracle(), name)


def test_w4a8_matches_generic_kernel(ctx):
    """Same launch through the literal per-element kernel."""
    eng, strm = ctx
    say("mfma_w4a8 vs generic")
    p = dynamic_quant(37, 256, 72, 7, wei_dt=dt.u4, gz=128, exact=True)
    a = p.run_gpu(eng, strm, impl=W4A8)
    b = p.run_gpu(eng, strm, impl=GENERIC)
    assert_bit_exact(a, b, "w4a8 vs generic")


@pytest.mark.parametrize("dst_dt", [dt.f32, dt.bf16, dt.f16])
def test_w4a8_arbitrary_scales(ctx, variant, dst_dt):
    eng, strm = ctx
    say("mfma_w4a8 arbitrary scales dst=%d variant=%d" % (dst_dt, variant))
    p = dynamic_quant(200, 1024, 264, 11, wei_dt=dt.u4, gz=128, dst_dt=dst_dt)
    got, pd = p.run_gpu(eng, strm, weights_any=True, return_pd=True)
    assert pd.impl_info_str() == W4A8
    want = p.run_oracle()
    g, w = O.to_f32(dst_dt, got), O.to_f32(dst_dt, want)
    if dst_dt == dt.f32:
        assert_f32_close(g, w, rel=1e-5, scale=p.term_scale, what="f32")
    elif dst_dt == dt.bf16:
        assert_bf16_within_1ulp(got, want, "bf16", abs_slack=1e-5 * p.term_scale)
    else:  # f16: one ulp is 2^-10 relative
        assert_f32_close(g, w, rel=2.0 ** -10, scale=p.term_scale, what="f16")


@pytest.mark.parametrize("M", [1, 3, 24, 40])
def test_w4a8_decode_rows_arbitrary_scales(ctx, M):
    """Rows <= 64 take the split-K kernel: slices are summed in slice order,
    which is not the oracle's group order, hence the f32 bar."""
    eng, strm = ctx
    say("mfma_w4a8 decode rows M=%d" % M)
    p = dynamic_quant(M, 4096, 520, 15 + M, wei_dt=dt.u4, gz=128)
    got, pd = p.run_gpu(eng, strm, weights_any=True, return_pd=True)
    assert pd.impl_info_str() == W4A8
    assert_f32_close(got, p.run_oracle(), rel=1e-5, scale=p.term_scale, what="decode rows")


def test_w4a8_single_token_long_k(ctx):
    """K = 14336: eight waves per workgroup, two chunks of tiles per wave."""
    eng, strm = ctx
    say("mfma_w4a8 M=2 K=14336")
    p = dynamic_quant(2, 14336, 96, 31, wei_dt=dt.u4, gz=128, zp_dt=dt.u4, dst_dt=dt.f32)
    got, pd = p.run_gpu(eng, strm, weights_any=True, return_pd=True)
    assert pd.impl_info_str() == W4A8
    assert_f32_close(got, p.run_oracle(), rel=1e-5, scale=p.term_scale, what="long K")


def test_w4a8_llm_post_ops(ctx):
    """swish then multiplication by an f16 tensor, f16 dst
    (tests/benchdnn/inputs/matmul/option_set_fwks_llm_gpu:36)."""
    eng, strm = ctx
    say("mfma_w4a8 swish + binary_mul f16")
    r = np.random.default_rng(5)
    M, K, N = 96, 512, 320
    gate = TensorSpec(dt.f16, [M, N], None, r.uniform(-2, 2, (M, N)).astype(np.float32))
    p = dynamic_quant(M, K, N, 12, dst_dt=dt.f16,
                      post_ops=[{"kind": "eltwise", "alg": A.eltwise_swish, "alpha": 1.0},
                                {"kind": "binary", "alg": A.binary_mul, "src1": gate}])
    got, pd = p.run_gpu(eng, strm, weights_any=True, return_pd=True)
    assert pd.impl_info_str() == W4A8
    want = p.run_oracle()
    g, w = O.to_f32(dt.f16, got), O.to_f32(dt.f16, want)
    assert_f32_close(g, w, rel=2.0 ** -9, scale=p.term_scale, what="swish*gate f16")


def test_w4a8_binary_add_f32(ctx):
    """residual add, f32 dst (option_set_fwks_llm_gpu:37)."""
    eng, strm = ctx
    say("mfma_w4a8 binary_add f32")
    r = np.random.default_rng(6)
    M, K, N = 40, 768, 256
    res = TensorSpec(dt.f32, [M, N], None, r.standard_normal((M, N)).astype(np.float32))
    p = dynamic_quant(M, K, N, 13, wei_dt=dt.u4, gz=128,
                      post_ops=[{"kind": "binary", "alg": A.binary_add, "src1": res}])
    got, pd = p.run_gpu(eng, strm, weights_any=True, return_pd=True)
    assert pd.impl_info_str() == W4A8
    assert_f32_close(got, p.run_oracle(), rel=1e-5, scale=max(p.term_scale, 1.0), what="add")


def test_w4a8_many_groups_full_width(ctx):
    """K = 4096 in 32 groups, enough tiles for the 128 x 128 configuration."""
    eng, strm = ctx
    say("mfma_w4a8 1100 x 4096 x 2048")
    p = dynamic_quant(1100, 4096, 2048, 14, exact=True)
    got, pd = p.run_gpu(eng, strm, weights_any=True, return_pd=True)
    assert pd.impl_info_str() == W4A8
    assert_bit_exact(got, p.run_oracle(nthreads=0), "full width")


def test_w4a8_prepack_round_trip(ctx):
    eng, strm = ctx
    say("W4K64 prepack round trip")
    r = np.random.default_rng(91)
    for code, dims, layout in ((dt.u4, [256, 48], "ab"), (dt.s4, [192, 34], "ba")):
        vals = r.integers(0, 16, dims) if code == dt.u4 else r.integers(-8, 8, dims)
        t = TensorSpec(code, dims, layout, vals)
        attr = dnnl.primitive_attr()
        attr.set_scales(dnnl.DNNL_ARG_WEIGHTS, 3, [64, 1], dt.f16)
        pd = dnnl.matmul.primitive_desc(eng, memory.desc([4, dims[0]], dt.s8, T("ab")),
                                        memory.desc(dims, code, tag.any),
                                        memory.desc([4, dims[1]], dt.f32, T("ab")), attr=attr)
        assert pd.impl_info_str() == W4A8
        wmd = pd.weights_desc()
        assert wmd.get_format_kind() == memory.format_kind.opaque
        plain = memory(t.md(), eng).write(t.raw)
        packed = memory(wmd, eng)
        back = memory(t.md(), eng).write(np.zeros_like(t.raw))
        dnnl.reorder(plain, packed).execute(strm, plain, packed)
        dnnl.reorder(packed, back).execute(strm, packed, back)
        strm.wait()
        assert np.array_equal(t.logical(back.read(t.raw.dtype)), t.logical()), (code, dims, layout)


def _extreme_zero_point(K, gk, zp_value=255):
    """Saturated activations against the largest u8 zero point: the group sum
    16 * sum s * (w - z) reaches 16 * 127 * 255 * gk."""
    M, N = 8, 64
    r = np.random.default_rng(77)
    s = np.full((M, K), 127)
    s[1::2] = -128
    w = r.integers(0, 16, (K, N))
    src = TensorSpec(dt.s8, [M, K], None, s)
    wei = TensorSpec(dt.u4, [K, N], "ab", w)
    dst = TensorSpec(dt.f32, [M, N])
    scales = {"src": (3, dt.f32, (1, gk), np.full((M, K // gk), 2.0 ** -20)),
              "wei": (3, dt.f32, (gk, 1), np.full((K // gk, N), 2.0 ** -8))}
    zps = {"wei": (3, dt.u8, (gk, 1), np.full((K // gk, N), zp_value))}
    return Problem(src, wei, dst, scales=scales, zps=zps)


def test_w4a8_largest_8bit_zero_point_stays_in_s32(ctx):
    """u8 zero point 255 with saturated activations: the largest group the
    MFMA implementation takes with 8-bit zero points (3968) is exact; a group of
    4096 would leave s32 in its 16 x scaled sums and goes to the generic
    implementation, which is exact as well."""
    eng, strm = ctx
    say("mfma_w4a8 u8 zp=255, gk=3968 (MFMA) and gk=4096 (generic)")
    p = _extreme_zero_point(3968, 3968)
    got, pd = p.run_gpu(eng, strm, weights_any=True, return_pd=True)
    assert pd.impl_info_str() == W4A8
    assert_bit_exact(got, p.run_oracle(), "gk 3968")
    # closed form: one group, (float)s32 rounds to nearest even, the scales are powers of two
    acc = p.src.logical().astype(np.int64) @ (p.wei.logical().astype(np.int64) - 255)
    assert 2 ** 30 < np.abs(acc).max() * 16 < 2 ** 31  # the 16 x scaled sum is within 5 % of the s32 range
    assert np.array_equal(got.view(np.float32).reshape(8, 64), acc.astype(np.float32) * np.float32(2.0 ** -28))
    p = _extreme_zero_point(4096, 4096)
    got, pd = p.run_gpu(eng, strm, return_pd=True)
    assert pd.impl_info_str() == GENERIC
    assert_bit_exact(got, p.run_oracle(), "gk 4096")


def test_w4a8_s32_zero_points_go_to_generic(ctx):
    eng, strm = ctx
    say("mfma_w4a8 refuses s32 zero points")
    p = dynamic_quant(16, 256, 64, 5, wei_dt=dt.u4, gz=128, zp_dt=dt.s32, exact=True)
    got, pd = p.run_gpu(eng, strm, return_pd=True)
    assert pd.impl_info_str() == GENERIC
    assert_bit_exact(got, p.run_oracle(), "s32 zp")
