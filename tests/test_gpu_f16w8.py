"""GPU parity of hip:gfx950:mfma_f16w8 (f16 activations x u8 / s8 weights with scales and zero points that do not
vary along K, 256 rows and more) against the CPU oracle, through the dnnl_* C API.

The shapes are those of the 8-bit weights-only prefill entries of the reference's LLM list
(tests/benchdnn/inputs/matmul/option_set_fwks_llm_gpu: --dt=f16:u8:f16|f32 --wtag=ba --attr-scales=wei:per_oc:f16
--attr-zero-points=wei:per_oc:u8 --attr-fpmath=f16:true, with swish / binary_add post-ops) at a reduced K and N.

Bars: the kernel converts the weights exactly and sums f16 x f16 products in f32 (MFMA order) where the reference sums
a x ((w - z) x scale) in f32 in k order: an f32 dst within 2e-5 of the summed magnitudes, an f16 dst within one f16
step (2^-10 relative) plus that."""
import sys

import numpy as np
import pytest

import onednn_amd as dnnl
import oracle as O
from qmm_harness import Problem, TensorSpec, dt

pytestmark = pytest.mark.gpu

A = dnnl.algorithm
F16W8, DECODE = "hip:gfx950:mfma_f16w8", "hip:gfx950:decode_w4"


def say(msg):
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def ctx():
    eng = dnnl.engine(dnnl.engine.kind.gpu, 0)
    return eng, dnnl.stream(eng)


def problem(M, K, N, seed, wei_dt=dt.u8, zp="per_column", zp_dt=dt.u8, scale="per_column", scale_dt=dt.f16,
            dst_dt=dt.f16, wei_layout="ba", post=None, lda=None, src_scale=None):
    r = np.random.default_rng(seed)
    a = r.standard_normal((M, K)).astype(np.float32)
    lo, hi = (0, 256) if wei_dt == dt.u8 else (-128, 128)
    w = r.integers(lo, hi, (K, N))
    src = TensorSpec(dt.f16, [M, K], [lda, 1] if lda else None, a)
    wei = TensorSpec(wei_dt, [K, N], wei_layout, w)
    dst = TensorSpec(dst_dt, [M, N])
    scales, zps = {}, {}
    if scale == "per_column":
        scales["wei"] = (2, scale_dt, None, r.uniform(0.0005, 0.002, N))
    elif scale == "common":
        scales["wei"] = (0, scale_dt, None, [0.00125])
    if src_scale is not None:
        scales["src"] = (0, dt.f32, None, [src_scale])
    zlo, zhi = {dt.u8: (0, 256), dt.s8: (-128, 128)}[zp_dt]
    if zp == "per_column":
        zps["wei"] = (2, zp_dt, None, r.integers(zlo, zhi, N))
    elif zp == "common":
        zps["wei"] = (0, zp_dt, None, [int(r.integers(zlo, zhi))])
    post_ops = []
    if post == "swish":
        post_ops = [{"kind": "eltwise", "alg": A.eltwise_swish, "alpha": 1.0}]
    elif post == "add":
        post_ops = [{"kind": "binary", "alg": A.binary_add,
                     "src1": TensorSpec(dt.f32, [M, N], None, r.standard_normal((M, N)).astype(np.float32))}]
    elif post == "gelu":
        post_ops = [{"kind": "eltwise", "alg": A.eltwise_gelu_erf, "alpha": 0.0}]
    return Problem(src, wei, dst, scales=scales, zps=zps, post_ops=post_ops, apply_to_int=True,
                   fpmath=dnnl.fpmath_mode.f16)


def term_scale(p):
    """sum_k |a| |w - z| scale per output (times the source scale)."""
    a = np.abs(p.src.logical().astype(np.float64))
    w = p.wei.logical().astype(np.float64)
    K, N = w.shape
    if "wei" in p.zps:
        w = w - np.asarray(p.zps["wei"][3], np.float64).reshape(1, -1)
    t = a @ np.abs(w)
    if "wei" in p.scales:
        code, vals = p.scales["wei"][1], p.scales["wei"][3]
        t = t * O.to_f32(code, Problem._quant_raw(code, vals)).astype(np.float64).reshape(1, -1)
    if "src" in p.scales:
        t = t * float(p.scales["src"][3][0])
    return t


def check(p, got, want, what):
    M, N = p.dst.dims
    code = p.dst.dt
    g, w = O.to_f32(code, got).reshape(M, N).astype(np.float64), O.to_f32(code, want).reshape(M, N).astype(np.float64)
    bar = 2e-5 * term_scale(p)
    if code == dt.f16:
        bar = bar + 2.0 ** -10 * np.abs(w)
    err = np.abs(g - w)
    worst = np.unravel_index(np.argmax(err - bar), err.shape)
    print("[%s] max error %.3e (bar there %.3e) at %r" % (what, err[worst], bar[worst], worst))
    assert np.all(np.isfinite(g)), what
    assert np.all(err <= bar), "%s: %d of %d beyond the bar, worst at %r: got %r want %r" % (
        what, int((err > bar).sum()), err.size, worst, g[worst], w[worst])


CASES = {
    # row and column tails, 12 k-steps
    "u8_per_column_tails": dict(M=1030, K=384, N=2040),
    # the fewest k-steps: 5 (odd, no paired iteration), 6 (even), 7, 8
    "u8_k160_f32_add": dict(M=512, K=160, N=256, dst_dt=dt.f32, post="add"),
    "u8_k192": dict(M=256, K=192, N=300),
    "s8_k224_swish": dict(M=300, K=224, N=520, wei_dt=dt.s8, zp_dt=dt.s8, post="swish"),
    "u8_k256_f32": dict(M=260, K=256, N=264, dst_dt=dt.f32),
    # an odd count with paired iterations (11), and a long sum
    "u8_k352_swish": dict(M=384, K=352, N=512, post="swish"),
    "u8_k4096_f32": dict(M=256, K=4096, N=256, dst_dt=dt.f32),
    # zero points / scales of the other shapes and types
    "s8_weights_u8_zero_points": dict(M=256, K=320, N=320, wei_dt=dt.s8, zp_dt=dt.u8),
    "u8_weights_s8_zero_points_f32_scales": dict(M=257, K=320, N=96, zp_dt=dt.s8, scale_dt=dt.f32),
    "u8_common_zero_point_bf16_scales": dict(M=300, K=256, N=130, zp="common", scale_dt=dt.bf16),
    "s8_no_zero_point_common_scale": dict(M=256, K=256, N=256, wei_dt=dt.s8, zp=None, scale="common"),
    "u8_no_scale_source_scale": dict(M=256, K=192, N=64, scale=None, src_scale=0.25, dst_dt=dt.f32),
    # weights rows N-contiguous, source rows with a pitch, dst rows that start at odd elements
    "u8_ab_weights_pitched_source": dict(M=300, K=256, N=1001, wei_layout="ab", lda=264),
    "u8_gelu_f16": dict(M=270, K=256, N=272, post="gelu"),
    # few tiles, long K: the K range runs as slices whose f32 sums a second kernel adds (8 slices for u8_k4096_f32
    # above; here 3 of 16 k-steps, 2 of 17, 4 with a binary operand, 2 with odd dst rows)
    "u8_k1536_three_slices_swish": dict(M=300, K=1536, N=520, post="swish"),
    "s8_k1088_two_odd_slices": dict(M=256, K=1088, N=260, wei_dt=dt.s8, zp_dt=dt.s8, dst_dt=dt.f32),
    "u8_k2048_four_slices_add": dict(M=512, K=2048, N=384, dst_dt=dt.f32, post="add"),
    "u8_k1024_slices_gelu_odd_columns": dict(M=260, K=1024, N=1001, post="gelu", src_scale=0.5),
}


@pytest.mark.parametrize("name", sorted(CASES))
@pytest.mark.parametrize("weights_any", [True, False])
def test_f16_activations_8bit_weights(ctx, name, weights_any):
    eng, strm = ctx
    say("mfma_f16w8 %s any=%s" % (name, weights_any))
    p = problem(seed=len(name) * 7 + 1, **CASES[name])
    got, pd = p.run_gpu(eng, strm, weights_any=weights_any, return_pd=True)
    assert pd.impl_info_str() == F16W8
    check(p, got, p.run_oracle(), name)


def test_extreme_weights_and_zero_points_convert_exactly(ctx):
    """Weights and zero points at the ends of their ranges (differences of +-255) against a one-hot source: every
    output is a single product a x (w - z) x scale, so any error in the byte -> f16 conversion shows undiluted."""
    eng, strm = ctx
    for wei_dt, zp_dt in ((dt.u8, dt.u8), (dt.s8, dt.s8), (dt.u8, dt.s8), (dt.s8, dt.u8)):
        say("mfma_f16w8 one-hot %s / %s" % (wei_dt, zp_dt))
        M, K, N = 256, 256, 256
        p = problem(M, K, N, 5, wei_dt=wei_dt, zp_dt=zp_dt, dst_dt=dt.f32, scale="common")
        a = np.zeros((M, K), np.float32)
        a[np.arange(M), np.arange(M) % K] = 1.0
        p.src.set(a)
        lo, hi = (0, 255) if wei_dt == dt.u8 else (-128, 127)
        w = np.where((np.arange(K)[:, None] + np.arange(N)[None, :]) % 2 == 0, lo, hi)
        w[::7] = np.arange(N) % (hi - lo + 1) + lo  # every value of the range
        p.wei.set(w)
        got, pd = p.run_gpu(eng, strm, weights_any=True, return_pd=True)
        assert pd.impl_info_str() == F16W8
        want = p.run_oracle()
        g, r = got.view(np.float32).reshape(M, N), want.view(np.float32).reshape(M, N)
        # one product and one scale multiplication in either order: 2 f32 roundings at most
        assert np.all(np.abs(g - r) <= 2.0 ** -22 * np.abs(r)), "one-hot %s / %s" % (wei_dt, zp_dt)


def test_slices_of_k_and_one_pass_agree(ctx, monkeypatch):
    """QMM_GEMM_VARIANT=1 keeps K in one pass: same problem both ways, each against the oracle's bar."""
    eng, strm = ctx
    p = problem(256, 2048, 512, 11, dst_dt=dt.f32)
    got_slices = p.run_gpu(eng, strm, weights_any=True)
    monkeypatch.setenv("QMM_GEMM_VARIANT", "1")
    got_one = p.run_gpu(eng, strm, weights_any=True)
    want = p.run_oracle()
    check(p, got_slices, want, "slices")
    check(p, got_one, want, "one pass")
    a, b = got_slices.view(np.float32), got_one.view(np.float32)
    assert not np.array_equal(a, b), "the two paths sum in different orders: identical results mean one path ran twice"


def test_fewer_than_256_rows_stay_with_the_decode_implementation(ctx):
    eng, strm = ctx
    p = problem(255, 256, 256, 3)
    _, pd = p.run_gpu(eng, strm, weights_any=True, return_pd=True)
    assert pd.impl_info_str() == DECODE
    # K that is not a multiple of 32, K-grouped scales: not this implementation's
    p = problem(256, 200, 256, 4)
    _, pd = p.run_gpu(eng, strm, weights_any=True, return_pd=True)
    assert pd.impl_info_str() != F16W8
