"""Every forward eltwise algorithm (21 + the 7 *_use_dst_for_bwd aliases) and every
binary algorithm (12) of the post-op chain, on the device, through the three
places that implement the chain: the generic kernel (one thread per element),
the general MFMA kernel's four-element interpreter, and the 256 x 256 kernels'
row interpreter. Reference: src/common/math_utils.hpp:129-416,
src/cpu/primitive_attr_postops.cpp:29-46.

Algorithms made of comparisons, selects and single IEEE operations are compared
bit for bit; those that call a transcendental routine (device libm against the
oracle's host libm) at rel 1e-5 of the result, as stated for f32 dst."""
import sys

import numpy as np
import pytest

import onednn_amd as dnnl
import oracle as O
from onednn_amd import _capi
from qmm_harness import TensorSpec, assert_bit_exact, assert_f32_close, dt
import test_gpu_parity as cases

pytestmark = pytest.mark.gpu
A = dnnl.algorithm

# name: (alpha, beta, exact)
ELTWISE = {
    "eltwise_relu": (0.1, 0.0, True), "eltwise_tanh": (0.0, 0.0, False), "eltwise_elu": (0.7, 0.0, False),
    "eltwise_square": (0.0, 0.0, True), "eltwise_abs": (0.0, 0.0, True), "eltwise_sqrt": (0.0, 0.0, True),
    "eltwise_linear": (0.75, -0.5, True), "eltwise_soft_relu": (1.5, 0.0, False),
    "eltwise_hardsigmoid": (0.2, 0.5, True), "eltwise_logistic": (0.0, 0.0, False), "eltwise_exp": (0.0, 0.0, False),
    "eltwise_gelu_tanh": (0.0, 0.0, False), "eltwise_swish": (0.9, 0.0, False), "eltwise_log": (0.0, 0.0, False),
    "eltwise_clip": (-1.0, 2.0, True), "eltwise_clip_v2": (-1.5, 1.0, True), "eltwise_pow": (0.5, 2.0, False),
    "eltwise_gelu_erf": (0.0, 0.0, False), "eltwise_round": (0.0, 0.0, True), "eltwise_mish": (0.0, 0.0, False),
    "eltwise_hardswish": (1.0 / 6, 0.5, True),
    "eltwise_relu_use_dst_for_bwd": (0.0, 0.0, True), "eltwise_tanh_use_dst_for_bwd": (0.0, 0.0, False),
    "eltwise_elu_use_dst_for_bwd": (0.7, 0.0, False), "eltwise_sqrt_use_dst_for_bwd": (0.0, 0.0, True),
    "eltwise_logistic_use_dst_for_bwd": (0.0, 0.0, False), "eltwise_exp_use_dst_for_bwd": (0.0, 0.0, False),
    "eltwise_clip_v2_use_dst_for_bwd": (-1.5, 1.0, True),
}
BINARY = ["binary_add", "binary_mul", "binary_max", "binary_min", "binary_div", "binary_sub", "binary_ge",
          "binary_gt", "binary_le", "binary_lt", "binary_eq", "binary_ne"]
# sqrt, log and pow see negative accumulators (NaN in both); the routes are compared NaN for NaN
ROUTES = ["generic", "general", "tile256", "two_per_cu"]


def say(msg):
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def ctx():
    eng = dnnl.engine(dnnl.engine.kind.gpu, 0)
    return eng, dnnl.stream(eng)


def _run(ctx, route, p):
    eng, strm = ctx
    if route == "generic":
        return p.run_gpu(eng, strm, impl=cases.GENERIC)
    # tile256: 256 x 256 tiles, one workgroup per CU; two_per_cu: 256 x 128 tiles; general: the 128 x 128 configuration
    with _capi.kernel_variants(gemm=2 if route == "general" else 6, b8x=2 if route == "two_per_cu" else 3):
        got, pd = p.run_gpu(eng, strm, weights_any=True, return_pd=True)
    assert pd.impl_info_str() == cases.MFMA
    return got


def _check(got, want, exact, what, term=None):
    if exact:
        assert_bit_exact(got, want, what)
        return
    g, w = got.view(np.float32).astype(np.float64), want.view(np.float32).astype(np.float64)
    # device libm against host libm: 1e-5 of the result; where the result underflows
    # towards 0 (exp, logistic, swish, mish of very negative inputs) 1e-5 of 1e-30.
    # `term`: magnitude of the terms of a form that cancels (gelu: 0.5 x (1 + erf) for
    # negative x is the difference of two numbers near 0.5 |x|)
    scale = 1e-30 if term is None else np.maximum(term.astype(np.float64).reshape(g.shape), 1e-30)
    assert_f32_close(g, w, rel=1e-5, scale=scale, what=what, max_slack_frac=0.05)


@pytest.mark.parametrize("route", ROUTES)
@pytest.mark.parametrize("name", sorted(ELTWISE))
def test_eltwise_algorithm(ctx, route, name):
    alpha, beta, exact = ELTWISE[name]
    say("eltwise %s via %s" % (name, route))
    # accumulators of both signs, scaled to |x| of a few units; 300 x 130: edge tiles on every route
    p = cases.int8_linear(300, 128, 130, 500 + len(name), src_dt=dt.s8, dst_dt=dt.f32, src_zp=None, src_scale=0.004,
                          post_ops=[{"kind": "eltwise", "alg": getattr(A, name), "alpha": alpha, "beta": beta}])
    term = None
    if "gelu" in name:
        po, p.post_ops = p.post_ops, []
        term = 0.5 * np.abs(p.run_oracle().view(np.float32))
        p.post_ops = po
    got, want = _run(ctx, route, p), p.run_oracle()
    _check(got, want, exact, "%s %s" % (name, route), term)
    if name == "eltwise_gelu_erf":
        # 0.5 x (1 + erf(x / sqrt 2)): for negative x the bracket is a difference of numbers near 1, so an erff that
        # is good to an ulp or two of ITS result (2^-24) leaves the product good to that many units of 2^-24 x 0.5 |x|
        # only. Both sides against the exact value (float64 erf): the device's erff must be as good as the host's.
        from scipy.special import erf
        po, p.post_ops = p.post_ops, []
        x = p.run_oracle().view(np.float32).astype(np.float64).reshape(-1)
        p.post_ops = po
        exact64 = 0.5 * x * (1.0 + erf(x / np.sqrt(2.0)))
        unit = 2.0 ** -24 * np.maximum(0.5 * np.abs(x), 1e-30)
        e_gpu = np.abs(got.view(np.float32).astype(np.float64).reshape(-1) - exact64) / unit
        e_ref = np.abs(want.view(np.float32).astype(np.float64).reshape(-1) - exact64) / unit
        print("[gelu_erf] %s: distance from the exact value in units of 2^-24 x 0.5|x|: kernel max %.2f mean %.3f, "
              "host libm (the oracle) max %.2f mean %.3f" % (route, e_gpu.max(), e_gpu.mean(), e_ref.max(), e_ref.mean()),
              flush=True)
        assert e_gpu.max() <= 6.0 and e_gpu.mean() <= 1.0, (e_gpu.max(), e_gpu.mean())


@pytest.mark.parametrize("route", ROUTES)
@pytest.mark.parametrize("name", BINARY)
def test_binary_algorithm(ctx, route, name):
    say("binary %s via %s" % (name, route))
    p = cases.int8_linear(300, 128, 130, 600 + len(name), src_dt=dt.s8, dst_dt=dt.f32, src_zp=None, src_scale=0.004)
    # an operand that ties with the accumulated value in places, so that eq / ge / le see both outcomes
    base = p.run_oracle().view(np.float32).reshape(300, 130).copy()
    r = np.random.default_rng(9)
    other = np.where(r.random((300, 130)) < 0.3, base, r.standard_normal((300, 130)).astype(np.float32) * 2 + 0.25)
    p.post_ops = [{"kind": "binary", "alg": getattr(A, name),
                   "src1": TensorSpec(dt.f32, [300, 130], None, other.astype(np.float32))}]
    _check(_run(ctx, route, p), p.run_oracle(), True, "%s %s" % (name, route))
