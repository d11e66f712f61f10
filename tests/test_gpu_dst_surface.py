"""GPU parity for the rest of the destination / epilogue surface:
f8_e5m2 x f8_e5m2 matmul, an f8_e5m2 destination of the fp8 MFMA kernels, the sum
post-op with a zero point and with a data type of its own, and destination scales
masked over N (M and M + N are refused, as in the reference).

Reference: src/cpu/matmul/ref_matmul.cpp:130-233 (float path), ref_matmul_int8.cpp:154-261,
src/cpu/primitive_attr_postops.cpp:187-198 (sum: scale * (dst_as_sum_dt - zero_point)),
src/common/matmul.cpp:147-159 and src/gpu/intel/ocl/ref_matmul.cl:239-245 (masked dst scales).
"""
import sys

import numpy as np
import pytest

import onednn_amd as dnnl
import oracle as O
from onednn_amd import _capi
from qmm_harness import Problem, TensorSpec, assert_bit_exact, assert_f32_close, dt
import test_gpu_parity as cases

pytestmark = pytest.mark.gpu
ROUTES = ["generic", "general", "tile256", "two_per_cu"]


def say(msg):
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def ctx():
    eng = dnnl.engine(dnnl.engine.kind.gpu, 0)
    return eng, dnnl.stream(eng)


def _run(ctx, route, p, dst_init=None):
    eng, strm = ctx
    if route == "generic":
        return p.run_gpu(eng, strm, impl=cases.GENERIC, dst_init=dst_init)
    # tile256: 256 x 256 tiles, one workgroup per CU; two_per_cu: 256 x 128 tiles; general: the 128 x 128 configuration
    with _capi.kernel_variants(gemm=2 if route == "general" else 6, b8x=2 if route == "two_per_cu" else 3):
        got, pd = p.run_gpu(eng, strm, weights_any=True, return_pd=True, dst_init=dst_init)
    assert pd.impl_info_str() == cases.MFMA
    return got


# ---------------------------------------------------------------------------
def _e5m2_problem(M, K, N, seed, dst_dt, with_sum):
    r = np.random.default_rng(seed)
    a = (r.standard_normal((M, K)) * 3).astype(np.float32)
    b = (r.standard_normal((K, N)) * 3).astype(np.float32)
    src = TensorSpec(dt.f8_e5m2, [M, K], None, a)
    wei = TensorSpec(dt.f8_e5m2, [K, N], "ba", b)
    dst = TensorSpec(dst_dt, [M, N], None, r.standard_normal((M, N)).astype(np.float32))
    scales = {"src": (0, dt.f32, None, [0.5]), "wei": (2, dt.f32, None, r.uniform(0.1, 0.5, N))}
    po = [{"kind": "sum", "scale": 0.5}] if with_sum else []
    po.append({"kind": "eltwise", "alg": dnnl.algorithm.eltwise_relu, "alpha": 0.1})
    return Problem(src, wei, dst, scales=scales, post_ops=po)


@pytest.mark.parametrize("dst_dt", [dt.f32, dt.bf16, dt.f16, dt.f8_e5m2, dt.f8_e4m3], ids=str)
def test_e5m2_matmul(ctx, dst_dt):
    """e5m2 x e5m2 has one implementation, the generic kernel, which adds the K products in the reference's
    order: every dst type bit for bit."""
    eng, strm = ctx
    say("f8_e5m2 x f8_e5m2 -> %s" % dst_dt)
    p = _e5m2_problem(70, 96, 50, 41, dst_dt, with_sum=True)
    got, pd = p.run_gpu(eng, strm, return_pd=True)
    assert pd.impl_info_str() == cases.GENERIC
    assert_bit_exact(got, p.run_oracle(), "e5m2 matmul")


def _f8_neighbours(code_dt, got_raw, want_raw):
    """Distance in representable values between two arrays of fp8 codes (sign-magnitude codes
    mapped onto a line)."""
    def line(raw):
        v = raw.astype(np.int32)
        return np.where(v & 0x80, -(v & 0x7F), v & 0x7F)
    return np.abs(line(got_raw) - line(want_raw))


@pytest.mark.parametrize("dst_dt", [dt.f8_e5m2, dt.f8_e4m3], ids=str)
def test_mfma_fp8_kernels_store_fp8(ctx, dst_dt):
    """The fp8 MFMA kernels with an fp8 destination. Their f32 sums differ from the reference's in the last
    bits (the MFMA's summation tree), so a result may round to the neighbouring fp8 value: at most one step,
    and for few elements."""
    eng, strm = ctx
    for route, (M, K, N) in (("general", (200, 256, 160)), ("tile256", (512, 512, 512))):
        say("mfma_b8 fp8 -> %s via %s" % (dst_dt, route))
        p = cases.fp8_gemm(M, K, N, 91, dst_dt=dst_dt, with_sum=False)
        p.scales = {"src": (0, dt.f32, None, [0.05]), "wei": (0, dt.f32, None, [0.05])}
        got, want = _run(ctx, route, p), p.run_oracle()
        d = _f8_neighbours(dst_dt, got, want)
        frac = float((d != 0).mean())
        # a result that cancels to nearly zero may land on the other side of it, several tiny values away:
        # there the f32 bar applies (1e-5 of the summed term magnitudes)
        term = (np.abs(p.src.logical().astype(np.float64)) @ np.abs(p.wei.logical().astype(np.float64))) * 0.05 * 0.05
        err = np.abs(O.to_f32(dst_dt, got).astype(np.float64) - O.to_f32(dst_dt, want).astype(np.float64))
        far = (d > 1) & (err > 1e-5 * term.reshape(-1))
        print("[fp8 dst] %s %s: %.4f %% of the elements differ, %d by more than one value, %d of those beyond 1e-5 of the terms"
              % (route, dst_dt, 100 * frac, int((d > 1).sum()), int(far.sum())))
        assert not far.any() and frac < 0.01, (int(far.sum()), frac)


# ---------------------------------------------------------------------------
@pytest.mark.parametrize("route", ROUTES)
@pytest.mark.parametrize("dst_dt,sum_dt", [(dt.s8, dt.undef), (dt.s8, dt.u8), (dt.u8, dt.s8), (dt.s32, dt.undef),
                                           (dt.f32, dt.s32)], ids=str)
def test_sum_zero_point_and_data_type(ctx, route, dst_dt, sum_dt):
    """sum: acc += scale * (old_dst read as sum_dt - zero_point). Integer results: bit for bit."""
    say("sum zero point, dst %s read as %s, via %s" % (dst_dt, sum_dt, route))
    r = np.random.default_rng(17)
    M, K, N = 300, 128, 130
    po = [{"kind": "sum", "scale": 0.75, "zero_point": -3, "dt": sum_dt},
          {"kind": "eltwise", "alg": dnnl.algorithm.eltwise_linear, "alpha": 0.5, "beta": 1.0}]
    p = cases.int8_linear(M, K, N, 77, src_dt=dt.s8, dst_dt=dst_dt, src_zp=None, src_scale=0.01, post_ops=po,
                          dst_zp=[2] if dst_dt in (dt.s8, dt.u8) else None)
    # old dst: every byte value appears, so that reading it with the other signedness matters
    if dst_dt in (dt.s8, dt.u8):
        init = r.integers(0, 256, M * N).astype(np.uint8).view(p.dst.raw.dtype)
    elif dst_dt == dt.s32:
        init = r.integers(-1000, 1000, M * N).astype(np.int32)
    else:
        init = r.integers(-1000, 1000, M * N).astype(np.int32).view(np.float32)
    got = _run(ctx, route, p, dst_init=init)
    want = p.run_oracle(dst_init=init)
    if dst_dt == dt.f32:
        a = np.abs(want.view(np.float32).astype(np.float64))
        assert_f32_close(got.view(np.float32), want.view(np.float32), rel=1e-5, scale=a, what="sum f32 read as s32")
    else:
        assert_bit_exact(got, want, "sum with zero point")


def test_sum_rules_rejected_at_creation(ctx):
    """A sum data type of another size than dst's, and a sum zero point on a non-integer problem, are refused
    (src/common/primitive_attr.cpp check_sum_consistency, src/common/matmul.cpp:264-266)."""
    eng, _ = ctx
    p = cases.int8_linear(32, 64, 32, 5, src_dt=dt.s8, dst_dt=dt.s8, src_zp=None,
                          post_ops=[{"kind": "sum", "scale": 1.0, "dt": dt.s32}])
    with pytest.raises(dnnl.error) as e:
        p.primitive_desc(eng)
    assert e.value.status == dnnl.status.unimplemented
    p = cases.fp8_gemm(32, 64, 32, 5, dst_dt=dt.f32, with_sum=False)
    p.post_ops = [{"kind": "sum", "scale": 1.0, "zero_point": 1}]
    with pytest.raises(dnnl.error) as e:
        p.primitive_desc(eng)
    assert e.value.status == dnnl.status.unimplemented


# ---------------------------------------------------------------------------
@pytest.mark.parametrize("batch", [(), (3,)], ids=["2d", "3d"])
@pytest.mark.parametrize("which", ["N"])
@pytest.mark.parametrize("dst_dt", [dt.f32, dt.s8], ids=str)
def test_masked_dst_scales(ctx, which, batch, dst_dt):
    """dst scales over N (a GPU-engine-only attribute): one implementation, the generic kernel.
    Checked against the oracle and, independently of its code, against the unscaled f32 result divided on the
    host (one IEEE division per element, then the dst conversion)."""
    eng, strm = ctx
    say("dst scale mask %s, dst %s, batch %s" % (which, dst_dt, batch))
    M, K, N = 40, 64, 48
    nd = len(batch) + 2
    r = np.random.default_rng(23)
    mask = {"N": 1 << (nd - 1), "M": 1 << (nd - 2), "MN": 3 << (nd - 2)}[which]
    shape = {"N": (1, N), "M": (M, 1), "MN": (M, N)}[which]
    sc = r.uniform(0.5, 4.0, shape).astype(np.float32)
    p = cases.int8_linear(M, K, N, 29, src_dt=dt.s8, dst_dt=dst_dt, src_zp=None, src_scale=0.02, batch=batch)
    plain = cases.int8_linear(M, K, N, 29, src_dt=dt.s8, dst_dt=dt.f32, src_zp=None, src_scale=0.02, batch=batch)
    p.scales["dst"] = (mask, dt.f32, None, sc)
    got, pd = p.run_gpu(eng, strm, return_pd=True)
    assert pd.impl_info_str() == cases.GENERIC
    assert_bit_exact(got, p.run_oracle(), "masked dst scale vs oracle")
    unscaled = plain.run_oracle().view(np.float32).reshape(list(batch) + [M, N])
    want = (unscaled / sc).astype(np.float32)
    if dst_dt == dt.s8:
        want = np.clip(np.rint(want), -128, 127).astype(np.int8)
    assert_bit_exact(got.view(want.dtype).reshape(want.shape), want, "masked dst scale vs host division")


def test_masked_dst_scale_over_batch_m_or_m_and_n_is_refused(ctx):
    """Of the masks the reference names for GPU engines (N, M, M + N) only N can be created there: its common
    check computes the M bit from the source's K position (src/common/matmul.cpp:91, 150-154: for 2-D tensors
    0, 2, 2 or 4) and the primitive descriptor's rule takes 0, N or M + N (src/common/matmul_pd.hpp:230-233),
    which leaves 0 and N. The same descriptors fail here with the same status."""
    eng, _ = ctx
    for mask, n in ((1, 16), (3, 16 * 32)):
        p = cases.int8_linear(16, 64, 32, 3, src_dt=dt.s8, dst_dt=dt.f32, src_zp=None)
        p.scales["dst"] = (mask, dt.f32, None, np.ones(n, np.float32))
        with pytest.raises(dnnl.error) as e:
            p.primitive_desc(eng)
        assert e.value.status == dnnl.status.unimplemented
    p = cases.int8_linear(16, 64, 32, 3, src_dt=dt.s8, dst_dt=dt.f32, src_zp=None, batch=(2,))
    p.scales["dst"] = (1, dt.f32, None, np.ones(2, np.float32))
    with pytest.raises(dnnl.error) as e:
        p.primitive_desc(eng)
    assert e.value.status == dnnl.status.unimplemented


# ---------------------------------------------------------------------------
@pytest.mark.parametrize("route", ROUTES)
@pytest.mark.parametrize("dst_dt", [dt.s8, dt.u8], ids=str)
def test_swish_into_quantized_dst(ctx, route, dst_dt):
    """swish followed by a dst scale, a dst zero point and the saturating integer store. A transcendental
    sits in front of the rounding (hardware exp2 / reciprocal in the straight-line epilogue, device libm elsewhere,
    host libm in the oracle), so a value within float rounding of a .5 boundary may land on the neighbouring
    integer: never further, and for few elements."""
    say("swish -> %s with dst scale and zero point via %s" % (dst_dt, route))
    M, K, N = (512, 256, 512) if route in ("tile256", "two_per_cu") else (300, 128, 130)
    p = cases.int8_linear(M, K, N, 57, src_dt=dt.s8, dst_dt=dst_dt, src_zp=None, src_scale=0.01,
                          post_ops=[{"kind": "eltwise", "alg": dnnl.algorithm.eltwise_swish, "alpha": 1.0}],
                          dst_scale=0.05, dst_zp=[7])
    got = _run(ctx, route, p).astype(np.int32)
    want = p.run_oracle().astype(np.int32)
    d = np.abs(got - want)
    frac = float((d != 0).mean())
    print("[swish q8] %s %s: %.4f %% of the elements one step off, max distance %d; distinct values %d"
          % (route, dst_dt, 100 * frac, d.max(), len(np.unique(want))))
    assert len(np.unique(want)) > 50  # the case exercises the range, not a saturated constant
    assert d.max() <= 1 and frac < 2e-3, (int(d.max()), frac)


# ---------------------------------------------------------------------------
@pytest.mark.parametrize("forced", [True, False], ids=["generic", "first_impl"])
def test_e8m0_grouped_weights_scales(ctx, forced):
    """Weights scales stored as e8m0 (src/common/primitive_attr.cpp:529 admits the type; decoded as
    src/common/float8.cpp:36-41: 2^(r - 127)), one per 32 k and column, on s8 x s8. Powers of two keep every
    product exact, so the result is the oracle's bit for bit whatever the order."""
    eng, strm = ctx
    say("e8m0 weights scales per 32 k, %s" % ("generic" if forced else "first implementation"))
    r = np.random.default_rng(23)
    M, K, N = 33, 128, 48
    src = TensorSpec(dt.s8, [M, K], None, r.integers(-9, 10, (M, K)))
    wei = TensorSpec(dt.s8, [K, N], None, r.integers(-9, 10, (K, N)))
    dst = TensorSpec(dt.f32, [M, N])
    ws = 2.0 ** r.integers(-6, 4, (K // 32, N))
    p = Problem(src, wei, dst, scales={"src": (0, dt.f32, None, [0.25]), "wei": (3, dt.e8m0, (32, 1), ws)})
    got, pd = p.run_gpu(eng, strm, impl=cases.GENERIC if forced else None, return_pd=True)
    say("  ran on " + pd.impl_info_str())
    want = p.run_oracle()
    assert_bit_exact(got, want, "e8m0 grouped weights scales")
    # and against the arithmetic itself: sum over groups of 2^e * (exact integer dot product of the group)
    a = src.logical().astype(np.int64)
    b = wei.logical().astype(np.int64)
    exact = sum((a[:, g * 32:(g + 1) * 32] @ b[g * 32:(g + 1) * 32]) * ws[g][None, :] for g in range(K // 32)) * 0.25
    assert np.array_equal(got.view(np.float32).reshape(M, N).astype(np.float64), exact)


@pytest.mark.parametrize("act", [dt.bf16, dt.f16], ids=str)
@pytest.mark.parametrize("scale", [2.0, 0.25])
def test_e8m0_dst_scale(ctx, act, scale):
    """The reference's CI case (tests/benchdnn/inputs/matmul/test_matmul_ci:110-114): a single destination scale of
    type e8m0 on bf16 / f16 matmuls, 4x256:256x64 and 6x256:256x100."""
    eng, strm = ctx
    for M, K, N in ((4, 256, 64), (6, 256, 100)):
        say("e8m0 dst scale %g, %s %dx%dx%d" % (scale, act, M, K, N))
        r = np.random.default_rng(M * N)
        src = TensorSpec(act, [M, K], None, r.integers(-4, 5, (M, K)).astype(np.float32))
        wei = TensorSpec(act, [K, N], None, r.integers(-4, 5, (K, N)).astype(np.float32))
        dst = TensorSpec(act, [M, N])
        p = Problem(src, wei, dst, scales={"dst": (0, dt.e8m0, None, [scale])})
        got, pd = p.run_gpu(eng, strm, return_pd=True)
        say("  ran on " + pd.impl_info_str())
        assert_bit_exact(got, p.run_oracle(), "e8m0 dst scale")
        exact = (src.logical().astype(np.float64) @ wei.logical().astype(np.float64)) / scale
        # the exact quotient (an integer or half-integer, exact in f32) rounded once to the dst type
        assert np.array_equal(got.view(np.uint16).reshape(-1), O.from_f32(act, exact.astype(np.float32)).reshape(-1))


# ---------------------------------------------------------------------------
@pytest.mark.parametrize("route", ROUTES)
@pytest.mark.parametrize("dst_dt", [dt.s8, dt.u8, dt.f32, dt.bf16, dt.s32], ids=str)
@pytest.mark.parametrize("N", [999, 1001, 998])
def test_rows_that_start_at_any_byte(ctx, route, dst_dt, N):
    """dst rows of 999 / 1001 / 998 elements: a row starts at any byte (s8 / u8), at 2 mod 4 (bf16) or off its 16-byte
    vector (f32 / s32), and the four-column stores of every epilogue are then vector stores at unaligned addresses,
    which global memory instructions take. Integer data, a relu and a power-of-two dst scale: every route must give the
    oracle's bits, in the last columns of a row and the first of the next one alike."""
    say("odd row length %d, dst %s via %s" % (N, dst_dt, route))
    M, K = (300, 320) if route in ("tile256", "two_per_cu") else (70, 128)
    quant = dst_dt in (dt.s8, dt.u8)
    p = cases.int8_linear(M, K, N, 91 + N, src_dt=dt.s8, dst_dt=dst_dt, src_zp=None,
                          src_scale=None if dst_dt == dt.s32 else 2.0 ** -6,
                          post_ops=None if dst_dt == dt.s32 else [{"kind": "eltwise", "alg": dnnl.algorithm.eltwise_relu,
                                                                   "alpha": 0.25}],
                          dst_scale=4.0 if quant else None, dst_zp=[3] if quant else None)
    if dst_dt == dt.s32:
        p.scales = {}
    else:
        r = np.random.default_rng(N)
        p.scales["wei"] = (2, dt.f32, None, 2.0 ** r.integers(-7, -3, N))
    assert_bit_exact(_run(ctx, route, p), p.run_oracle(), "odd rows %d %s %s" % (N, dst_dt, route))


@pytest.mark.parametrize("route", ROUTES)
@pytest.mark.parametrize("op_dt", [dt.f32, dt.f16, dt.s8], ids=str)
@pytest.mark.parametrize("N", [999, 1001])
def test_binary_operand_rows_that_start_at_any_byte(ctx, route, op_dt, N):
    """The same for the second tensor of a binary post-op: a dense [M, N] operand whose rows start off their vectors
    (f32 at 4 mod 16, f16 at 2 mod 8, s8 at any byte), added to an f32 result. Integer data: bit for bit."""
    say("binary add operand %s, odd row length %d via %s" % (op_dt, N, route))
    M, K = (300, 320) if route in ("tile256", "two_per_cu") else (70, 128)
    r = np.random.default_rng(7 * N + op_dt)
    src1 = TensorSpec(op_dt, [M, N], None, r.integers(-50, 51, (M, N)).astype(np.float32))
    p = cases.int8_linear(M, K, N, 17 + N, src_dt=dt.s8, dst_dt=dt.f32, src_zp=None, src_scale=2.0 ** -6,
                          post_ops=[{"kind": "binary", "alg": dnnl.algorithm.binary_add, "src1": src1}])
    p.scales["wei"] = (2, dt.f32, None, 2.0 ** r.integers(-7, -3, N))
    assert_bit_exact(_run(ctx, route, p), p.run_oracle(), "binary operand rows %d %s %s" % (N, op_dt, route))
