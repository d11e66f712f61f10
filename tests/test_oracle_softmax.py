"""Pins oracle.softmax (oracle/qmm_oracle.c orc_softmax, a restatement of src/cpu/ref_softmax.cpp:40-312) with
checks that do not repeat its code: float64 closed forms from scipy, rows whose result is exact in binary
arithmetic, the C library's own expf combined step by step with numpy float32 operations (which separates the
reference's two loops: times-the-reciprocal for a dense same-type row, division otherwise), scales, the saturating
integer store, other axes and strided layouts against numpy on a moved axis."""
import ctypes

import numpy as np
import pytest
import scipy.special

import oracle as O


def T(code, a, dims=None, strides=None):
    return O.Tensor(code, list(a.shape) if dims is None else list(dims), a, strides)


def _libm_expf(x):
    m = ctypes.CDLL("libm.so.6")
    m.expf.restype = ctypes.c_float
    m.expf.argtypes = [ctypes.c_float]
    return np.array([m.expf(float(v)) for v in np.asarray(x, np.float32).reshape(-1)], np.float32).reshape(np.shape(x))


def test_against_float64_closed_forms():
    r = np.random.default_rng(1)
    x = (r.standard_normal((7, 5, 33)) * 4).astype(np.float32)
    for axis in (0, 1, 2):
        out = np.zeros_like(x)
        O.softmax(T(O.F32, x), T(O.F32, out), axis)
        want = scipy.special.softmax(x.astype(np.float64), axis=axis)
        assert np.max(np.abs(out - want) / want) < 2e-6
        assert np.allclose(out.sum(axis=axis), 1.0, atol=2e-6)
        O.softmax(T(O.F32, x), T(O.F32, out), axis, log=True)
        want = scipy.special.log_softmax(x.astype(np.float64), axis=axis)
        assert np.max(np.abs(out - want)) < 2e-6 * np.max(np.abs(want))


def test_exact_rows():
    # 2^k equal values: exp(0) = 1, the sum 2^k and its reciprocal are exact
    for k in (0, 3, 10):
        x = np.full((3, 1 << k), 2.5, np.float32)
        out = np.zeros_like(x)
        O.softmax(T(O.F32, x), T(O.F32, out), 1)
        assert np.all(out == np.float32(2.0 ** -k))
    # a masked row: -1e4 below the maximum underflows to exactly 0 and leaves the rest untouched
    x = np.array([[1.0, 1.0, -1e4, 1.0, 1.0, -1e4]], np.float32)
    out = np.zeros_like(x)
    O.softmax(T(O.F32, x), T(O.F32, out), 1)
    assert np.array_equal(out, np.array([[0.25, 0.25, 0, 0.25, 0.25, 0]], np.float32))


def test_dense_rows_multiply_by_the_reciprocal_other_cases_divide():
    """ref_softmax.hpp:137-139 picks the loop: innermost axis + one dense layout + ONE data type -> d * (1 / sum)
    (ref_softmax.cpp:160-172); anything else -> d / sum (:283-287). The two differ in the last bit for some
    elements; the expected bits come from libm's expf and numpy float32 operations, summed in index order."""
    r = np.random.default_rng(2)
    x = (r.standard_normal((16, 24)) * 3).astype(np.float32)
    e = _libm_expf(x - x.max(axis=1, keepdims=True))
    s = np.zeros(16, np.float32)
    for c in range(24):
        s = s + e[:, c]
    recip = e * (np.float32(1) / s)[:, None]
    divided = e / s[:, None]
    assert not np.array_equal(recip.view(np.uint32), divided.view(np.uint32))  # the data tell the two apart
    out = np.zeros_like(x)
    O.softmax(T(O.F32, x), T(O.F32, out), 1)
    assert np.array_equal(out.view(np.uint32), recip.view(np.uint32))
    # same row data, destination of another type: the generic loop, then one conversion
    out16 = np.zeros(x.shape, np.uint16)
    O.softmax(T(O.F32, x), T(O.F16, out16), 1)
    assert np.array_equal(out16, divided.astype(np.float16).view(np.uint16))
    # same type, but the axis is not the innermost one: the generic loop
    xt = np.ascontiguousarray(x.T)  # [24, 16], softmax over axis 0
    outt = np.zeros_like(xt)
    O.softmax(T(O.F32, xt), T(O.F32, outt), 0)
    assert np.array_equal(outt.T.view(np.uint32), divided.view(np.uint32))


def test_scales_and_saturating_integer_store():
    r = np.random.default_rng(3)
    x = (r.standard_normal((8, 40)) * 2).astype(np.float32)
    e = _libm_expf(x - x.max(axis=1, keepdims=True))
    s = np.zeros(8, np.float32)
    for c in range(40):
        s = s + e[:, c]
    ss, ds = np.array([1.7], np.float32), np.array([0.003], np.float32)
    val = (e / s[:, None]) * ss[0]            # f32 -> u8: the generic loop
    val = val * (np.float32(1) / ds[0])       # the destination scale enters inverted
    want = np.clip(np.rint(val), 0, 255).astype(np.uint8)
    assert want.max() == 255 and len(np.unique(want)) > 20  # saturation and a spread of values both occur
    out = np.zeros(x.shape, np.uint8)
    O.softmax(T(O.F32, x), T(O.U8, out), 1, src_scale=O.Quant(0, O.F32, ss), dst_scale=O.Quant(0, O.F32, ds))
    assert np.array_equal(out, want)


def test_other_axes_and_strided_layouts():
    r = np.random.default_rng(4)
    x = (r.standard_normal((3, 6, 10)) * 3).astype(np.float32)
    # a permuted physical layout of the same logical tensor: logical [3, 6, 10] stored as [10, 3, 6]
    phys = np.ascontiguousarray(np.transpose(x, (2, 0, 1)))
    strides = [6, 1, 18]  # of the logical dims in that storage
    for axis in (0, 1, 2):
        out = np.zeros_like(x)
        O.softmax(O.Tensor(O.F32, [3, 6, 10], phys, strides), T(O.F32, out), axis)
        want = scipy.special.softmax(x.astype(np.float64), axis=axis)
        assert np.max(np.abs(out - want) / want) < 2e-6
    # bf16 source values are converted first (ref_io_helper load), results rounded once at the end
    xb = O.from_f32(O.BF16, x)
    outb = np.zeros(x.shape, np.uint16)
    O.softmax(T(O.BF16, xb), T(O.BF16, outb), 2)
    want = scipy.special.softmax(O.to_f32(O.BF16, xb).reshape(x.shape).astype(np.float64), axis=2)
    got = O.to_f32(O.BF16, outb).reshape(x.shape)
    assert np.max(np.abs(got - want) / want) < 2.0 ** -8
