"""Pins the oracle's scalar type layer against independent implementations.

Sources of truth: numpy's IEEE float16, torch's bfloat16 / float8 tensors,
closed-form decoders, and the properties the reference's own unit tests assert
(tests/gtests/internals/test_float8.cpp:31-118, test_nibble.cpp:36-80,
test_bfloat16.cpp).
"""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle as O


def _rand_f32(n, seed):
    rng = np.random.default_rng(seed)
    bits = rng.integers(0, 2**32, size=n, dtype=np.uint64).astype(np.uint32)
    vals = bits.view(np.float32)
    scaled = (rng.standard_normal(n) * np.exp(rng.uniform(-12, 12, n))).astype(np.float32)
    return np.concatenate([vals, scaled])


def test_bf16_matches_round_to_nearest_even_closed_form():
    x = _rand_f32(200000, 1)
    x = x[np.isfinite(x) & (np.abs(x) >= np.finfo(np.float32).tiny)]
    got = O.from_f32(O.BF16, x)
    u = x.view(np.uint32).astype(np.uint64)
    want = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    assert np.array_equal(got, want)
    # and against torch's converter (an independent implementation)
    t = torch.from_numpy(x.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, t)


def test_bf16_specials():
    L = O.lib()
    assert L.orc_f32_to_bf16(0.0) == 0x0000
    assert L.orc_f32_to_bf16(-0.0) == 0x8000
    assert L.orc_f32_to_bf16(float("inf")) == 0x7F80
    assert L.orc_f32_to_bf16(float("-inf")) == 0xFF80
    nan = L.orc_f32_to_bf16(float("nan"))
    assert (nan & 0x7F80) == 0x7F80 and (nan & 0x7F) != 0 and (nan & 0x40)
    # f32 subnormals flush to a signed zero (src/common/bfloat16.cpp:29-33)
    sub = np.array([1e-40, -1e-40], dtype=np.float32)
    assert list(O.from_f32(O.BF16, sub)) == [0x0000, 0x8000]
    # ties go to even: 1 + 2^-8 is exactly between 1.0 and 1 + 2^-7
    assert L.orc_f32_to_bf16(1.0 + 2.0**-8) == 0x3F80
    assert L.orc_f32_to_bf16(1.0 + 2.0**-7 + 2.0**-8) == 0x3F82
    # widening is a 16-bit shift
    for r in (0x3F80, 0xC000, 0x0001, 0x7F7F):
        assert np.float32(L.orc_bf16_to_f32(r)).view(np.uint32) == r << 16


def test_f16_from_f32_matches_numpy():
    x = _rand_f32(300000, 2)
    x = x[~np.isnan(x)]
    got = O.from_f32(O.F16, x)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(got, want)
    # half-way points between neighbouring f16 values, including subnormals
    h = np.arange(0, 0x7BFF, dtype=np.uint16)
    lo = h.view(np.float16).astype(np.float64)
    hi = (h + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    mid = ((lo + hi) / 2).astype(np.float32)
    assert np.array_equal(((lo + hi) / 2), mid.astype(np.float64))
    got = O.from_f32(O.F16, mid)
    assert np.array_equal(got, mid.astype(np.float16).view(np.uint16))
    assert np.all(got % 2 == 0)  # ties to even


def test_f16_to_f32_all_values():
    h = np.arange(0, 0x10000, dtype=np.uint32).astype(np.uint16)
    got = O.to_f32(O.F16, h)
    want = h.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def _e4m3_closed_form(r):
    s = -1.0 if r & 0x80 else 1.0
    e, m = (r >> 3) & 0xF, r & 7
    if e == 0xF and m == 7:
        return float("nan")
    if e == 0:
        return s * m * 2.0**-9
    return s * (1 + m / 8.0) * 2.0 ** (e - 7)


def test_e4m3_decode_closed_form_and_round_trip():
    L = O.lib()
    for r in range(256):
        v = L.orc_e4m3_to_f32(r)
        w = _e4m3_closed_form(r)
        if w != w:
            assert v != v
            continue
        assert v == w
        # tests/gtests/internals/test_float8.cpp:60-89: f8 -> f32 -> f8 is identity
        assert L.orc_f32_to_e4m3(v) == r
    assert L.orc_e4m3_to_f32(0x7E) == 448.0


def test_e4m3_encode_matches_torch_on_every_f16_input():
    h = np.arange(0, 0x10000, dtype=np.uint32).astype(np.uint16)
    f = h.view(np.float16).astype(np.float32)
    got = O.from_f32(O.F8_E4M3, f)
    want = torch.from_numpy(f.copy()).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    gn = (got & 0x7F) == 0x7F
    wn = (want & 0x7F) == 0x7F
    assert np.array_equal(gn, wn)  # overflow / inf / nan all map to the NaN code
    assert np.array_equal(got[~gn], want[~wn])
    # sign is kept on the NaN code for overflow (src/common/float8.cpp:103-109)
    assert O.lib().orc_f32_to_e4m3(-1000.0) == 0xFF
    assert O.lib().orc_f32_to_e4m3(1000.0) == 0x7F
    # no saturation: 464 is the last value that still rounds to 448
    assert O.lib().orc_f32_to_e4m3(464.0) == 0x7E
    assert O.lib().orc_f32_to_e4m3(465.0) == 0x7F
    # |x| <= 2^-10 flushes to signed zero
    assert O.lib().orc_f32_to_e4m3(2.0**-10) == 0x00
    assert O.lib().orc_f32_to_e4m3(-(2.0**-10)) == 0x80


def test_e4m3_goes_through_f16():
    # 1.0625 is the tie between 1.0 and 1.125; a value just above it rounds to
    # the tie in f16 first and then to even: the documented double rounding
    L = O.lib()
    x = np.float32(1.0625) + np.float32(2.0**-20)
    assert L.orc_f32_to_e4m3(float(x)) == L.orc_f16_to_e4m3(L.orc_f32_to_f16(float(x)))
    assert L.orc_f32_to_e4m3(float(x)) == 0x38  # 1.0


def test_e5m2_matches_torch_and_round_trip():
    L = O.lib()
    for r in range(256):
        v = L.orc_e5m2_to_f32(r)
        back = L.orc_f32_to_e5m2(v)
        # tests/gtests/internals/test_float8.cpp:31-58: identity but sNaN -> qNaN
        assert back == (r | 0x02 if r in (0x7D, 0xFD) else r)
    h = np.arange(0, 0x10000, dtype=np.uint32).astype(np.uint16)
    f = h.view(np.float16).astype(np.float32)
    ok = ~np.isnan(f)
    got = O.from_f32(O.F8_E5M2, f[ok])
    want = torch.from_numpy(f[ok].copy()).to(torch.float8_e5m2).view(torch.uint8).numpy()
    assert np.array_equal(got, want)


def test_e8m0_decode_closed_form_all_codes():
    # src/common/float8.cpp:36-41: the code is the f32 exponent field, no sign, no mantissa:
    # r in 1..254 is 2^(r-127); 0xff is the only NaN (the "real indefinite" pattern); r = 0 has
    # an all-zero f32 pattern, i.e. +0.0 (not the 2^-127 an OCP decoder would give).
    codes = np.arange(256, dtype=np.uint8)
    got = O.to_f32(O.E8M0, codes)
    L = O.lib()
    for r in range(256):
        one = L.orc_load_float(O.E8M0, codes.ctypes.data, r)
        if r == 0xFF:
            assert np.isnan(got[r]) and np.isnan(one)
            assert got[r:r + 1].view(np.uint32)[0] == 0xFFC00000
        elif r == 0:
            assert got[r] == 0.0 and not np.signbit(got[r]) and one == 0.0
        else:
            want = np.float32(2.0 ** (r - 127))       # exact: a normal f32 power of two
            assert got[r] == want and one == want, r
            assert np.frexp(np.float64(got[r])) == (0.5, r - 126)
    # a second decoder: torch's e8m0 type agrees wherever the value is a normal f32
    t = torch.from_numpy(codes[1:255].copy()).view(torch.float8_e8m0fnu).to(torch.float32).numpy()
    assert np.array_equal(t, got[1:255])
    # src/common/float8.cpp:28-34: the encoder keeps the exponent field and drops sign and
    # mantissa (round toward zero), so decode(encode(x)) is the power of two at or below |x|
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(4096) * np.exp(rng.uniform(-60, 60, 4096))).astype(np.float32)
    x = x[np.abs(x) >= np.float32(2.0 ** -126)]
    enc = ((x.view(np.uint32) >> 23) & 0xFF).astype(np.uint8)
    dec = O.to_f32(O.E8M0, enc)
    assert np.array_equal(dec, np.float32(2.0) ** np.floor(np.log2(np.abs(x.astype(np.float64)))).astype(np.float32))


def test_nibble_order_and_ranges():
    # tests/gtests/internals/test_nibble.cpp:36-80: low nibble is the even index
    buf = np.array([0x21, 0xF8], dtype=np.uint8)
    L = O.lib()
    p = buf.ctypes.data
    assert [L.orc_load_int(O.U4, p, i) for i in range(4)] == [1, 2, 8, 15]
    assert [L.orc_load_int(O.S4, p, i) for i in range(4)] == [1, 2, -8, -1]
    assert [L.orc_load_float(O.S4, p, i) for i in range(4)] == [1.0, 2.0, -8.0, -1.0]
    allv = O.pack4(np.arange(16))
    assert list(O.unpack4(allv, 16, False)) == list(range(16))
    assert list(O.unpack4(allv, 16, True)) == [0, 1, 2, 3, 4, 5, 6, 7, -8, -7, -6, -5, -4, -3, -2, -1]
    assert [L.orc_load_int(O.S4, allv.ctypes.data, i) for i in range(16)] == list(O.unpack4(allv, 16, True))


@pytest.mark.parametrize("dt,vals,want", [
    (O.S8, [0.5, 1.5, 2.5, -0.5, -1.5, 127.4, 127.5, 300.0, -128.5, -1e9], [0, 2, 2, 0, -2, 127, 127, 127, -128, -128]),
    (O.U8, [0.5, 1.5, 2.5, -3.0, 254.5, 255.5, 1e9], [0, 2, 2, 0, 254, 255, 255]),
    (O.S32, [2.5, -2.5, 3e9, -3e9, 2147483520.0], [2, -2, 2147483520, -2147483648, 2147483520]),
])
def test_saturating_round_half_even(dt, vals, want):
    # src/cpu/simple_q10n.hpp:41-81: clamp to the type's range, then nearbyintf
    got = O.from_f32(dt, np.array(vals, dtype=np.float32))
    assert list(got.astype(np.int64)) == want


def test_eltwise_formulas():
    L = O.lib()
    xs = np.linspace(-12, 12, 97).astype(np.float32)
    RELU, TANH, ELU, SQUARE, ABS, SQRT, LINEAR, SOFT_RELU, HARDSIGMOID, LOGISTIC, EXP, GELU_TANH, SWISH, LOG, CLIP, CLIP_V2, POW, GELU_ERF, ROUND, MISH, HARDSWISH = range(0x20, 0x20 + 21)
    import math

    def close(a, b, tol=3e-6):
        return abs(a - b) <= tol * max(1.0, abs(b))

    for x in map(float, xs):
        assert L.orc_eltwise(RELU, x, 0.25, 0) == (x if x > 0 else np.float32(x) * np.float32(0.25))
        assert L.orc_eltwise(LINEAR, x, 2.0, -1.0) == np.float32(np.float32(2.0) * np.float32(x)) + np.float32(-1.0)
        assert L.orc_eltwise(CLIP, x, -1.0, 3.0) == min(max(x, -1.0), 3.0)
        assert L.orc_eltwise(CLIP_V2, x, -1.0, 3.0) == min(max(x, -1.0), 3.0)
        assert L.orc_eltwise(ROUND, x, 0, 0) == float(np.rint(np.float32(x)))
        assert L.orc_eltwise(ABS, x, 0, 0) == abs(x)
        assert L.orc_eltwise(SQUARE, x, 0, 0) == float(np.float32(x) * np.float32(x))
        assert close(L.orc_eltwise(TANH, x, 0, 0), math.tanh(x))
        assert close(L.orc_eltwise(LOGISTIC, x, 0, 0), 1 / (1 + math.exp(-x)))
        assert close(L.orc_eltwise(SWISH, x, 1.5, 0), x / (1 + math.exp(-1.5 * x)))
        assert close(L.orc_eltwise(EXP, x, 0, 0), math.exp(x), 1e-6)
        assert close(L.orc_eltwise(ELU, x, 0.5, 0), x if x > 0 else 0.5 * math.expm1(x))
        assert close(L.orc_eltwise(GELU_ERF, x, 0, 0), 0.5 * x * (1 + math.erf(x / math.sqrt(2))))
        assert close(L.orc_eltwise(GELU_TANH, x, 0, 0), 0.5 * x * (1 + math.tanh(math.sqrt(2 / math.pi) * x * (1 + 0.044715 * x * x))))
        assert close(L.orc_eltwise(SOFT_RELU, x, 2.0, 0), math.log1p(math.exp(2.0 * x)) / 2.0)
        sp = math.log1p(math.exp(x))
        assert close(L.orc_eltwise(MISH, x, 0, 0), x * math.tanh(sp))
        hs = min(max(0.2 * x + 0.5, 0.0), 1.0)
        assert close(L.orc_eltwise(HARDSIGMOID, x, 0.2, 0.5), hs)
        assert close(L.orc_eltwise(HARDSWISH, x, 0.2, 0.5), x * hs)
        if x > 0:
            assert close(L.orc_eltwise(SQRT, x, 0, 0), math.sqrt(x))
            assert close(L.orc_eltwise(LOG, x, 0, 0), math.log(x))
            assert close(L.orc_eltwise(POW, x, 0.5, 1.5), 0.5 * x**1.5, 1e-5)
    # logistic guards the exp overflow (src/common/math_utils.hpp:239-245)
    assert L.orc_eltwise(LOGISTIC, -100.0, 0, 0) == 0.0
    assert L.orc_eltwise(SWISH, -100.0, 1.0, 0) == 0.0


def test_binary_formulas():
    L = O.lib()
    ADD = 0x1FFF0
    x, y = 3.5, -2.0
    want = [x + y, x * y, max(x, y), min(x, y), x / y, x - y, x >= y, x > y, x <= y, x < y, x == y, x != y]
    for i, w in enumerate(want):
        assert L.orc_binary(ADD + i, x, y) == float(w)
