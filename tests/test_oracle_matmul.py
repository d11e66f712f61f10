"""Pins the oracle's matmul / reorder against what the mathematics fixes.

No stored golden tensors exist in the reference (its tests compute expected
values on the fly), so each check here is chosen so that a plausible mistake
(dropped zero-point, wrong group index, transposed operand, swapped scale
order, wrong broadcast) fails it:
  * exact integer dot products by brute force (numpy int64),
  * the zero-point compensation identity of
    src/cpu/matmul/gemm_x8s8s32x_matmul.cpp:165-193,
  * integer-valued data with power-of-two scales, where every intermediate is
    exactly representable so any evaluation order gives the same bits (the
    reason benchdnn can compare matmul with a zero threshold,
    tests/benchdnn/utils/compare.hpp:74),
  * pure-Python loops with hand-written index arithmetic for grouped scales
    and zero points,
  * a sequential float32 accumulation written with numpy for the float path.
"""
import numpy as np
import pytest

import oracle as O

SWISH, RELU, LINEAR = 0x2C, 0x20, 0x26
ADD, MUL = 0x1FFF0, 0x1FFF1


def T(dt, arr, strides=None, dims=None):
    arr = np.ascontiguousarray(arr)
    return O.Tensor(dt, dims if dims is not None else arr.shape, arr, strides)


def test_s32_accumulators_are_the_exact_integer_dot_product():
    rng = np.random.default_rng(0)
    M, K, N = 7, 96, 10
    src = rng.integers(0, 256, (M, K)).astype(np.uint8)
    wei = rng.integers(-128, 128, (K, N)).astype(np.int8)
    dst = np.zeros((M, N), np.int32)
    zp = np.array([131], np.int32)
    acc = O.matmul_s32_acc(T(O.U8, src), T(O.S8, wei), T(O.S32, dst),
                           zps={O.Q_SRC: O.Quant(0, O.S32, zp)})
    want = (src.astype(np.int64) - 131) @ wei.astype(np.int64)
    assert np.array_equal(acc, want)
    # compensation identity: sum((s-zp)*w) == sum(s*w) - zp*colsum(w)
    plain = O.matmul_s32_acc(T(O.U8, src), T(O.S8, wei), T(O.S32, dst))
    assert np.array_equal(acc, plain - 131 * wei.astype(np.int64).sum(0))
    # a transposed operand must not pass: strides select the layout
    wt = np.ascontiguousarray(wei.T)
    acc_t = O.matmul_s32_acc(T(O.U8, src), O.Tensor(O.S8, (K, N), wt, (1, K)), T(O.S32, dst),
                             zps={O.Q_SRC: O.Quant(0, O.S32, zp)})
    assert np.array_equal(acc_t, want)


def test_int8_exact_arithmetic_any_order():
    """Small integers and power-of-two scales: all intermediates exact."""
    rng = np.random.default_rng(1)
    B, M, K, N = 3, 5, 64, 6
    src = rng.integers(-4, 5, (B, M, K)).astype(np.int8)
    wei = rng.integers(-4, 5, (B, K, N)).astype(np.int8)
    ws = (2.0 ** rng.integers(-2, 3, N)).astype(np.float32)
    ss = np.array([0.5], np.float32)
    bias = rng.integers(-8, 9, (1, 1, N)).astype(np.float32)
    dzp = np.array([3], np.int32)
    dsc = np.array([2.0], np.float32)
    dst = np.zeros((B, M, N), np.int8)
    O.matmul(T(O.S8, src), T(O.S8, wei), T(O.S8, dst), bias=T(O.F32, bias),
             scales={O.Q_SRC: O.Quant(0, O.F32, ss), O.Q_WEI: O.Quant(1 << 2, O.F32, ws),
                     O.Q_DST: O.Quant(0, O.F32, dsc)},
             zps={O.Q_DST: O.Quant(0, O.S32, dzp)},
             post_ops=[{"kind": "eltwise", "alg": RELU, "alpha": 0.0}])
    acc = np.einsum("bmk,bkn->bmn", src.astype(np.float64), wei.astype(np.float64))
    want = np.maximum(acc * 0.5 * ws + bias, 0) / 2.0 + 3
    want = np.clip(np.rint(want), -128, 127).astype(np.int8)
    assert np.array_equal(dst, want)


def _py_int8_reference(src, wei, ss, ws, sz, wz, gs, gw, gsz, gwz):
    """Pure-Python int8 matmul with K-grouped src/wei scales and zero points.
    Layouts: src quant [M, K/g], wei quant [K/g, N] (row-major)."""
    M, K = src.shape
    N = wei.shape[1]
    gk = min(gs, gw, gsz, gwz)
    out = np.zeros((M, N), np.float32)
    for m in range(M):
        for n in range(N):
            d = np.float32(0)
            for g in range(K // gk):
                acc = 0
                for k in range(g * gk, (g + 1) * gk):
                    s = int(src[m, k]) - int(sz[m, k // gsz])
                    w = int(wei[k, n]) - int(wz[k // gwz, n])
                    acc += s * w
                k_last = (g + 1) * gk - 1
                a = np.float32(acc)
                a = a * ss[m, k_last // gs]
                a = a * ws[k_last // gw, n]
                d = d + a
            out[m, n] = d
    return out


def test_int8_grouped_scales_and_zero_points_indexing():
    rng = np.random.default_rng(2)
    M, K, N = 4, 128, 6
    gs, gw, gsz, gwz = 64, 32, 128, 64
    src = rng.integers(-128, 128, (M, K)).astype(np.int8)
    wei = rng.integers(-128, 128, (K, N)).astype(np.int8)
    ss = rng.uniform(0.01, 0.1, (M, K // gs)).astype(np.float32)
    ws = rng.uniform(0.01, 0.1, (K // gw, N)).astype(np.float32)
    sz = rng.integers(-5, 6, (M, K // gsz)).astype(np.int32)
    wz = rng.integers(-5, 6, (K // gwz, N)).astype(np.int8)
    dst = np.zeros((M, N), np.float32)
    O.matmul(T(O.S8, src), T(O.S8, wei), T(O.F32, dst),
             scales={O.Q_SRC: O.Quant(3, O.F32, ss, (1, gs)), O.Q_WEI: O.Quant(3, O.F32, ws, (gw, 1))},
             zps={O.Q_SRC: O.Quant(3, O.S32, sz, (1, gsz)), O.Q_WEI: O.Quant(3, O.S8, wz, (gwz, 1))})
    want = _py_int8_reference(src, wei, ss, ws, sz, wz, gs, gw, gsz, gwz)
    assert np.array_equal(dst.view(np.uint32), want.view(np.uint32))


def test_int8_scale_order_is_src_then_weights():
    """((float)acc * s_src) * s_wei, not acc * (s_src * s_wei):
    src/cpu/matmul/ref_matmul_int8.cpp:195-218."""
    rng = np.random.default_rng(3)
    M, K, N = 64, 256, 64
    src = rng.integers(-127, 128, (M, K)).astype(np.int8)
    wei = rng.integers(-127, 128, (K, N)).astype(np.int8)
    ss = rng.uniform(0.005, 0.05, (M, 1)).astype(np.float32)
    ws = rng.uniform(0.0005, 0.005, N).astype(np.float32)
    dst = np.zeros((M, N), np.float32)
    O.matmul(T(O.S8, src), T(O.S8, wei), T(O.F32, dst),
             scales={O.Q_SRC: O.Quant(3, O.F32, ss, (1, K)), O.Q_WEI: O.Quant(2, O.F32, ws)})
    acc = (src.astype(np.int64) @ wei.astype(np.int64)).astype(np.float32)
    want = (acc * ss) * ws[None, :]
    other = acc * (ss * ws[None, :])
    assert np.array_equal(dst.view(np.uint32), want.view(np.uint32))
    assert not np.array_equal(want.view(np.uint32), other.view(np.uint32))


def test_int8_literal_k_grouping_sums_in_f32_one_k_at_a_time():
    """As written, v3.8 closes the K group after every k when an entry carries no
    explicit groups (src/cpu/matmul/ref_matmul_int8.cpp:139-144 with
    src/common/primitive_attr_quant.hpp:83-90): d = sum_k f32(s*w)*ss*ws in f32."""
    rng = np.random.default_rng(33)
    M, K, N = 5, 200, 6
    src = rng.integers(0, 256, (M, K)).astype(np.uint8)
    wei = rng.integers(-128, 128, (K, N)).astype(np.int8)
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    ss = np.array([0.02], np.float32)
    zp = np.array([128], np.int32)
    dst = np.zeros((M, N), np.float32)
    args = dict(scales={O.Q_SRC: O.Quant(0, O.F32, ss), O.Q_WEI: O.Quant(2, O.F32, ws)},
                zps={O.Q_SRC: O.Quant(0, O.S32, zp)})
    O.matmul(T(O.U8, src), T(O.S8, wei), T(O.F32, dst), k_group_mode=O.KGROUP_LITERAL, **args)
    d = np.zeros((M, N), np.float32)
    for k in range(K):
        prod = ((src[:, k].astype(np.int32) - 128)[:, None] * wei[k].astype(np.int32)[None, :]).astype(np.float32)
        d = d + (prod * ss[0]) * ws[None, :]
    assert np.array_equal(dst.view(np.uint32), d.view(np.uint32))
    # the whole-K integer accumulation differs only by f32 summation error
    dst2 = np.zeros((M, N), np.float32)
    O.matmul(T(O.U8, src), T(O.S8, wei), T(O.F32, dst2), **args)
    acc = ((src.astype(np.int64) - 128) @ wei.astype(np.int64)).astype(np.float32)
    assert np.array_equal(dst2.view(np.uint32), ((acc * ss[0]) * ws[None, :]).view(np.uint32))
    scale = (np.abs(src.astype(np.float64) - 128) @ np.abs(wei.astype(np.float64))) * 0.02 * ws[None, :]
    assert np.max(np.abs(dst - dst2) / scale) < 1e-6
    assert not np.array_equal(dst, dst2)


def test_int8_accumulator_rounds_to_f32_above_2_pow_24():
    K = 4096
    src = np.full((1, K), 127, np.int8)
    wei = np.full((K, 2), 127, np.int8)
    wei[0, 1] = 126  # 66064383 is not representable in f32
    dst = np.zeros((1, 2), np.float32)
    O.matmul(T(O.S8, src), T(O.S8, wei), T(O.F32, dst))
    assert dst[0, 0] == np.float32(127 * 127 * K)
    assert 127 * 127 * K - 127 == 66064257 and int(dst[0, 1]) == 66064256  # f32 spacing is 4 there


def _bf16(a):
    return O.from_f32(O.BF16, np.asarray(a, np.float32))


def test_weights_decompression_sequential_f32():
    """bf16 x u4 with group-K f16 scales and u4 zero points, f32 accumulate in k
    order: src/cpu/matmul/ref_matmul.cpp:140-173."""
    rng = np.random.default_rng(4)
    M, K, N, G = 3, 256, 16, 128
    a = rng.standard_normal((M, K)).astype(np.float32)
    a_bf = _bf16(a)
    a = O.to_f32(O.BF16, a_bf)
    w = rng.integers(0, 16, (K, N))
    sc = O.from_f32(O.F16, rng.uniform(0.005, 0.02, (K // G, N)).astype(np.float32))
    zp = rng.integers(6, 10, (K // G, N))
    dst = np.zeros((M, N), np.uint16)
    O.matmul(T(O.BF16, a_bf), O.Tensor(O.U4, (K, N), O.pack4(w)), T(O.BF16, dst),
             scales={O.Q_WEI: O.Quant(3, O.F16, sc, (G, 1))},
             zps={O.Q_WEI: O.Quant(3, O.U4, O.pack4(zp), (G, 1))}, apply_to_int=True)
    scf = sc.view(np.float16).astype(np.float32)
    acc = np.zeros((M, N), np.float32)
    for k in range(K):
        wk = (w[k].astype(np.float32) - zp[k // G].astype(np.float32)) * scf[k // G]
        acc = acc + a[:, k, None] * wk[None, :]
    assert np.array_equal(dst, _bf16(acc))
    # dropping the zero point or using the wrong group must change the answer
    acc2 = a @ ((w - 8) * scf.repeat(G, 0)).astype(np.float32)
    assert not np.array_equal(dst, _bf16(acc2))


def test_fp8_path_and_sum_post_op():
    rng = np.random.default_rng(5)
    M, K, N = 8, 64, 8
    a8 = O.from_f32(O.F8_E4M3, np.clip(rng.standard_normal((M, K)) * 4, -448, 448).astype(np.float32))
    b8 = O.from_f32(O.F8_E4M3, np.clip(rng.standard_normal((K, N)) * 4, -448, 448).astype(np.float32))
    old = _bf16(rng.standard_normal((M, N)))
    dst = old.copy()
    O.matmul(T(O.F8_E4M3, a8), T(O.F8_E4M3, b8), T(O.BF16, dst),
             scales={O.Q_SRC: O.Quant(0, O.F32, np.array([0.5], np.float32)),
                     O.Q_WEI: O.Quant(0, O.F32, np.array([0.25], np.float32))},
             post_ops=[{"kind": "sum", "scale": 1.0}])
    a, b = O.to_f32(O.F8_E4M3, a8), O.to_f32(O.F8_E4M3, b8)
    acc = np.zeros((M, N), np.float32)
    for k in range(K):
        acc = acc + a[:, k, None] * b[None, k, :]
    want = (acc * np.float32(0.5)) * np.float32(0.25) + O.to_f32(O.BF16, old)
    assert np.array_equal(dst, _bf16(want))


@pytest.mark.parametrize("dst_dt,sum_dt,zp,scale", [
    ("u8", "s8", 5, 0.5), ("s8", "u8", -3, 0.75), ("u8", "s8", -128, 1.0), ("s8", None, 7, 0.5),
    ("s32", None, 11, 2.0), ("f32", None, 9, 0.25)])
def test_sum_post_op_zero_point_and_data_type(dst_dt, sum_dt, zp, scale):
    """src/cpu/primitive_attr_postops.cpp:286-293: res += scale * (dst_val - float(zero_point)), where dst_val is the
    old destination element read through the sum's own data type when it has one
    (src/common/primitive_attr.hpp:448-455, src/cpu/matmul/ref_matmul_int8.cpp:231,246). Written here with numpy
    float32 steps on the raw bytes: reading the old bytes in the destination's signedness, dropping the zero point or
    flipping its sign each changes the expected bytes."""
    rng = np.random.default_rng(11)
    M, K, N = 6, 48, 9
    np_of = {"u8": np.uint8, "s8": np.int8, "s32": np.int32, "f32": np.float32}
    src = rng.integers(-6, 7, (M, K)).astype(np.int8)
    wei = rng.integers(-6, 7, (K, N)).astype(np.int8)
    if dst_dt in ("u8", "s8"):
        old_bytes = rng.integers(0, 256, (M, N)).astype(np.uint8)      # both halves of the byte range
        old = old_bytes.view(np_of[dst_dt])
    elif dst_dt == "s32":
        old = rng.integers(-300, 300, (M, N)).astype(np.int32)
    else:
        old = rng.integers(-300, 300, (M, N)).astype(np.float32)
    dst = old.copy()
    ws = np.float32(0.125)
    po = {"kind": "sum", "scale": scale, "zero_point": zp}
    if sum_dt:
        po["dt"] = O.DT_NAMES[sum_dt]
    O.matmul(T(O.S8, src), T(O.S8, wei), T(O.DT_NAMES[dst_dt], dst),
             scales={O.Q_WEI: O.Quant(0, O.F32, np.array([ws], np.float32))}, post_ops=[po])
    acc = (src.astype(np.int64) @ wei.astype(np.int64)).astype(np.float32)
    res = acc * ws
    seen = old.view(np_of[sum_dt]) if sum_dt else old                  # same bytes, the sum's own type
    res = res + np.float32(scale) * (seen.astype(np.float32) - np.float32(zp))
    if dst_dt == "f32":
        want = res
    else:
        info = np.iinfo(np_of[dst_dt])
        want = np.rint(np.clip(res, np.float32(info.min), np.float32(info.max))).astype(np_of[dst_dt])
    assert np.array_equal(dst, want)
    if sum_dt:      # the two readings of the old bytes must differ on this data, or the case pins nothing
        other = res - np.float32(scale) * seen.astype(np.float32) + np.float32(scale) * old.astype(np.float32)
        assert not np.array_equal(other, res)
    assert zp != 0


def test_float_path_sum_reads_old_dst_in_its_own_type():
    """src/cpu/matmul/ref_matmul.cpp:190,215: the float path reads the old destination through get_sum_dt too. With a
    bf16 destination and an f16 sum type the same 16 bits are another number."""
    rng = np.random.default_rng(12)
    M, K, N = 4, 16, 6
    a = rng.integers(-3, 4, (M, K)).astype(np.float32)
    b = rng.integers(-3, 4, (K, N)).astype(np.float32)
    old = rng.integers(0x3000, 0x4800, (M, N)).astype(np.uint16)       # positive, normal in both formats
    dst = old.copy()
    O.matmul(T(O.F32, a), T(O.F32, b), T(O.BF16, dst), post_ops=[{"kind": "sum", "scale": 2.0, "dt": O.F16}])
    want = (a.astype(np.float64) @ b.astype(np.float64)).astype(np.float32) \
        + np.float32(2.0) * old.view(np.float16).astype(np.float32)
    assert np.array_equal(dst, _bf16(want))
    assert not np.array_equal(old.view(np.float16).astype(np.float32), O.to_f32(O.BF16, old))


def test_binary_post_op_broadcast_and_batch():
    rng = np.random.default_rng(6)
    B, M, K, N = 4, 6, 32, 5
    q = rng.integers(-127, 128, (B, M, K)).astype(np.int8)
    kt = rng.integers(-127, 128, (B, N, K)).astype(np.int8)  # stored as K^T: acb view
    mask = np.where(np.arange(N)[None, :] > np.arange(M)[:, None], -1e4, 0).astype(np.float32)[None]
    dst = np.zeros((B, M, N), np.float32)
    wei = O.Tensor(O.S8, (B, K, N), kt, (N * K, 1, K))
    O.matmul(T(O.S8, q), wei, T(O.F32, dst),
             scales={O.Q_SRC: O.Quant(0, O.F32, np.array([0.01], np.float32)),
                     O.Q_WEI: O.Quant(0, O.F32, np.array([0.012], np.float32))},
             post_ops=[{"kind": "binary", "alg": ADD, "src1": T(O.F32, mask)}])
    acc = np.einsum("bmk,bnk->bmn", q.astype(np.int64), kt.astype(np.int64)).astype(np.float32)
    want = (acc * np.float32(0.01)) * np.float32(0.012) + mask
    assert np.array_equal(dst.view(np.uint32), want.view(np.uint32))
    # batch broadcast of the weights (dims 1 on the batch axis)
    dst2 = np.zeros((B, M, N), np.float32)
    O.matmul(T(O.S8, q), O.Tensor(O.S8, (1, K, N), kt[:1], (N * K, 1, K)), T(O.F32, dst2))
    want2 = np.einsum("bmk,nk->bmn", q.astype(np.int64), kt[0].astype(np.int64)).astype(np.float32)
    assert np.array_equal(dst2, want2)


def test_post_op_chain_order_bias_and_prelu():
    rng = np.random.default_rng(7)
    M, K, N = 5, 32, 7
    src = rng.integers(-8, 9, (M, K)).astype(np.int8)
    wei = rng.integers(-8, 9, (K, N)).astype(np.int8)
    bias = rng.integers(-4, 5, (1, N)).astype(np.int32)
    col = rng.integers(1, 4, (1, N)).astype(np.float32)
    pw = (2.0 ** rng.integers(-2, 2, N)).astype(np.float32)
    old = rng.integers(-10, 10, (M, N)).astype(np.float32)
    dst = old.copy()
    O.matmul(T(O.S8, src), T(O.S8, wei), T(O.F32, dst), bias=T(O.S32, bias),
             post_ops=[{"kind": "binary", "alg": MUL, "src1": T(O.F32, col)},
                       {"kind": "sum", "scale": 0.5},
                       {"kind": "prelu", "mask": 2, "weights": pw},
                       {"kind": "eltwise", "alg": LINEAR, "alpha": 2.0, "beta": 1.0, "scale": 0.25}])
    acc = (src.astype(np.int64) @ wei.astype(np.int64)).astype(np.float64)
    v = (acc + bias) * col + 0.5 * old
    v = np.where(v < 0, v * pw[None, :], v)
    v = (2.0 * v + 1.0) * 0.25
    assert np.array_equal(dst, v.astype(np.float32))


@pytest.mark.parametrize("mask", [0, 1, 2, 4, 3, 5, 6, 7])
def test_prelu_weights_layout_3d(mask):
    # src/cpu/primitive_attr_postops.cpp:190-225: the weights tensor has dst's
    # dims where the mask bit is set and 1 elsewhere, in the layout acb for a
    # 3-D dst (the N axis is the *outer* of the two matrix axes), ab for 2-D.
    rng = np.random.default_rng(40 + mask)
    B, M, K, N = 3, 4, 16, 5
    src = rng.integers(-8, 9, (B, M, K)).astype(np.int8)
    wei = rng.integers(-8, 9, (B, K, N)).astype(np.int8)
    wd = [B if mask & 1 else 1, M if mask & 2 else 1, N if mask & 4 else 1]
    # physical order a, c, b
    phys = (2.0 ** rng.integers(-3, 3, (wd[0], wd[2], wd[1]))).astype(np.float32)
    dst = np.zeros((B, M, N), np.float32)
    O.matmul(T(O.S8, src), T(O.S8, wei), T(O.F32, dst),
             post_ops=[{"kind": "prelu", "mask": mask, "weights": phys.reshape(-1)}])
    acc = np.einsum("bmk,bkn->bmn", src.astype(np.int64), wei.astype(np.int64)).astype(np.float32)
    logical = np.broadcast_to(phys.transpose(0, 2, 1), (B, M, N))
    want = np.where(acc >= 0, acc, acc * logical)
    assert np.array_equal(dst, want)


def test_zero_dim_is_a_no_op():
    dst = np.full((0, 4), 7, np.float32)
    O.matmul(T(O.S8, np.zeros((0, 8), np.int8)), T(O.S8, np.zeros((8, 4), np.int8)), T(O.F32, dst, dims=(0, 4)))
    dst = np.full((3, 4), 7, np.float32)
    O.matmul(O.Tensor(O.S8, (3, 0), np.zeros(1, np.int8)), O.Tensor(O.S8, (0, 4), np.zeros(1, np.int8)), T(O.F32, dst))
    assert np.all(dst == 7)  # src/cpu/matmul/ref_matmul_int8.cpp:64-66


def test_reorder_quantize_and_transpose():
    rng = np.random.default_rng(8)
    K, N = 64, 12
    w = (rng.standard_normal((K, N)) * 3).astype(np.float32)
    sc = (2.0 ** rng.integers(-3, 0, N)).astype(np.float32)
    out = np.zeros((N, K), np.int8)  # ba layout of a [K, N] tensor
    O.reorder(T(O.F32, w), O.Tensor(O.S8, (K, N), out, (1, K)),
              dst_scale=O.Quant(2, O.F32, sc))
    want = np.clip(np.rint(w / sc[None, :]), -128, 127).astype(np.int8)
    assert np.array_equal(out.T, want)
    # u4 <- s8 pure conversion keeps nibble order
    v = rng.integers(0, 16, (K, N)).astype(np.int8)
    out4 = np.zeros(K * N // 2, np.uint8)
    O.reorder(T(O.S8, v), O.Tensor(O.U4, (K, N), out4))
    assert np.array_equal(out4, O.pack4(v))


def test_reorder_every_quantization_entry_against_numpy_float32():
    """d = src_scale * (in - src_zp); d = d * (1 / dst_scale) + dst_zp; saturating round-to-nearest-even store
    (src/cpu/reorder/simple_reorder.hpp:2500-2640), with scales that are not powers of two, so that every float32
    rounding step counts. numpy float32 arithmetic performs the same single IEEE operations step by step; a dropped
    step, a division where the reference multiplies by the reciprocal, a swapped scale or a wrong group index changes
    bits here."""
    rng = np.random.default_rng(18)
    R, Ccols, G = 24, 64, 32
    # s8 source with per-row-and-column-group scales and zero points (groups along the last dim)
    src = rng.integers(-128, 128, (R, Ccols)).astype(np.int8)
    ss = rng.uniform(0.01, 0.3, (R, Ccols // G)).astype(np.float32)
    sz = rng.integers(-5, 6, (R, Ccols // G)).astype(np.int32)
    ds = np.array([0.037], np.float32)
    dz = np.array([3], np.int32)
    for dst_code, lo, hi, store in ((O.S8, -128, 127, np.int8), (O.U8, 0, 255, np.uint8)):
        out = np.zeros((R, Ccols), store)
        O.reorder(T(O.S8, src), T(dst_code, out), src_scale=O.Quant(3, O.F32, ss, (1, G)),
                  src_zp=O.Quant(3, O.S32, sz, (1, G)), dst_scale=O.Quant(0, O.F32, ds), dst_zp=O.Quant(0, O.S32, dz))
        s_full = np.repeat(ss, G, axis=1)
        z_full = np.repeat(sz, G, axis=1).astype(np.float32)
        d = s_full * (src.astype(np.float32) - z_full)                # one multiply, one subtract, both float32
        d = d * (np.float32(1.0) / ds[0]) + np.float32(dz[0])         # reciprocal first, then multiply, then add
        want = np.clip(np.rint(d), lo, hi).astype(store)
        assert np.array_equal(out, want)
    # the same entries into an f32 destination: every bit of the float32 chain is visible, and the variant that
    # divides by the destination scale instead of multiplying by its reciprocal differs on this data
    outf = np.zeros((R, Ccols), np.float32)
    O.reorder(T(O.S8, src), T(O.F32, outf), src_scale=O.Quant(3, O.F32, ss, (1, G)),
              src_zp=O.Quant(3, O.S32, sz, (1, G)), dst_scale=O.Quant(0, O.F32, ds))
    base = s_full * (src.astype(np.float32) - z_full)
    assert np.array_equal(outf.view(np.uint32), (base * (np.float32(1.0) / ds[0])).view(np.uint32))
    assert not np.array_equal(outf.view(np.uint32), (base / ds[0]).view(np.uint32))
    # f32 -> bf16 / f16 with a per-column destination scale: numpy / torch conversions as the independent rounding
    import torch
    x = (rng.standard_normal((R, Ccols)) * 5).astype(np.float32)
    dsc = rng.uniform(0.3, 3.0, Ccols).astype(np.float32)
    scaled = x * (np.float32(1.0) / dsc)[None, :]
    out16 = np.zeros((R, Ccols), np.uint16)
    O.reorder(T(O.F32, x), T(O.F16, out16), dst_scale=O.Quant(2, O.F32, dsc))
    assert np.array_equal(out16, scaled.astype(np.float16).view(np.uint16))
    outb = np.zeros((R, Ccols), np.uint16)
    O.reorder(T(O.F32, x), T(O.BF16, outb), dst_scale=O.Quant(2, O.F32, dsc))
    assert np.array_equal(outb, torch.from_numpy(scaled).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16))


@pytest.mark.parametrize("src_dt", ["s8", "u8"])
@pytest.mark.parametrize("M,K,N,gk,wei_t", [(5, 100, 7, None, False), (9, 256, 33, 64, False), (3, 4096, 20, 128, True),
                                            (4, 16, 5, None, False), (2, 191, 3, None, True), (6, 512, 65, 32, False)])
def test_byte_dot_product_instruction_gives_the_scalar_loops_bits(monkeypatch, src_dt, M, K, N, gk, wei_t):
    """The integer path forms a K group's sum of products 64 at a time where the host has AVX-512 VNNI (u8 x s8 dot
    products; an s8 source enters as s + 128 and 128 x the column's sum leaves again). Integer sums wrap the same in any
    order: the destination (f32 with scales per row and per group and column, a swish behind them) and the raw s32
    accumulators must be the scalar loop's bit for bit. Extreme values included (-128 x -128 four times in a row is the
    instruction's largest intermediate sum)."""
    rng = np.random.default_rng(M * 1000 + K + N)
    if src_dt == "s8":
        src = rng.integers(-128, 128, (M, K)).astype(np.int8)
        src[0, :8] = -128
        sdt = O.S8
    else:
        src = rng.integers(0, 256, (M, K)).astype(np.uint8)
        src[0, :8] = 255
        sdt = O.U8
    wei = rng.integers(-128, 128, (K, N)).astype(np.int8)
    wei[:8, 0] = -128
    wt = O.Tensor(O.S8, [K, N], np.ascontiguousarray(wei.T), [1, K]) if wei_t else T(O.S8, wei)
    if gk:
        scales = {O.Q_SRC: O.Quant(3, O.F32, rng.uniform(0.01, 0.1, (M, K // gk)).astype(np.float32), (1, gk)),
                  O.Q_WEI: O.Quant(3, O.F32, rng.uniform(0.01, 0.1, (K // gk, N)).astype(np.float32), (gk, 1))}
    else:
        scales = {O.Q_SRC: O.Quant(1, O.F32, rng.uniform(0.01, 0.1, M).astype(np.float32)),
                  O.Q_WEI: O.Quant(2, O.F32, rng.uniform(0.01, 0.1, N).astype(np.float32))}
    out = {}
    for mode in ("1", "0"):
        monkeypatch.setenv("QMM_ORACLE_SCALAR", mode)
        dst = np.zeros((M, N), np.float32)
        O.matmul(T(sdt, src), wt, T(O.F32, dst), scales=scales)
        acc = O.matmul_s32_acc(T(sdt, src), wt, T(O.S32, np.zeros((M, N), np.int32)))
        out[mode] = (dst.view(np.uint32).copy(), acc.copy())
    assert np.array_equal(out["0"][0], out["1"][0])
    assert np.array_equal(out["0"][1], out["1"][1])
    # and both are the integer product itself
    exact = src.astype(np.int64) @ wei.astype(np.int64)
    assert np.array_equal(out["0"][1].astype(np.int64), exact)
