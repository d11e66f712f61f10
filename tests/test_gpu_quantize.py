"""GPU parity of the row-wise quantizing reorder (hip:gfx950:quantize) against
the CPU oracle's reorder, bit for bit: the kernel performs the reference's
operations in the reference's order (src/cpu/reorder/simple_reorder.hpp:2500-2640)."""
import sys

import numpy as np
import pytest

import onednn_amd as dnnl
import oracle as O
from onednn_amd import memory
from qmm_harness import T, TensorSpec, assert_bit_exact, dt

pytestmark = pytest.mark.gpu

QUANTIZE, REORDER = "hip:gfx950:quantize", "hip:gfx950:reorder"


def say(msg):
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def ctx():
    eng = dnnl.engine(dnnl.engine.kind.gpu, 0)
    return eng, dnnl.stream(eng)


def _raw(code, values):
    v = np.asarray(values).reshape(-1)
    if code in (dt.s32, dt.s8, dt.u8):
        return v.astype(O.STORAGE[code])
    return O.from_f32(code, v.astype(np.float32))


def run_case(eng, strm, src_dt, dst_dt, dims, seed, src_scale=None, dst_scale=None, src_zp=None, dst_zp=None,
             layout=None, dst_layout=None, expect=QUANTIZE, amp=3.0, src_values=None):
    """Each of *_scale / src_zp: (mask, dt, groups or None, values); dst_zp: int."""
    r = np.random.default_rng(seed)
    x = (r.standard_normal(dims) * amp).astype(np.float32) if src_values is None else src_values
    src = TensorSpec(src_dt, list(dims), layout, x)
    dst = TensorSpec(dst_dt, list(dims), dst_layout or layout)
    attr = dnnl.primitive_attr()
    quants, args = {}, {}
    for name, arg, q, zp in (("src_scale", dnnl.DNNL_ARG_SRC, src_scale, False), ("dst_scale", dnnl.DNNL_ARG_DST, dst_scale, False),
                             ("src_zp", dnnl.DNNL_ARG_SRC, src_zp, True)):
        if q is None:
            continue
        mask, code, groups, values = q
        raw = _raw(code, values)
        if zp:
            attr.set_zero_points(arg, mask, list(groups or []), code)
            key = dnnl.DNNL_ARG_ATTR_ZERO_POINTS | arg
        else:
            attr.set_scales(arg, mask, list(groups or []), code)
            key = dnnl.DNNL_ARG_ATTR_SCALES | arg
        quants[name] = O.Quant(mask, code, raw, groups)
        args[key] = memory(memory.desc([raw.nbytes], dt.u8, T("a")), eng).write(raw)
    if dst_zp is not None:
        attr.set_zero_points_mask(dnnl.DNNL_ARG_DST, 0)
        raw = np.array([dst_zp], np.int32)
        quants["dst_zp"] = O.Quant(0, dt.s32, raw)
        args[dnnl.DNNL_ARG_ATTR_ZERO_POINTS | dnnl.DNNL_ARG_DST] = memory(memory.desc([1], dt.s32, T("a")), eng).write(raw)
    pd = dnnl.reorder.primitive_desc(eng, src.md(), eng, dst.md(), attr=attr)
    assert pd.impl_info_str() == expect, pd.impl_info_str()
    s_mem = memory(src.md(), eng).write(src.raw)
    d_mem = memory(dst.md(), eng).write(dst.raw)
    args[dnnl.DNNL_ARG_FROM], args[dnnl.DNNL_ARG_TO] = s_mem, d_mem
    dnnl.reorder(pd).execute(strm, args)
    strm.wait()
    want = dst.raw.copy()
    O.reorder(src.oracle(), dst.oracle(want), **quants)
    assert_bit_exact(d_mem.read(dst.raw.dtype), want, "%s -> %s %s" % (src_dt, dst_dt, dims))


def test_weights_f32_to_s8_per_column(ctx):
    eng, strm = ctx
    say("quantize f32 -> s8, per-column scales")
    N = 200
    run_case(eng, strm, dt.f32, dt.s8, (96, N), 1, dst_scale=(2, dt.f32, None, np.random.default_rng(2).uniform(0.01, 0.1, N)))


def test_activations_bf16_to_s8_per_row_and_to_u8_with_zero_point(ctx):
    eng, strm = ctx
    say("quantize bf16 -> s8 per-row scales; f16 -> u8 with dst zero point")
    M = 70
    run_case(eng, strm, dt.bf16, dt.s8, (M, 256), 3, dst_scale=(1, dt.f32, None, np.random.default_rng(4).uniform(0.02, 0.05, M)))
    run_case(eng, strm, dt.f16, dt.u8, (M, 64), 5, dst_scale=(0, dt.f32, None, [0.04]), dst_zp=128)


@pytest.mark.parametrize("src_dt", [dt.f32, dt.bf16, dt.f16], ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("dims,scale,zp,dst_dt", [
    ((1, 8), "row", None, dt.s8), ((5, 24), "one", 3, dt.u8), ((300, 40), "row", None, dt.u8),
    ((37, 4104), "row", -7, dt.s8), ((129, 4096), "none", None, dt.s8), ((2, 9, 520), "one", None, dt.s8),
    ((1000, 16), "row", 100, dt.u8), ((3, 12296), "row", None, dt.s8),
    ((97, 200), "col", None, dt.s8), ((13, 4104), "col", -3, dt.s8), ((3, 21, 64), "col", 9, dt.u8),
    ((2050, 8), "col", None, dt.u8),
], ids=str)
def test_activation_quantizer_shapes(ctx, src_dt, dims, scale, zp, dst_dt):
    """The specialised 8-bit kernels (one dst scale for the tensor, per row or per column, dst zero point): rows and
    columns that do not fill their workgroups, a thread's second chunk past the row's end, row blocks past the last
    row, values that saturate, a NaN."""
    eng, strm = ctx
    say("activation quantizer %s -> %s %s scale=%s zp=%s" % (src_dt, dst_dt, dims, scale, zp))
    r = np.random.default_rng(sum(dims) + src_dt)
    x = (r.standard_normal(dims) * 40).astype(np.float32)
    x.reshape(-1)[::97] *= 50  # saturating values
    x.reshape(-1)[5 % x.size] = np.nan
    rows = int(np.prod(dims[:-1]))
    ds = None
    if scale == "row" and len(dims) == 2:
        ds = (1, dt.f32, None, r.uniform(0.2, 0.9, rows))
    elif scale == "col":
        ds = (1 << (len(dims) - 1), dt.f32, None, r.uniform(0.2, 0.9, dims[-1]))
    elif scale != "none":
        ds = (0, dt.f32, None, [0.37])
    run_case(eng, strm, src_dt, dst_dt, dims, 0, dst_scale=ds, dst_zp=zp, src_values=x)


def test_grouped_source_scales(ctx):
    """Groups are a source-side attribute in the reference (src/common/reorder.cpp:121-143)."""
    eng, strm = ctx
    say("f32 -> s8 with f16 source scales per row and 128 columns; per 64 rows and column")
    M, K, G = 33, 512, 128
    sc = np.random.default_rng(6).uniform(2.0, 6.0, (M, K // G))
    run_case(eng, strm, dt.f32, dt.s8, (M, K), 7, src_scale=(3, dt.f16, (1, G), sc))
    sc = np.random.default_rng(60).uniform(2.0, 6.0, (256 // 64, 48))
    run_case(eng, strm, dt.bf16, dt.s8, (256, 48), 70, src_scale=(3, dt.f32, (64, 1), sc), dst_scale=(0, dt.f32, None, [0.5]))


def test_weights_to_int4(ctx):
    eng, strm = ctx
    say("quantize f32 -> u4 / s4, per-column scales, dst zero point")
    K, N = 256, 48
    sc = np.random.default_rng(8).uniform(0.3, 0.6, N)
    run_case(eng, strm, dt.f32, dt.u4, (K, N), 9, dst_scale=(2, dt.f32, None, sc), dst_zp=8)
    run_case(eng, strm, dt.bf16, dt.s4, (K, N), 10, dst_scale=(2, dt.bf16, None, sc))


def test_to_fp8_and_float_types_with_both_scales(ctx):
    eng, strm = ctx
    say("f32 -> f8_e4m3 / f8_e5m2 / bf16 / f16 / f32 with src and dst scales")
    # (zero points go with integral types only: src/common/reorder.cpp:98-106)
    for code in (dt.f8_e4m3, dt.f8_e5m2, dt.bf16, dt.f16, dt.f32):
        run_case(eng, strm, dt.f32, code, (40, 72), 11 + code, src_scale=(0, dt.f32, None, [0.37]),
                 dst_scale=(2, dt.f32, None, np.random.default_rng(12).uniform(0.5, 2, 72)))


def test_three_dims_last_dim_scales(ctx):
    eng, strm = ctx
    say("quantize f16 [3, 20, 64] -> s8, scales over the last dim")
    run_case(eng, strm, dt.f16, dt.s8, (3, 20, 64), 13, dst_scale=(4, dt.f32, None, np.random.default_rng(14).uniform(0.02, 0.05, 64)))


def test_other_shapes_stay_with_the_general_reorder(ctx):
    eng, strm = ctx
    say("ragged rows, permutations of three dims and integer sources take the per-element kernel")
    N = 24
    sc = (2, dt.f32, None, np.random.default_rng(15).uniform(0.01, 0.1, N))
    run_case(eng, strm, dt.f32, dt.s8, (4, 16, N), 16, dst_scale=(4, dt.f32, None, sc[3]), layout="abc", dst_layout="acb",
             expect=REORDER)
    run_case(eng, strm, dt.f32, dt.s8, (64, 20), 17, dst_scale=(0, dt.f32, None, [0.05]), expect=REORDER)
    run_case(eng, strm, dt.f32, dt.s8, (3, 8, 16), 18, dst_scale=(1, dt.f32, None, [0.05, 0.07, 0.09]), expect=REORDER)


def test_dequantize_int4_and_int8_weights_with_grouped_scales_and_zero_points(ctx):
    """The decompression direction (src/cpu/reorder/simple_reorder.hpp:2240-2400,
    :2560-2640): dst = scale[k / g, n] * (w[k, n] - zp[k / g, n]), scale and zero
    point each with its own groups and type."""
    eng, strm = ctx
    say("u4 / s4 / s8 -> f32 / bf16 / f16 with grouped source scales and zero points")
    K, N = 256, 48
    r = np.random.default_rng(80)
    w = r.integers(0, 16, (K, N))
    for out in (dt.f32, dt.bf16, dt.f16):
        run_case(eng, strm, dt.u4, out, (K, N), 81, expect=REORDER, src_values=w,
                 src_scale=(3, dt.f16, (64, 1), r.uniform(0.01, 0.1, (K // 64, N))),
                 src_zp=(3, dt.u4, (64, 1), r.integers(5, 11, (K // 64, N))))
    run_case(eng, strm, dt.s4, dt.f32, (K, N), 82, expect=REORDER, src_values=r.integers(-8, 8, (K, N)),
             src_scale=(3, dt.bf16, (32, 1), r.uniform(0.01, 0.1, (K // 32, N))),
             src_zp=(3, dt.s8, (128, 1), r.integers(-3, 4, (K // 128, N))))
    run_case(eng, strm, dt.s8, dt.f32, (K, N), 83, expect=REORDER, src_values=r.integers(-128, 128, (K, N)),
             src_scale=(2, dt.f32, None, r.uniform(0.01, 0.1, N)), src_zp=(0, dt.s32, None, [3]))
    # groups along the last dim (activations quantized per row and 64 columns)
    run_case(eng, strm, dt.s8, dt.bf16, (40, K), 84, expect=REORDER, src_values=r.integers(-128, 128, (40, K)),
             src_scale=(3, dt.f32, (1, 64), r.uniform(0.01, 0.1, (40, K // 64))))


TRANSPOSE = "hip:gfx950:quantize_transpose"


@pytest.mark.parametrize("src_dt", [dt.f32, dt.bf16, dt.f16], ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("dims,src_layout,dst_dt,scale,zp", [
    # weights stored [N, K] (column-major as a [K, N] tensor) quantized into row-major [K, N], one scale per column
    ((256, 200), "ba", dt.s8, "col", None),
    # tile tails on both dims, a dst zero point, scales per row
    ((77, 130), "ba", dt.u8, "row", 5),
    # row-major source into a column-major destination
    ((130, 77), "ab", dt.s8, "col", -3),
    # source scales per group of 32 rows and column (2-D mask with groups), 4-bit destination (pairs along the stride-1 dim)
    ((128, 96), "ba", dt.s4, "grouped", None),
    ((64, 192), "ab", dt.u4, "one", 8),
    # 16-bit and fp8 destinations, a source scale on the way
    ((100, 64), "ba", dt.bf16, "src", None),
    ((66, 70), "ab", dt.f8_e4m3, "one", None),
    ((2, 4098), "ba", dt.s8, "row", None), ((4098, 2), "ab", dt.u8, "none", 1),
], ids=str)
def test_transposing_quantizer(ctx, src_dt, dims, src_layout, dst_dt, scale, zp):
    """The sides disagree on the dim order: a 64 x 64 tile through LDS, the row kernel's arithmetic per element. Bit for
    bit against the oracle's reorder, with saturating values and a NaN in the source."""
    eng, strm = ctx
    say("transposing quantizer %s(%s) -> %s %s scale=%s zp=%s" % (src_dt, src_layout, dst_dt, dims, scale, zp))
    r = np.random.default_rng(sum(dims) + src_dt + dst_dt)
    amp = 3.0 if dst_dt in (dt.s4, dt.u4) else 40.0
    x = (r.standard_normal(dims) * amp).astype(np.float32)
    x.reshape(-1)[::97] *= 50
    x.reshape(-1)[7 % x.size] = np.nan
    R, C = dims
    kw = {}
    if scale == "col":
        kw["dst_scale"] = (2, dt.f32, None, r.uniform(0.2, 0.9, C))
    elif scale == "row":
        kw["dst_scale"] = (1, dt.f32, None, r.uniform(0.2, 0.9, R))
    elif scale == "one":
        kw["dst_scale"] = (0, dt.f32, None, [0.37])
    elif scale == "grouped":
        kw["src_scale"] = (3, dt.f16, (32, 1), r.uniform(1.0, 3.0, (R // 32, C)))
    elif scale == "src":
        kw["src_scale"] = (2, dt.f32, None, r.uniform(0.5, 2.0, C))
        kw["dst_scale"] = (0, dt.f32, None, [0.5])
    dst_layout = "ab" if src_layout == "ba" else "ba"
    run_case(eng, strm, src_dt, dst_dt, dims, 0, dst_zp=zp, layout=src_layout, dst_layout=dst_layout, expect=TRANSPOSE,
             src_values=x, **kw)
