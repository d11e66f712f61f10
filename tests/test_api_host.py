"""Host-side contract of the C ABI, runnable without a GPU.

The library is loaded through ctypes; a descriptor-only engine
(DNNL_AMD_DESCRIPTOR_ONLY=1) lets primitive descriptors be created and queried
on a host with no device -- descriptor creation is pure host work in the
reference too (src/common/primitive_desc_iface.cpp:32-55). The expected
statuses are the reference's: the case list follows
tests/gtests/test_iface_attr_quantization.cpp:455-545 and
tests/gtests/test_matmul.cpp:400-470.
"""
import ctypes as C
import glob
import os
import re

import pytest

os.environ.setdefault("DNNL_AMD_DESCRIPTOR_ONLY", "1")

import onednn_amd as dnnl  # noqa: E402
from onednn_amd import _capi, memory, status  # noqa: E402

dt = memory.data_type
tag = memory.format_tag
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def T(name):
    return 2 + tag._plain.index(name)


@pytest.fixture(scope="module")
def eng():
    return dnnl.engine(dnnl.engine.kind.gpu, 0)


def expect(st, fn):
    if st == status.success:
        return fn()
    with pytest.raises(dnnl.error) as e:
        fn()
    assert e.value.status == st, e.value


def test_library_exports_every_declared_symbol():
    names = set()
    for path in glob.glob(os.path.join(ROOT, "include", "**", "*.h"), recursive=True):
        text = open(path).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"DNNL_API\s*\*?\s*(dnnl_\w+)\s*\(", text))
        names |= set(re.findall(r"\b(qmm_\w+)\s*\(", text))
    names -= {"qmm_w4_nibble_pos"}
    assert len(names) > 80
    L = C.CDLL(_capi.LIB_PATH)
    missing = [n for n in sorted(names) if not hasattr(L, n)]
    assert not missing, missing
    assert dnnl.version() == (3, 8, 0)


def test_no_cpu_engine_and_bad_index():
    expect(status.invalid_arguments, lambda: dnnl.engine(dnnl.engine.kind.cpu, 0))
    expect(status.invalid_arguments, lambda: dnnl.engine(dnnl.engine.kind.gpu, 77))
    assert dnnl.engine.get_count(dnnl.engine.kind.cpu) == 0


def test_memory_desc_tags_strides_sizes():
    md = memory.desc([3, 4, 5], dt.f32, T("abc"))
    assert md.get_strides() == [20, 5, 1] and md.get_size() == 240
    md = memory.desc([3, 4, 5], dt.s8, T("acb"))
    assert md.get_strides() == [20, 1, 4]
    md = memory.desc([64, 20], dt.s8, T("ba"))
    assert md.get_strides() == [1, 64]
    assert memory.desc([7, 6], dt.u4, T("ab")).get_size() == 21
    assert memory.desc([4096, 4096], dt.u4, T("ab")).get_size() == 8 * 2**20
    assert memory.desc([0, 6], dt.f32, T("ab")).get_size() == 0
    a = memory.desc([3, 4], dt.bf16, [4, 1])
    assert a == memory.desc([3, 4], dt.bf16, T("ab")) and a != memory.desc([3, 4], dt.bf16, T("ba"))
    assert a.get_data_type() == dt.bf16 and a.get_format_kind() == memory.format_kind.blocked
    assert memory.desc([3, 4], dt.f32, tag.any).get_format_kind() == memory.format_kind.any
    # K^T view: permuting axes swaps dims and strides
    kt = memory.desc([2, 128, 16], dt.s8, T("abc")).permute_axes([0, 2, 1])
    assert kt.get_dims() == [2, 16, 128] and kt.get_strides() == [2048, 1, 16]
    assert memory.desc([2, 3, 4], dt.f32, T("abc")).reshape([6, 4]).get_strides() == [4, 1]
    assert memory.desc().is_zero()
    # malformed descriptors
    expect(status.invalid_arguments, lambda: memory.desc([3, -4], dt.f32, T("ab")))
    expect(status.invalid_arguments, lambda: memory.desc([3, 4], dt.f32, T("abc")))
    expect(status.invalid_arguments, lambda: memory.desc([3, 4], dt.f32, [1, 1]))
    expect(status.invalid_arguments, lambda: memory.desc([3, 4], 99, T("ab")))


def test_attr_and_post_ops_setters():
    attr = dnnl.primitive_attr()
    expect(status.invalid_arguments, lambda: attr.set_scales_mask(dnnl.DNNL_ARG_SRC, -1))
    expect(status.invalid_arguments, lambda: attr.set_scales(dnnl.DNNL_ARG_WEIGHTS, 3, [128, 1], dt.s8))
    expect(status.invalid_arguments, lambda: attr.set_zero_points(dnnl.DNNL_ARG_WEIGHTS, 3, [128, 1], dt.f32))
    # int4 zero points need a mask (src/common/primitive_attr.cpp:552-553)
    expect(status.invalid_arguments, lambda: attr.set_zero_points(dnnl.DNNL_ARG_WEIGHTS, 0, [], dt.u4))
    # dst zero points are s32 without groups
    expect(status.invalid_arguments, lambda: attr.set_zero_points(dnnl.DNNL_ARG_DST, 0, [], dt.u8))
    attr.set_zero_points(dnnl.DNNL_ARG_WEIGHTS, 3, [128, 1], dt.u4)
    attr.set_fpmath_mode(dnnl.fpmath_mode.bf16, True)
    assert attr.get_fpmath_mode() == (dnnl.fpmath_mode.bf16, True)
    attr.set_scratchpad_mode(dnnl.scratchpad_mode.user)
    assert attr.get_scratchpad_mode() == dnnl.scratchpad_mode.user

    po = dnnl.post_ops()
    po.append_sum(2.0, 3, dt.u8)
    po.append_eltwise(dnnl.algorithm.eltwise_swish, 1.0, 0.0)
    po.append_binary(dnnl.algorithm.binary_add, memory.desc([1, 8], dt.f32, T("ab")))
    po.append_prelu(2)
    assert po.len() == 4
    assert [po.kind(i) for i in range(4)] == [dnnl.primitive_kind.sum, dnnl.primitive_kind.eltwise,
                                              dnnl.primitive_kind.binary, dnnl.primitive_kind.prelu]
    assert po.get_params_sum(0) == (2.0, 3, dt.u8)
    assert po.get_params_eltwise(1) == (dnnl.algorithm.eltwise_swish, 1.0, 0.0)
    alg, md = po.get_params_binary(2)
    assert alg == dnnl.algorithm.binary_add and md.get_dims() == [1, 8]
    assert po.get_params_prelu(3) == 2
    expect(status.invalid_arguments, lambda: po.get_params_sum(1))
    expect(status.invalid_arguments, lambda: po.append_eltwise(dnnl.algorithm.eltwise_clip, 2.0, 1.0))
    expect(status.invalid_arguments, lambda: po.append_eltwise(dnnl.algorithm.binary_add, 0.0, 0.0))
    expect(status.invalid_arguments, lambda: po.append_binary(dnnl.algorithm.eltwise_relu, memory.desc([1, 8], dt.f32, T("ab"))))
    attr.set_post_ops(po)
    assert attr.get_post_ops().len() == 4
    po2 = dnnl.post_ops()
    for _ in range(32):
        po2.append_eltwise(dnnl.algorithm.eltwise_relu, 0.0, 0.0)
    expect(status.out_of_memory, lambda: po2.append_prelu(1))


def test_dropout_and_rounding_mode_are_stored_and_refused_by_matmul(eng):
    """The setters behave as the reference's (src/common/primitive_attr.cpp:430-442, 564-575; primitive_attr.hpp:
    207-238: a non-default rounding mode only for dst and the gradients); no implementation on this path computes
    dropout or stochastic rounding, so the matmul descriptor is unimplemented with either."""
    env, sto = 0, 1  # dnnl_rounding_mode_environment / _stochastic
    a_md = memory.desc([16, 64], dt.bf16, T("ab"))
    b_md = memory.desc([64, 32], dt.bf16, T("ab"))
    c_md = memory.desc([16, 32], dt.bf16, T("ab"))
    attr = dnnl.primitive_attr()
    assert attr.get_rounding_mode(dnnl.DNNL_ARG_DST) == env and attr.get_dropout_ndims() == 0
    expect(status.invalid_arguments, lambda: attr.set_rounding_mode(dnnl.DNNL_ARG_SRC, sto))
    attr.set_rounding_mode(dnnl.DNNL_ARG_SRC, env)  # the default is accepted for any argument
    expect(status.success, lambda: dnnl.matmul.primitive_desc(eng, a_md, b_md, c_md, attr=attr))
    attr.set_rounding_mode(dnnl.DNNL_ARG_DST, sto)
    assert attr.get_rounding_mode(dnnl.DNNL_ARG_DST) == sto
    expect(status.unimplemented, lambda: dnnl.matmul.primitive_desc(eng, a_md, b_md, c_md, attr=attr))
    attr2 = dnnl.primitive_attr()
    attr2.set_dropout(memory.desc([16, 32], dt.u8, T("ab")))
    assert attr2.get_dropout_ndims() == 2
    expect(status.unimplemented, lambda: dnnl.matmul.primitive_desc(eng, a_md, b_md, c_md, attr=attr2))


def _scales(arg=None, mask=0, data_type=dt.f32, groups=()):
    attr = dnnl.primitive_attr()
    for a in ([arg] if arg is not None else [dnnl.DNNL_ARG_SRC, dnnl.DNNL_ARG_WEIGHTS, dnnl.DNNL_ARG_DST]):
        attr.set_scales(a, mask, list(groups), data_type)
    return attr


def _zp(arg, mask=0, data_type=dt.s32, groups=()):
    attr = dnnl.primitive_attr()
    attr.set_zero_points(arg, mask, list(groups), data_type)
    return attr


def test_matmul_attr_quantization_case_list(eng):
    """tests/gtests/test_iface_attr_quantization.cpp:455-545, GPU-engine branch."""
    OK, UNIMPL = status.success, status.unimplemented
    for a_dt in (dt.f32, dt.u8):
        b_dt = dt.f32 if a_dt == dt.f32 else dt.s8
        a_md = memory.desc([10, 64], a_dt, T("ab"))
        b_md = memory.desc([64, 20], b_dt, T("ba"))
        c_md = memory.desc([10, 20], dt.f32, T("ab"))

        def pd(attr=None):
            return lambda: dnnl.matmul.primitive_desc(eng, a_md, b_md, c_md, attr=attr)

        expect(OK, pd())
        expect(OK, pd(_scales()))
        for arg in (dnnl.DNNL_ARG_SRC, dnnl.DNNL_ARG_WEIGHTS, dnnl.DNNL_ARG_DST):
            if a_dt != dt.u8:
                expect(UNIMPL, pd(_zp(arg)))
            else:
                expect(OK, pd(_zp(arg)))
                expect(OK, pd(_zp(arg, 1 << 1)))
                if arg == dnnl.DNNL_ARG_WEIGHTS:
                    expect(OK, pd(_zp(arg, 3)))
                    expect(OK, pd(_zp(arg, 3, b_dt, (32, 1))))
                elif arg == dnnl.DNNL_ARG_SRC:
                    expect(OK, pd(_zp(arg, 3)))
                    expect(OK, pd(_zp(arg, 3, b_dt, (1, 32))))
                else:
                    expect(UNIMPL, pd(_zp(arg, 3)))
            expect(OK, pd(_scales(arg)))
            if arg == dnnl.DNNL_ARG_WEIGHTS:
                expect(OK, pd(_scales(arg, 1 << 1)))
                if b_dt == dt.s8:
                    expect(OK, pd(_scales(arg, 3)))
                    expect(UNIMPL, pd(_scales(arg, 3, dt.f32, (3, 1))))
                    expect(OK, pd(_scales(arg, 3, dt.f32, (32, 1))))
                else:
                    expect(UNIMPL, pd(_scales(arg, 3, dt.f32, (32, 1))))
            elif arg == dnnl.DNNL_ARG_SRC:
                if a_dt == dt.u8:
                    expect(OK, pd(_scales(arg, 1 << 1, dt.f32, (1, 32))))
                    expect(UNIMPL, pd(_scales(arg, 3, dt.f32, (1, 3))))
                    expect(OK, pd(_scales(arg, 3, dt.f32, (1, 32))))
                else:
                    expect(UNIMPL, pd(_scales(arg, 1 << 1, dt.f32, (1, 32))))
                    expect(UNIMPL, pd(_scales(arg, 3, dt.f32, (1, 32))))
    # per-token source scales cannot be written without groups
    # (tests/gtests/test_iface_attr_quantization.cpp:523-528, src/common/matmul_pd.hpp:219-229)
    a_md = memory.desc([10, 64], dt.s8, T("ab"))
    b_md = memory.desc([64, 20], dt.s8, T("ab"))
    c_md = memory.desc([10, 20], dt.bf16, T("ab"))
    expect(UNIMPL, lambda: dnnl.matmul.primitive_desc(eng, a_md, b_md, c_md, attr=_scales(dnnl.DNNL_ARG_SRC, 1 << 0)))
    expect(UNIMPL, lambda: dnnl.matmul.primitive_desc(eng, a_md, b_md, c_md, attr=_scales(dnnl.DNNL_ARG_SRC, 3)))
    expect(OK, lambda: dnnl.matmul.primitive_desc(eng, a_md, b_md, c_md, attr=_scales(dnnl.DNNL_ARG_SRC, 3, dt.f32, (1, 64))))


def test_matmul_shape_errors(eng):
    """src/common/matmul.cpp:284-409: malformed problems are invalid_arguments."""
    BAD = status.invalid_arguments

    def pd(s, w, d, b=None, sdt=dt.f32, wdt=dt.f32, ddt=dt.f32):
        def mk(dims, t):
            return memory.desc(dims, t, T("abcdef"[:len(dims)]))
        return lambda: dnnl.matmul.primitive_desc(eng, mk(s, sdt), mk(w, wdt), mk(d, ddt),
                                                  bias_md=mk(b, dt.f32) if b else None)

    expect(status.success, pd([10, 64], [64, 20], [10, 20]))
    expect(BAD, pd([10, 64], [63, 20], [10, 20]))  # K mismatch
    expect(BAD, pd([10, 64], [64, 20], [11, 20]))  # M mismatch
    expect(BAD, pd([10, 64], [64, 20], [10, 21]))  # N mismatch
    expect(BAD, pd([2, 10, 64], [64, 20], [2, 10, 20]))  # ndims mismatch
    expect(BAD, pd([3, 10, 64], [2, 64, 20], [3, 10, 20]))  # bad broadcast
    expect(status.success, pd([3, 10, 64], [1, 64, 20], [3, 10, 20]))
    expect(status.success, pd([1, 10, 64], [3, 64, 20], [3, 10, 20]))
    expect(BAD, pd([1, 10, 64], [3, 64, 20], [1, 10, 20]))
    expect(status.success, pd([10, 64], [64, 20], [10, 20], b=[1, 20]))
    expect(BAD, pd([10, 64], [64, 20], [10, 20], b=[1, 19]))
    expect(BAD, pd([10, 64], [64, 20], [10, 20], b=[20]))
    expect(BAD, pd([10, 64], [64, 21], [10, 21], sdt=dt.bf16, wdt=dt.u4, ddt=dt.bf16))  # odd N with int4
    expect(BAD, pd([10, 64], [64, 20], [10, 20], sdt=dt.s32, wdt=dt.s32, ddt=dt.s32))  # no accumulation type
    expect(BAD, lambda: dnnl.matmul.primitive_desc(eng, memory.desc([4], dt.f32, T("a")), memory.desc([4], dt.f32, T("a")), memory.desc([4], dt.f32, T("a"))))


def _config_pd(eng, name, wtag=tag.any):
    A = dnnl
    if name == "c1":
        attr = A.primitive_attr()
        attr.set_scales_mask(A.DNNL_ARG_SRC, 0)
        attr.set_zero_points_mask(A.DNNL_ARG_SRC, 0)
        attr.set_scales_mask(A.DNNL_ARG_WEIGHTS, 2)
        return A.matmul.primitive_desc(eng, memory.desc([256, 1024], dt.u8, T("ab")), memory.desc([1024, 1024], dt.s8, wtag),
                                       memory.desc([256, 1024], dt.f32, T("ab")), attr=attr)
    if name == "c2":
        attr = A.primitive_attr()
        attr.set_scales(A.DNNL_ARG_SRC, 3, [1, 4096], dt.f32)
        attr.set_scales_mask(A.DNNL_ARG_WEIGHTS, 2)
        po = A.post_ops()
        po.append_eltwise(A.algorithm.eltwise_swish, 1.0, 0.0)
        attr.set_post_ops(po)
        return A.matmul.primitive_desc(eng, memory.desc([4096, 4096], dt.s8, T("ab")), memory.desc([4096, 14336], dt.s8, wtag),
                                       memory.desc([4096, 14336], dt.bf16, T("ab")), attr=attr)
    if name == "c3":
        attr = A.primitive_attr()
        attr.set_fpmath_mode(A.fpmath_mode.bf16, True)
        attr.set_scales(A.DNNL_ARG_WEIGHTS, 3, [128, 1], dt.f16)
        attr.set_zero_points(A.DNNL_ARG_WEIGHTS, 3, [128, 1], dt.u4)
        return A.matmul.primitive_desc(eng, memory.desc([1, 4096], dt.bf16, T("ab")), memory.desc([4096, 4096], dt.u4, wtag),
                                       memory.desc([1, 4096], dt.bf16, T("ab")), attr=attr)
    if name == "c4":
        attr = A.primitive_attr()
        attr.set_scales_mask(A.DNNL_ARG_SRC, 0)
        attr.set_scales_mask(A.DNNL_ARG_WEIGHTS, 0)
        po = A.post_ops()
        po.append_binary(A.algorithm.binary_add, memory.desc([1, 2048, 2048], dt.f32, T("abc")))
        attr.set_post_ops(po)
        return A.matmul.primitive_desc(eng, memory.desc([32, 2048, 128], dt.s8, T("abc")), memory.desc([32, 128, 2048], dt.s8, wtag),
                                       memory.desc([32, 2048, 2048], dt.f32, T("abc")), attr=attr)
    if name == "c5":
        attr = A.primitive_attr()
        attr.set_scales_mask(A.DNNL_ARG_SRC, 0)
        attr.set_scales_mask(A.DNNL_ARG_WEIGHTS, 0)
        po = A.post_ops()
        po.append_sum(1.0)
        attr.set_post_ops(po)
        return A.matmul.primitive_desc(eng, memory.desc([8192, 8192], dt.f8_e4m3, T("ab")), memory.desc([8192, 8192], dt.f8_e4m3, wtag),
                                       memory.desc([8192, 8192], dt.bf16, T("ab")), attr=attr)
    raise KeyError(name)


@pytest.mark.parametrize("name,impl,wei_bytes", [
    ("c1", "hip:gfx950:mfma_b8", 1024 * 1024 + 4 * 1024),
    ("c2", "hip:gfx950:mfma_b8", 4096 * 14336 + 4 * 14336),
    ("c3", "hip:gfx950:decode_w4", 4096 * 4096 // 2),
    ("c4", "hip:gfx950:mfma_b8", 32 * (128 * 2048 + 4 * 2048)),
    ("c5", "hip:gfx950:mfma_b8", 8192 * 8192 + 4 * 8192),
])
def test_headline_configs_dispatch_to_the_mfma_kernels(eng, name, impl, wei_bytes):
    pd = _config_pd(eng, name)
    assert pd.impl_info_str() == impl
    w = pd.weights_desc()
    # format any resolves to an opaque prepacked layout
    assert w.get_format_kind() == memory.format_kind.opaque
    assert w.get_size() == wei_bytes
    assert w.clone() == w
    assert pd.n_inputs() == (3 if name == "c4" else 2) and pd.n_outputs() == 1
    # the implementation list ends; plain weights are what the last entry takes
    names = [pd.impl_info_str()]
    while pd.next_impl():
        names.append(pd.impl_info_str())
    assert names[-1] == "hip:gfx950:generic"
    assert pd.weights_desc().get_format_kind() == memory.format_kind.blocked
    # plain weights also run on the tiled kernels (packed on the fly into the scratchpad)
    pd2 = _config_pd(eng, name, T("abc" if name == "c4" else "ab"))
    assert pd2.impl_info_str() == impl
    assert pd2.weights_desc().get_format_kind() == memory.format_kind.blocked


def test_user_scratchpad_is_reported(eng):
    attr = dnnl.primitive_attr()
    attr.set_scratchpad_mode(dnnl.scratchpad_mode.user)
    pd = dnnl.matmul.primitive_desc(eng, memory.desc([64, 64], dt.s8, T("ab")), memory.desc([64, 64], dt.s8, T("ab")),
                                    memory.desc([64, 64], dt.s32, T("ab")), attr=attr)
    assert pd.impl_info_str() == "hip:gfx950:mfma_b8"
    assert pd.scratchpad_desc().get_size() == 128 * 64 + 64 * 4
    pd = dnnl.matmul.primitive_desc(eng, memory.desc([64, 64], dt.s8, T("ab")), memory.desc([64, 64], dt.s8, tag.any),
                                    memory.desc([64, 64], dt.s32, T("ab")), attr=attr)
    assert pd.scratchpad_desc().is_zero()


def test_generic_takes_what_the_tiled_kernels_do_not(eng):
    # K-grouped dynamic quantization: s8 x u4 with grouped src and weights scales
    # goes to the int8 x int4 kernel when the groups are whole 64-k tiles ...
    attr = dnnl.primitive_attr()
    attr.set_scales(dnnl.DNNL_ARG_SRC, 3, [1, 64], dt.f16)
    attr.set_scales(dnnl.DNNL_ARG_WEIGHTS, 3, [64, 1], dt.f16)
    pd = dnnl.matmul.primitive_desc(eng, memory.desc([4, 128], dt.s8, T("ab")), memory.desc([128, 32], dt.u4, tag.any),
                                    memory.desc([4, 32], dt.f16, T("ab")), attr=attr)
    assert pd.impl_info_str() == "hip:gfx950:mfma_w4a8"
    assert pd.weights_desc().get_format_kind() == memory.format_kind.opaque
    assert pd.weights_desc().get_size() == 128 * 32 // 2
    # groups of 32 (half a tile) too
    attr = dnnl.primitive_attr()
    attr.set_scales(dnnl.DNNL_ARG_SRC, 3, [1, 32], dt.f16)
    attr.set_scales(dnnl.DNNL_ARG_WEIGHTS, 3, [32, 1], dt.f16)
    pd = dnnl.matmul.primitive_desc(eng, memory.desc([4, 128], dt.s8, T("ab")), memory.desc([128, 32], dt.u4, tag.any),
                                    memory.desc([4, 32], dt.f16, T("ab")), attr=attr)
    assert pd.impl_info_str() == "hip:gfx950:mfma_w4a8"
    # ... and to the generic kernel otherwise (groups of 96, s32 source zero points)
    attr = dnnl.primitive_attr()
    attr.set_scales(dnnl.DNNL_ARG_SRC, 3, [1, 96], dt.f16)
    attr.set_scales(dnnl.DNNL_ARG_WEIGHTS, 3, [96, 1], dt.f16)
    pd = dnnl.matmul.primitive_desc(eng, memory.desc([4, 192], dt.s8, T("ab")), memory.desc([192, 32], dt.u4, tag.any),
                                    memory.desc([4, 32], dt.f16, T("ab")), attr=attr)
    assert pd.impl_info_str() == "hip:gfx950:generic"
    assert pd.weights_desc().get_format_kind() == memory.format_kind.blocked
    attr = dnnl.primitive_attr()
    attr.set_scales(dnnl.DNNL_ARG_WEIGHTS, 3, [64, 1], dt.f16)
    attr.set_zero_points(dnnl.DNNL_ARG_SRC, 3, [1, 64], dt.s32)
    pd = dnnl.matmul.primitive_desc(eng, memory.desc([4, 128], dt.s8, T("ab")), memory.desc([128, 32], dt.s4, T("ab")),
                                    memory.desc([4, 32], dt.f32, T("ab")), attr=attr)
    assert pd.impl_info_str() == "hip:gfx950:generic"
    # 8-bit source zero points per row and K group, and u8 sources, stay on the MFMA path
    attr = dnnl.primitive_attr()
    attr.set_scales(dnnl.DNNL_ARG_WEIGHTS, 3, [64, 1], dt.f16)
    attr.set_zero_points(dnnl.DNNL_ARG_SRC, 3, [1, 64], dt.u8)
    pd = dnnl.matmul.primitive_desc(eng, memory.desc([4, 128], dt.u8, T("ab")), memory.desc([128, 32], dt.s4, T("ab")),
                                    memory.desc([4, 32], dt.f32, T("ab")), attr=attr)
    assert pd.impl_info_str() == "hip:gfx950:mfma_w4a8"
    # transposed source
    pd = dnnl.matmul.primitive_desc(eng, memory.desc([64, 64], dt.s8, T("ba")), memory.desc([64, 64], dt.s8, T("ab")),
                                    memory.desc([64, 64], dt.s32, T("ab")))
    assert pd.impl_info_str() == "hip:gfx950:generic"
    # unsupported type combinations stay unimplemented
    expect(status.unimplemented, lambda: dnnl.matmul.primitive_desc(
        eng, memory.desc([8, 8], dt.f32, T("ab")), memory.desc([8, 8], dt.f32, T("ab")), memory.desc([8, 8], dt.bf16, T("ab"))))
    expect(status.unimplemented, lambda: dnnl.matmul.primitive_desc(
        eng, memory.desc([8, 8], dt.bf16, T("ab")), memory.desc([8, 8], dt.s8, T("ab")), memory.desc([8, 8], dt.bf16, T("ab"))))


def test_reorder_descriptor_rules(eng):
    """src/common/reorder.cpp:66-160."""
    pd = _config_pd(eng, "c1")
    plain = memory.desc([1024, 1024], dt.s8, T("ab"))
    r = dnnl.reorder.primitive_desc(eng, plain, eng, pd.weights_desc())
    assert r.impl_info_str() == "hip:gfx950:prepack"
    r = dnnl.reorder.primitive_desc(eng, pd.weights_desc(), eng, plain)
    assert r.impl_info_str() == "hip:gfx950:prepack"
    r = dnnl.reorder.primitive_desc(eng, memory.desc([8, 8], dt.f32, T("ab")), eng, memory.desc([8, 8], dt.s8, T("ba")))
    assert r.impl_info_str() == "hip:gfx950:quantize_transpose"
    r = dnnl.reorder.primitive_desc(eng, memory.desc([8, 8], dt.s8, T("ab")), eng, memory.desc([8, 8], dt.f32, T("ba")))
    assert r.impl_info_str() == "hip:gfx950:reorder"
    BAD = status.invalid_arguments
    expect(BAD, lambda: dnnl.reorder.primitive_desc(eng, memory.desc([8, 8], dt.f32, tag.any), eng, plain))
    expect(BAD, lambda: dnnl.reorder.primitive_desc(eng, memory.desc([8, 9], dt.f32, T("ab")), eng, memory.desc([8, 8], dt.f32, T("ab"))))
    # zero points only for integral types
    expect(BAD, lambda: dnnl.reorder.primitive_desc(eng, memory.desc([8, 8], dt.f32, T("ab")), eng, memory.desc([8, 8], dt.s8, T("ab")),
                                                    attr=_zp(dnnl.DNNL_ARG_SRC)))
    # packed layouts only by plain copy of the same type
    expect(status.unimplemented, lambda: dnnl.reorder.primitive_desc(eng, memory.desc([1024, 1024], dt.f32, T("ab")), eng, pd.weights_desc()))


def test_memory_without_device_fails_loudly(eng):
    if _capi.lib().qmm_device_count() > 0:
        pytest.skip("a GPU is present")
    md = memory.desc([4, 4], dt.f32, T("ab"))
    expect(status.runtime_error, lambda: memory(md, eng))
    expect(status.runtime_error, lambda: dnnl.stream(eng))
    pd = dnnl.matmul.primitive_desc(eng, md, md, md)
    expect(status.runtime_error, lambda: dnnl.matmul(pd))


def test_inner_product_descriptor_is_lowered_to_matmul(eng):
    src = memory.desc([8, 16, 2, 2], dt.s8, T("abcd"))
    wei = memory.desc([32, 16, 2, 2], dt.s8, tag.any)
    dst = memory.desc([8, 32], dt.f32, T("ab"))
    pd = dnnl.inner_product_forward.primitive_desc(eng, dnnl.prop_kind.forward_inference, src, wei, dst)
    assert pd.impl_info_str() == "hip:gfx950:mfma_b8"
    assert pd.src_desc().get_dims() == [8, 16, 2, 2]
    w = pd.weights_desc()
    assert w.get_dims() == [32, 16, 2, 2] and w.get_format_kind() == memory.format_kind.opaque
    # the prepacking reorder takes the user's OC-major tensor
    r = dnnl.reorder.primitive_desc(eng, memory.desc([32, 16, 2, 2], dt.s8, T("abcd")), eng, w)
    assert r.impl_info_str() == "hip:gfx950:prepack"
    # shape errors and unsupported attributes
    expect(status.invalid_arguments, lambda: dnnl.inner_product_forward.primitive_desc(
        eng, dnnl.prop_kind.forward_inference, src, memory.desc([32, 8, 2, 2], dt.s8, tag.any), dst))
    attr = dnnl.primitive_attr()
    attr.set_zero_points_mask(dnnl.DNNL_ARG_SRC, 0)
    expect(status.unimplemented, lambda: dnnl.inner_product_forward.primitive_desc(
        eng, dnnl.prop_kind.forward_inference, src, wei, dst, attr=attr))



def test_runtime_dims_descriptor(eng):
    """Descriptors holding DNNL_RUNTIME_DIM_VAL: the dims stay open until
    execute; format any cannot be resolved without them
    (src/common/matmul_pd.hpp:266-277) and the batch dims are runtime together
    or not at all (src/common/matmul.cpp:375-386)."""
    R = dnnl.DNNL_RUNTIME_DIM_VAL
    src = memory.desc([R, 256], dt.s8, T("ab"))
    wei = memory.desc([256, 128], dt.s8, T("ab"))
    dst = memory.desc([R, 128], dt.f32, T("ab"))
    assert src.get_strides() == [256, 1]
    assert src.get_size() == dnnl.DNNL_RUNTIME_SIZE_VAL
    pd = dnnl.matmul.primitive_desc(eng, src, wei, dst)
    assert pd.impl_info_str() == "hip:gfx950:runtime_dims"
    assert pd.src_desc().get_dims() == [R, 256]
    assert pd.dst_desc() == dst
    assert pd.scratchpad_desc().is_zero()
    assert not pd.next_impl()
    # format any: refused on a descriptor that has runtime dims itself, resolved on
    # weights whose own dims are known (src/common/matmul_pd.hpp:266-277,
    # examples/tutorials/matmul/inference_int8_matmul.cpp:104-125)
    expect(status.unimplemented, lambda: dnnl.matmul.primitive_desc(
        eng, memory.desc([R, 256], dt.s8, tag.any), wei, dst))
    pd_any = dnnl.matmul.primitive_desc(eng, src, memory.desc([256, 128], dt.s8, tag.any), dst)
    assert pd_any.impl_info_str() == "hip:gfx950:runtime_dims"
    assert pd_any.weights_desc().get_format_kind() == memory.format_kind.opaque
    expect(status.invalid_arguments, lambda: dnnl.matmul.primitive_desc(
        eng, memory.desc([R, 8, 256], dt.s8, T("abc")), memory.desc([4, 256, 128], dt.s8, T("abc")),
        memory.desc([R, 8, 128], dt.f32, T("abc"))))
    # fully open
    pd = dnnl.matmul.primitive_desc(eng, memory.desc([R, R], dt.s8, T("ab")), memory.desc([R, R], dt.s8, T("ab")),
                                    memory.desc([R, R], dt.f32, T("ab")))
    assert pd.impl_info_str() == "hip:gfx950:runtime_dims"
