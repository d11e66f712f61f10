"""Python mirror of the dnnl C++ API subset (dnnl::engine, stream, memory,
primitive_attr, post_ops, matmul, reorder) over the C ABI of libdnnl_amd.so.

Names, argument meaning and error behaviour follow the reference's
include/oneapi/dnnl/dnnl.hpp (engine dnnl_common.hpp:238, stream :322,
memory dnnl.hpp:834, memory::desc :2749, post_ops :3639, primitive_attr :3965,
reorder :5028, matmul :12808, primitive::execute :215), so tests written against
it read like the reference's own. Every call goes through the exported C entry
points; nothing here computes.
"""
import ctypes as C

import numpy as np

from . import _capi
from ._capi import error  # noqa: F401  (re-export, mirrors dnnl::error)

# ---- argument indices (include/oneapi/dnnl/dnnl_types.h:2476-2700) ----------
DNNL_ARG_SRC = DNNL_ARG_FROM = 1
DNNL_ARG_SRC_1 = 2
DNNL_ARG_DST = DNNL_ARG_TO = 17
DNNL_ARG_WEIGHTS = 33
DNNL_ARG_BIAS = 41
DNNL_ARG_SCRATCHPAD = 80
DNNL_ARG_ATTR_SCALES = 4096
DNNL_ARG_ATTR_ZERO_POINTS = 8192
DNNL_ARG_ATTR_MULTIPLE_POST_OP_BASE = 32768
DNNL_RUNTIME_DIM_VAL = -(2 ** 63)
DNNL_RUNTIME_SIZE_VAL = 2 ** 63  # (size_t)DNNL_RUNTIME_DIM_VAL
DNNL_MEMORY_ALLOCATE = C.c_void_p(2 ** 64 - 1)
DNNL_MEMORY_NONE = None


def DNNL_ARG_ATTR_MULTIPLE_POST_OP(idx):
    return DNNL_ARG_ATTR_MULTIPLE_POST_OP_BASE * (idx + 1)


class status:
    success, out_of_memory, invalid_arguments, unimplemented = 0, 1, 2, 3
    last_impl_reached, runtime_error, not_required = 4, 5, 6


class algorithm:
    undef = 0
    (eltwise_relu, eltwise_tanh, eltwise_elu, eltwise_square, eltwise_abs,
     eltwise_sqrt, eltwise_linear, eltwise_soft_relu, eltwise_hardsigmoid,
     eltwise_logistic, eltwise_exp, eltwise_gelu_tanh, eltwise_swish,
     eltwise_log, eltwise_clip, eltwise_clip_v2, eltwise_pow, eltwise_gelu_erf,
     eltwise_round, eltwise_mish, eltwise_hardswish) = range(0x20, 0x20 + 21)
    (eltwise_relu_use_dst_for_bwd, eltwise_tanh_use_dst_for_bwd,
     eltwise_elu_use_dst_for_bwd, eltwise_sqrt_use_dst_for_bwd,
     eltwise_logistic_use_dst_for_bwd, eltwise_exp_use_dst_for_bwd,
     eltwise_clip_v2_use_dst_for_bwd) = range(0x100, 0x100 + 7)
    (binary_add, binary_mul, binary_max, binary_min, binary_div, binary_sub,
     binary_ge, binary_gt, binary_le, binary_lt, binary_eq, binary_ne,
     binary_select) = range(0x1FFF0, 0x1FFF0 + 13)
    softmax_accurate, softmax_log = 0x30000, 0x30001


class fpmath_mode:
    strict, bf16, f16, any, tf32 = range(5)


class scratchpad_mode:
    library, user = 0, 1


class primitive_kind:
    undef, reorder, sum, eltwise, binary, matmul, prelu = 0, 1, 4, 7, 13, 14, 18


class query:
    engine, primitive_kind, num_of_inputs_s32, num_of_outputs_s32 = 1, 2, 3, 4
    memory_consumption_s64, impl_info_str = 6, 8
    strides = 14
    src_md, weights_md, dst_md, scratchpad_md, exec_arg_md = 129, 131, 133, 136, 255
    ndims_s32, dims, data_type, format_kind = 256, 257, 258, 262


class engine:
    class kind:
        any, cpu, gpu = 0, 1, 2

    def __init__(self, kind=2, index=0):
        h = C.c_void_p()
        _capi.call("dnnl_engine_create", C.byref(h), kind, index)
        self._h = h

    @staticmethod
    def get_count(kind):
        return _capi.lib().dnnl_engine_get_count(kind)

    def get_kind(self):
        k = C.c_int()
        _capi.call("dnnl_engine_get_kind", self._h, C.byref(k))
        return k.value

    def __del__(self):
        if getattr(self, "_h", None):
            _capi.lib().dnnl_engine_destroy(self._h)
            self._h = None


class stream:
    class flags:
        in_order, out_of_order, default_flags = 1, 2, 1

    def __init__(self, eng, flags=1, hip_stream=None):
        h = C.c_void_p()
        if hip_stream is None:
            _capi.call("dnnl_stream_create", C.byref(h), eng._h, flags)
        else:  # wrap a caller-owned hipStream_t (e.g. torch's current stream)
            _capi.call("dnnl_hip_interop_stream_create", C.byref(h), eng._h,
                       C.c_void_p(hip_stream))
        self._h, self._eng = h, eng

    def wait(self):
        _capi.call("dnnl_stream_wait", self._h)
        return self

    def get_engine(self):
        return self._eng

    def __del__(self):
        if getattr(self, "_h", None):
            _capi.lib().dnnl_stream_destroy(self._h)
            self._h = None


class memory:
    class data_type:
        undef, f16, bf16, f32, s32, s8, u8, f64, boolean = range(9)
        f8_e5m2, f8_e4m3, s4, u4, e8m0, f4_e2m1, f4_e3m0 = range(9, 16)

    class format_kind:
        undef, any, blocked, opaque = range(4)

    class format_tag:
        undef, any = 0, 1
        _plain = ("a ab abc abcd abcde abcdef abcdefg abcdefgh abcdefghi "
                  "abcdefghij abcdefghijk abcdefghijkl ba acb bac bca cab cba "
                  "abdc acbd acdb adbc adcb bacd bcda cdab cdba dcab abced abdec "
                  "acbde acdeb adecb bacde bcdea cdeab cdeba decab abcdfe abdefc "
                  "abdfce acbdef adefcb defcab abcdegf abcdefhg abcdefgih "
                  "abcdefghji abcdefghikj abcdefghijlk").split()

    class desc:
        """memory::desc: dims + data type + (tag | strides)."""

        def __init__(self, dims=None, data_type=None, fmt=None, _handle=None,
                     _borrowed=False):
            self._borrowed = _borrowed
            if _handle is not None:
                self._h = _handle
                return
            h = C.c_void_p()
            if dims is None:
                _capi.call("dnnl_memory_desc_create_with_tag", C.byref(h), 0,
                           None, 0, 0)
            elif isinstance(fmt, (list, tuple)):
                _capi.call("dnnl_memory_desc_create_with_strides", C.byref(h),
                           len(dims), _capi.make_dims(dims), data_type,
                           _capi.make_dims(fmt))
            else:
                _capi.call("dnnl_memory_desc_create_with_tag", C.byref(h),
                           len(dims), _capi.make_dims(dims), data_type, fmt)
            self._h = h

        def _query_dims(self, what):
            p = C.POINTER(C.c_int64)()
            _capi.call("dnnl_memory_desc_query", self._h, what, C.byref(p))
            return [p[i] for i in range(self.get_ndims())]

        def get_ndims(self):
            v = C.c_int32()
            _capi.call("dnnl_memory_desc_query", self._h, query.ndims_s32,
                       C.byref(v))
            return v.value

        def get_dims(self):
            return self._query_dims(query.dims)

        def get_strides(self):
            return self._query_dims(query.strides)

        def get_data_type(self):
            v = C.c_int()
            _capi.call("dnnl_memory_desc_query", self._h, query.data_type,
                       C.byref(v))
            return v.value

        def get_format_kind(self):
            v = C.c_int()
            _capi.call("dnnl_memory_desc_query", self._h, query.format_kind,
                       C.byref(v))
            return v.value

        def get_size(self):
            return _capi.lib().dnnl_memory_desc_get_size(self._h)

        def is_zero(self):
            return self.get_ndims() == 0

        def reshape(self, dims):
            h = C.c_void_p()
            _capi.call("dnnl_memory_desc_reshape", C.byref(h), self._h,
                       len(dims), _capi.make_dims(dims))
            return memory.desc(_handle=h)

        def permute_axes(self, perm):
            h = C.c_void_p()
            arr = (C.c_int * len(perm))(*perm)
            _capi.call("dnnl_memory_desc_permute_axes", C.byref(h), self._h, arr)
            return memory.desc(_handle=h)

        def clone(self):
            h = C.c_void_p()
            _capi.call("dnnl_memory_desc_clone", C.byref(h), self._h)
            return memory.desc(_handle=h)

        def __eq__(self, other):
            return bool(_capi.lib().dnnl_memory_desc_equal(self._h, other._h))

        def __ne__(self, other):
            return not self == other

        def __del__(self):
            if getattr(self, "_h", None) and not self._borrowed:
                _capi.lib().dnnl_memory_desc_destroy(self._h)
            self._h = None

    def __init__(self, md, eng, handle="allocate"):
        h = C.c_void_p()
        if isinstance(handle, str):
            raw = DNNL_MEMORY_ALLOCATE
        else:
            raw = C.c_void_p(handle) if handle is not None else None
        _capi.call("dnnl_memory_create", C.byref(h), md._h, eng._h, raw)
        self._h, self._eng = h, eng
        self._md = md if not md._borrowed else md.clone()

    def get_desc(self):
        return self._md

    def get_engine(self):
        return self._eng

    def get_data_handle(self):
        p = C.c_void_p()
        _capi.call("dnnl_memory_get_data_handle", self._h, C.byref(p))
        return p.value

    def set_data_handle(self, handle):
        _capi.call("dnnl_memory_set_data_handle", self._h, C.c_void_p(handle))

    def map_data(self):
        p = C.c_void_p()
        _capi.call("dnnl_memory_map_data", self._h, C.byref(p))
        return p.value

    def unmap_data(self, ptr):
        _capi.call("dnnl_memory_unmap_data", self._h, C.c_void_p(ptr))

    # ---- convenience on top of map/unmap (examples/example_utils.hpp) ----
    def write(self, array):
        """Copy a numpy buffer (raw bytes of the layout) into the memory."""
        buf = np.ascontiguousarray(array)
        size = self._md.get_size()
        if buf.nbytes != size:
            raise ValueError("buffer has %d bytes, memory needs %d"
                             % (buf.nbytes, size))
        if size == 0:
            return self
        p = self.map_data()
        C.memmove(p, buf.ctypes.data, size)
        self.unmap_data(p)
        return self

    def read(self, dtype=np.uint8, shape=None):
        size = self._md.get_size()
        out = np.empty(size, dtype=np.uint8)
        if size:
            p = self.map_data()
            C.memmove(out.ctypes.data, p, size)
            self.unmap_data(p)
        out = out.view(dtype)
        return out.reshape(shape) if shape is not None else out

    def __del__(self):
        if getattr(self, "_h", None):
            _capi.lib().dnnl_memory_destroy(self._h)
            self._h = None


class post_ops:
    def __init__(self, _handle=None):
        if _handle is None:
            _handle = C.c_void_p()
            _capi.call("dnnl_post_ops_create", C.byref(_handle))
        self._h = _handle
        self._keep = []

    def len(self):
        return _capi.lib().dnnl_post_ops_len(self._h)

    def kind(self, index):
        return _capi.lib().dnnl_post_ops_get_kind(self._h, index)

    def append_sum(self, scale=1.0, zero_point=0, data_type=0):
        _capi.call("dnnl_post_ops_append_sum", self._h, scale, zero_point,
                   data_type)

    def append_eltwise(self, alg, alpha, beta):
        _capi.call("dnnl_post_ops_append_eltwise", self._h, alg, alpha, beta)

    def append_binary(self, alg, src1_desc):
        _capi.call("dnnl_post_ops_append_binary", self._h, alg, src1_desc._h)
        self._keep.append(src1_desc)

    def append_prelu(self, mask):
        _capi.call("dnnl_post_ops_append_prelu", self._h, mask)

    def get_params_sum(self, index):
        s, z, d = C.c_float(), C.c_int32(), C.c_int()
        _capi.call("dnnl_post_ops_get_params_sum", self._h, index, C.byref(s),
                   C.byref(z), C.byref(d))
        return s.value, z.value, d.value

    def get_params_eltwise(self, index):
        a, al, be = C.c_int(), C.c_float(), C.c_float()
        _capi.call("dnnl_post_ops_get_params_eltwise", self._h, index,
                   C.byref(a), C.byref(al), C.byref(be))
        return a.value, al.value, be.value

    def get_params_binary(self, index):
        a, md = C.c_int(), C.c_void_p()
        _capi.call("dnnl_post_ops_get_params_binary", self._h, index,
                   C.byref(a), C.byref(md))
        return a.value, memory.desc(_handle=md, _borrowed=True)

    def get_params_prelu(self, index):
        m = C.c_int()
        _capi.call("dnnl_post_ops_get_params_prelu", self._h, index, C.byref(m))
        return m.value

    def __del__(self):
        if getattr(self, "_h", None):
            _capi.lib().dnnl_post_ops_destroy(self._h)
            self._h = None


class primitive_attr:
    def __init__(self):
        h = C.c_void_p()
        _capi.call("dnnl_primitive_attr_create", C.byref(h))
        self._h = h

    def set_scales_mask(self, arg, mask):
        _capi.call("dnnl_primitive_attr_set_scales_mask", self._h, arg, mask)

    def set_scales(self, arg, mask, groups, data_type=memory.data_type.f32):
        _capi.call("dnnl_primitive_attr_set_scales", self._h, arg, mask,
                   len(groups), _capi.make_dims(groups), data_type)

    def set_zero_points_mask(self, arg, mask):
        _capi.call("dnnl_primitive_attr_set_zero_points_mask", self._h, arg,
                   mask)

    def set_zero_points(self, arg, mask, groups,
                        data_type=memory.data_type.s32):
        _capi.call("dnnl_primitive_attr_set_zero_points", self._h, arg, mask,
                   len(groups), _capi.make_dims(groups), data_type)

    def set_fpmath_mode(self, mode, apply_to_int=False):
        _capi.call("dnnl_primitive_attr_set_fpmath_mode_v2", self._h, mode,
                   int(apply_to_int))

    def get_fpmath_mode(self):
        m, a = C.c_int(), C.c_int()
        _capi.call("dnnl_primitive_attr_get_fpmath_mode_v2", self._h,
                   C.byref(m), C.byref(a))
        return m.value, bool(a.value)

    def set_rounding_mode(self, arg, mode):
        _capi.call("dnnl_primitive_attr_set_rounding", self._h, arg, mode)

    def get_rounding_mode(self, arg):
        m = C.c_int()
        _capi.call("dnnl_primitive_attr_get_rounding", self._h, arg, C.byref(m))
        return m.value

    def set_dropout(self, mask_desc):
        _capi.call("dnnl_primitive_attr_set_dropout", self._h, mask_desc._h)

    def get_dropout_ndims(self):
        """ndims of the stored dropout mask descriptor (0: no dropout)."""
        p = C.c_void_p()
        _capi.call("dnnl_primitive_attr_get_dropout", self._h, C.byref(p))
        n = C.c_int()
        _capi.call("dnnl_memory_desc_query", p, query.ndims_s32, C.byref(n))
        return n.value

    def set_scratchpad_mode(self, mode):
        _capi.call("dnnl_primitive_attr_set_scratchpad_mode", self._h, mode)

    def get_scratchpad_mode(self):
        m = C.c_int()
        _capi.call("dnnl_primitive_attr_get_scratchpad_mode", self._h,
                   C.byref(m))
        return m.value

    def set_post_ops(self, po):
        _capi.call("dnnl_primitive_attr_set_post_ops", self._h, po._h)

    def get_post_ops(self):
        p = C.c_void_p()
        _capi.call("dnnl_primitive_attr_get_post_ops", self._h, C.byref(p))
        c = C.c_void_p()
        _capi.call("dnnl_post_ops_clone", C.byref(c), p)
        return post_ops(_handle=c)

    def __del__(self):
        if getattr(self, "_h", None):
            _capi.lib().dnnl_primitive_attr_destroy(self._h)
            self._h = None


class _primitive_desc:
    def __init__(self, handle, eng):
        self._h, self._eng = handle, eng

    def _md(self, what, index=0):
        p = _capi.lib().dnnl_primitive_desc_query_md(self._h, what, index)
        if not p:
            raise error(status.invalid_arguments, "query_md")
        return memory.desc(_handle=C.c_void_p(p), _borrowed=True)

    def src_desc(self):
        return self._md(query.src_md)

    def weights_desc(self):
        return self._md(query.weights_md)

    def bias_desc(self):
        return self._md(query.weights_md, 1)

    def dst_desc(self):
        return self._md(query.dst_md)

    def scratchpad_desc(self):
        return self._md(query.scratchpad_md)

    def query_md(self, what, index=0):
        return self._md(what, index)

    def impl_info_str(self):
        s = C.c_char_p()
        _capi.call("dnnl_primitive_desc_query", self._h, query.impl_info_str, 0,
                   C.byref(s))
        return s.value.decode()

    def next_impl(self):
        st = _capi.lib().dnnl_primitive_desc_next_impl(self._h)
        if st == status.last_impl_reached:
            return False
        _capi.check(st, "dnnl_primitive_desc_next_impl")
        return True

    def n_inputs(self):
        return _capi.lib().dnnl_primitive_desc_query_s32(
            self._h, query.num_of_inputs_s32, 0)

    def n_outputs(self):
        return _capi.lib().dnnl_primitive_desc_query_s32(
            self._h, query.num_of_outputs_s32, 0)

    def get_engine(self):
        return self._eng

    def __del__(self):
        if getattr(self, "_h", None):
            _capi.lib().dnnl_primitive_desc_destroy(self._h)
            self._h = None


class _primitive:
    def __init__(self, pd):
        h = C.c_void_p()
        _capi.call("dnnl_primitive_create", C.byref(h), pd._h)
        self._h, self._pd = h, pd

    def execute(self, strm, args):
        """args: {DNNL_ARG_*: memory}"""
        n = len(args)
        arr = (_capi.exec_arg_t * max(n, 1))()
        for i, (k, m) in enumerate(args.items()):
            arr[i].arg = k
            arr[i].memory = m._h if m is not None else None
        _capi.call("dnnl_primitive_execute", self._h, strm._h, n, arr)

    def get_primitive_desc(self):
        return self._pd

    def __del__(self):
        if getattr(self, "_h", None):
            _capi.lib().dnnl_primitive_destroy(self._h)
            self._h = None


class matmul(_primitive):
    class primitive_desc(_primitive_desc):
        def __init__(self, eng, src_md, weights_md, dst_md, bias_md=None,
                     attr=None):
            h = C.c_void_p()
            _capi.call("dnnl_matmul_primitive_desc_create", C.byref(h), eng._h,
                       src_md._h, weights_md._h,
                       bias_md._h if bias_md is not None else None, dst_md._h,
                       attr._h if attr is not None else None)
            super().__init__(h, eng)


class prop_kind:
    forward_training, forward_inference = 64, 96
    forward = forward_training


class inner_product_forward(_primitive):
    """dnnl::inner_product_forward: src [MB, IC, spatial...] x weights
    [OC, IC, spatial...] -> dst [MB, OC], run by the matmul implementations."""

    class primitive_desc(_primitive_desc):
        def __init__(self, eng, aprop_kind, src_md, weights_md, dst_md,
                     bias_md=None, attr=None):
            h = C.c_void_p()
            _capi.call("dnnl_inner_product_forward_primitive_desc_create",
                       C.byref(h), eng._h, aprop_kind, src_md._h, weights_md._h,
                       bias_md._h if bias_md is not None else None, dst_md._h,
                       attr._h if attr is not None else None)
            super().__init__(h, eng)


class reorder(_primitive):
    class primitive_desc(_primitive_desc):
        def __init__(self, src_engine, src_md, dst_engine, dst_md, attr=None):
            h = C.c_void_p()
            _capi.call("dnnl_reorder_primitive_desc_create", C.byref(h),
                       src_md._h, src_engine._h, dst_md._h, dst_engine._h,
                       attr._h if attr is not None else None)
            super().__init__(h, src_engine)

    def __init__(self, pd_or_src_mem, dst_mem=None, attr=None):
        if dst_mem is not None:  # reorder(src_memory, dst_memory) convenience
            pd_or_src_mem = reorder.primitive_desc(
                pd_or_src_mem.get_engine(), pd_or_src_mem.get_desc(),
                dst_mem.get_engine(), dst_mem.get_desc(), attr)
        super().__init__(pd_or_src_mem)

    def execute(self, strm, src, dst=None):
        if dst is None:
            return super().execute(strm, src)
        return super().execute(strm, {DNNL_ARG_FROM: src, DNNL_ARG_TO: dst})


class softmax_forward(_primitive):
    """dnnl::softmax_forward over one axis (softmax_accurate / softmax_log)."""

    class primitive_desc(_primitive_desc):
        def __init__(self, eng, aprop_kind, aalgorithm, src_md, dst_md, axis, attr=None):
            h = C.c_void_p()
            _capi.call("dnnl_softmax_forward_primitive_desc_create", C.byref(h), eng._h, aprop_kind, aalgorithm,
                       src_md._h, dst_md._h, axis, attr._h if attr is not None else None)
            super().__init__(h, eng)

    def execute(self, strm, src, dst=None):
        if dst is None:
            return super().execute(strm, src)
        return super().execute(strm, {DNNL_ARG_SRC: src, DNNL_ARG_DST: dst})


DNNL_ARG_QUERIES, DNNL_ARG_KEYS, DNNL_ARG_VALUES = 1, 2, 3
DNNL_ARG_SCALE, DNNL_ARG_ATTN_MASK = 51, 52


class sdpa(_primitive):
    """The reference's internal scaled dot-product attention primitive (tests/gtests/internals/sdpa_internal.hpp):
    dst = softmax(scale * Q x K + mask) x V. kq_attr / vs_attr carry the scales and zero points of a quantized
    key / value cache as DNNL_ARG_WEIGHTS entries."""

    class primitive_desc(_primitive_desc):
        def __init__(self, eng, query_md, key_md, value_md, mask_md, scale_dt, dst_md, invert_scale=False,
                     kv_head_number=0, causal_mask=False, attr=None, kq_attr=None, vs_attr=None):
            h = C.c_void_p()
            opt = lambda a: a._h if a is not None else None
            _capi.call("sdpa_primitive_desc_create", C.byref(h), eng._h, query_md._h, key_md._h, value_md._h,
                       dst_md._h, opt(mask_md), scale_dt, bool(invert_scale), kv_head_number, bool(causal_mask),
                       opt(attr), opt(kq_attr), opt(vs_attr))
            super().__init__(h, eng)


def version():
    v = _capi.lib().dnnl_version().contents
    return v.major, v.minor, v.patch
