"""ctypes binding of the dnnl C API subset exported by libdnnl_amd.so.

The library must have been built (python -m onednn_amd.build, or
__graft_entry__.build()); loading fails loudly otherwise. There is no CPU
fallback of any kind.
"""
import contextlib
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdnnl_amd.so")

MAX_NDIMS = 12
dims_t = C.c_int64 * MAX_NDIMS

STATUS_NAMES = {0: "success", 1: "out_of_memory", 2: "invalid_arguments",
                3: "unimplemented", 4: "last_impl_reached", 5: "runtime_error",
                6: "not_required"}


class error(RuntimeError):
    """Mirror of dnnl::error: carries the dnnl_status_t of a failed call."""

    def __init__(self, status, what):
        super().__init__("%s: %s" % (what, STATUS_NAMES.get(status, status)))
        self.status = status


class exec_arg_t(C.Structure):
    _fields_ = [("arg", C.c_int), ("memory", C.c_void_p)]


class version_t(C.Structure):
    _fields_ = [("major", C.c_int), ("minor", C.c_int), ("patch", C.c_int),
                ("hash", C.c_char_p), ("cpu_runtime", C.c_uint),
                ("gpu_runtime", C.c_uint)]


_P = C.c_void_p
_PP = C.POINTER(C.c_void_p)
_I = C.c_int
_F = C.c_float
_DIMS = C.POINTER(C.c_int64)

# name -> (restype, argtypes); restype None means dnnl_status_t
_SIGNATURES = {
    "dnnl_engine_get_count": (C.c_size_t, [_I]),
    "dnnl_engine_create": (None, [_PP, _I, C.c_size_t]),
    "dnnl_engine_get_kind": (None, [_P, C.POINTER(_I)]),
    "dnnl_engine_destroy": (None, [_P]),
    "dnnl_stream_create": (None, [_PP, _P, C.c_uint]),
    "dnnl_stream_get_engine": (None, [_P, _PP]),
    "dnnl_stream_wait": (None, [_P]),
    "dnnl_stream_destroy": (None, [_P]),
    "dnnl_get_default_fpmath_mode": (None, [C.POINTER(_I)]),
    "dnnl_set_default_fpmath_mode": (None, [_I]),
    "dnnl_set_verbose": (None, [_I]),
    "dnnl_version": (C.POINTER(version_t), []),
    "dnnl_primitive_desc_next_impl": (None, [_P]),
    "dnnl_primitive_desc_clone": (None, [_PP, _P]),
    "dnnl_primitive_desc_get_attr": (None, [_P, _PP]),
    "dnnl_primitive_desc_destroy": (None, [_P]),
    "dnnl_primitive_desc_query": (None, [_P, _I, _I, _P]),
    "dnnl_primitive_desc_query_md": (_P, [_P, _I, _I]),
    "dnnl_primitive_desc_query_s32": (_I, [_P, _I, _I]),
    "dnnl_primitive_create": (None, [_PP, _P]),
    "dnnl_primitive_execute": (None, [_P, _P, _I, C.POINTER(exec_arg_t)]),
    "dnnl_primitive_get_primitive_desc": (None, [_P, _PP]),
    "dnnl_primitive_destroy": (None, [_P]),
    "dnnl_primitive_attr_create": (None, [_PP]),
    "dnnl_primitive_attr_clone": (None, [_PP, _P]),
    "dnnl_primitive_attr_destroy": (None, [_P]),
    "dnnl_primitive_attr_get_fpmath_mode": (None, [_P, C.POINTER(_I)]),
    "dnnl_primitive_attr_set_fpmath_mode": (None, [_P, _I]),
    "dnnl_primitive_attr_get_fpmath_mode_v2":
        (None, [_P, C.POINTER(_I), C.POINTER(_I)]),
    "dnnl_primitive_attr_set_fpmath_mode_v2": (None, [_P, _I, _I]),
    "dnnl_softmax_forward_primitive_desc_create": (None, [_PP, _P, _I, _I, _P, _P, _I, _P]),
    "sdpa_primitive_desc_create": (None, [_PP, _P, _P, _P, _P, _P, _P, _I, C.c_bool, C.c_int64, C.c_bool, _P, _P, _P]),
    "dnnl_primitive_attr_get_dropout": (None, [_P, _PP]),
    "dnnl_primitive_attr_set_dropout": (None, [_P, _P]),
    "dnnl_primitive_attr_get_rounding": (None, [_P, _I, C.POINTER(_I)]),
    "dnnl_primitive_attr_set_rounding": (None, [_P, _I, _I]),
    "dnnl_primitive_attr_get_deterministic": (None, [_P, C.POINTER(_I)]),
    "dnnl_primitive_attr_set_deterministic": (None, [_P, _I]),
    "dnnl_primitive_attr_get_accumulation_mode": (None, [_P, C.POINTER(_I)]),
    "dnnl_primitive_attr_set_accumulation_mode": (None, [_P, _I]),
    "dnnl_primitive_attr_get_scratchpad_mode": (None, [_P, C.POINTER(_I)]),
    "dnnl_primitive_attr_set_scratchpad_mode": (None, [_P, _I]),
    "dnnl_primitive_attr_set_scales_mask": (None, [_P, _I, _I]),
    "dnnl_primitive_attr_set_scales": (None, [_P, _I, _I, _I, _DIMS, _I]),
    "dnnl_primitive_attr_set_zero_points_mask": (None, [_P, _I, _I]),
    "dnnl_primitive_attr_set_zero_points": (None, [_P, _I, _I, _I, _DIMS, _I]),
    "dnnl_primitive_attr_get_post_ops": (None, [_P, _PP]),
    "dnnl_primitive_attr_set_post_ops": (None, [_P, _P]),
    "dnnl_post_ops_create": (None, [_PP]),
    "dnnl_post_ops_clone": (None, [_PP, _P]),
    "dnnl_post_ops_destroy": (None, [_P]),
    "dnnl_post_ops_len": (_I, [_P]),
    "dnnl_post_ops_get_kind": (_I, [_P, _I]),
    "dnnl_post_ops_append_sum": (None, [_P, _F, C.c_int32, _I]),
    "dnnl_post_ops_get_params_sum":
        (None, [_P, _I, C.POINTER(_F), C.POINTER(C.c_int32), C.POINTER(_I)]),
    "dnnl_post_ops_append_eltwise": (None, [_P, _I, _F, _F]),
    "dnnl_post_ops_get_params_eltwise":
        (None, [_P, _I, C.POINTER(_I), C.POINTER(_F), C.POINTER(_F)]),
    "dnnl_post_ops_append_binary": (None, [_P, _I, _P]),
    "dnnl_post_ops_get_params_binary": (None, [_P, _I, C.POINTER(_I), _PP]),
    "dnnl_post_ops_append_prelu": (None, [_P, _I]),
    "dnnl_post_ops_get_params_prelu": (None, [_P, _I, C.POINTER(_I)]),
    "dnnl_memory_desc_destroy": (None, [_P]),
    "dnnl_memory_desc_clone": (None, [_PP, _P]),
    "dnnl_memory_desc_create_with_strides": (None, [_PP, _I, _DIMS, _I, _DIMS]),
    "dnnl_memory_desc_create_with_tag": (None, [_PP, _I, _DIMS, _I, _I]),
    "dnnl_memory_desc_reshape": (None, [_PP, _P, _I, _DIMS]),
    "dnnl_memory_desc_permute_axes": (None, [_PP, _P, C.POINTER(_I)]),
    "dnnl_memory_desc_query": (None, [_P, _I, _P]),
    "dnnl_memory_desc_equal": (_I, [_P, _P]),
    "dnnl_memory_desc_get_size": (C.c_size_t, [_P]),
    "dnnl_data_type_size": (C.c_size_t, [_I]),
    "dnnl_memory_create": (None, [_PP, _P, _P, _P]),
    "dnnl_memory_get_memory_desc": (None, [_P, _PP]),
    "dnnl_memory_get_engine": (None, [_P, _PP]),
    "dnnl_memory_map_data": (None, [_P, _PP]),
    "dnnl_memory_unmap_data": (None, [_P, _P]),
    "dnnl_memory_get_data_handle": (None, [_P, _PP]),
    "dnnl_memory_set_data_handle": (None, [_P, _P]),
    "dnnl_memory_destroy": (None, [_P]),
    "dnnl_reorder_primitive_desc_create": (None, [_PP, _P, _P, _P, _P, _P]),
    "dnnl_matmul_primitive_desc_create": (None, [_PP, _P, _P, _P, _P, _P, _P]),
    "dnnl_inner_product_forward_primitive_desc_create": (None, [_PP, _P, _I, _P, _P, _P, _P, _P]),
    # HIP interop and the kernel-level ABI (include/qmm_hip.h)
    "dnnl_hip_interop_stream_create": (None, [_PP, _P, _P]),
    "dnnl_hip_interop_stream_get_stream": (None, [_P, _PP]),
    "qmm_device_count": (_I, []),
    "qmm_last_error": (C.c_char_p, []),
    "qmm_matmul_impl_count": (_I, []),
    "qmm_matmul_impl_name": (C.c_char_p, [_I]),
    "qmm_reorder_impl_name": (C.c_char_p, [_P]),
    "qmm_stream_read": (_I, [_P, C.c_size_t, _P, C.c_size_t, _P, C.c_size_t, _P, _P]),
    "qmm_stream_write": (_I, [_P, C.c_size_t, _I, _P]),
    "qmm_stream_copy": (_I, [_P, _P, C.c_size_t, _I, _P]),
    "qmm_gemm_stamps_read": (_I, [_P, C.c_size_t]),
    "qmm_mfma_ceiling": (_I, [_I, _I, _I, _I, _P, _P, C.POINTER(C.c_double)]),
}

_lib = None


def lib():
    """The loaded shared library (raises if it has not been built)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                "%s is missing: build it with `python -m onednn_amd.build`"
                % LIB_PATH)
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            f = getattr(L, name)
            f.argtypes = args
            f.restype = _I if res is None else res
        _lib = L
    return _lib


@contextlib.contextmanager
def kernel_variants(gemm=None, w4a8=None, b8x=None, measure=None):
    """Kernel-selection overrides (include/qmm_hip.h) for the plans created inside the block: environment variables
    the library reads at plan creation, restored on exit."""
    names = {"QMM_GEMM_VARIANT": gemm, "QMM_W4A8_VARIANT": w4a8, "QMM_B8X_VARIANT": b8x, "QMM_MEASURE": measure}
    old = {k: os.environ.get(k) for k in names}
    try:
        for k, v in names.items():
            if v is not None:
                os.environ[k] = str(int(v))
        yield
    finally:
        for k, v in old.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v


def check(status, what):
    if status != 0:
        raise error(status, what)


def call(name, *args):
    """Call a status-returning entry point, raising `error` on failure."""
    check(getattr(lib(), name)(*args), name)


def make_dims(values):
    a = dims_t()
    for i, v in enumerate(values):
        a[i] = int(v)
    return a
