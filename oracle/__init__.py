"""ctypes front-end of the CPU oracle (TEST INFRASTRUCTURE ONLY).

Only the test-suite, the smoke check and the benchmark's CPU-baseline leg may
import this package; the shipped library never does.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libqmm_oracle.so")

# data-type codes (the reference's public enum values)
UNDEF, F16, BF16, F32, S32, S8, U8 = 0, 1, 2, 3, 4, 5, 6
F8_E5M2, F8_E4M3, S4, U4, E8M0 = 9, 10, 11, 12, 13
PO_SUM, PO_ELTWISE, PO_BINARY, PO_PRELU = 1, 2, 3, 4
Q_SRC, Q_WEI, Q_DST = 0, 1, 2
MAX_NDIMS, MAX_PO = 12, 32

DT_NAMES = {"f16": F16, "bf16": BF16, "f32": F32, "s32": S32, "s8": S8,
            "u8": U8, "f8_e5m2": F8_E5M2, "f8_e4m3": F8_E4M3, "s4": S4,
            "u4": U4, "e8m0": E8M0}

# numpy storage dtype of one element (4-bit types: two per byte)
STORAGE = {F16: np.uint16, BF16: np.uint16, F32: np.float32, S32: np.int32,
           S8: np.int8, U8: np.uint8, F8_E5M2: np.uint8, F8_E4M3: np.uint8,
           S4: np.uint8, U4: np.uint8, E8M0: np.uint8}


def build(force=False):
    """Compile the C restatement with gcc (no FMA contraction)."""
    src = os.path.join(_HERE, "qmm_oracle.c")
    if (not force and os.path.exists(_LIB_PATH)
            and os.path.getmtime(_LIB_PATH) >= os.path.getmtime(src)):
        return _LIB_PATH
    subprocess.check_call(["make", "-C", _HERE, "-B", "libqmm_oracle.so"],
                          stdout=subprocess.DEVNULL)
    return _LIB_PATH


class _Tensor(C.Structure):
    _fields_ = [("dt", C.c_int32), ("ndims", C.c_int32),
                ("dims", C.c_int64 * MAX_NDIMS),
                ("strides", C.c_int64 * MAX_NDIMS), ("ptr", C.c_void_p)]


class _Quant(C.Structure):
    _fields_ = [("set", C.c_int32), ("mask", C.c_int32), ("dt", C.c_int32),
                ("pad_", C.c_int32), ("g0", C.c_int64), ("g1", C.c_int64),
                ("ptr", C.c_void_p)]


class _PostOp(C.Structure):
    _fields_ = [("kind", C.c_int32), ("alg", C.c_int32), ("alpha", C.c_float),
                ("beta", C.c_float), ("scale", C.c_float),
                ("zero_point", C.c_int32), ("sum_dt", C.c_int32),
                ("prelu_mask", C.c_int32), ("src1", _Tensor)]


class _Matmul(C.Structure):
    _fields_ = [("src", _Tensor), ("wei", _Tensor), ("bias", _Tensor),
                ("dst", _Tensor), ("scales", _Quant * 3), ("zps", _Quant * 3),
                ("apply_to_int", C.c_int32), ("npo", C.c_int32),
                ("po", _PostOp * MAX_PO), ("nthreads", C.c_int32),
                ("k_group_mode", C.c_int32)]


class _Reorder(C.Structure):
    _fields_ = [("src", _Tensor), ("dst", _Tensor), ("src_scale", _Quant),
                ("dst_scale", _Quant), ("src_zp", _Quant), ("dst_zp", _Quant)]


class _Softmax(C.Structure):
    _fields_ = [("src", _Tensor), ("dst", _Tensor), ("axis", C.c_int32), ("log_softmax", C.c_int32),
                ("src_scale", _Quant), ("dst_scale", _Quant)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        L.orc_matmul.argtypes = [C.POINTER(_Matmul)]
        L.orc_matmul.restype = C.c_int
        L.orc_matmul_s32_acc.argtypes = [C.POINTER(_Matmul), C.c_void_p]
        L.orc_matmul_s32_acc.restype = C.c_int
        L.orc_reorder.argtypes = [C.POINTER(_Reorder)]
        L.orc_reorder.restype = C.c_int
        for name, res, args in [
                ("orc_f32_to_bf16", C.c_uint16, [C.c_float]),
                ("orc_bf16_to_f32", C.c_float, [C.c_uint16]),
                ("orc_f32_to_f16", C.c_uint16, [C.c_float]),
                ("orc_f16_to_f32", C.c_float, [C.c_uint16]),
                ("orc_f16_to_e4m3", C.c_uint8, [C.c_uint16]),
                ("orc_f32_to_e4m3", C.c_uint8, [C.c_float]),
                ("orc_e4m3_to_f16", C.c_uint16, [C.c_uint8]),
                ("orc_e4m3_to_f32", C.c_float, [C.c_uint8]),
                ("orc_f32_to_e5m2", C.c_uint8, [C.c_float]),
                ("orc_e5m2_to_f32", C.c_float, [C.c_uint8]),
                ("orc_eltwise", C.c_float,
                 [C.c_int, C.c_float, C.c_float, C.c_float]),
                ("orc_binary", C.c_float, [C.c_int, C.c_float, C.c_float])]:
            f = getattr(L, name)
            f.restype, f.argtypes = res, args
        L.orc_load_int.argtypes = [C.c_int, C.c_void_p, C.c_int64]
        L.orc_load_int.restype = C.c_int
        L.orc_load_float.argtypes = [C.c_int, C.c_void_p, C.c_int64]
        L.orc_load_float.restype = C.c_float
        L.orc_cvt_from_f32.argtypes = [C.c_int, C.c_void_p, C.c_void_p,
                                       C.c_int64]
        L.orc_cvt_to_f32.argtypes = [C.c_int, C.c_void_p, C.c_void_p,
                                     C.c_int64]
        _lib = L
    return _lib


def from_f32(dt, a):
    """Convert an f32 array to the storage of `dt` with the reference rounding."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    out = np.empty(a.shape, dtype=STORAGE[dt])
    lib().orc_cvt_from_f32(dt, a.ctypes.data, out.ctypes.data, a.size)
    return out


def to_f32(dt, a, n=None):
    a = np.ascontiguousarray(a)
    n = a.size if n is None else n
    out = np.empty(n, dtype=np.float32)
    lib().orc_cvt_to_f32(dt, a.ctypes.data, out.ctypes.data, n)
    return out if n != a.size else out.reshape(a.shape)


def pack4(vals):
    """Pack integer values (flat, logical order) two per byte, even index low."""
    v = np.asarray(vals).astype(np.int64).ravel() & 0xF
    if v.size % 2:
        v = np.concatenate([v, [0]])
    return (v[0::2] | (v[1::2] << 4)).astype(np.uint8)


def unpack4(buf, n, signed):
    b = np.asarray(buf, dtype=np.uint8).ravel()
    v = np.empty(b.size * 2, dtype=np.int32)
    v[0::2] = b & 0xF
    v[1::2] = b >> 4
    v = v[:n]
    if signed:
        v = np.where(v >= 8, v - 16, v)
    return v


def dense_strides(dims):
    s, out = 1, []
    for d in reversed(dims):
        out.append(s)
        s *= max(int(d), 1)
    return list(reversed(out))


class Tensor:
    """A strided tensor: `data` is a numpy buffer in the storage type of `dt`."""

    def __init__(self, dt, dims, data, strides=None):
        self.dt = dt
        self.dims = [int(d) for d in dims]
        self.strides = ([int(s) for s in strides] if strides is not None
                        else dense_strides(self.dims))
        self.data = data

    def c(self):
        t = _Tensor()
        t.dt, t.ndims = self.dt, len(self.dims)
        for i, (d, s) in enumerate(zip(self.dims, self.strides)):
            t.dims[i], t.strides[i] = d, s
        t.ptr = self.data.ctypes.data if self.data is not None else None
        return t


class Quant:
    """Scales or zero-points entry: mask, dt, (g0, g1) groups and the buffer."""

    def __init__(self, mask, dt, data, groups=None):
        self.mask, self.dt, self.data = mask, dt, data
        self.groups = tuple(groups) if groups else None

    def c(self):
        q = _Quant()
        q.set, q.mask, q.dt = 1, self.mask, self.dt
        q.g0, q.g1 = self.groups if self.groups else (0, 0)
        q.ptr = self.data.ctypes.data
        return q


KGROUP_LITERAL, KGROUP_WHOLE = 0, 1


def _fill(p, src, wei, dst, bias, scales, zps, post_ops, apply_to_int,
          nthreads, k_group_mode=KGROUP_WHOLE):
    p.k_group_mode = k_group_mode
    keep = [src, wei, dst, bias]
    p.src, p.wei, p.dst = src.c(), wei.c(), dst.c()
    if bias is not None:
        p.bias = bias.c()
    for i in range(3):
        if scales and scales.get(i) is not None:
            p.scales[i] = scales[i].c()
            keep.append(scales[i])
        if zps and zps.get(i) is not None:
            p.zps[i] = zps[i].c()
            keep.append(zps[i])
    p.apply_to_int = int(bool(apply_to_int))
    p.npo = len(post_ops or [])
    for i, po in enumerate(post_ops or []):
        e = p.po[i]
        kind = po["kind"]
        if kind == "sum":
            e.kind, e.scale = PO_SUM, po.get("scale", 1.0)
            e.zero_point, e.sum_dt = po.get("zero_point", 0), po.get("dt", 0)
        elif kind == "eltwise":
            e.kind, e.alg = PO_ELTWISE, po["alg"]
            e.alpha, e.beta = po.get("alpha", 0.0), po.get("beta", 0.0)
            e.scale = po.get("scale", 1.0)
        elif kind == "binary":
            e.kind, e.alg, e.src1 = PO_BINARY, po["alg"], po["src1"].c()
            keep.append(po["src1"])
        elif kind == "prelu":
            e.kind, e.prelu_mask = PO_PRELU, po["mask"]
            e.src1.ptr = po["weights"].ctypes.data
            keep.append(po["weights"])
        else:
            raise ValueError(kind)
    p.nthreads = nthreads
    return keep


def matmul(src, wei, dst, bias=None, scales=None, zps=None, post_ops=None,
           apply_to_int=False, nthreads=0, k_group_mode=KGROUP_WHOLE):
    """Run the reference-semantics matmul; writes into dst.data.

    k_group_mode (integer path only): KGROUP_WHOLE accumulates in s32 over
    each scale group (all of K when no groups are given); KGROUP_LITERAL
    follows the v3.8 source literally, where an entry without explicit groups
    closes the group after every k and the sum runs in f32.
    """
    p = _Matmul()
    keep = _fill(p, src, wei, dst, bias, scales, zps, post_ops, apply_to_int,
                 nthreads, k_group_mode)
    rc = lib().orc_matmul(C.byref(p))
    del keep
    if rc != 0:
        raise RuntimeError("oracle: unsupported combination (%d)" % rc)
    return dst.data


def matmul_s32_acc(src, wei, dst, zps=None, nthreads=0):
    """Exact s32 accumulators (batch*M*N) of the integer path."""
    p = _Matmul()
    keep = _fill(p, src, wei, dst, None, None, zps, None, False, nthreads)
    n = 1
    for d in dst.dims:
        n *= d
    acc = np.zeros(n, dtype=np.int32)
    rc = lib().orc_matmul_s32_acc(C.byref(p), acc.ctypes.data)
    del keep
    if rc != 0:
        raise RuntimeError("oracle: unsupported combination (%d)" % rc)
    return acc.reshape(dst.dims)


def reorder(src, dst, src_scale=None, dst_scale=None, src_zp=None,
            dst_zp=None):
    p = _Reorder()
    p.src, p.dst = src.c(), dst.c()
    for name, q in (("src_scale", src_scale), ("dst_scale", dst_scale),
                    ("src_zp", src_zp), ("dst_zp", dst_zp)):
        if q is not None:
            setattr(p, name, q.c())
    rc = lib().orc_reorder(C.byref(p))
    if rc != 0:
        raise RuntimeError("oracle reorder failed (%d)" % rc)
    return dst.data


def softmax(src, dst, axis, log=False, src_scale=None, dst_scale=None):
    """Reference softmax forward over `axis` (src/cpu/ref_softmax.cpp); scales are single-value Quant entries."""
    p = _Softmax()
    p.src, p.dst = src.c(), dst.c()
    p.axis, p.log_softmax = axis, 1 if log else 0
    for name, q in (("src_scale", src_scale), ("dst_scale", dst_scale)):
        if q is not None:
            setattr(p, name, q.c())
    rc = lib().orc_softmax(C.byref(p))
    if rc != 0:
        raise RuntimeError("oracle softmax failed (%d)" % rc)
    return dst.data
