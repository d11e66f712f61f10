"""qmm_matmul_launch_static_scratch (include/qmm_hip.h): the launch entry point for
callers that cannot allocate. Called through the C ABI with ctypes mirrors of the
header's structs and checked bit for bit against qmm_matmul_launch with an
allocated scratch buffer, on two calls in a row, the second on a smaller problem
(the static buffer keeps the first call's contents). Further cases put every region
of the scratch layout into the static buffer (the s8 copy of a u8 source behind the
packed weights; the row sums that weights zero points need), and every call is
bracketed by hipMemGetInfo: the device's free memory must not move."""
import ctypes as C

import numpy as np
import pytest

import onednn_amd as dnnl
from onednn_amd import _capi, hiprt, memory
from qmm_harness import T

pytestmark = pytest.mark.gpu

MAX_NDIMS, MAX_PO = 12, 32
DT_F32, DT_S32, DT_S8, DT_U8 = 3, 4, 5, 6  # dnnl_data_type_t
LAYOUT_PLAIN = 0
IMPL_MFMA_B8 = 0
STATIC_SCRATCH_BYTES = 32 << 20


class tensor_t(C.Structure):
    _fields_ = [("dt", C.c_int32), ("ndims", C.c_int32), ("dims", C.c_int64 * MAX_NDIMS),
                ("strides", C.c_int64 * MAX_NDIMS)]


class quant_t(C.Structure):
    _fields_ = [("set", C.c_int32), ("mask", C.c_int32), ("dt", C.c_int32), ("has_groups", C.c_int32),
                ("g0", C.c_int64), ("g1", C.c_int64)]


class postop_t(C.Structure):
    _fields_ = [("kind", C.c_int32), ("alg", C.c_int32), ("alpha", C.c_float), ("beta", C.c_float),
                ("scale", C.c_float), ("zero_point", C.c_int32), ("dt", C.c_int32), ("mask", C.c_int32),
                ("src1", tensor_t)]


class desc_t(C.Structure):
    _fields_ = [("src", tensor_t), ("wei", tensor_t), ("bias", tensor_t), ("dst", tensor_t),
                ("wei_layout", C.c_int32), ("apply_to_int", C.c_int32), ("scales", quant_t * 3),
                ("zps", quant_t * 3), ("npo", C.c_int32), ("reserved", C.c_int32), ("po", postop_t * MAX_PO)]


class args_t(C.Structure):
    _fields_ = [("src", C.c_void_p), ("wei", C.c_void_p), ("bias", C.c_void_p), ("dst", C.c_void_p),
                ("scales", C.c_void_p * 3), ("zps", C.c_void_p * 3), ("po_arg", C.c_void_p * MAX_PO),
                ("scratch", C.c_void_p)]


def _lib():
    L = _capi.lib()
    L.qmm_matmul_scratch_size.restype = C.c_size_t
    L.qmm_matmul_scratch_size.argtypes = [C.c_int, C.POINTER(desc_t)]
    L.qmm_matmul_impl_supports.argtypes = [C.c_int, C.POINTER(desc_t)]
    L.qmm_matmul_plan_create.argtypes = [C.POINTER(C.c_void_p), C.c_int, C.POINTER(desc_t)]
    L.qmm_matmul_plan_destroy.argtypes = [C.c_void_p]
    L.qmm_matmul_plan_destroy.restype = None
    for f in (L.qmm_matmul_launch, L.qmm_matmul_launch_static_scratch):
        f.argtypes = [C.c_void_p, C.POINTER(args_t), C.c_void_p]
        f.restype = C.c_int
    L.qmm_last_error.restype = C.c_char_p
    return L


def _plain(dt_code, shape):
    t = tensor_t()
    t.dt, t.ndims = dt_code, len(shape)
    stride = 1
    for d in reversed(range(len(shape))):
        t.dims[d], t.strides[d] = shape[d], stride
        stride *= shape[d]
    return t


def _desc(M, K, N, src_dt=DT_S8, wei_dt=DT_S8, wei_zp=False):
    """[M,K] x plain [K,N] -> f32 with per-column weights scales: the plain weights are packed into the scratch
    buffer at every launch. wei_zp: one s32 zero point per column."""
    d = desc_t()
    d.src, d.wei, d.dst = _plain(src_dt, (M, K)), _plain(wei_dt, (K, N)), _plain(DT_F32, (M, N))
    d.wei_layout = LAYOUT_PLAIN
    d.scales[1].set, d.scales[1].mask, d.scales[1].dt = 1, 2, DT_F32
    d.scales[1].g0 = d.scales[1].g1 = 1
    for q in (d.scales[0], d.scales[2], d.zps[0], d.zps[1], d.zps[2]):
        q.g0 = q.g1 = 1
    if wei_zp:
        d.zps[1].set, d.zps[1].mask, d.zps[1].dt = 1, 2, DT_S32
    return d


def _free_bytes():
    free, total = C.c_size_t(), C.c_size_t()
    hiprt.check(hiprt.rt().hipMemGetInfo(C.byref(free), C.byref(total)), "hipMemGetInfo")
    return free.value


def _stream_handle(strm):
    p = C.c_void_p()
    _capi.call("dnnl_hip_interop_stream_get_stream", strm._h, C.byref(p))
    return p.value


def _run_case(L, eng, strm, hs, M, K, N, seed, src_dt=DT_S8, wei_dt=DT_S8, wei_zp=False):
    dt = memory.data_type
    r = np.random.default_rng(seed)
    np_of = {DT_S8: np.int8, DT_U8: np.uint8}
    lo = {DT_S8: -128, DT_U8: 0}
    src = r.integers(lo[src_dt], lo[src_dt] + 256, (M, K)).astype(np_of[src_dt])
    wei = r.integers(lo[wei_dt], lo[wei_dt] + 256, (K, N)).astype(np_of[wei_dt])
    if K > 1024:      # keep |acc| below 2^24 so that the f32 product with the scale is the exact one
        src = (src.astype(np.int32) // 8).astype(np_of[src_dt])
    ws = r.uniform(0.001, 0.01, N).astype(np.float32)
    zp = r.integers(100, 140, N).astype(np.int32) if wei_zp else None
    d = _desc(M, K, N, src_dt, wei_dt, wei_zp)
    assert L.qmm_matmul_impl_supports(IMPL_MFMA_B8, C.byref(d)) == 0, L.qmm_last_error()
    need = L.qmm_matmul_scratch_size(IMPL_MFMA_B8, C.byref(d))
    assert 0 < need <= STATIC_SCRATCH_BYTES
    plan = C.c_void_p()
    assert L.qmm_matmul_plan_create(C.byref(plan), IMPL_MFMA_B8, C.byref(d)) == 0, L.qmm_last_error()
    sdt = {DT_S8: dt.s8, DT_U8: dt.u8}
    m_src = memory(memory.desc([M, K], sdt[src_dt], T("ab")), eng).write(src)
    m_wei = memory(memory.desc([K, N], sdt[wei_dt], T("ab")), eng).write(wei)
    m_ws = memory(memory.desc([N], dt.f32, T("a")), eng).write(ws)
    m_zp = memory(memory.desc([N], dt.s32, T("a")), eng).write(zp) if wei_zp else None
    m_scr = memory(memory.desc([need], dt.u8, T("a")), eng)
    m_dsts = [memory(memory.desc([M, N], dt.f32, T("ab")), eng).write(np.full((M, N), np.nan, np.float32))
              for _ in range(2)]
    outs = []
    for entry, m_dst in zip((L.qmm_matmul_launch, L.qmm_matmul_launch_static_scratch), m_dsts):
        a = args_t()
        a.src, a.wei, a.dst = m_src.get_data_handle(), m_wei.get_data_handle(), m_dst.get_data_handle()
        a.scales[1] = m_ws.get_data_handle()
        if wei_zp:
            a.zps[1] = m_zp.get_data_handle()
        # the static-scratch entry point ignores args->scratch
        a.scratch = m_scr.get_data_handle() if entry is L.qmm_matmul_launch else None
        strm.wait()
        before = _free_bytes()
        assert entry(plan, C.byref(a), hs) == 0, L.qmm_last_error()
        strm.wait()
        if entry is L.qmm_matmul_launch_static_scratch:
            assert _free_bytes() == before, "the static-scratch launch changed the device's free memory"
        outs.append(m_dst.read(np.float32, (M, N)).copy())
    L.qmm_matmul_plan_destroy(plan)
    w = wei.astype(np.float64) - (zp.astype(np.float64)[None, :] if wei_zp else 0.0)
    acc = src.astype(np.float64) @ w
    assert np.abs(acc).max() < 2 ** 24
    want = acc.astype(np.float32) * ws  # exact: |acc| < 2^24
    assert np.array_equal(outs[0], want), "existing entry point against the exact product"
    assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32)), \
        "static-scratch entry point differs from qmm_matmul_launch (%dx%dx%d)" % (M, K, N)


def test_static_scratch_entry_point_matches_launch():
    L = _lib()
    eng = dnnl.engine(dnnl.engine.kind.gpu, 0)
    strm = dnnl.stream(eng)
    hs = _stream_handle(strm)
    _run_case(L, eng, strm, hs, 192, 512, 320, 11)
    # second call, smaller problem: the buffer still holds the first call's packed weights
    _run_case(L, eng, strm, hs, 48, 128, 96, 12)


def test_static_scratch_holds_every_scratch_region():
    """The s8 copy of a u8 source (problems large enough for the 256 x 256 kernels: the copy lies behind the packed
    weights) and the per-row sums of weights zero points, u8 weights included, through the static buffer; then a
    small plain case again, over whatever those left behind."""
    L = _lib()
    eng = dnnl.engine(dnnl.engine.kind.gpu, 0)
    strm = dnnl.stream(eng)
    hs = _stream_handle(strm)
    _run_case(L, eng, strm, hs, 4096, 320, 3072, 13, src_dt=DT_U8)
    _run_case(L, eng, strm, hs, 192, 512, 320, 14, wei_dt=DT_U8, wei_zp=True)
    _run_case(L, eng, strm, hs, 200, 256, 160, 15, src_dt=DT_U8, wei_zp=True)
    _run_case(L, eng, strm, hs, 48, 128, 96, 16)


def test_static_scratch_rejects_oversized_problem():
    L = _lib()
    d = _desc(64, 8192, 8192)  # 64 MiB of packed weights
    assert L.qmm_matmul_scratch_size(IMPL_MFMA_B8, C.byref(d)) > STATIC_SCRATCH_BYTES
    plan = C.c_void_p()
    assert L.qmm_matmul_plan_create(C.byref(plan), IMPL_MFMA_B8, C.byref(d)) == 0
    a = args_t()
    rc = L.qmm_matmul_launch_static_scratch(plan, C.byref(a), None)
    L.qmm_matmul_plan_destroy(plan)
    assert rc == 2  # QMM_INVALID_ARGUMENTS
    assert b"static" in L.qmm_last_error()
