#!/usr/bin/env python3
"""Benchmark of the quantized matmul path on one MI355X.

A "step" is one execute() of the primitive over one batch of synthetic input
already resident in HBM. The headline workload is BASELINE.json's config 2
(W8A8 LLM linear layer: s8 [4096,4096] x s8 [4096,14336], per-token src scales,
per-N weights scales, swish, bf16 dst); the decode GEMV (config 3) and the fp8
GEMM (config 5) are measured in the same run and reported as extra objects of
the same JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2]
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

PEAK_INT8 = 5000.0  # TOP/s, dense MFMA int8 (published MI355X figure)
PEAK_FP8 = 5000.0  # TFLOP/s, dense MFMA fp8
PEAK_HBM = 8000.0  # GB/s
# HBM bytes per launch of the config-2 kernel come from the committed rocprofv3
# summary: its "traffic-record" line holds FETCH_SIZE and WRITE_SIZE (KiB per
# dispatch), the factor each counter needs (what it reads for a 1 GiB device
# copy, --calibrate-copy) and a hash of the kernel's source file at the time.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "gemm_b8y_config2_pmc.txt")
TRAFFIC_SOURCE = os.path.join(ROOT, "onednn_amd", "csrc", "qmm_gemm_b8x.hip")


def traffic_from_profile(kernel="gemm_b8y_kernel"):
    """(bytes per launch or None, note): None when the summary is missing, has no record for the kernel, or was
    taken from another version of the kernel's source file."""
    import hashlib
    try:
        lines = open(TRAFFIC_PROFILE).read().splitlines()
        src_hash = hashlib.sha256(open(TRAFFIC_SOURCE, "rb").read()).hexdigest()[:16]
    except OSError as e:
        return None, "no traffic figure: %s" % e
    for ln in lines:
        tok = ln.split()
        if len(tok) > 2 and tok[0] == "traffic-record:" and tok[1] == kernel:
            kv = dict(t.split("=", 1) for t in tok[2:])
            if kv.get("source_sha256") != src_hash:
                return None, ("the counters in profiles/%s were read on another version of %s"
                              % (os.path.basename(TRAFFIC_PROFILE), os.path.basename(TRAFFIC_SOURCE)))
            nbytes = (float(kv["fetch_kib"]) * float(kv["fetch_factor"])
                      + float(kv["write_kib"]) * float(kv["write_factor"])) * 1024.0
            return nbytes, "profiles/%s: FETCH_SIZE %s KiB x %s + WRITE_SIZE %s KiB x %s" % (
                os.path.basename(TRAFFIC_PROFILE), kv["fetch_kib"], kv["fetch_factor"], kv["write_kib"], kv["write_factor"])
    return None, "no traffic-record for %s in profiles/%s" % (kernel, os.path.basename(TRAFFIC_PROFILE))


def build_c2(dnnl, dt, T, M=4096, K=4096, N=14336, seed=2):
    """Config 2: returns (problem tensors on host, attr builder)."""
    r = np.random.default_rng(seed)
    src = np.clip(np.rint(r.standard_normal((M, K)) * 32), -127, 127).astype(np.int8)
    wei = r.integers(-127, 128, (K, N), dtype=np.int8)
    ss = r.uniform(0.005, 0.05, M).astype(np.float32)
    ws = r.uniform(0.0005, 0.005, N).astype(np.float32)
    return src, wei, ss, ws


# side measurements reported next to the headline configuration: key -> function
EXTRAS = {"decode_gemv": "bench_decode", "fp8_gemm": "bench_fp8", "int8_small": "bench_c1",
          "attention_scores": "bench_c4", "attention_chain": "bench_attention_chain", "attention_fused": "bench_attention_fused", "attention_decode": "bench_attention_decode", "int8_int4_grouped": "bench_w4a8", "quantize_reorder": "bench_quantize",
          "attention_products_f16": "bench_f16_products", "int8_decode_rows": "bench_int8_rows",
          "mfma_ceiling": "bench_mfma_ceiling", "gemm_anatomy": "bench_gemm_anatomy",
          "f16_u8_prefill": "bench_f16_u8_prefill"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="c2", choices=["c2"])
    ap.add_argument("--variant", type=int, default=0, help="mfma_b8 tile configuration (0 = heuristic)")
    ap.add_argument("--no-extras", action="store_true", help="skip the decode / fp8 side measurements")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--only", default=None, choices=sorted(EXTRAS),
                    help="run one of the side measurements alone and print its JSON (for profiling)")
    ap.add_argument("--clock-warmup-s", type=float, default=2.0,
                    help="seconds of untimed launches of the same primitive before the timed steps (after --warmup)")
    ap.add_argument("--cpu-rows", type=int, default=4096, help="rows of config 2 timed on the CPU oracle")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run only a 1 GiB copy kernel (reference point for the rocprofv3 "
                         "FETCH_SIZE / WRITE_SIZE counters) and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (the path shards "
              "along N with each GPU holding its own column slice and no exchange step); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    if args.calibrate_copy:
        from onednn_amd import hiprt as H
        n = 1 << 30
        a, b = H.malloc(n), H.malloc(n)
        H.memset(a, 0x5A, n)
        from onednn_amd import _capi as CA
        for _ in range(3):
            CA.call("qmm_stream_copy", b, a, n, 2048, None)  # stream_copy_kernel: n bytes in, n bytes out
        H.device_synchronize()
        print(json.dumps({"calibrate_copy_bytes": n, "launches": 3, "kernel": "stream_copy_kernel"}))
        return

    import onednn_amd as dnnl
    from onednn_amd import _capi, hiprt, memory
    from qmm_harness import T, assert_bf16_within_1ulp
    dt = memory.data_type
    tag = memory.format_tag
    A = dnnl

    eng = dnnl.engine(dnnl.engine.kind.gpu, 0)
    strm = dnnl.stream(eng)
    hs = C_stream(strm)
    if args.variant:
        os.environ["QMM_GEMM_VARIANT"] = str(args.variant)  # read by the library when a plan is created
    if args.only:
        print(json.dumps({args.only: globals()[EXTRAS[args.only]](A, memory, dt, tag, T, eng, strm, hs, hiprt)}))
        return

    # ------------------------------------------------------------------ c2
    M, K, N = 4096, 4096, 14336
    src, wei, ss, ws = build_c2(dnnl, dt, T)
    attr = A.primitive_attr()
    attr.set_scales(A.DNNL_ARG_SRC, 3, [1, K], dt.f32)
    attr.set_scales_mask(A.DNNL_ARG_WEIGHTS, 2)
    po = A.post_ops()
    po.append_eltwise(A.algorithm.eltwise_swish, 1.0, 0.0)
    attr.set_post_ops(po)
    pd = A.matmul.primitive_desc(eng, memory.desc([M, K], dt.s8, T("ab")), memory.desc([K, N], dt.s8, tag.any),
                                 memory.desc([M, N], dt.bf16, T("ab")), attr=attr)
    prim = A.matmul(pd)
    m_src = memory(pd.src_desc(), eng).write(src)
    m_plain = memory(memory.desc([K, N], dt.s8, T("ab")), eng).write(wei)
    m_wei = memory(pd.weights_desc(), eng)
    A.reorder(m_plain, m_wei).execute(strm, m_plain, m_wei)  # prepack, once, untimed
    m_dst = memory(pd.dst_desc(), eng)
    m_ss = memory(memory.desc([M], dt.f32, T("a")), eng).write(ss)
    m_ws = memory(memory.desc([N], dt.f32, T("a")), eng).write(ws)
    exec_args = {A.DNNL_ARG_SRC: m_src, A.DNNL_ARG_WEIGHTS: m_wei, A.DNNL_ARG_DST: m_dst,
                 A.DNNL_ARG_ATTR_SCALES | A.DNNL_ARG_SRC: m_ss, A.DNNL_ARG_ATTR_SCALES | A.DNNL_ARG_WEIGHTS: m_ws}
    strm.wait()
    del m_plain

    for _ in range(args.warmup):
        prim.execute(strm, exec_args)
    strm.wait()
    # The card idles at a low clock and takes on the order of a second of
    # sustained load to settle at its working point; a handful of 0.2 ms
    # launches does not get there. Run the same launch for a fixed wall time,
    # whatever --warmup says, so the timed steps see the settled clock.
    t_end = time.perf_counter() + args.clock_warmup_s
    while time.perf_counter() < t_end:
        for _ in range(50):
            prim.execute(strm, exec_args)
        strm.wait()
    hiprt.device_synchronize()
    e0, e1 = hiprt.Event(), hiprt.Event()
    t0 = time.perf_counter()
    e0.record(hs)
    for _ in range(args.steps):
        prim.execute(strm, exec_args)
    e1.record(hs)
    strm.wait()
    hiprt.device_synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    ev_ms = e1.elapsed_ms(e0) / args.steps
    ops = 2.0 * M * K * N
    tops = ops / (wall_ms * 1e-3) / 1e12
    kern_tops = ops / (ev_ms * 1e-3) / 1e12

    traffic = traffic_from_profile()
    out = {
        "metric": "int8/fp8 matmul TOPS + % MFMA peak; int4-weight GEMV HBM GB/s, 1 MI355X",
        "value": round(tops, 2), "unit": "TOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "s8", "data": "synthetic",
        "config": {"workload": "config 2: W8A8 linear, s8[4096,4096] x s8[4096,14336] -> bf16, per-token src scales, "
                               "per-N weights scales, swish; weights prepacked via format_tag any",
                   "impl": pd.impl_info_str(), "tile_variant": args.variant,
                   "clock_warmup": "%g s of untimed launches of the same primitive after the --warmup steps, "
                                   "so the timed steps run at the settled clock" % args.clock_warmup_s},
        "roofline": {"bound": "mfma", "achieved": round(kern_tops, 2), "peak": PEAK_INT8, "unit": "TOP/s",
                     "frac": round(kern_tops / PEAK_INT8, 4),
                     "traffic": traffic[0] if args.variant == 0 else None, "traffic_source": traffic[1],
                     "kernel": "gemm_b8y_kernel (int8, 256x256 tile, 16x16x64 MFMA, persistent grid of one workgroup per CU)" if args.variant in (0, 6) else "gemm_b8_kernel (int8)", "kernel_ms": round(ev_ms, 5),
                     "algorithmic_ops_per_launch": ops},
    }
    # what the matrix cores sustain on this card in this run (MFMA-only loop, random operands), next to the published peak
    practical = mfma_ceiling(hiprt, hs, MFMA_KINDS["int8_16x16x64"])
    out["roofline"]["practical_peak"] = round(practical, 1)
    out["roofline"]["frac_of_practical_peak"] = round(kern_tops / practical, 4)
    out["roofline"]["practical_peak_source"] = ("qmm_mfma_ceiling, v_mfma_i32_16x16x64_i8 on register-resident operands drawn "
                                                "like config 2's, same process, measured right after the timed steps")

    # ------------------------------------------------------- CPU baseline
    if not args.no_cpu_baseline:
        import oracle as O
        host = host_cpu()
        # the whole problem where the oracle's K sums run on byte dot products (about a second), a sample of 640 rows
        # (about 10 s) where they run scalar
        rows = min(args.cpu_rows if host["oracle_isa"] != "scalar" else min(args.cpu_rows, 640), M)
        sel = np.linspace(0, M - 1, rows).astype(np.int64)
        s_sub = np.ascontiguousarray(src[sel])
        d_sub = np.zeros((rows, N), np.uint16)
        ncores = min(host["usable_cpus"], int(os.environ.get("OMP_NUM_THREADS", "16")))
        t = time.perf_counter()
        O.matmul(O.Tensor(O.S8, [rows, K], s_sub), O.Tensor(O.S8, [K, N], wei), O.Tensor(O.BF16, [rows, N], d_sub),
                 scales={O.Q_SRC: O.Quant(3, O.F32, np.ascontiguousarray(ss[sel]), (1, K)), O.Q_WEI: O.Quant(2, O.F32, ws)},
                 post_ops=[{"kind": "eltwise", "alg": A.algorithm.eltwise_swish, "alpha": 1.0}], nthreads=ncores)
        cpu_s = time.perf_counter() - t
        out["cpu_baseline"] = {"value": round(2.0 * rows * K * N / cpu_s / 1e12, 5), "unit": "TOP/s", "cores": ncores,
                               "kind": "port", "host": host,
                               # what the reference's own CPU implementation reached where it could be built and run:
                               # a different, smaller host than the one timed here, quoted for scale only
                               "reference_brgemm_elsewhere": {
                                   "where": "a CPU-only container (8 vCPU) where the reference was built, isa avx10_1_512_amx (brg_matmul:avx10_1_512_amx), benchdnn",
                                   "config2_TOPs": 11.3, "config1_TOPs": 17.7, "config4_TOPs": 1.9,
                                   "decode_common_zp_M1_ms": 20.1,
                                   "note": "config 2 there ran with one common src scale: the reference's brgemm has no "
                                           "per-token src scales, and its scalar fallback was not timed"},
                               "sample": "%d of the 4096 rows of config 2 (evenly spaced), full K and N, the C oracle with "
                                         "OpenMP: its K sums on %s, everything else (scales, swish through libm, the bf16 "
                                         "store) per element as the reference's scalar code, %.1f s"
                                         % (rows, "AVX-512 VNNI byte dot products (64 products an instruction)"
                                            if host["oracle_isa"] == "avx512_vnni" else "the scalar loop", cpu_s)}
        # the same rows double as a parity check of the timed kernel's output
        got = m_dst.read(np.uint16, (M, N))[sel]
        import contextlib
        with contextlib.redirect_stdout(sys.stderr):  # stdout carries the one JSON line only
            frac = assert_bf16_within_1ulp(got, d_sub, "bench parity sample", abs_slack=1e-30)  # x*rcp(1+e^-x) is 0 where libm keeps 1e-37
        out["parity_sample"] = {"rows": rows, "max_bf16_ulp": 1, "frac_off_by_one": round(frac, 6)}

    if not args.no_extras:
        for name in EXTRAS:
            out[name] = globals()[EXTRAS[name]](A, memory, dt, tag, T, eng, strm, hs, hiprt)
    print(json.dumps(out))


def host_cpu():
    """Model name, usable CPU count and the widest matmul-relevant ISA of the host."""
    model, flags = "unknown", set()
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name") and model == "unknown":
                    model = line.split(":", 1)[1].strip()
                elif line.startswith("flags") and not flags:
                    flags = set(line.split(":", 1)[1].split())
    except OSError:
        pass
    isa = next((name for name, flag in (("amx_int8", "amx_int8"), ("avx512_vnni", "avx512_vnni"), ("avx512", "avx512f"),
                                        ("avx_vnni", "avx_vnni"), ("avx2", "avx2")) if flag in flags), "baseline")
    try:
        usable = len(os.sched_getaffinity(0))
    except AttributeError:
        usable = os.cpu_count() or 1
    vnni = {"avx512f", "avx512bw", "avx512_vnni"} <= flags and os.environ.get("QMM_ORACLE_SCALAR") != "1"
    return {"model": model, "logical_cpus": os.cpu_count(), "usable_cpus": usable, "widest_isa": isa,
            "oracle_isa": "avx512_vnni" if vnni else "scalar",
            "note": "the oracle is C with OpenMP; the K sums of its integer path run on AVX-512 VNNI byte dot products where "
                    "the host has them (bit-identical to its scalar loop), the rest is scalar"}


def C_stream(strm):
    import ctypes as C
    from onednn_amd import _capi
    p = C.c_void_p()
    _capi.call("dnnl_hip_interop_stream_get_stream", strm._h, C.byref(p))
    return p.value


def bench_decode(A, memory, dt, tag, T, eng, strm, hs, hiprt, sets=64, reps=20, K=4096, N=4096, rows=(1, 4, 8, 16, 1024)):
    """Config 3: bf16 x u4 GEMV, G=128 f16 scales + u4 zero points. The 8.7 MB
    of one weights set would sit in the last-level cache, so `sets` distinct
    copies are cycled; the launches are replayed from a HIP graph so that the
    host does not pace them. After config 3's own shape: the same layer with 8-bit weights, and the decode shape of
    the reference's LLM list (4096 x 14336, f16 and bf16 activations, 29 MB of weights per launch), where the launch
    is long enough for bandwidth rather than launch latency to show, and the list's output projection over 128256
    columns (525 MB of 8-bit weights), where nothing but bandwidth is left."""
    import oracle as O
    G = 128
    r = np.random.default_rng(3)
    res = {}
    cache = {}

    def weights(Kx, Nx, w8):
        key = (Kx, Nx, w8)
        if key not in cache:
            if w8:
                # 8-bit weights-only quantization, one f16 scale and u8 zero point per column
                # (tests/benchdnn/inputs/matmul/option_set_fwks_llm_gpu: --dt=f16:u8:f16, wei:per_oc)
                cache[key] = (r.integers(0, 256, (Kx, Nx)).astype(np.uint8),
                              O.from_f32(O.F16, r.uniform(0.0005, 0.002, Nx).astype(np.float32)),
                              r.integers(100, 156, Nx).astype(np.uint8))
            else:
                cache[key] = (O.pack4(r.integers(0, 16, (Kx, Nx))),
                              O.from_f32(O.F16, r.uniform(0.005, 0.02, (Kx // G, Nx)).astype(np.float32)),
                              O.pack4(r.integers(6, 10, (Kx // G, Nx))))
        return cache[key]

    # (key, M, K, N, activations f16, 8-bit weights, weight sets)
    cases = [("M%d" % m, m, K, N, False, False, sets) for m in rows]
    cases.append(("M1_u8_weights", 1, K, N, True, True, sets))
    for act16 in (True, False):
        for m in (1, 16):
            cases.append(("N14336_%s_M%d" % ("f16" if act16 else "bf16", m), m, 4096, 14336, act16, False, 20))
    # the output projection of the list's decode step (--dt=f16:u8:f32 1x4096:4096x128256, one f16 scale and u8 zero
    # point per column): 525 MB of weights per launch, two sets alternating (one set is twice the last-level cache)
    cases.append(("lm_head_f16_u8_M1", 1, 4096, 128256, True, True, 2))
    # config 3's own format (bf16 x u4, groups of 128) at that width: 262 MB of weights and 12 MB of scales and zero
    # points per launch, three sets in turn
    cases.append(("lm_head_bf16_u4_M1", 1, 4096, 128256, False, False, 3))
    cases.append(("lm_head_bf16_u4_M16", 16, 4096, 128256, False, False, 3))
    for key, M, Kx, Nx, act16, w8, nsets in cases:
        w, sc, zp = weights(Kx, Nx, w8)
        attr = A.primitive_attr()
        adt = dt.f16 if act16 else dt.bf16
        attr.set_fpmath_mode(A.fpmath_mode.f16 if act16 else A.fpmath_mode.bf16, True)
        if w8:
            attr.set_scales(A.DNNL_ARG_WEIGHTS, 2, [], dt.f16)
            attr.set_zero_points(A.DNNL_ARG_WEIGHTS, 2, [], dt.u8)
            wdt = dt.u8
        else:
            attr.set_scales(A.DNNL_ARG_WEIGHTS, 3, [G, 1], dt.f16)
            attr.set_zero_points(A.DNNL_ARG_WEIGHTS, 3, [G, 1], dt.u4)
            wdt = dt.u4
        pd = A.matmul.primitive_desc(eng, memory.desc([M, Kx], adt, T("ab")), memory.desc([Kx, Nx], wdt, tag.any),
                                     memory.desc([M, Nx], adt, T("ab")), attr=attr)
        prim = A.matmul(pd)
        a = O.from_f32(O.F16 if act16 else O.BF16, r.standard_normal((M, Kx)).astype(np.float32))
        m_src = memory(pd.src_desc(), eng).write(a)
        m_dst = memory(pd.dst_desc(), eng)
        plain = memory(memory.desc([Kx, Nx], wdt, T("ab")), eng).write(w)
        wsets, ssets, zsets = [], [], []
        nb = pd.weights_desc().get_size()
        ro = None
        for i in range(nsets):
            # every set is packed by the library's own reorder (a kernel on the stream): the bench issues no
            # device-to-device copy through the HIP runtime
            m = memory(pd.weights_desc(), eng)
            ro = ro or A.reorder(plain, m)
            ro.execute(strm, plain, m)
            wsets.append(m)
        strm.wait()
        for i in range(nsets):
            ssets.append(memory(memory.desc([sc.nbytes], dt.u8, T("a")), eng).write(sc))
            zsets.append(memory(memory.desc([zp.nbytes], dt.u8, T("a")), eng).write(zp))

        def one(i):
            prim.execute(strm, {A.DNNL_ARG_SRC: m_src, A.DNNL_ARG_WEIGHTS: wsets[i], A.DNNL_ARG_DST: m_dst,
                                A.DNNL_ARG_ATTR_SCALES | A.DNNL_ARG_WEIGHTS: ssets[i],
                                A.DNNL_ARG_ATTR_ZERO_POINTS | A.DNNL_ARG_WEIGHTS: zsets[i]})

        for i in range(nsets):
            one(i)
        strm.wait()
        graph = hiprt.Graph(hs, lambda: [one(i) for i in range(nsets)])
        graph.launch()
        strm.wait()
        e0, e1 = hiprt.Event(), hiprt.Event()
        e0.record(hs)
        for _ in range(reps):
            graph.launch()
        e1.record(hs)
        strm.wait()
        us = e1.elapsed_ms(e0) * 1e3 / (reps * nsets)
        nbytes = (Kx * Nx if w8 else Kx * Nx // 2) + sc.nbytes + zp.nbytes + M * Kx * 2 + M * Nx * 2
        floor = None
        if M == 1 and not w8:
            # the same bytes, the same weight sets and the same graph harness, read by a kernel that
            # does nothing else (qmm_stream_read): what the launch gaps and a cold read cost alone
            from onednn_amd import _capi
            sink = memory(memory.desc([8192], dt.u8, T("a")), eng)
            L = _capi.lib()

            def rd(i):
                rc = L.qmm_stream_read(wsets[i].get_data_handle(), nb, ssets[i].get_data_handle(), sc.nbytes,
                                       zsets[i].get_data_handle(), zp.nbytes, sink.get_data_handle(), hs)
                assert rc == 0, rc

            for i in range(nsets):
                rd(i)
            strm.wait()
            g2 = hiprt.Graph(hs, lambda: [rd(i) for i in range(nsets)])
            g2.launch()
            strm.wait()
            f0, f1 = hiprt.Event(), hiprt.Event()
            f0.record(hs)
            for _ in range(reps):
                g2.launch()
            f1.record(hs)
            strm.wait()
            floor = round(f1.elapsed_ms(f0) * 1e3 / (reps * nsets), 3)
        res[key] = {"us_per_launch": round(us, 3), "algorithmic_bytes": nbytes,
                    "GBps": round(nbytes / us / 1e3, 1), "frac_of_hbm_peak": round(nbytes / us / 1e3 / PEAK_HBM, 4),
                    "impl": pd.impl_info_str(), "weight_sets": nsets, "timing": "hip graph of %d launches x %d" % (nsets, reps)}
        if (Kx, Nx) != (K, N):
            res[key]["shape"] = "%d x %d x %d" % (M, Kx, Nx)
        if M > 64:  # the prefill step of the same layer: the tiled kernel, arithmetic-bound
            res[key]["TFLOPs"] = round(2.0 * M * Kx * Nx / us / 1e6, 1)
            res[key]["frac_of_f16_peak"] = round(2.0 * M * Kx * Nx / us / 1e6 / 2500.0, 4)
        if floor is not None:
            res[key]["read_floor_us"] = floor
            res[key]["read_floor_kernel"] = ("qmm_stream_read: 256 workgroups x 512 lanes, 16-byte loads of the same "
                                              "weights + scales + zero points, same graph of %d launches x %d" % (nsets, reps))
        del wsets, ssets, zsets, graph
    return res


def bench_fp8(A, memory, dt, tag, T, eng, strm, hs, hiprt, steps=20, rounds=5, settle_s=1.5):
    """Config 5: f8_e4m3 8192^3, scales 0.5 / 0.25, sum post-op, bf16 dst."""
    import oracle as O
    n = 8192
    r = np.random.default_rng(5)
    # e4m3 codes drawn directly: clip(N(0,1)*4) quantised with the reference rounding on a 1M sample, tiled
    base = O.from_f32(O.F8_E4M3, np.clip(r.standard_normal(1 << 20) * 4, -448, 448).astype(np.float32))
    a = np.resize(base, n * n)
    b = np.resize(np.roll(base, 12345), n * n)
    attr = A.primitive_attr()
    attr.set_scales_mask(A.DNNL_ARG_SRC, 0)
    attr.set_scales_mask(A.DNNL_ARG_WEIGHTS, 0)
    po = A.post_ops()
    po.append_sum(1.0)
    attr.set_post_ops(po)
    pd = A.matmul.primitive_desc(eng, memory.desc([n, n], dt.f8_e4m3, T("ab")), memory.desc([n, n], dt.f8_e4m3, tag.any),
                                 memory.desc([n, n], dt.bf16, T("ab")), attr=attr)
    prim = A.matmul(pd)
    m_src = memory(pd.src_desc(), eng).write(a)
    plain = memory(memory.desc([n, n], dt.f8_e4m3, T("ab")), eng).write(b)
    m_wei = memory(pd.weights_desc(), eng)
    A.reorder(plain, m_wei).execute(strm, plain, m_wei)
    strm.wait()
    del plain
    m_dst = memory(pd.dst_desc(), eng).write(O.from_f32(O.BF16, np.resize(r.standard_normal(1 << 20).astype(np.float32), n * n)))
    m_s = memory(memory.desc([1], dt.f32, T("a")), eng).write(np.array([0.5], np.float32))
    m_w = memory(memory.desc([1], dt.f32, T("a")), eng).write(np.array([0.25], np.float32))
    ex = {A.DNNL_ARG_SRC: m_src, A.DNNL_ARG_WEIGHTS: m_wei, A.DNNL_ARG_DST: m_dst,
          A.DNNL_ARG_ATTR_SCALES | A.DNNL_ARG_SRC: m_s, A.DNNL_ARG_ATTR_SCALES | A.DNNL_ARG_WEIGHTS: m_w}
    # the same protocol as the headline: a fixed wall time of untimed launches so that the clock has settled, then
    # `rounds` groups of `steps` launches between events; min, median and max over the groups are reported and the
    # median is the figure the fraction is quoted on
    ms_all = _settled_times(prim, strm, hs, hiprt, ex, steps, rounds, settle_s)
    ms = float(np.median(ms_all))
    tf = 2.0 * n ** 3 / (ms * 1e-3) / 1e12
    return {"ms_per_launch": round(ms, 4), "ms_min": round(min(ms_all), 4), "ms_max": round(max(ms_all), 4),
            "TFLOPs": round(tf, 1), "frac_of_fp8_peak": round(tf / PEAK_FP8, 4),
            "TFLOPs_best": round(2.0 * n ** 3 / (min(ms_all) * 1e-3) / 1e12, 1),
            "timing": "%g s of untimed launches, then %d groups of %d launches between events; median group" % (settle_s, rounds, steps),
            "impl": pd.impl_info_str()}


def _settled_times(prim, strm, hs, hiprt, ex, steps, rounds, settle_s):
    """ms per launch of `rounds` groups of `steps` launches, after `settle_s` seconds of the same launch."""
    t_end = time.perf_counter() + settle_s
    while time.perf_counter() < t_end:
        for _ in range(20):
            prim.execute(strm, ex)
        strm.wait()
    out = []
    for _ in range(rounds):
        e0, e1 = hiprt.Event(), hiprt.Event()
        e0.record(hs)
        for _ in range(steps):
            prim.execute(strm, ex)
        e1.record(hs)
        strm.wait()
        out.append(e1.elapsed_ms(e0) / steps)
    return out


def _c2_primitive(A, memory, dt, tag, T, eng, strm, data):
    """Config 2's primitive and execute arguments (weights prepacked); `data` = build_c2()."""
    src, wei, ss, ws = data
    M, K = src.shape
    N = wei.shape[1]
    attr = A.primitive_attr()
    attr.set_scales(A.DNNL_ARG_SRC, 3, [1, K], dt.f32)
    attr.set_scales_mask(A.DNNL_ARG_WEIGHTS, 2)
    po = A.post_ops()
    po.append_eltwise(A.algorithm.eltwise_swish, 1.0, 0.0)
    attr.set_post_ops(po)
    pd = A.matmul.primitive_desc(eng, memory.desc([M, K], dt.s8, T("ab")), memory.desc([K, N], dt.s8, tag.any),
                                 memory.desc([M, N], dt.bf16, T("ab")), attr=attr)
    prim = A.matmul(pd)
    m_plain = memory(memory.desc([K, N], dt.s8, T("ab")), eng).write(wei)
    m_wei = memory(pd.weights_desc(), eng)
    A.reorder(m_plain, m_wei).execute(strm, m_plain, m_wei)
    strm.wait()
    ex = {A.DNNL_ARG_SRC: memory(pd.src_desc(), eng).write(src), A.DNNL_ARG_WEIGHTS: m_wei,
          A.DNNL_ARG_DST: memory(pd.dst_desc(), eng),
          A.DNNL_ARG_ATTR_SCALES | A.DNNL_ARG_SRC: memory(memory.desc([M], dt.f32, T("a")), eng).write(ss),
          A.DNNL_ARG_ATTR_SCALES | A.DNNL_ARG_WEIGHTS: memory(memory.desc([N], dt.f32, T("a")), eng).write(ws)}
    return pd, prim, ex


def bench_gemm_anatomy(A, memory, dt, tag, T, eng, strm, hs, hiprt, steps=20, rounds=3, settle_s=1.5):
    """Where a config-2 launch spends its time, from the 256 x 256 kernel's own measurement switches (QMM_MEASURE):
    the launch as it is, the same launch ending after the main loop (no epilogue, nothing stored), and per-tile time
    stamps (core clock counter and a constant 100 MHz counter at kernel entry, loop entry, loop exit and the end of
    the epilogue, and inside the epilogue), which give the cycles per k-step and the clock each phase ran at. Next to
    it the same problem on the 256 x 128 kernel with two workgroups per CU (the default up to K 2048), timed only."""
    import ctypes as C
    from onednn_amd import _capi
    data = build_c2(A, dt, T)
    M, K, N = 4096, 4096, 14336
    ops = 2.0 * M * K * N
    res = {}
    for name, measure, b8x in (("as_is", 0, 3), ("main_loop_only", 1, 3), ("tile_256x128_two_per_cu", 0, 2)):
        with _capi.kernel_variants(measure=measure, b8x=b8x):
            pd, prim, ex = _c2_primitive(A, memory, dt, tag, T, eng, strm, data)
        ms = float(np.median(_settled_times(prim, strm, hs, hiprt, ex, steps, rounds, settle_s)))
        res[name] = {"ms_per_launch": round(ms, 4), "TOPs": round(ops / ms / 1e9, 1),
                     "frac_of_int8_peak": round(ops / ms / 1e9 / PEAK_INT8, 4)}
        del prim, ex
    res["epilogue_share_of_launch"] = round(1.0 - res["main_loop_only"]["ms_per_launch"] / res["as_is"]["ms_per_launch"], 4)
    with _capi.kernel_variants(measure=2, b8x=3):
        pd, prim, ex = _c2_primitive(A, memory, dt, tag, T, eng, strm, data)
    _settled_times(prim, strm, hs, hiprt, ex, steps, 1, settle_s)       # the stamps kept are the last launch's
    strm.wait()
    ntiles = (M // 256) * (N // 256)
    grid = min((ntiles + 7) // 8 * 8, 4096)
    buf = (C.c_uint64 * (grid * 16))()
    rc = _capi.lib().qmm_gemm_stamps_read(buf, C.sizeof(buf))
    assert rc == 0, rc
    t8 = np.frombuffer(buf, dtype=np.uint64).reshape(grid, 8, 2).astype(np.float64)
    t8 = t8[t8[:, 3, 0] > 0]
    t = t8[:, :4]
    cyc = np.diff(t[:, :, 0], axis=1)            # core-clock cycles per phase: prologue, main loop, epilogue
    ns = np.diff(t[:, :, 1], axis=1) * 10.0      # the constant counter ticks at 100 MHz
    ksteps = K // 64
    ghz = cyc / np.maximum(ns, 1.0)
    med = lambda a: float(np.median(a))
    res["stamps"] = {
        "tiles": int(t.shape[0]), "k_steps_per_tile": ksteps,
        "prologue_us": round(med(ns[:, 0]) / 1e3, 2), "main_loop_us": round(med(ns[:, 1]) / 1e3, 2),
        "epilogue_us": round(med(ns[:, 2]) / 1e3, 2),
        "main_loop_cycles_per_k_step": round(med(cyc[:, 1]) / ksteps, 1), "mfma_cycles_per_k_step": 1024,
        "main_loop_clock_GHz": round(med(ghz[:, 1]), 3), "epilogue_clock_GHz": round(med(ghz[:, 2]), 3),
        "epilogue_cycles": round(med(cyc[:, 2]), 0),
        # inside the epilogue: staging of the first half of the tile, its rows (arithmetic + stores), staging of the
        # second half, its rows
        "epilogue_parts_cycles": {
            "stage_half_0": round(med(t8[:, 4, 0] - t8[:, 2, 0]), 0), "rows_half_0": round(med(t8[:, 5, 0] - t8[:, 4, 0]), 0),
            "stage_half_1": round(med(t8[:, 6, 0] - t8[:, 5, 0]), 0), "rows_half_1": round(med(t8[:, 3, 0] - t8[:, 6, 0]), 0)},
        "launch_span_us": round(float(t[:, 3, 1].max() - t[:, 0, 1].min()) * 10.0 / 1e3, 1),
        "note": "medians over the block tiles of one launch; clock = core-clock cycles / time of the constant 100 MHz counter "
                "(10 ns resolution); the stamp code costs a scalar branch per phase"}
    return res


MFMA_KINDS = {"int8_16x16x64": 0, "int8_32x32x32": 1, "fp8_16x16x128": 2, "fp8_32x32x64": 3,
              "int8_16x16x64_weights_held": 4}


def mfma_ceiling(hiprt, hs, kind, data=2, settle_s=1.0, steps=20, rounds=3, groups=256):
    """What the matrix cores sustain on this card: qmm_mfma_ceiling (nothing but the main loop's MFMAs on
    register-resident pseudo-random operands, one wave per SIMD on every CU), timed like the GEMMs: settle, then the
    median of `rounds` groups of `steps` launches. A launch is as long as a GEMM launch (224 k-steps of 64 k = 3.5
    rounds of config 2's tiles; half as many of the 128-k fp8 instruction). Returns T(FL)OP/s."""
    import ctypes as C
    from onednn_amd import _capi
    L = _capi.lib()
    ksteps = 112 if kind == 2 else (448 if kind == 1 else 224)  # kinds 0 and 4: 224
    sink = hiprt.malloc(groups * 1024)
    ops = C.c_double()

    def one():
        rc = L.qmm_mfma_ceiling(kind, ksteps, groups, data, sink, hs, C.byref(ops))
        assert rc == 0, rc

    t_end = time.perf_counter() + settle_s
    while time.perf_counter() < t_end:
        for _ in range(20):
            one()
        hiprt.device_synchronize()
    ms = []
    for _ in range(rounds):
        e0, e1 = hiprt.Event(), hiprt.Event()
        e0.record(hs)
        for _ in range(steps):
            one()
        e1.record(hs)
        hiprt.device_synchronize()
        ms.append(e1.elapsed_ms(e0) / steps)
    hiprt.free(sink)
    return ops.value / (float(np.median(ms)) * 1e-3) / 1e12


def bench_mfma_ceiling(A, memory, dt, tag, T, eng, strm, hs, hiprt):
    """The practical ceilings next to the published 5.0 P(FL)OP/s: MFMA-only loops, random and all-zero operands."""
    res = {"kernel": "qmm_mfma_ceiling: 256 workgroups x 4 waves, only the MFMAs of a 128 x 128 wave tile's k-steps, operands in "
                     "registers (config_data: the value distributions of config 2 / config 5; random_bytes: uniform bytes; two operand sets "
                     "alternating per k-step), no LDS / memory / barrier; "
                     "1 s of untimed launches, then the median of 3 groups of 20 launches"}
    for name, kind in MFMA_KINDS.items():
        res[name] = {"config_data_TOPs": round(mfma_ceiling(hiprt, hs, kind, data=2), 1),
                     "random_bytes_TOPs": round(mfma_ceiling(hiprt, hs, kind, data=0), 1),
                     "zeros_TOPs": round(mfma_ceiling(hiprt, hs, kind, data=1), 1)}
    return res


def _time(prim, strm, hs, hiprt, ex, steps, warm=3):
    for _ in range(warm):
        prim.execute(strm, ex)
    strm.wait()
    e0, e1 = hiprt.Event(), hiprt.Event()
    e0.record(hs)
    for _ in range(steps):
        prim.execute(strm, ex)
    e1.record(hs)
    strm.wait()
    return e1.elapsed_ms(e0) / steps


def bench_c1(A, memory, dt, tag, T, eng, strm, hs, hiprt, steps=200):
    """Config 1: u8 [256,1024] (zero point 128, scale 0.02) x s8 [1024,1024], per-N scales, f32 dst.
    0.54 GOP and 2.4 MB: a launch-latency case, reported for completeness."""
    M, K, N = 256, 1024, 1024
    r = np.random.default_rng(1)
    attr = A.primitive_attr()
    attr.set_scales_mask(A.DNNL_ARG_SRC, 0)
    attr.set_zero_points_mask(A.DNNL_ARG_SRC, 0)
    attr.set_scales_mask(A.DNNL_ARG_WEIGHTS, 2)
    pd = A.matmul.primitive_desc(eng, memory.desc([M, K], dt.u8, T("ab")), memory.desc([K, N], dt.s8, tag.any),
                                 memory.desc([M, N], dt.f32, T("ab")), attr=attr)
    prim = A.matmul(pd)
    m_src = memory(pd.src_desc(), eng).write(r.integers(0, 256, (M, K), dtype=np.uint8))
    plain = memory(memory.desc([K, N], dt.s8, T("ab")), eng).write(r.integers(-128, 128, (K, N), dtype=np.int8))
    m_wei = memory(pd.weights_desc(), eng)
    A.reorder(plain, m_wei).execute(strm, plain, m_wei)
    strm.wait()
    ex = {A.DNNL_ARG_SRC: m_src, A.DNNL_ARG_WEIGHTS: m_wei, A.DNNL_ARG_DST: memory(pd.dst_desc(), eng),
          A.DNNL_ARG_ATTR_SCALES | A.DNNL_ARG_SRC: memory(memory.desc([1], dt.f32, T("a")), eng).write(np.array([0.02], np.float32)),
          A.DNNL_ARG_ATTR_ZERO_POINTS | A.DNNL_ARG_SRC: memory(memory.desc([1], dt.s32, T("a")), eng).write(np.array([128], np.int32)),
          A.DNNL_ARG_ATTR_SCALES | A.DNNL_ARG_WEIGHTS: memory(memory.desc([N], dt.f32, T("a")), eng).write(
              r.uniform(0.001, 0.01, N).astype(np.float32))}
    ms = _time(prim, strm, hs, hiprt, ex, steps, warm=10)
    return {"us_per_launch": round(ms * 1e3, 2), "TOPs": round(2.0 * M * K * N / (ms * 1e-3) / 1e12, 1),
            "impl": pd.impl_info_str(), "note": "back-to-back launches on one stream; launch-latency bound"}


def bench_int8_rows(A, memory, dt, tag, T, eng, strm, hs, hiprt, steps=100, K=4096, N=14336):
    """The decode step of config 2's layer (s8 x s8, per-token and per-column scales, bf16 dst) and of the W8A8 layers of
    the reference's LLM list (--dt=s8:u8:f16, a u8 zero point per column) at 1, 32 and 64 rows: the streaming kernel;
    and the same layers' prefill at 1024 rows (the MFMA kernels; a weights zero point costs a row-sum pre-pass and a
    correction of the staged s32 sums in the epilogue). The 59 MB of weights stay in the last-level cache between
    launches, so the rate is not an HBM figure."""
    out = {}
    r = np.random.default_rng(11)
    for name, wdt, zp in (("s8_s8", dt.s8, False), ("s8_u8_zp_per_column", dt.u8, True)):
        for M in (1, 32, 64, 1024):
            attr = A.primitive_attr()
            attr.set_scales(A.DNNL_ARG_SRC, 3, [1, K], dt.f32)  # per token, as in config 2
            attr.set_scales_mask(A.DNNL_ARG_WEIGHTS, 2)
            if zp:
                attr.set_zero_points(A.DNNL_ARG_WEIGHTS, 2, [], dt.u8)
            pd = A.matmul.primitive_desc(eng, memory.desc([M, K], dt.s8, T("ab")), memory.desc([K, N], wdt, tag.any),
                                         memory.desc([M, N], dt.bf16, T("ab")), attr=attr)
            prim = A.matmul(pd)
            w = r.integers(0, 256, (K, N)).astype(np.uint8) if zp else r.integers(-127, 128, (K, N)).astype(np.int8)
            plain = memory(memory.desc([K, N], wdt, T("ab")), eng).write(w)
            m_wei = memory(pd.weights_desc(), eng)
            A.reorder(plain, m_wei).execute(strm, plain, m_wei)
            strm.wait()
            ex = {A.DNNL_ARG_SRC: memory(pd.src_desc(), eng).write(r.integers(-127, 128, (M, K)).astype(np.int8)),
                  A.DNNL_ARG_WEIGHTS: m_wei, A.DNNL_ARG_DST: memory(pd.dst_desc(), eng),
                  A.DNNL_ARG_ATTR_SCALES | A.DNNL_ARG_SRC: memory(memory.desc([M], dt.f32, T("a")), eng).write(
                      r.uniform(0.005, 0.05, M).astype(np.float32)),
                  A.DNNL_ARG_ATTR_SCALES | A.DNNL_ARG_WEIGHTS: memory(memory.desc([N], dt.f32, T("a")), eng).write(
                      r.uniform(0.0005, 0.005, N).astype(np.float32))}
            if zp:
                ex[A.DNNL_ARG_ATTR_ZERO_POINTS | A.DNNL_ARG_WEIGHTS] = memory(memory.desc([N], dt.u8, T("a")), eng).write(
                    r.integers(100, 156, N).astype(np.uint8))
            ms = _time(prim, strm, hs, hiprt, ex, steps, warm=5)
            nbytes = K * N + M * K + 2 * M * N + 8 * N
            out["%s_M%d" % (name, M)] = {"us_per_launch": round(ms * 1e3, 2), "TOPs": round(2.0 * M * K * N / (ms * 1e-3) / 1e12, 1),
                                         "algorithmic_bytes": nbytes, "GBps_from_cache": round(nbytes / (ms * 1e-3) / 1e9, 1),
                                         "impl": pd.impl_info_str()}
    out["note"] = "back-to-back launches on one stream, one weight set (resident in the last-level cache)"
    return out


PEAK_F16 = 2500.0  # TFLOP/s, dense MFMA f16


def bench_f16_u8_prefill(A, memory, dt, tag, T, eng, strm, hs, hiprt, steps=20):
    """Prefill of the 8-bit weights-only layers of the reference's LLM list (tests/benchdnn/inputs/matmul/
    option_set_fwks_llm_gpu: --dt=f16:u8:f16|f32 --attr-scales=wei:per_oc:f16 --attr-zero-points=wei:per_oc:u8
    --attr-fpmath=f16:true): f16 activations, u8 weights prepacked through format_tag any, one scale and one zero point
    per column. Bound: the f16 matrix cores (the weights are converted in registers between the MFMAs)."""
    out = {}
    r = np.random.default_rng(13)
    for (M, K, N, dst, swish) in ((2176, 4096, 14336, dt.f16, True), (1024, 4096, 14336, dt.f16, False),
                                  (1024, 4096, 4096, dt.f16, False), (1024, 11008, 4096, dt.f32, False),
                                  (2048, 4096, 128256, dt.f32, False)):
        attr = A.primitive_attr()
        attr.set_fpmath_mode(A.fpmath_mode.f16, True)
        attr.set_scales(A.DNNL_ARG_WEIGHTS, 2, [], dt.f16)
        attr.set_zero_points(A.DNNL_ARG_WEIGHTS, 2, [], dt.u8)
        if swish:
            po = A.post_ops()
            po.append_eltwise(A.algorithm.eltwise_swish, 1.0, 0.0)
            attr.set_post_ops(po)
        pd = A.matmul.primitive_desc(eng, memory.desc([M, K], dt.f16, T("ab")), memory.desc([K, N], dt.u8, tag.any),
                                     memory.desc([M, N], dst, T("ab")), attr=attr)
        prim = A.matmul(pd)
        m_wei = memory(pd.weights_desc(), eng)
        plain = memory(memory.desc([K, N], dt.u8, T("ba")), eng).write(r.integers(0, 256, K * N, dtype=np.uint8))
        A.reorder(plain, m_wei).execute(strm, plain, m_wei)
        strm.wait()
        del plain
        ex = {A.DNNL_ARG_SRC: memory(pd.src_desc(), eng).write(r.standard_normal((M, K)).astype(np.float16).view(np.uint16)),
              A.DNNL_ARG_WEIGHTS: m_wei, A.DNNL_ARG_DST: memory(pd.dst_desc(), eng),
              A.DNNL_ARG_ATTR_SCALES | A.DNNL_ARG_WEIGHTS: memory(memory.desc([N], dt.f16, T("a")), eng).write(
                  r.uniform(0.0005, 0.002, N).astype(np.float16).view(np.uint16)),
              A.DNNL_ARG_ATTR_ZERO_POINTS | A.DNNL_ARG_WEIGHTS: memory(memory.desc([N], dt.u8, T("a")), eng).write(
                  r.integers(100, 156, N).astype(np.uint8))}
        ms = _time(prim, strm, hs, hiprt, ex, steps, warm=5)
        tf = 2.0 * M * K * N / (ms * 1e-3) / 1e12
        out["%dx%dx%d_%s%s" % (M, K, N, "f16" if dst == dt.f16 else "f32", "_swish" if swish else "")] = {
            "us_per_launch": round(ms * 1e3, 1), "TFLOPs": round(tf, 1), "frac_of_f16_peak": round(tf / PEAK_F16, 4),
            "impl": pd.impl_info_str()}
    out["note"] = "back-to-back launches on one stream; peak = 2.5 PFLOP/s dense f16"
    return out


def bench_f16_products(A, memory, dt, tag, T, eng, strm, hs, hiprt, steps=100):
    """The attention products as frameworks issue them unfused, shapes of the reference's LLM matmul list
    (tests/benchdnn/inputs/matmul/option_set_fwks_llm_gpu: --dt=f16:f16:f16, abcd tags, 32 heads of 128): one token's
    scores and context over about 1000 keys, and the prefill products at 998 tokens (rows that are only 4-byte
    granular). No quantization attributes; the scores carry the list's clip post-op."""
    out = {}
    r = np.random.default_rng(9)
    h16 = lambda x: x.astype(np.float16).view(np.uint16)
    clip = A.post_ops()
    clip.append_eltwise(A.algorithm.eltwise_clip, -65504.0, 65504.0)
    for name, sd, wd, po in (("decode_scores_1x128x1000", [1, 32, 1, 128], [1, 32, 128, 1000], True),
                             ("decode_context_1x1000x128", [1, 32, 1, 1000], [1, 32, 1000, 128], False),
                             ("decode_scores_1x128x999", [1, 32, 1, 128], [1, 32, 128, 999], True),
                             ("prefill_scores_998x128x998", [1, 32, 998, 128], [1, 32, 128, 998], True),
                             ("prefill_context_998x998x128", [1, 32, 998, 998], [1, 32, 998, 128], False)):
        dd = sd[:-1] + [wd[-1]]
        attr = A.primitive_attr()
        if po:
            attr.set_post_ops(clip)
        pd = A.matmul.primitive_desc(eng, memory.desc(sd, dt.f16, T("abcd")), memory.desc(wd, dt.f16, T("abcd")),
                                     memory.desc(dd, dt.f16, T("abcd")), attr=attr)
        prim = A.matmul(pd)
        ex = {A.DNNL_ARG_SRC: memory(pd.src_desc(), eng).write(h16(r.standard_normal(sd))),
              A.DNNL_ARG_WEIGHTS: memory(pd.weights_desc(), eng).write(h16(r.standard_normal(wd))),
              A.DNNL_ARG_DST: memory(pd.dst_desc(), eng)}
        ms = _time(prim, strm, hs, hiprt, ex, steps, warm=5)
        nbytes = 2 * (int(np.prod(sd)) + int(np.prod(wd)) + int(np.prod(dd)))
        out[name] = {"us_per_launch": round(ms * 1e3, 2), "TFLOPs": round(2.0 * np.prod(sd) * wd[-1] / (ms * 1e-3) / 1e12, 2),
                     "algorithmic_bytes": nbytes, "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1),
                     "frac_of_hbm_peak": round(nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM, 4), "impl": pd.impl_info_str()}
    out["note"] = "back-to-back launches on one stream"
    return out


def bench_c4(A, memory, dt, tag, T, eng, strm, hs, hiprt, steps=20):
    """Config 4: s8 [32,2048,128] x s8 [32,128,2048], per-tensor scales, f32 dst + binary add of a causal
    mask [1,2048,2048]. 34.4 GOP against 537 MB of f32 output: bound by the HBM write stream."""
    B, S, D = 32, 2048, 128
    r = np.random.default_rng(4)
    q = np.clip(np.rint(r.standard_normal((B, S, D)) * 40), -127, 127).astype(np.int8)
    k = np.clip(np.rint(r.standard_normal((B, D, S)) * 40), -127, 127).astype(np.int8)
    mask = np.where(np.arange(S)[None, :] > np.arange(S)[:, None], -1e4, 0).astype(np.float32)[None]
    attr = A.primitive_attr()
    attr.set_scales_mask(A.DNNL_ARG_SRC, 0)
    attr.set_scales_mask(A.DNNL_ARG_WEIGHTS, 0)
    po = A.post_ops()
    mask_md = memory.desc([1, S, S], dt.f32, T("abc"))
    po.append_binary(A.algorithm.binary_add, mask_md)
    attr.set_post_ops(po)
    pd = A.matmul.primitive_desc(eng, memory.desc([B, S, D], dt.s8, T("abc")), memory.desc([B, D, S], dt.s8, tag.any),
                                 memory.desc([B, S, S], dt.f32, T("abc")), attr=attr)
    prim = A.matmul(pd)
    m_src = memory(pd.src_desc(), eng).write(q)
    plain = memory(memory.desc([B, D, S], dt.s8, T("abc")), eng).write(k)
    m_wei = memory(pd.weights_desc(), eng)
    A.reorder(plain, m_wei).execute(strm, plain, m_wei)
    strm.wait()
    ex = {A.DNNL_ARG_SRC: m_src, A.DNNL_ARG_WEIGHTS: m_wei, A.DNNL_ARG_DST: memory(pd.dst_desc(), eng),
          A.DNNL_ARG_ATTR_SCALES | A.DNNL_ARG_SRC: memory(memory.desc([1], dt.f32, T("a")), eng).write(np.array([0.01], np.float32)),
          A.DNNL_ARG_ATTR_SCALES | A.DNNL_ARG_WEIGHTS: memory(memory.desc([1], dt.f32, T("a")), eng).write(np.array([0.012], np.float32)),
          A.DNNL_ARG_ATTR_MULTIPLE_POST_OP(0) | A.DNNL_ARG_SRC_1: memory(mask_md, eng).write(mask)}
    ms = _time(prim, strm, hs, hiprt, ex, steps)
    nbytes = 2 * B * S * D + 4 * B * S * S + 4 * S * S
    # what a launch that only writes the same 537 MB reaches (qmm_stream_write, the best of a few grid sizes): the
    # practical ceiling of a destination-bound launch on this card, next to the published 8 TB/s
    from onednn_amd import _capi
    L = _capi.lib()
    dst_bytes = 4 * B * S * S
    dptr = ex[A.DNNL_ARG_DST].get_data_handle()
    best = None
    for groups in (1024, 2048, 4096, 8192):
        for _ in range(3):
            assert L.qmm_stream_write(dptr, dst_bytes, groups, hs) == 0
        e0, e1 = hiprt.Event(), hiprt.Event()
        e0.record(hs)
        for _ in range(steps):
            L.qmm_stream_write(dptr, dst_bytes, groups, hs)
        e1.record(hs)
        strm.wait()
        t = e1.elapsed_ms(e0) / steps
        if best is None or t < best[0]:
            best = (t, groups)
    return {"ms_per_launch": round(ms, 4), "TOPs": round(2.0 * B * S * S * D / (ms * 1e-3) / 1e12, 1),
            "algorithmic_bytes": nbytes, "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1),
            "frac_of_hbm_peak": round(nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM, 4), "impl": pd.impl_info_str(),
            "write_only_floor": {"ms": round(best[0], 4), "GBps": round(dst_bytes / (best[0] * 1e-3) / 1e9, 1),
                                 "kernel": "qmm_stream_write: %d workgroups x 256 lanes, 16-byte stores over the same 537 MB dst" % best[1]},
            "frac_of_write_only_rate": round((nbytes / ms) / (dst_bytes / best[0]), 4)}


def bench_attention_chain(A, memory, dt, tag, T, eng, strm, hs, hiprt, steps=10):
    """The attention block around config 4 as a chain of primitives: s8 Q x s8 K^T -> f32 scores + causal mask
    (config 4 itself), softmax over the keys -> u8 probabilities (dst scale 1/255), u8 P x s8 V -> bf16. The
    537 MB f32 scores and the 134 MB u8 probabilities cross HBM between the stages: that traffic, not the 68.7 GOP,
    sets the time."""
    B, S, D = 32, 2048, 128
    r = np.random.default_rng(4)
    f = A.prop_kind.forward_inference
    one = lambda v: memory(memory.desc([1], dt.f32, T("a")), eng).write(np.array([v], np.float32))
    q = np.clip(np.rint(r.standard_normal((B, S, D)) * 40), -127, 127).astype(np.int8)
    k = np.clip(np.rint(r.standard_normal((B, S, D)) * 40), -127, 127).astype(np.int8)
    v = np.clip(np.rint(r.standard_normal((B, S, D)) * 40), -127, 127).astype(np.int8)
    mask = np.where(np.arange(S)[None, :] > np.arange(S)[:, None], -1e4, 0).astype(np.float32)[None]
    a1 = A.primitive_attr()
    a1.set_scales_mask(A.DNNL_ARG_SRC, 0)
    a1.set_scales_mask(A.DNNL_ARG_WEIGHTS, 0)
    po = A.post_ops()
    mask_md = memory.desc([1, S, S], dt.f32, T("abc"))
    po.append_binary(A.algorithm.binary_add, mask_md)
    a1.set_post_ops(po)
    s_md = memory.desc([B, S, S], dt.f32, T("abc"))
    p_md = memory.desc([B, S, S], dt.u8, T("abc"))
    o_md = memory.desc([B, S, D], dt.bf16, T("abc"))
    kt_md = memory.desc([B, D, S], dt.s8, T("acb"))  # the K cache [heads, keys, d] viewed as K^T
    pd1 = A.matmul.primitive_desc(eng, memory.desc([B, S, D], dt.s8, T("abc")), kt_md, s_md, attr=a1)
    a2 = A.primitive_attr()
    a2.set_scales_mask(A.DNNL_ARG_DST, 0)
    pd2 = A.softmax_forward.primitive_desc(eng, f, A.algorithm.softmax_accurate, s_md, p_md, 2, a2)
    a3 = A.primitive_attr()
    a3.set_scales_mask(A.DNNL_ARG_SRC, 0)
    a3.set_scales_mask(A.DNNL_ARG_WEIGHTS, 0)
    v_md = memory.desc([B, S, D], dt.s8, T("abc"))
    pd3 = A.matmul.primitive_desc(eng, p_md, v_md, o_md, attr=a3)
    p1, p2, p3 = A.matmul(pd1), A.softmax_forward(pd2), A.matmul(pd3)
    score, prob, out = memory(s_md, eng), memory(p_md, eng), memory(o_md, eng)
    ex1 = {A.DNNL_ARG_SRC: memory(pd1.src_desc(), eng).write(q), A.DNNL_ARG_WEIGHTS: memory(kt_md, eng).write(k),
           A.DNNL_ARG_DST: score, A.DNNL_ARG_ATTR_SCALES | A.DNNL_ARG_SRC: one(0.01),
           A.DNNL_ARG_ATTR_SCALES | A.DNNL_ARG_WEIGHTS: one(0.012),
           A.DNNL_ARG_ATTR_MULTIPLE_POST_OP(0) | A.DNNL_ARG_SRC_1: memory(mask_md, eng).write(mask)}
    ex2 = {A.DNNL_ARG_SRC: score, A.DNNL_ARG_DST: prob, A.DNNL_ARG_ATTR_SCALES | A.DNNL_ARG_DST: one(1.0 / 255.0)}
    ex3 = {A.DNNL_ARG_SRC: prob, A.DNNL_ARG_WEIGHTS: memory(v_md, eng).write(v), A.DNNL_ARG_DST: out,
           A.DNNL_ARG_ATTR_SCALES | A.DNNL_ARG_SRC: one(1.0 / 255.0), A.DNNL_ARG_ATTR_SCALES | A.DNNL_ARG_WEIGHTS: one(0.02)}
    stages = ((p1, ex1), (p2, ex2), (p3, ex3))

    def run():
        for prim, ex in stages:
            prim.execute(strm, ex)

    for _ in range(3):
        run()
    strm.wait()
    ev = [hiprt.Event() for _ in range(4)]
    per = [0.0, 0.0, 0.0]
    for _ in range(steps):
        ev[0].record(hs)
        for i, (prim, ex) in enumerate(stages):
            prim.execute(strm, ex)
            ev[i + 1].record(hs)
        strm.wait()
        for i in range(3):
            per[i] += ev[i + 1].elapsed_ms(ev[i]) / steps
    total = sum(per)
    ops = 2 * 2.0 * B * S * S * D
    moved = (2 * B * S * D + 4 * B * S * S + 4 * S * S) + (4 * B * S * S + B * S * S) + (B * S * S + B * S * D + 2 * B * S * D)
    fused = 3 * B * S * D + 2 * B * S * D  # what one fused kernel would have to move: Q, K, V in, bf16 out
    return {"ms_per_block": round(total, 4), "stages_ms": {"scores": round(per[0], 4), "softmax": round(per[1], 4),
                                                           "values": round(per[2], 4)},
            "TOPs": round(ops / (total * 1e-3) / 1e12, 1), "bytes_moved": moved,
            "GBps": round(moved / (total * 1e-3) / 1e9, 1), "frac_of_hbm_peak": round(moved / (total * 1e-3) / 1e9 / PEAK_HBM, 4),
            "bytes_if_fused": fused,
            "impl": [pd1.impl_info_str(), pd2.impl_info_str(), pd3.impl_info_str()]}


def bench_attention_fused(A, memory, dt, tag, T, eng, strm, hs, hiprt, steps=20, causal=True, S=2048):
    """The same attention block (32 heads, 2048 queries and keys, head size 128, causal) in one kernel: f16 Q and
    dst, K / V either f16 or an s8 cache with per-key f16 scales and zero points. 2 x 2 x 32 x 2048 x 2048 x 128 =
    68.7 GFLOP nominal (the causal half is skipped); bytes: Q, K, V in and dst out."""
    import oracle as O
    B, D = 32, 128
    r = np.random.default_rng(4)
    h16 = lambda x: O.from_f32(O.F16, np.ascontiguousarray(x, np.float32))
    res = {}
    q_md = memory.desc([1, B, S, D], dt.f16, T("abcd"))
    o_md = memory.desc([1, B, S, D], dt.f16, T("abcd"))
    q = memory(q_md, eng).write(h16(r.standard_normal((B, S, D))))
    out = memory(o_md, eng)
    scale = memory(memory.desc([1], dt.f16, T("a")), eng).write(h16(np.array([1.0 / np.sqrt(D)])))
    for name, code in (("f16_cache", dt.f16), ("s8_cache", dt.s8)):
        kt_md = memory.desc([1, B, D, S], code, T("abdc"))
        v_md = memory.desc([1, B, S, D], code, T("abcd"))
        ex = {A.DNNL_ARG_QUERIES: q, A.DNNL_ARG_DST: out, A.DNNL_ARG_SCALE: scale}
        kq = vs = None
        if code == dt.f16:
            ex[A.DNNL_ARG_KEYS] = memory(kt_md, eng).write(h16(r.standard_normal((B, S, D))))
            ex[A.DNNL_ARG_VALUES] = memory(v_md, eng).write(h16(r.standard_normal((B, S, D))))
            nbytes = 4 * B * S * D * 2
        else:
            ex[A.DNNL_ARG_KEYS] = memory(kt_md, eng).write(r.integers(-128, 128, (B, S, D), dtype=np.int8))
            ex[A.DNNL_ARG_VALUES] = memory(v_md, eng).write(r.integers(-128, 128, (B, S, D), dtype=np.int8))
            kq, vs = A.primitive_attr(), A.primitive_attr()
            for a, groups, which in ((kq, [D, 1], A.DNNL_ARG_KEYS), (vs, [1, D], A.DNNL_ARG_VALUES)):
                a.set_scales(A.DNNL_ARG_WEIGHTS, 0b1110, groups, dt.f16)
                a.set_zero_points(A.DNNL_ARG_WEIGHTS, 0b1110, groups, dt.s8)
                sc = h16(r.uniform(0.005, 0.02, (B, S)))
                zp = r.integers(-6, 7, (B, S), dtype=np.int8)
                ex[A.DNNL_ARG_ATTR_SCALES | which] = memory(memory.desc([sc.nbytes], dt.u8, T("a")), eng).write(sc)
                ex[A.DNNL_ARG_ATTR_ZERO_POINTS | which] = memory(memory.desc([zp.nbytes], dt.u8, T("a")), eng).write(zp)
            nbytes = 2 * B * S * D * 2 + 2 * B * S * D + 2 * B * S * 3
        pd = A.sdpa.primitive_desc(eng, q_md, kt_md, v_md, None, dt.f16, o_md, False, B, causal, None, kq, vs)
        ms = _time(A.sdpa(pd), strm, hs, hiprt, ex, steps)
        flops = 2 * 2.0 * B * S * S * D
        res[name] = {"ms_per_block": round(ms, 4), "TFLOPs_nominal": round(flops / (ms * 1e-3) / 1e12, 1),
                     "TFLOPs_computed": round(flops / (2 if causal else 1) / (ms * 1e-3) / 1e12, 1), "algorithmic_bytes": nbytes,
                     "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1), "impl": pd.impl_info_str()}
    return res


def bench_attention_decode(A, memory, dt, tag, T, eng, strm, hs, hiprt, steps=50):
    """One query per head against a long K / V cache (32 heads, head size 128): the decode step of the same block.
    The keys are cut into ranges (one workgroup each), partial results merged by a second small kernel. Bytes: the
    cache once (+ per-key scales and zero points for the 8-bit cache)."""
    import oracle as O
    H, D = 32, 128
    r = np.random.default_rng(8)
    h16 = lambda x: O.from_f32(O.F16, np.ascontiguousarray(x, np.float32))
    res = {}
    q_md = memory.desc([1, H, 1, D], dt.f16, T("abcd"))
    for S in (8192, 32768):
        for name, code in (("f16_cache", dt.f16), ("s8_cache", dt.s8)):
            kt_md = memory.desc([1, H, D, S], code, T("abdc"))
            v_md = memory.desc([1, H, S, D], code, T("abcd"))
            ex = {A.DNNL_ARG_QUERIES: memory(q_md, eng).write(h16(r.standard_normal((H, 1, D)))),
                  A.DNNL_ARG_DST: memory(q_md, eng)}
            kq = vs = None
            if code == dt.f16:
                ex[A.DNNL_ARG_KEYS] = memory(kt_md, eng).write(h16(r.standard_normal((H, S, D))))
                ex[A.DNNL_ARG_VALUES] = memory(v_md, eng).write(h16(r.standard_normal((H, S, D))))
                nbytes = 2 * H * S * D * 2
            else:
                ex[A.DNNL_ARG_KEYS] = memory(kt_md, eng).write(r.integers(-128, 128, (H, S, D), dtype=np.int8))
                ex[A.DNNL_ARG_VALUES] = memory(v_md, eng).write(r.integers(-128, 128, (H, S, D), dtype=np.int8))
                kq, vs = A.primitive_attr(), A.primitive_attr()
                for a, groups, which in ((kq, [D, 1], A.DNNL_ARG_KEYS), (vs, [1, D], A.DNNL_ARG_VALUES)):
                    a.set_scales(A.DNNL_ARG_WEIGHTS, 0b1110, groups, dt.f16)
                    a.set_zero_points(A.DNNL_ARG_WEIGHTS, 0b1110, groups, dt.s8)
                    sc = h16(r.uniform(0.005, 0.02, (H, S)))
                    zp = r.integers(-6, 7, (H, S), dtype=np.int8)
                    ex[A.DNNL_ARG_ATTR_SCALES | which] = memory(memory.desc([sc.nbytes], dt.u8, T("a")), eng).write(sc)
                    ex[A.DNNL_ARG_ATTR_ZERO_POINTS | which] = memory(memory.desc([zp.nbytes], dt.u8, T("a")), eng).write(zp)
                nbytes = 2 * H * S * D + 2 * H * S * 3
            pd = A.sdpa.primitive_desc(eng, q_md, kt_md, v_md, None, dt.undef, q_md, False, H, False, None, kq, vs)
            ms = _time(A.sdpa(pd), strm, hs, hiprt, ex, steps, warm=5)
            res["keys%d_%s" % (S, name)] = {"us_per_step": round(ms * 1e3, 2), "algorithmic_bytes": nbytes,
                                             "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1),
                                             "frac_of_hbm_peak": round(nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM, 4),
                                             "impl": pd.impl_info_str()}
    return res


def bench_w4a8(A, memory, dt, tag, T, eng, strm, hs, hiprt):
    """Dynamic quantization: s8 [M,4096] with f16 scales per row and 128 k, s4 [4096,14336] with f16 scales per
    128 k and column, f16 dst (tests/benchdnn/inputs/matmul/option_set_fwks_llm_gpu:39,51,63,77). M = 2176 is
    the prefill shape (MFMA-bound), M = 32 and 1 the decode shapes (bound by the 29 MB weights stream; 8 weight
    sets are cycled so they do not sit in the last-level cache)."""
    import oracle as O
    K, N, G = 4096, 14336, 128
    r = np.random.default_rng(6)
    w = O.pack4(r.integers(-8, 8, (K, N)))
    sw = O.from_f32(O.F16, r.uniform(0.002, 0.02, (K // G, N)).astype(np.float32))
    plain = memory(memory.desc([K, N], dt.s4, T("ab")), eng).write(w)
    res = {}
    wsets = None
    # the last entry: asymmetric activations (u8 with a u8 zero point per row and 128 k)
    for M, sets, steps, szp in ((2176, 1, 10, False), (32, 8, 40, False), (1, 8, 40, False), (2176, 1, 10, True)):
        attr = A.primitive_attr()
        attr.set_scales(A.DNNL_ARG_SRC, 3, [1, G], dt.f16)
        attr.set_scales(A.DNNL_ARG_WEIGHTS, 3, [G, 1], dt.f16)
        if szp:
            attr.set_zero_points(A.DNNL_ARG_SRC, 3, [1, G], dt.u8)
        pd = A.matmul.primitive_desc(eng, memory.desc([M, K], dt.u8 if szp else dt.s8, T("ab")),
                                     memory.desc([K, N], dt.s4, tag.any),
                                     memory.desc([M, N], dt.f16, T("ab")), attr=attr)
        prim = A.matmul(pd)
        if wsets is None:
            first = memory(pd.weights_desc(), eng)
            A.reorder(plain, first).execute(strm, plain, first)
            strm.wait()
            wsets = [first]
            for _ in range(7):
                m = memory(pd.weights_desc(), eng)
                A.reorder(plain, m).execute(strm, plain, m)
                wsets.append(m)
            strm.wait()
        a8 = np.clip(np.rint(r.standard_normal((M, K)) * 40), -128, 127)
        m_src = memory(pd.src_desc(), eng).write((a8 + 128).astype(np.uint8) if szp else a8.astype(np.int8))
        m_sz = memory(memory.desc([M * (K // G)], dt.u8, T("a")), eng).write(
            r.integers(100, 156, M * (K // G)).astype(np.uint8))
        ss = O.from_f32(O.F16, r.uniform(0.005, 0.05, (M, K // G)).astype(np.float32))
        m_ss = memory(memory.desc([ss.nbytes], dt.u8, T("a")), eng).write(ss)
        m_sw = memory(memory.desc([sw.nbytes], dt.u8, T("a")), eng).write(sw)
        m_dst = memory(pd.dst_desc(), eng)

        def one(i):
            ex = {A.DNNL_ARG_SRC: m_src, A.DNNL_ARG_WEIGHTS: wsets[i % sets], A.DNNL_ARG_DST: m_dst,
                  A.DNNL_ARG_ATTR_SCALES | A.DNNL_ARG_SRC: m_ss, A.DNNL_ARG_ATTR_SCALES | A.DNNL_ARG_WEIGHTS: m_sw}
            if szp:
                ex[A.DNNL_ARG_ATTR_ZERO_POINTS | A.DNNL_ARG_SRC] = m_sz
            prim.execute(strm, ex)

        for i in range(8):
            one(i)
        strm.wait()
        e0, e1 = hiprt.Event(), hiprt.Event()
        e0.record(hs)
        for i in range(steps):
            one(i)
        e1.record(hs)
        strm.wait()
        ms = e1.elapsed_ms(e0) / steps
        ops = 2.0 * M * K * N
        nbytes = K * N // 2 + sw.nbytes + ss.nbytes + M * K + M * N * 2
        res["M%d%s" % (M, "_u8_src_zero_points" if szp else "")] = {"ms_per_launch": round(ms, 4), "TOPs": round(ops / (ms * 1e-3) / 1e12, 1),
                          "frac_of_int8_peak": round(ops / (ms * 1e-3) / 1e12 / PEAK_INT8, 4),
                          "algorithmic_bytes": nbytes, "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1),
                          "frac_of_hbm_peak": round(nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM, 4),
                          "impl": pd.impl_info_str(),
                          "includes": "scale pre-pass%s + GEMM" % (" with weights column sums" if szp else "")}
    return res


def bench_quantize(A, memory, dt, tag, T, eng, strm, hs, hiprt, steps=20):
    """The reorder as a quantizer on the tensors of config 2: its weights f32 [4096,14336] -> s8 with per-column
    scales (once per model), its activations bf16 [4096,4096] -> s8 with per-row scales (every step), and the weights
    again from their [N, K] storage (the transposing kernel). A stream: bytes read + written against HBM bandwidth."""
    r = np.random.default_rng(8)
    res = {}
    for name, sdt, dims, mask, nsc, stag in (("weights_f32_s8_per_column", dt.f32, [4096, 14336], 2, 14336, "ab"),
                                             ("activations_bf16_s8_per_row", dt.bf16, [4096, 4096], 1, 4096, "ab"),
                                             # the same weights as a framework keeps them, [N, K]: a transposing pass
                                             ("weights_f32_stored_n_k_s8_per_column", dt.f32, [4096, 14336], 2, 14336, "ba")):
        attr = A.primitive_attr()
        attr.set_scales_mask(A.DNNL_ARG_DST, mask)
        s_md, d_md = memory.desc(dims, sdt, T(stag)), memory.desc(dims, dt.s8, T("ab"))
        pd = A.reorder.primitive_desc(eng, s_md, eng, d_md, attr=attr)
        prim = A.reorder(pd)
        n = dims[0] * dims[1]
        x = np.resize(r.standard_normal(1 << 20).astype(np.float32), n)
        if sdt == dt.bf16:
            import oracle as O
            x = O.from_f32(O.BF16, x)
        ex = {A.DNNL_ARG_FROM: memory(s_md, eng).write(x), A.DNNL_ARG_TO: memory(d_md, eng),
              A.DNNL_ARG_ATTR_SCALES | A.DNNL_ARG_DST: memory(memory.desc([nsc], dt.f32, T("a")), eng).write(
                  r.uniform(0.01, 0.05, nsc).astype(np.float32))}
        ms = _time(prim, strm, hs, hiprt, ex, steps)
        nbytes = n * (4 if sdt == dt.f32 else 2) + n + nsc * 4
        res[name] = {"us_per_launch": round(ms * 1e3, 2), "algorithmic_bytes": nbytes,
                     "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1),
                     "frac_of_hbm_peak": round(nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM, 4), "impl": pd.impl_info_str()}
    return res


if __name__ == "__main__":
    main()
