"""Every distinct attribute combination of the quantized entries of the reference's LLM matmul list
(tests/benchdnn/inputs/matmul/option_set_fwks_llm_gpu; shapes dropped, kept as the fixture
tests/golden/llm_matmul_combos.json with the script that wrote it) at a reduced shape, at one decode and one prefill
row count, against the CPU oracle.

Integer-source combinations run on exact-arithmetic data (small integers, power-of-two scales, post-op operands with few
bits), where every summation order gives the same bits: bit-exact, except behind a swish / gelu (the device's exp / erf /
tanh are not the host libm's: one f16 step, 2e-6 relative in f32). 16-bit-source (weights decompression) combinations:
the bar of that path, rel 1e-2 of the mean magnitude."""
import json
import os
import sys

import numpy as np
import pytest

import onednn_amd as dnnl
import oracle as O
from qmm_harness import Problem, TensorSpec, assert_bit_exact, assert_f32_close, dt

pytestmark = pytest.mark.gpu
A = dnnl.algorithm
DT = {"f16": dt.f16, "bf16": dt.bf16, "f32": dt.f32, "s8": dt.s8, "u8": dt.u8, "s4": dt.s4, "u4": dt.u4, "s32": dt.s32}
COMBOS = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "llm_matmul_combos.json")))
K, N = 256, 96
RANGE = {dt.s8: (-128, 128), dt.u8: (0, 256), dt.s4: (-8, 8), dt.u4: (0, 16)}


def say(msg):
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def ctx():
    eng = dnnl.engine(dnnl.engine.kind.gpu, 0)
    return eng, dnnl.stream(eng)


def quant_entries(spec, M, r, zero_points, wide_weights):
    """benchdnn's ARG:POLICY[:DT[:GROUPS]] entries -> the harness's {name: (mask, dt, groups, values)}."""
    out = {}
    for entry in filter(None, spec.split("+")):
        f = entry.split(":")
        name = "src" if f[0].startswith("src") else f[0]
        code = DT[f[2]]
        groups = None
        if len(f) > 3:
            groups = tuple(K if g == "K" else int(g) for g in f[3].split("x"))
        rows = M if name == "src" else K
        cols = K if name == "src" else N
        if f[1] == "per_oc":
            mask, shape = 2, (N,)
        else:  # per_ocic with groups
            mask, shape = 3, (rows // groups[0], cols // groups[1])
        if zero_points:
            lo, hi = (100, 156) if (name == "src" or wide_weights) else (5, 12)
            vals = r.integers(lo, hi, shape)
        else:
            vals = 2.0 ** r.integers(-6, -3, shape)
        out[name] = (mask, code, groups, vals)
    return out


def build(c, M, seed):
    r = np.random.default_rng(seed)
    s_dt, w_dt, d_dt = [DT[x] for x in c["dt"].split(":")]
    int_src = s_dt in (dt.s8, dt.u8)
    if int_src:
        lo, hi = RANGE[s_dt]
        s = np.clip(np.rint(r.standard_normal((M, K)) * 20) + (128 if s_dt == dt.u8 else 0), lo, hi - 1)
    else:
        s = r.standard_normal((M, K)).astype(np.float32)
    w = r.integers(*RANGE[w_dt], (K, N))
    src = TensorSpec(s_dt, [M, K], c["stag"], s)
    wei = TensorSpec(w_dt, [K, N], c["wtag"], w)
    dst = TensorSpec(d_dt, [M, N], c["dtag"])
    wide = w_dt in (dt.u8, dt.s8)
    scales = quant_entries(c["scales"], M, r, False, wide)
    zps = quant_entries(c["zero_points"], M, r, True, wide)
    post_ops, smooth = [], False
    for e in filter(None, c["post_ops"].split("+")):
        f = e.split(":")
        if f[0].startswith("eltwise_"):
            smooth = True
            post_ops.append({"kind": "eltwise", "alg": getattr(A, f[0]), "alpha": float(f[1]) if len(f) > 1 else 0.0,
                             "beta": float(f[2]) if len(f) > 2 else 0.0})
        else:
            mask = int(f[2])
            dims = [M if mask & 1 else 1, N if mask & 2 else 1]
            vals = r.integers(-8, 9, dims) * 0.25
            post_ops.append({"kind": "binary", "alg": getattr(A, f[0]), "src1": TensorSpec(DT[f[1]], dims, None, vals.astype(np.float32))})
    bias = None
    if c["bia_dt"]:
        bm = int(c["bia_mask"])
        bias = TensorSpec(DT[c["bia_dt"]], [M if bm & 1 else 1, N if bm & 2 else 1], None,
                          (r.integers(-8, 9, N) * 0.25).astype(np.float32).reshape(1, N))
    mode, apply_to_int = (c["fpmath"].split(":") + ["false"])[:2] if c["fpmath"] else ("strict", "false")
    p = Problem(src, wei, dst, bias=bias, scales=scales, zps=zps, post_ops=post_ops, apply_to_int=apply_to_int == "true",
                fpmath=getattr(dnnl.fpmath_mode, mode))
    return p, int_src, smooth, d_dt


@pytest.mark.parametrize("M", [1, 70])
@pytest.mark.parametrize("idx", range(len(COMBOS)))
def test_combination(ctx, idx, M):
    eng, strm = ctx
    c = COMBOS[idx]
    say("llm combination %d M=%d: %s sc=%s zp=%s po=%s bias=%s" % (idx, M, c["dt"], c["scales"], c["zero_points"],
                                                                   c["post_ops"], c["bia_dt"]))
    p, int_src, smooth, d_dt = build(c, M, 1000 + idx)
    got, pd = p.run_gpu(eng, strm, weights_any=True, return_pd=True)
    assert pd.impl_info_str() != "hip:gfx950:generic", pd.impl_info_str()
    want = p.run_oracle()
    if int_src and not smooth:
        assert_bit_exact(got, want, "combination %d" % idx)
        return
    g, w = O.to_f32(d_dt, got).reshape(M, N), O.to_f32(d_dt, want).reshape(M, N)
    if int_src:
        rel = 2.0 ** -10 if d_dt == dt.f16 else 2e-6
        assert_f32_close(g, w, rel=rel, scale=np.abs(w).mean(), what="combination %d" % idx, max_slack_frac=1.0)
    else:
        assert_f32_close(g, w, rel=1e-2, scale=np.abs(w).mean(), what="combination %d" % idx, max_slack_frac=1.0)
