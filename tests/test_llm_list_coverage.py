"""Which implementation each entry of the reference's own LLM matmul list gets (host only: descriptor creation).

The list is tests/benchdnn/inputs/matmul/option_set_fwks_llm_gpu of the reference tree (1388 benchdnn lines: data
types, tags, scales / zero points with their groups, post-ops, bias, shapes). It is read where it lies when the
reference tree is present and the test is skipped otherwise; nothing of it is kept here. Every line must yield a
primitive descriptor, and every line with a quantized operand (8-bit or 4-bit source or weights) must land on one of
the MFMA / decode kernels, not on the per-element kernel."""
import collections
import os
import re

import pytest

os.environ.setdefault("DNNL_AMD_DESCRIPTOR_ONLY", "1")

import onednn_amd as dnnl  # noqa: E402
from onednn_amd import memory  # noqa: E402

dt = memory.data_type
tag = memory.format_tag
LIST = "/root/reference/tests/benchdnn/inputs/matmul/option_set_fwks_llm_gpu"
DT = {"f16": dt.f16, "bf16": dt.bf16, "f32": dt.f32, "s8": dt.s8, "u8": dt.u8, "s4": dt.s4, "u4": dt.u4, "s32": dt.s32}
ARG = {"src0": dnnl.DNNL_ARG_SRC, "src": dnnl.DNNL_ARG_SRC, "wei": dnnl.DNNL_ARG_WEIGHTS, "dst": dnnl.DNNL_ARG_DST}
A = dnnl.algorithm


def T(name):
    return 2 + tag._plain.index(name)


def eltwise(name):
    return getattr(A, "eltwise_" + name)


def quant_attr(attr, spec, zero_points, nd):
    """benchdnn's --attr-scales / --attr-zero-points: ARG:POLICY[:DT[:GROUPS]] joined by '+'."""
    last, prev = 1 << (nd - 1), 1 << (nd - 2)
    for entry in spec.split("+"):
        f = entry.split(":")
        arg, policy = ARG[f[0]], f[1]
        code = DT[f[2]] if len(f) > 2 else (dt.s32 if zero_points else dt.f32)
        groups = [int(x) for x in f[3].split("x")] if len(f) > 3 else []
        mask = {"common": 0, "per_oc": last, "per_ocic": last | prev, "per_tensor": (1 << nd) - 1}[policy]
        (attr.set_zero_points if zero_points else attr.set_scales)(arg, mask, groups, code)


def descriptor(eng, line):
    o = dict(re.findall(r"--([a-z_-]+)=(\S*)", line))
    m = re.search(r"\s(\d+(?:x\d+)*):(\d+(?:x\d+)*)(?:_n|\s|$)", line)
    sd = [int(x) for x in m.group(1).split("x")]
    wd = [int(x) for x in m.group(2).split("x")]
    nd = len(sd)
    dd = [max(a, b) for a, b in zip(sd[:-2], wd[:-2])] + [sd[-2], wd[-1]]
    s_dt, w_dt, d_dt = [DT[x] for x in o["dt"].split(":")]
    attr = dnnl.primitive_attr()
    if o.get("attr-fpmath"):
        mode, apply_to_int = (o["attr-fpmath"].split(":") + ["false"])[:2]
        attr.set_fpmath_mode(getattr(dnnl.fpmath_mode, mode), apply_to_int == "true")
    if o.get("attr-scales"):
        quant_attr(attr, o["attr-scales"], False, nd)
    if o.get("attr-zero-points"):
        quant_attr(attr, o["attr-zero-points"], True, nd)
    if o.get("attr-post-ops"):
        po = dnnl.post_ops()
        for e in o["attr-post-ops"].split("+"):
            f = e.split(":")
            if f[0].startswith("eltwise_"):
                po.append_eltwise(eltwise(f[0][8:]), float(f[1]) if len(f) > 1 else 0.0, float(f[2]) if len(f) > 2 else 0.0)
            else:
                mask = int(f[2])
                dims = [dd[i] if (mask >> i) & 1 else 1 for i in range(nd)]
                po.append_binary(getattr(A, "binary_" + f[0][7:]), memory.desc(dims, DT[f[1]], T("abcd"[:nd])))
        attr.set_post_ops(po)
    b_md = None
    if o.get("bia-dt"):
        bm = int(o["bia_mask"])
        b_md = memory.desc([dd[i] if (bm >> i) & 1 else 1 for i in range(nd)], DT[o["bia-dt"]], T("abcd"[:nd]))
    pd = dnnl.matmul.primitive_desc(eng, memory.desc(sd, s_dt, T(o["stag"])), memory.desc(wd, w_dt, T(o["wtag"])),
                                    memory.desc(dd, d_dt, T(o["dtag"])), bias_md=b_md, attr=attr)
    quantized = any(c in (dt.s8, dt.u8, dt.s4, dt.u4) for c in (s_dt, w_dt))
    return pd.impl_info_str(), quantized, o["dt"]


@pytest.mark.skipif(not os.path.exists(LIST), reason="the reference tree is not present")
def test_every_quantized_entry_of_the_reference_llm_list_has_a_kernel():
    eng = dnnl.engine(dnnl.engine.kind.gpu, 0)
    count, on_generic = collections.Counter(), []
    total = 0
    for ln, line in enumerate(open(LIST), 1):
        if not line.startswith("--reset"):
            continue
        total += 1
        impl, quantized, dts = descriptor(eng, line)  # raises if the descriptor is refused
        count[(impl, dts)] += 1
        if quantized and impl == "hip:gfx950:generic":
            on_generic.append(ln)
    by_impl = collections.Counter()
    for (impl, _), c in count.items():
        by_impl[impl] += c
    print("[llm list] %d entries: %s" % (total, dict(by_impl)))
    assert total > 1000
    assert not on_generic, "quantized entries on the per-element kernel, lines %s" % on_generic[:20]
    # what is left on the per-element kernel is the list's plain f16 matmuls
    assert {d for (impl, d), _ in count.items() if impl == "hip:gfx950:generic"} <= {"f16:f16:f16"}
