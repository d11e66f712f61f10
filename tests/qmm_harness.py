"""Shared machinery of the parity tests: one problem description that is run
both by the CPU oracle and by the library through its C ABI (the dnnl mirror in
onednn_amd), plus the comparison rules of the path:

    s32 / s8 / u8 dst   bit-exact
    f32 dst             rel 1e-5
    bf16 dst            within 1 bf16 ulp of the rounded reference
    int4 decompression  rel 1e-2
"""
import numpy as np

import onednn_amd as dnnl
import oracle as O
from onednn_amd import memory

dt = memory.data_type
tag = memory.format_tag

ARG = {"src": dnnl.DNNL_ARG_SRC, "wei": dnnl.DNNL_ARG_WEIGHTS, "dst": dnnl.DNNL_ARG_DST}
QIDX = {"src": O.Q_SRC, "wei": O.Q_WEI, "dst": O.Q_DST}


def T(name):
    return 2 + tag._plain.index(name)


def plain_tag(nd):
    return T("abcdefghijkl"[:nd])


def tag_strides(dims, name):
    """Element strides of a plain tag, e.g. 'acb'."""
    strides = [0] * len(dims)
    s = 1
    for ch in reversed(name):
        d = ord(ch) - ord("a")
        strides[d] = s
        s *= max(dims[d], 1)
    return strides


def storage(dtype_code, n):
    """Zeroed numpy buffer holding n elements of a dnnl data type."""
    if dtype_code in (dt.s4, dt.u4):
        return np.zeros((n + 1) // 2, np.uint8)
    return np.zeros(n, O.STORAGE[dtype_code])


def span(dims, strides):
    if any(d == 0 for d in dims):
        return 0
    return 1 + sum((d - 1) * s for d, s in zip(dims, strides))


class TensorSpec:
    """dims + dt + layout ('ab', 'acb', ... or explicit strides) + data.

    `data` is given in LOGICAL row-major order (numpy array of logical values:
    ints for integer types, float32 for float types) and is laid out / encoded
    here; `raw` is the resulting storage buffer."""

    def __init__(self, dtype_code, dims, layout=None, values=None):
        self.dt = dtype_code
        self.dims = [int(d) for d in dims]
        nd = len(dims)
        if layout is None:
            layout = "abcdefghijkl"[:nd]
        self.layout = layout
        self.strides = (tag_strides(self.dims, layout) if isinstance(layout, str)
                        else [int(s) for s in layout])
        self.raw = storage(dtype_code, span(self.dims, self.strides))
        if values is not None:
            self.set(values)

    def _offsets(self):
        idx = np.indices(self.dims).reshape(len(self.dims), -1)
        return (idx * np.array(self.strides)[:, None]).sum(0)

    def set(self, values):
        v = np.asarray(values).reshape(-1)
        off = self._offsets()
        if self.dt in (dt.s4, dt.u4):
            nib = np.zeros(self.raw.size * 2, np.uint8)
            nib[off] = v.astype(np.int64) & 0xF
            self.raw[:] = nib[0::2] | (nib[1::2] << 4)
        elif self.dt in (dt.f32, dt.s32, dt.s8, dt.u8):
            self.raw[off] = v.astype(self.raw.dtype)
        else:
            self.raw[off] = O.from_f32(self.dt, v.astype(np.float32))

    def logical(self, raw=None):
        """Decode a storage buffer back to logical row-major values (f32/int)."""
        raw = self.raw if raw is None else raw.view(self.raw.dtype)
        off = self._offsets()
        if self.dt in (dt.s4, dt.u4):
            v = O.unpack4(raw, raw.size * 2, self.dt == dt.s4)[off]
        elif self.dt in (dt.f32, dt.s32, dt.s8, dt.u8):
            v = raw[off]
        else:
            v = O.to_f32(self.dt, raw)[off]
        return v.reshape(self.dims)

    def oracle(self, raw=None):
        return O.Tensor(self.dt, self.dims, self.raw if raw is None else raw, self.strides)

    def md(self, any_layout=False):
        if any_layout:
            return memory.desc(self.dims, self.dt, tag.any)
        return memory.desc(self.dims, self.dt, self.strides)


class Problem:
    """A matmul problem: tensors, attributes, post-ops."""

    def __init__(self, src, wei, dst, bias=None, scales=None, zps=None, post_ops=None,
                 apply_to_int=False, fpmath=dnnl.fpmath_mode.strict):
        self.src, self.wei, self.dst, self.bias = src, wei, dst, bias
        # scales / zps: {"src"|"wei"|"dst": (mask, dt, groups or None, values)}
        self.scales, self.zps = scales or {}, zps or {}
        self.post_ops = post_ops or []
        self.apply_to_int, self.fpmath = apply_to_int, fpmath

    # ---- quant buffers ----
    @staticmethod
    def _quant_raw(code, values):
        v = np.asarray(values).reshape(-1)
        if code in (dt.s4, dt.u4):
            return O.pack4(v)
        if code in (dt.s32, dt.s8, dt.u8):
            return v.astype(O.STORAGE[code])
        if code == dt.e8m0:
            # the reference's encoder keeps the f32 exponent field (src/common/float8.cpp:28-34)
            return ((v.astype(np.float32).view(np.uint32) >> 23) & 0xFF).astype(np.uint8)
        return O.from_f32(code, v.astype(np.float32))

    # ---- oracle ----
    def run_oracle(self, k_group_mode=O.KGROUP_WHOLE, nthreads=0, dst_init=None):
        dst_raw = self.dst.raw.copy() if dst_init is None else dst_init.copy()
        scales, zps, keep = {}, {}, []
        for name, (mask, code, groups, values) in self.scales.items():
            raw = self._quant_raw(code, values)
            scales[QIDX[name]] = O.Quant(mask, code, raw, groups)
        for name, (mask, code, groups, values) in self.zps.items():
            raw = self._quant_raw(code, values)
            zps[QIDX[name]] = O.Quant(mask, code, raw, groups)
        pos = []
        for po in self.post_ops:
            po = dict(po)
            if po["kind"] == "binary":
                po["src1"] = po["src1"].oracle()
            elif po["kind"] == "prelu":
                po["weights"] = np.ascontiguousarray(po["weights"], np.float32)
            pos.append(po)
        O.matmul(self.src.oracle(), self.wei.oracle(), self.dst.oracle(dst_raw),
                 bias=self.bias.oracle() if self.bias is not None else None,
                 scales=scales, zps=zps, post_ops=pos, apply_to_int=self.apply_to_int,
                 nthreads=nthreads, k_group_mode=k_group_mode)
        return dst_raw

    # ---- library ----
    def attr(self, scratchpad_user=False):
        a = dnnl.primitive_attr()
        for name, (mask, code, groups, _) in self.scales.items():
            if groups is None and code == dt.f32:
                a.set_scales_mask(ARG[name], mask)
            else:
                a.set_scales(ARG[name], mask, list(groups or []), code)
        for name, (mask, code, groups, _) in self.zps.items():
            if groups is None and code == dt.s32:
                a.set_zero_points_mask(ARG[name], mask)
            else:
                a.set_zero_points(ARG[name], mask, list(groups or []), code)
        if self.apply_to_int or self.fpmath != dnnl.fpmath_mode.strict:
            a.set_fpmath_mode(self.fpmath, self.apply_to_int)
        if self.post_ops:
            po = dnnl.post_ops()
            for e in self.post_ops:
                if e["kind"] == "sum":
                    po.append_sum(e.get("scale", 1.0), e.get("zero_point", 0), e.get("dt", 0))
                elif e["kind"] == "eltwise":
                    po.append_eltwise(e["alg"], e.get("alpha", 0.0), e.get("beta", 0.0))
                elif e["kind"] == "binary":
                    po.append_binary(e["alg"], e["src1"].md())
                elif e["kind"] == "prelu":
                    po.append_prelu(e["mask"])
            a.set_post_ops(po)
        if scratchpad_user:
            a.set_scratchpad_mode(dnnl.scratchpad_mode.user)
        return a

    def primitive_desc(self, eng, weights_any=False, impl=None, scratchpad_user=False):
        pd = dnnl.matmul.primitive_desc(
            eng, self.src.md(), self.wei.md(weights_any), self.dst.md(),
            bias_md=self.bias.md() if self.bias is not None else None,
            attr=self.attr(scratchpad_user))
        if impl is not None:
            while pd.impl_info_str() != impl:
                if not pd.next_impl():
                    raise RuntimeError("implementation %s does not take this problem" % impl)
        return pd

    def runtime_primitive_desc(self, eng, runtime, weights_any=False):
        """`runtime`: {"src" / "wei" / "dst" / "bias": dim indices that become
        DNNL_RUNTIME_DIM_VAL}; layouts must be tags. weights_any: the weights
        (all of their dims known) are given as format_tag::any."""
        def md(spec, name):
            dims = list(spec.dims)
            for i in runtime.get(name, ()):
                dims[i] = dnnl.DNNL_RUNTIME_DIM_VAL
            if name == "wei" and weights_any:
                return memory.desc(dims, spec.dt, tag.any)
            return memory.desc(dims, spec.dt, T(spec.layout))
        return dnnl.matmul.primitive_desc(
            eng, md(self.src, "src"), md(self.wei, "wei"), md(self.dst, "dst"),
            bias_md=md(self.bias, "bias") if self.bias is not None else None, attr=self.attr())

    def run_gpu(self, eng, strm, weights_any=False, impl=None, dst_init=None,
                scratchpad_user=False, return_pd=False, prim=None, prim_wei_md=None):
        """`prim`: a primitive made from runtime_primitive_desc (its memory
        objects then carry this problem's own descriptors; prim_wei_md: the
        prepacked weights descriptor that primitive descriptor reports)."""
        if prim is not None:
            pd = _ConcreteDescs(self, prim_wei_md)
        else:
            pd = self.primitive_desc(eng, weights_any, impl, scratchpad_user)
            prim = dnnl.matmul(pd)
        args = {}
        args[dnnl.DNNL_ARG_SRC] = memory(pd.src_desc(), eng).write(self.src.raw)
        wmd = pd.weights_desc()
        if wmd.get_format_kind() == memory.format_kind.opaque:
            plain = memory(self.wei.md(), eng).write(self.wei.raw)
            packed = memory(wmd, eng)
            dnnl.reorder(plain, packed).execute(strm, plain, packed)
            args[dnnl.DNNL_ARG_WEIGHTS] = packed
        else:
            args[dnnl.DNNL_ARG_WEIGHTS] = memory(wmd, eng).write(self.wei.raw)
        dst_mem = memory(pd.dst_desc(), eng)
        dst_mem.write(self.dst.raw if dst_init is None else dst_init)
        args[dnnl.DNNL_ARG_DST] = dst_mem
        if self.bias is not None:
            args[dnnl.DNNL_ARG_BIAS] = memory(pd.bias_desc(), eng).write(self.bias.raw)
        for name, (mask, code, groups, values) in self.scales.items():
            raw = self._quant_raw(code, values)
            md = memory.desc([raw.nbytes], dt.u8, T("a"))
            args[dnnl.DNNL_ARG_ATTR_SCALES | ARG[name]] = memory(md, eng).write(raw)
        for name, (mask, code, groups, values) in self.zps.items():
            raw = self._quant_raw(code, values)
            md = memory.desc([raw.nbytes], dt.u8, T("a"))
            args[dnnl.DNNL_ARG_ATTR_ZERO_POINTS | ARG[name]] = memory(md, eng).write(raw)
        for i, e in enumerate(self.post_ops):
            if e["kind"] == "binary":
                args[dnnl.DNNL_ARG_ATTR_MULTIPLE_POST_OP(i) | dnnl.DNNL_ARG_SRC_1] = \
                    memory(e["src1"].md(), eng).write(e["src1"].raw)
            elif e["kind"] == "prelu":
                w = np.ascontiguousarray(e["weights"], np.float32)
                md = memory.desc([w.size], dt.f32, T("a"))
                args[dnnl.DNNL_ARG_ATTR_MULTIPLE_POST_OP(i) | dnnl.DNNL_ARG_WEIGHTS] = \
                    memory(md, eng).write(w)
        if scratchpad_user and not pd.scratchpad_desc().is_zero():
            args[dnnl.DNNL_ARG_SCRATCHPAD] = memory(pd.scratchpad_desc(), eng)
        prim.execute(strm, args)
        strm.wait()
        out = dst_mem.read(self.dst.raw.dtype)
        return (out, pd) if return_pd else out


class _ConcreteDescs:
    """Stands in for a primitive descriptor when the primitive was created with
    runtime dims: the descriptors are the problem's own."""

    def __init__(self, p, wei_md=None):
        self.p = p
        self.wei_md = wei_md

    def src_desc(self):
        return self.p.src.md()

    def weights_desc(self):
        return self.wei_md if self.wei_md is not None else self.p.wei.md()

    def dst_desc(self):
        return self.p.dst.md()

    def bias_desc(self):
        return self.p.bias.md()

    def scratchpad_desc(self):
        return memory.desc()


# ---------------------------------------------------------------------------
# comparison rules
def assert_bit_exact(got, want, what=""):
    got, want = np.asarray(got), np.asarray(want)
    if not np.array_equal(got.view(np.uint8), want.view(np.uint8)):
        bad = np.flatnonzero(got.reshape(-1) != want.reshape(-1))
        raise AssertionError("%s: %d of %d elements differ, first at %d: got %r want %r"
                             % (what, bad.size, got.size, bad[0], got.reshape(-1)[bad[0]],
                                want.reshape(-1)[bad[0]]))


# Where a tolerance is widened (`scale` / `abs_slack` below), the share of elements
# that needed the wider bound is measured, printed and capped: a regression that
# pushes a large part of the outputs into the slack must not pass.
SLACK_FRAC_MAX = 0.02


def _report_slack(what, frac, ceiling):
    if frac > 0:
        print("[slack] %s: %.4f %% of the elements needed the widened bound (ceiling %.2f %%)"
              % (what, 100 * frac, 100 * ceiling), flush=True)
    assert frac <= ceiling, "%s: %.3f %% of the elements needed the widened bound (ceiling %.2f %%)" % (
        what, 100 * frac, 100 * ceiling)


def assert_f32_close(got, want, rel=1e-5, scale=None, what="", max_slack_frac=SLACK_FRAC_MAX):
    """|got - want| <= rel * max(|want|, scale): `scale` is the magnitude of the
    terms of the sum (a result that cancels to ~0 cannot be compared relative to
    itself). Returns the fraction of elements that were outside rel * |want| and
    only passed through `scale`; that fraction may not exceed max_slack_frac."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    ref = np.abs(want) if scale is None else np.maximum(np.abs(want), scale)
    err = np.abs(got - want)
    same = (got == want) | (np.isnan(got) & np.isnan(want))
    ok = (err <= rel * ref) | same
    if not ok.all():
        i = np.argmax(err / np.maximum(ref, 1e-300))
        raise AssertionError("%s: max rel err %.3g at %d (got %r want %r)"
                             % (what, (err / np.maximum(ref, 1e-300)).reshape(-1)[i], i,
                                got.reshape(-1)[i], want.reshape(-1)[i]))
    strict = (err <= rel * np.abs(want)) | same
    frac = float(1.0 - strict.mean()) if strict.size else 0.0
    if scale is not None:
        _report_slack(what, frac, max_slack_frac)
    return frac


def bf16_ulp_distance(a_raw, b_raw):
    """Distance in bf16 representable values between two raw bf16 arrays."""
    def key(r):
        r = r.astype(np.int32)
        return np.where(r & 0x8000, -(r & 0x7FFF), r & 0x7FFF)
    return np.abs(key(np.asarray(a_raw)) - key(np.asarray(b_raw)))


def assert_bf16_within_1ulp(got_raw, want_raw, what="", abs_slack=None, max_slack_frac=SLACK_FRAC_MAX):
    """bf16 results at most one representable value apart. `abs_slack` (array or
    scalar) additionally accepts |got - want| <= abs_slack: a kernel that sums
    in another order than the reference carries the f32 bar (1e-5 of the
    magnitude of the summed terms) into results that cancel towards zero, where
    one bf16 ulp is arbitrarily small. The fraction of elements more than one
    representable value apart that only passed through abs_slack may not exceed
    max_slack_frac. Returns the fraction of elements that differ at all."""
    d = bf16_ulp_distance(got_raw, want_raw).reshape(-1)
    if abs_slack is not None:
        g = O.to_f32(O.BF16, np.asarray(got_raw)).astype(np.float64).reshape(-1)
        w = O.to_f32(O.BF16, np.asarray(want_raw)).astype(np.float64).reshape(-1)
        slack = np.asarray(abs_slack, np.float64).reshape(-1)
        ok = np.abs(g - w) <= (slack if slack.size == g.size else slack[0])
        needed = float(((d > 1) & ok).mean()) if d.size else 0.0
        d = np.where(ok, np.minimum(d, 1), d)
        _report_slack(what, needed, max_slack_frac)
    if d.max(initial=0) > 1:
        i = int(np.argmax(d))
        raise AssertionError("%s: bf16 distance %d at %d (got 0x%04x want 0x%04x)"
                             % (what, d.max(), i, np.asarray(got_raw).reshape(-1)[i],
                                np.asarray(want_raw).reshape(-1)[i]))
    return float((d > 0).mean())
