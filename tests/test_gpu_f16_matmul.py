"""GPU parity of hip:gfx950:mfma_f16 (plain f16 / bf16 batched matmul, f32 accumulation) against the CPU oracle
(src/cpu/matmul/ref_matmul.cpp:130-233): the unfused attention products of the reference's LLM list
(tests/benchdnn/inputs/matmul/option_set_fwks_llm_gpu, --dt=f16:f16:f16 --stag=abcd --wtag=abcd --dtag=abcd, K and N
such as 998, 999, 1000 that are not multiples of the vector width). The kernel sums in another order than the oracle's
k loop, so results are compared within one step of the dst type on the magnitude of the summed terms; integer-valued
data, where every order gives the same bits, is compared bit for bit."""
import sys

import numpy as np
import pytest

import onednn_amd as dnnl
import oracle as O
from qmm_harness import Problem, TensorSpec, assert_bit_exact, assert_f32_close, dt

pytestmark = pytest.mark.gpu
A = dnnl.algorithm
F16MM, GENERIC = "hip:gfx950:mfma_f16", "hip:gfx950:generic"


def say(msg):
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def ctx():
    eng = dnnl.engine(dnnl.engine.kind.gpu, 0)
    return eng, dnnl.stream(eng)


def problem(sd, wd, seed, code=dt.f16, dst_dt=None, exact=False, post_ops=None, bias=False):
    r = np.random.default_rng(seed)
    nd = len(sd)
    dd = [max(a, b) for a, b in zip(sd[:-2], wd[:-2])] + [sd[-2], wd[-1]]
    if exact:
        s, w = r.integers(-4, 5, sd).astype(np.float32), r.integers(-4, 5, wd).astype(np.float32)
    else:
        s, w = r.standard_normal(sd).astype(np.float32), r.standard_normal(wd).astype(np.float32)
    b = None
    if bias:
        b = TensorSpec(dt.f32, [1] * (nd - 1) + [wd[-1]], None, r.integers(-3, 4, wd[-1]).astype(np.float32))
    return Problem(TensorSpec(code, sd, None, s), TensorSpec(code, wd, None, w), TensorSpec(dst_dt or code, dd), bias=b,
                   post_ops=post_ops)


CASES = {
    "decode_scores_clip": dict(sd=[1, 8, 1, 128], wd=[1, 8, 128, 999], post_ops=[{"kind": "eltwise", "alg": A.eltwise_clip, "alpha": -1.0, "beta": 1.0}]),
    "decode_context_k999": dict(sd=[1, 8, 1, 999], wd=[1, 8, 999, 128]),
    "prefill_scores_998": dict(sd=[1, 4, 198, 128], wd=[1, 4, 128, 198]),
    "prefill_context_k198": dict(sd=[1, 4, 198, 198], wd=[1, 4, 198, 128]),
    "two_dims_bf16_f32_dst": dict(sd=[70, 256], wd=[256, 100], code=dt.bf16, dst_dt=dt.f32),
    "broadcast_weights_bias": dict(sd=[3, 2, 33, 64], wd=[1, 1, 64, 72], bias=True),
    # M <= 4 per batch entry runs the lane-per-column kernel instead of the MFMA tile
    "decode_scores_n1000_vector": dict(sd=[1, 8, 1, 128], wd=[1, 8, 128, 1000]),
    "decode_scores_bf16": dict(sd=[1, 8, 1, 128], wd=[1, 8, 128, 1001], code=dt.bf16),
    "three_rows_vector": dict(sd=[2, 6, 3, 200], wd=[2, 6, 200, 264], bias=True),
    "four_rows_scalar_f32_dst": dict(sd=[5, 4, 2043], wd=[5, 2043, 77], dst_dt=dt.f32),
    "two_rows_narrow": dict(sd=[3, 2, 64], wd=[3, 64, 8]),
    "one_row_long_k": dict(sd=[1, 8192], wd=[8192, 520]),
    "two_rows_k_past_the_table": dict(sd=[2, 4100], wd=[4100, 96]),
    "odd_rows_with_bias_and_f32_dst": dict(sd=[2, 70, 250], wd=[2, 250, 99], bias=True, dst_dt=dt.f32),
    "odd_rows_with_bias_bf16": dict(sd=[3, 33, 77], wd=[3, 77, 51], bias=True, code=dt.bf16),
    "tiny_k": dict(sd=[2, 5, 8], wd=[2, 8, 16]),
    "odd_everything": dict(sd=[2, 67, 45], wd=[2, 45, 51]),
}


@pytest.mark.parametrize("name", sorted(CASES))
@pytest.mark.parametrize("exact", [True, False])
def test_f16_matmul(ctx, name, exact):
    eng, strm = ctx
    say("mfma_f16 %s exact=%s" % (name, exact))
    kw = CASES[name]
    p = problem(seed=len(name), exact=exact, **kw)
    got, pd = p.run_gpu(eng, strm, return_pd=True)
    assert pd.impl_info_str() == F16MM
    want = p.run_oracle()
    if exact:
        assert_bit_exact(got, want, name)
        return
    code = kw.get("dst_dt") or kw.get("code", dt.f16)
    g, w = O.to_f32(code, got), O.to_f32(code, want)
    K = kw["sd"][-1]
    step = {dt.f16: 2.0 ** -10, dt.bf16: 2.0 ** -7, dt.f32: 1e-5}[code]
    assert_f32_close(g, w, rel=step, scale=np.sqrt(K), what=name, max_slack_frac=1.0)


BIG_TILE_CASES = {
    "prefill_scores_198": CASES["prefill_scores_998"],
    "prefill_context_k198": CASES["prefill_context_k198"],
    "two_dims_bf16_f32_dst": CASES["two_dims_bf16_f32_dst"],
    "odd_rows_with_bias_and_f32_dst": CASES["odd_rows_with_bias_and_f32_dst"],
    "aligned_bias_clip_bf16": dict(sd=[2, 136, 256], wd=[2, 256, 200], bias=True, code=dt.bf16,
                                   post_ops=[{"kind": "eltwise", "alg": A.eltwise_clip, "alpha": -2.0, "beta": 2.0}]),
    "three_tiles_each_way_k520": dict(sd=[300, 520], wd=[520, 264],
                                      post_ops=[{"kind": "eltwise", "alg": A.eltwise_relu, "alpha": 0.0, "beta": 0.0}]),
    "unaligned_rows_999": dict(sd=[2, 131, 999], wd=[2, 999, 999]),
    "k_one_step_broadcast_weights": dict(sd=[3, 129, 24], wd=[1, 24, 130]),
    # many column tiles over a short K: what the walking kernel is for
    "scores_k64_nine_column_tiles_clip_bf16": dict(sd=[1, 2, 300, 64], wd=[1, 2, 64, 1100], code=dt.bf16,
                                                   post_ops=[{"kind": "eltwise", "alg": A.eltwise_clip, "alpha": -3.0,
                                                              "beta": 3.0}]),
    "scores_k128_unaligned_998": dict(sd=[1, 3, 260, 128], wd=[1, 3, 128, 998]),
    "ragged_k40_n1000_f32_dst": dict(sd=[2, 150, 40], wd=[2, 40, 1000], dst_dt=dt.f32),
    "k288_five_column_tiles": dict(sd=[131, 288], wd=[288, 600]),
}


@pytest.mark.parametrize("name", sorted(BIG_TILE_CASES))
@pytest.mark.parametrize("exact", [True, False])
@pytest.mark.parametrize("tiling", [2, 3], ids=["tiles128", "walk"])
def test_f16_matmul_128x128_tiles(ctx, name, exact, tiling):
    """The same products forced onto the 128 x 128 tiling (by default problems with at least 256 such tiles and K >= 256
    take it) and onto the kernel whose workgroups walk the column tiles of a 128-row block (the default for K <= 256 over
    at least four column tiles; epilogues it does not take fall back to the tiled kernels)."""
    from onednn_amd import _capi
    eng, strm = ctx
    say("mfma_f16 128x128 tiles %s exact=%s tiling=%d" % (name, exact, tiling))
    kw = BIG_TILE_CASES[name]
    p = problem(seed=len(name) + 40, exact=exact, **kw)
    with _capi.kernel_variants(gemm=tiling):
        got, pd = p.run_gpu(eng, strm, return_pd=True)
    assert pd.impl_info_str() == F16MM
    want = p.run_oracle()
    if exact:
        assert_bit_exact(got, want, name)
        with _capi.kernel_variants(gemm=1):
            assert_bit_exact(p.run_gpu(eng, strm), want, name + " (64 x 64 tiles)")
        return
    code = kw.get("dst_dt") or kw.get("code", dt.f16)
    g, w = O.to_f32(code, got), O.to_f32(code, want)
    step = {dt.f16: 2.0 ** -10, dt.bf16: 2.0 ** -7, dt.f32: 1e-5}[code]
    assert_f32_close(g, w, rel=step, scale=np.sqrt(kw["sd"][-1]), what=name, max_slack_frac=1.0)


def test_f16_matmul_tilings_are_different_kernels(ctx):
    """Forcing the tiling changes the summation grouping not at all (both sum 32 k per MFMA in the same order), so results
    agree bit for bit on random data as well; what shows that the override took is the default choice: a problem with
    256 tiles of 128 x 128 and one with fewer must both run, and the forced runs must equal the default ones."""
    from onednn_amd import _capi
    eng, strm = ctx
    for sd, wd in (([16, 512, 64], [16, 64, 512]), ([2, 200, 64], [2, 64, 200])):
        p = problem(sd, wd, 77)
        base = p.run_gpu(eng, strm)
        for v in (1, 2, 3):
            with _capi.kernel_variants(gemm=v):
                assert_bit_exact(p.run_gpu(eng, strm), base, "tile variant %d" % v)


def test_matches_the_per_element_kernel(ctx):
    eng, strm = ctx
    say("mfma_f16 vs generic")
    p = problem([2, 3, 40, 96], [2, 3, 96, 80], 5, exact=True)
    assert_bit_exact(p.run_gpu(eng, strm, impl=F16MM), p.run_gpu(eng, strm, impl=GENERIC), "vs generic")


def test_what_it_does_not_take(ctx):
    """Transposed weights (k contiguous) and f32 operands stay with the per-element kernel."""
    eng, strm = ctx
    p = Problem(TensorSpec(dt.f16, [16, 32], None, np.ones((16, 32), np.float32)),
                TensorSpec(dt.f16, [32, 24], "ba", np.ones((32, 24), np.float32)), TensorSpec(dt.f16, [16, 24]))
    got, pd = p.run_gpu(eng, strm, return_pd=True)
    assert pd.impl_info_str() == GENERIC
    assert_bit_exact(got, p.run_oracle(), "ba weights")


@pytest.mark.parametrize("code", [dt.f16, dt.bf16], ids=str)
@pytest.mark.parametrize("M,N", [(1, 1000), (3, 1000), (1, 264), (3, 264), (2, 1001), (4, 40)])
def test_few_rows_with_sum_post_op_stores_each_column_once(ctx, code, M, N):
    """The few-rows kernel moves its last column chunk back inside the row when N is not a multiple of the chunk; the
    columns two workgroups then both compute must be stored by one of them only, or a sum post-op (which reads the old
    dst) would be applied twice there. Integer-valued data: bit for bit."""
    eng, strm = ctx
    say("mfma_f16 few rows, sum post-op, %s M=%d N=%d" % (code, M, N))
    K = 96
    p = problem([2, 3, M, K], [2, 3, K, N], 7 * N + M, code=code, exact=True,
                post_ops=[{"kind": "sum", "scale": 0.5}])
    r = np.random.default_rng(N)
    init = O.from_f32(code, r.integers(-20, 21, 2 * 3 * M * N).astype(np.float32) * 2)
    got, pd = p.run_gpu(eng, strm, return_pd=True, dst_init=init)
    assert pd.impl_info_str() == F16MM
    assert_bit_exact(got, p.run_oracle(dst_init=init), "few rows + sum")
