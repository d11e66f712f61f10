"""GPU parity of the persistent form of the int8 256 x 256 kernel (hip:gfx950:mfma_b8): one workgroup per CU walks the
tiles w, w + W, ... of its XCD's share, reusing its LDS ring, staging area and operand tables from tile to tile.

Integer sums: which workgroup computes a tile cannot change a bit, so every case is bit-exact against the oracle AND
identical to the same problem with one workgroup per tile (QMM_B8X_VARIANT=4). The shapes give an XCD 33 ... 48 tiles
(more than its 32 CUs, so workgroups take a second tile with other rows, columns, scales and tails than their first),
with QMM_B8X_VARIANT=3 so that K = 1024 -- sized for the oracle -- reaches the kernel that K > 2048 reaches by itself."""
import sys

import pytest

import onednn_amd as dnnl
from onednn_amd import _capi
from qmm_harness import assert_bf16_within_1ulp, assert_bit_exact, dt
import test_gpu_parity as cases
import test_gpu_int8_wei_zp as zp_cases

pytestmark = pytest.mark.gpu

A = dnnl.algorithm
MFMA = "hip:gfx950:mfma_b8"
SWISH = [{"kind": "eltwise", "alg": A.eltwise_swish, "alpha": 1.0}]


def say(msg):
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def ctx():
    eng = dnnl.engine(dnnl.engine.kind.gpu, 0)
    return eng, dnnl.stream(eng)


CASES = {
    # 8 x 33 tiles: one workgroup per XCD takes a second tile; config 2's attributes (per-token and per-column scales,
    # swish, bf16): the second tile must see its own rows' and columns' scales in the tables
    "second_tile_swish_bf16": lambda: cases.int8_linear(2048, 1024, 8448, 301, src_dt=dt.s8, dst_dt=dt.bf16, src_zp=None,
                                                         per_token=True, post_ops=SWISH),
    # 7 x 37 = 259 tiles, 33 slots per XCD: the last XCD's share ends early
    "short_last_share_s32": lambda: cases.int8_linear(1792, 1024, 9472, 302, src_dt=dt.s8, dst_dt=dt.s32, src_zp=None,
                                                      src_scale=None),
    # 8 x 48 tiles with row and column tails in the tiles taken second
    "tails_in_second_tiles_f32": lambda: cases.int8_linear(2040, 1024, 12200, 303, src_dt=dt.s8, dst_dt=dt.f32,
                                                           src_zp=None, per_token=True),
    # weights zero points: the row-sum table is per tile as well
    "weights_zero_points_f16": lambda: zp_cases.w8a8(M=2048, K=1024, N=8448, seed=304, dst_dt=dt.f16),
    # a source zero point (column-sum compensation table) and an odd number of k-steps (the other instantiation)
    "source_zero_point_k1088": lambda: cases.int8_linear(2048, 1088, 8448, 305, src_dt=dt.s8, dst_dt=dt.f32, src_zp=3),
    # three walks: 8 x 72 tiles are 72 per XCD
    # two matrices of 4 x 40 tiles: an XCD's share (20) is smaller than its CUs, one grid row per matrix
    "batched_small_share_f32": lambda: cases.int8_linear(1024, 1024, 10240, 307, src_dt=dt.s8, dst_dt=dt.f32, src_zp=None,
                                                         batch=(2,)),
    # 8 x 80 tiles, 80 per XCD = two whole rounds and 16 more: the 16 workgroups without a tile in the last round start
    # late and the whole rounds hand each half of the workgroups a 4 x 4 block of tiles (another tile order)
    "late_half_square_blocks_s8": lambda: cases.int8_linear(2048, 1024, 20480, 308, src_dt=dt.s8, dst_dt=dt.s8,
                                                            src_zp=None, per_token=True),
    # 12 x 53 tiles, 80 per XCD again, but rounds that straddle the 8-row groups or lie in the 4-row group keep the
    # plain order
    "late_half_partial_row_group_f32": lambda: cases.int8_linear(3072, 1024, 13568, 309, src_dt=dt.s8, dst_dt=dt.f32,
                                                                 src_zp=None, per_token=True),
    "three_tiles_each_s8": lambda: cases.int8_linear(2048, 1024, 18432, 306, src_dt=dt.s8, dst_dt=dt.s8, src_zp=None,
                                                     per_token=True),
}


@pytest.mark.parametrize("name", sorted(CASES))
def test_persistent_walk_is_exact_and_changes_no_bit(ctx, name):
    eng, strm = ctx
    say("mfma_b8 persistent tiles %s" % name)
    p = CASES[name]()
    with _capi.kernel_variants(gemm=6, b8x=3):
        got, pd = p.run_gpu(eng, strm, weights_any=True, return_pd=True)
    assert pd.impl_info_str() == MFMA
    with _capi.kernel_variants(gemm=6, b8x=4):
        per_tile = p.run_gpu(eng, strm, weights_any=True)
    assert_bit_exact(got, per_tile, name + " (persistent against one workgroup per tile)")
    if "swish" in name:  # hardware exp2 / rcp in the kernel, libm in the oracle
        assert_bf16_within_1ulp(got, p.run_oracle(), name, abs_slack=1e-30)
    else:
        assert_bit_exact(got, p.run_oracle(), name)
