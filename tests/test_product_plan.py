"""The host-side plan of a matrix product (how many float32 shares of k): no
device is needed for it.  A decode step captured as a graph of 128 or 256 rows
stands for any number of sequences up to that; graph and kernel-by-kernel
execution agree bit for bit only if the plan is the same for all of them."""

import pytest

from shrike_amd.kernels import ops

MATRICES = [(4608, 3584), (3584, 3584), (3584, 18944), (5120, 13824), (7168, 5120), (5120, 5120),
            (152064, 3584), (503, 128), (2100, 16400)]


@pytest.mark.parametrize("m, k", MATRICES)
def test_the_plan_is_the_same_for_every_row_count_of_a_graph_bucket(m, k):
    for lo, hi in ((1, 16), (17, 32), (33, 64), (65, 128), (129, 256)):
        plans = {ops.gemm_splits(n, m, k) for n in range(lo, hi + 1)}
        assert len(plans) == 1, f"rows {lo}..{hi} of [{m}, {k}]: {sorted(plans)}"


@pytest.mark.parametrize("m, k", MATRICES)
def test_shares_keep_enough_of_k(m, k):
    """Every share has at least 16 tiles of 32 of k, and there are at most 16 shares."""
    for n in (1, 8, 16, 24, 64, 100, 256, 512, 2048, 4096):
        s = ops.gemm_splits(n, m, k)
        assert 1 <= s <= 16
        assert s == 1 or -(-k // 32) // s >= 16


def test_matrices_that_fill_the_chip_are_not_split():
    assert ops.gemm_splits(8, 152064, 3584) == 1      # 9504 row blocks
    assert ops.gemm_splits(4096, 18944, 3584) == 1    # 592 tiles of 256 x 256
    assert ops.gemm_splits(8, 3584, 18944) > 1        # 224 row blocks, a long k
    assert ops.gemm_splits(512, 5120, 13824) > 1      # 80 tiles of 256 x 128
