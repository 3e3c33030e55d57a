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


def test_key_splits_of_decode_attention_depend_on_the_buckets_only():
    """A graph is captured for a bucket of sequences and of context; every step
    that it replays must split the keys as the captured one did."""
    from shrike_amd.engine.runtime import bucket, decode_splits

    for kv_heads in (1, 4, 8):
        for seqs_lo, seqs_hi in ((1, 1), (3, 4), (5, 8), (33, 64), (129, 256)):
            for ctx_lo, ctx_hi in ((1, 256), (257, 512), (2049, 4096), (16385, 32768)):
                plans = {decode_splits(s, kv_heads, c)
                         for s in (seqs_lo, seqs_hi) for c in (ctx_lo, (ctx_lo + ctx_hi) // 2, ctx_hi)}
                assert len(plans) == 1
                (n,) = plans
                assert 1 <= n <= 64 and n <= max(1, bucket(ctx_hi, 256) // 256)
    assert decode_splits(8, 4, 2100) == 8 and decode_splits(64, 4, 4000) == 1 and decode_splits(1, 4, 100) == 1
