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


def test_small_matrices_of_a_decode_step_take_few_shares():
    """Up to 16 tokens, a matrix below 96 MiB: the count of shares that keeps the busiest
    compute unit's workgroups shortest, each share costing something by itself."""
    assert ops.gemm_splits(8, 3584, 3584) == 2    # 112 pairs of row blocks: 224 workgroups, one each
    assert ops.gemm_splits(8, 4608, 3584) == 3    # 144 pairs: 2 shares would give 32 compute units two each
    assert ops.gemm_splits(8, 5120, 5120) == 3
    assert ops.gemm_splits(8, 7168, 5120) == 1    # 224 pairs fill the chip unsplit
    assert ops.gemm_splits(8, 3584, 18944) == 9   # 130 MiB: a matter of bandwidth, many workgroups
    assert ops.gemm_splits(8, 896, 896) == 1      # 28 k-tiles: too few to share


def test_key_splits_of_decode_attention_depend_on_the_buckets_only():
    """A graph is captured for a bucket of sequences and of context; every step
    that it replays must split the keys as the captured one did."""
    from shrike_amd.engine.context import bucket
    from shrike_amd.parts.attention import decode_splits

    for kv_heads in (1, 4, 8):
        for seqs_lo, seqs_hi in ((1, 1), (3, 4), (5, 8), (33, 64), (129, 256)):
            for ctx_lo, ctx_hi in ((1, 256), (257, 512), (2049, 4096), (16385, 32768)):
                plans = {decode_splits(s, kv_heads, c)
                         for s in (seqs_lo, seqs_hi) for c in (ctx_lo, (ctx_lo + ctx_hi) // 2, ctx_hi)}
                assert len(plans) == 1
                (n,) = plans
                assert 1 <= n <= 64 and n <= max(1, bucket(ctx_hi, 256) // 256)
    assert decode_splits(8, 4, 2100) == 8 and decode_splits(64, 4, 4000) == 1 and decode_splits(1, 4, 100) == 1


def test_non_temporal_loads_from_a_size_on_and_alike_within_a_bucket():
    from shrike_amd.parts.attention import decode_streams

    # 7B heads: 8 sequences at 2,100 keys stay as they were, 64 of them or 8 at 16,000 stream
    assert not decode_streams(8, 4, 128, 2100) and not decode_streams(1, 4, 128, 4000)
    assert decode_streams(64, 4, 128, 2100) and decode_streams(8, 4, 128, 16000) and decode_streams(16, 4, 128, 2100)
    # a window bounds what is read
    assert not decode_streams(64, 4, 128, 100000, window=256)
    for seqs_lo, seqs_hi in ((3, 4), (5, 8), (33, 64), (129, 256)):
        for ctx_lo, ctx_hi in ((257, 512), (2049, 4096), (16385, 32768)):
            assert len({decode_streams(s, 4, 128, c) for s in (seqs_lo, seqs_hi) for c in (ctx_lo, ctx_hi)}) == 1


def test_decode_graphs_are_keyed_by_buckets_and_few():
    """The key of a decode graph: batch bucket, table widths in steps of 64
    pages, and what the parts' launches depend on (here the split of the keys).
    Walking batch sizes and contexts far and wide makes a few dozen keys, not
    one per context length."""
    import numpy as np
    import torch

    from shrike_amd.cache import CacheManager
    from shrike_amd.config import AttentionSpec, BlockSpec, ModelSpec, RMSNormSpec, SwiGLUSpec
    from shrike_amd.engine.runner import GRAPH_BATCH_BUCKETS, ModelRunner, StepEntry
    from shrike_amd.engine.runtime import Runtime
    from shrike_amd.models import DecoderModel

    norm = RMSNormSpec(eps=1e-6)
    mixer = AttentionSpec(num_heads=28, num_kv_heads=4, head_dim=128, qkv_bias=True, out_bias=False, scale=0.1)
    block = BlockSpec(name="model.layers.0", mixer=mixer, ffn=SwiGLUSpec(intermediate_size=64),
                      mixer_norm=norm, ffn_norm=norm)
    model = DecoderModel(ModelSpec(architecture="t", hidden_size=3584, vocab_size=100, blocks=(block,),
                                   final_norm=norm, tie_word_embeddings=False))
    model.blocks[0].mixer.dtype = torch.bfloat16  # what load() would set
    cache = CacheManager(model.cache_specs(), 16, 1 << 20)  # book-keeping only, nothing allocated
    runner = ModelRunner(model, cache, Runtime("cuda:0", torch.bfloat16))
    keys = {}
    for batch in (1, 2, 3, 8, 9, 60, 64, 65, 200, 256):
        seqs = [cache.new_sequence() for _ in range(batch)]
        for ctx in (1, 100, 256, 257, 1000, 1024, 1025, 2047, 2049, 4000, 4097, 8000):
            for s in seqs:
                cache.append(s, 0, ctx)
            entries = [StepEntry(s, [0], ctx - 1, [0]) for s in seqs]
            key = runner._graph_key(entries)
            assert key[0] == next(b for b in GRAPH_BATCH_BUCKETS if b >= batch)
            assert key[1] == (-(-(-(-ctx // 16)) // 64) * 64,)
            keys.setdefault(key, []).append((batch, ctx))
        for s in seqs:
            cache.free(s)
    assert len(keys) <= 64  # of 120 (batch, context) pairs over 8 batch buckets and 6 table widths
    # more than 256 rows, a portion, or a row that wants no logits: no graph
    seqs = [cache.new_sequence() for _ in range(2)]
    for s in seqs:
        cache.append(s, 0, 8)
    assert runner._graph_key([StepEntry(seqs[0], [0, 1], 0, [1])]) is None
    assert runner._graph_key([StepEntry(seqs[0], [0], 0, [])]) is None
    assert runner._graph_key([StepEntry(seqs[0], [0], 0, [0])] * 257) is None
    assert np.all([len(v) >= 1 for v in keys.values()])


def test_prompt_portions_are_launched_heaviest_first():
    """The list of workgroups that the attention part hands to the prefill
    kernel: runs of queries of every portion, each exactly once, the one whose
    last query reads the most keys first."""
    import numpy as np

    from shrike_amd.parts.attention import QUERY_TILE, heavy_first, portion_runs

    q_lens, starts = np.array([1, 1, 300, 40, 2048]), np.array([77, 5, 1900, 0, 0])
    run = 2 * QUERY_TILE
    seqs, q0 = portion_runs(q_lens[2:], 2, run)
    assert sorted(zip(seqs.tolist(), q0.tolist())) == (
        [(2, q) for q in range(0, 300, run)] + [(3, q) for q in range(0, 40, run)] + [(4, q) for q in range(0, 2048, run)])
    keys = starts[seqs] + q0 + run
    order = heavy_first(keys)
    assert sorted(order.tolist()) == list(range(seqs.size))
    assert (np.diff(keys[order]) <= 0).all()
    # the 300-token portion at position 1,900 reads more keys than the whole prompt's last run
    assert seqs[order][0] == 2 and q0[order][0] == 288
    assert (seqs[order][-1], q0[order][-1]) in ((3, 0), (4, 0))


def test_shares_of_a_portions_keys():
    from shrike_amd.parts.attention import portion_splits

    assert portion_splits(512, 1000) == 1  # a whole 2,048-token prompt: enough workgroups already
    assert portion_splits(128, 264) == 1   # 512 queries from position 0: too few keys to share
    assert portion_splits(128, 1800) == 4 and portion_splits(256, 3600) == 2
    assert portion_splits(32, 8000) == 16 and portion_splits(4, 100000) == 64
    assert portion_splits(0, 5) == 1


@pytest.mark.parametrize("gated", [False, True])
@pytest.mark.parametrize("m, k", MATRICES)
def test_a_product_in_two_parts_is_the_same_for_every_row_count_of_a_graph_bucket(m, k, gated):
    """A product of many tokens may run as two (whole rounds of tiles, then the
    rest): graphs of 128 and 256 rows must decide as every row count they stand for."""
    for lo, hi in ((65, 128), (129, 256)):
        assert len({ops.gemm_parts(n, m, k, gated) for n in range(lo, hi + 1)}) == 1
    assert ops.gemm_parts(64, m, k, gated) == 1


def test_where_a_product_runs_in_two_parts():
    assert ops.gemm_parts(512, 18944, 3584, True) == 2    # 296 tiles of 256 x 256: 256 + 40
    assert ops.gemm_parts(2048, 18944, 3584, True) == 1   # 1,184 tiles: the rest would take a round of its own anyway
    assert ops.gemm_parts(512, 3584, 18944) == 1          # shares of k instead
    assert ops.gemm_parts(2048, 13824, 5120, True) == 2   # 864 tiles: three whole rounds, then 96 tiles' rows in smaller tiles
