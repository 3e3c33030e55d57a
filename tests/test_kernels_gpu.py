"""Each HIP kernel alone against a plain float32/float64 torch computation of
the same operation, at sizes the engine's tiny models do not use."""

import math

import pytest
import torch

from .plain import model as plain

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
TOL = {torch.float32: 5e-6, torch.bfloat16: 1e-2}


@pytest.fixture(scope="module")
def ops():
    from shrike_amd.kernels import ops

    return ops


def dev(t, dtype=None):
    return t.to("cuda", dtype) if dtype else t.to("cuda")


def close(got, want, dtype, scale=None):
    """scale None: errors are measured against the largest wanted value.  With a
    number: element by element against max(scale, |wanted|), since a stored value
    cannot be closer to the truth than its format's spacing, which grows with the
    value (bfloat16 values near 2.4 lie 0.0156 apart)."""
    want = want.double().cpu()
    if scale is None:
        scale = want.abs().max().clamp_min(1e-30)
    else:
        scale = want.abs().clamp_min(scale)
    err = ((got.double().cpu() - want).abs() / scale).max().item()
    assert err <= TOL[dtype], f"rel err {err:.3e} > {TOL[dtype]}"


def rounded(t, dtype):
    """The values a tensor has after it is stored in `dtype`."""
    return t.to(dtype).double()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden, vocab", [(72, 101), (3584, 777)])
def test_embed(ops, dtype, hidden, vocab):
    torch.manual_seed(1)
    table = torch.randn(vocab, hidden)
    ids = torch.randint(0, vocab, (13,), dtype=torch.int32)
    out = torch.empty(13, hidden, device="cuda")
    ops.embed(dev(table, dtype), dev(ids), out)
    assert torch.equal(out.cpu(), table.to(dtype).float()[ids.long()])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden, eps", [(72, 1e-6), (1000, 1e-5), (5120, 3e-3)])
def test_add_rmsnorm(ops, dtype, hidden, eps):
    torch.manual_seed(2)
    n = 9
    resid, delta, w = torch.randn(n, hidden) * 3, torch.randn(n, hidden), 1 + 0.1 * torch.randn(hidden)
    r = dev(resid.clone())
    out = torch.empty(n, hidden, device="cuda", dtype=dtype)
    ops.add_rmsnorm(r, dev(delta, dtype), dev(w), eps, out)
    summed = resid.double() + rounded(delta, dtype)
    close(r, summed, torch.float32)  # the residual sum stays float32 in both modes
    close(out, plain.rms_norm(summed, w.double(), eps), dtype)
    # without delta, on chosen rows, without touching the residual
    rows = torch.tensor([4, 0, 7], dtype=torch.int32)
    before = r.clone()
    out2 = torch.empty(3, hidden, device="cuda", dtype=dtype)
    ops.add_rmsnorm(r, dev(delta, dtype), dev(w), eps, out2, rows=dev(rows), write_resid=False)
    assert torch.equal(r, before)
    x = before.double().cpu()[rows.long()] + rounded(delta, dtype)[rows.long()]
    close(out2, plain.rms_norm(x, w.double(), eps), dtype)
    # a norm in the wrong place (mean subtracted, eps outside the root) fails this
    const = torch.full((1, hidden), 2.0, device="cuda")
    out3 = torch.empty(1, hidden, device="cuda", dtype=dtype)
    ops.add_rmsnorm(const, None, torch.ones(hidden, device="cuda"), eps, out3)
    close(out3, torch.full((1, hidden), 2.0 / math.sqrt(4.0 + eps)), dtype)


def gate_reference(gate, activation):
    """SiLU, or GELU in its tanh form, by the library's own routines, in float64."""
    if activation == "silu":
        return torch.nn.functional.silu(gate)
    return torch.nn.functional.gelu(gate, approximate="tanh")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("activation", ["silu", "gelu_tanh"])
@pytest.mark.parametrize("n, inter", [(1, 172), (7, 18944), (33, 100)])
def test_act_mul(ops, dtype, n, inter, activation):
    torch.manual_seed(3)
    gu = torch.randn(n, 2 * inter) * 4
    out = torch.empty(n, inter, device="cuda", dtype=dtype)
    ops.act_mul(dev(gu, dtype), out, activation)
    g, u = rounded(gu, dtype)[:, :inter], rounded(gu, dtype)[:, inter:]
    close(out, gate_reference(g, activation) * u, dtype)
    with pytest.raises(Exception, match="activation"):
        ops.act_mul(dev(gu, dtype), out, "relu")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n, m, k", [(1, 503, 128), (5, 64, 172), (70, 130, 96), (130, 200, 333), (64, 3584, 512)])
def test_gemm(ops, dtype, n, m, k):
    torch.manual_seed(4)
    a, w, b = torch.randn(n, k), torch.randn(m, k) / math.sqrt(k), torch.randn(m)
    want = rounded(a, dtype) @ rounded(w, dtype).t() + b.double()
    out = torch.empty(n, m, device="cuda", dtype=dtype)
    ops.gemm(dev(a, dtype), dev(w, dtype), out, bias=dev(b))
    close(out, want, dtype)
    # float32 output from bfloat16 inputs (logits), without bias, accumulated on top
    out32 = torch.ones(n, m, device="cuda")
    ops.gemm(dev(a, dtype), dev(w, dtype), out32, accumulate=True)
    close(out32, want - b.double() + 1.0, torch.float32 if dtype == torch.float32 else dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_gemm_rows_do_not_depend_on_the_rest_of_the_batch(ops, dtype):
    torch.manual_seed(5)
    a, w = dev(torch.randn(77, 200), dtype), dev(torch.randn(150, 200), dtype)
    full = torch.empty(77, 150, device="cuda", dtype=torch.float32)
    ops.gemm(a, w, full)
    one = torch.empty(1, 150, device="cuda", dtype=torch.float32)
    ops.gemm(a[40:41], w, one)
    assert torch.equal(one[0], full[40])


def test_gemm_refuses_what_it_cannot_do(ops):
    from shrike_amd.kernels import KernelError

    a, w = torch.zeros(2, 8, device="cuda"), torch.zeros(4, 9, device="cuda")
    with pytest.raises(KernelError):
        ops.gemm(a, w, torch.zeros(2, 4, device="cuda"))
    with pytest.raises(KernelError, match="device"):
        ops.gemm(torch.zeros(2, 8), torch.zeros(4, 8), torch.zeros(2, 4))
    with pytest.raises(KernelError):
        ops.gemm(a, torch.zeros(4, 8, device="cuda", dtype=torch.bfloat16), torch.zeros(2, 4, device="cuda"))


# ------------------------------------------------------------ rotation + cache


def paged_setup(seq_lens, page_size, num_pages, kv_heads, head_dim, dtype, seed=0):
    """Random distinct pages per sequence; tables padded with 0 as the runner builds them."""
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(num_pages, generator=g).tolist()
    tables, width = [], max(-(-n // page_size) for n in seq_lens)
    for n in seq_lens:
        need = -(-n // page_size)
        tables.append([perm.pop() for _ in range(need)] + [0] * (width - need))
    slab = 32 if head_dim % 32 == 0 else head_dim
    k_pool = torch.full((num_pages, kv_heads, head_dim // slab, page_size, slab), float("nan"), dtype=dtype, device="cuda")
    v_pool = torch.full((num_pages, kv_heads, head_dim, page_size), float("nan"), dtype=dtype, device="cuda")
    return torch.tensor(tables, dtype=torch.int32, device="cuda"), k_pool, v_pool


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, kv_heads, head_dim, page_size, theta", [(6, 3, 48, 8, 5e4), (14, 2, 64, 16, 1e6), (5, 5, 80, 4, 1e4),
                                                                   (4, 2, 128, 16, 1e6), (3, 1, 72, 8, 1e4)])
def test_rope_kv_store(ops, dtype, heads, kv_heads, head_dim, page_size, theta):
    torch.manual_seed(6)
    seq_lens = [37, 1, 40]  # 78 tokens: bfloat16 rows that are rotated whole take the vector kernel
    starts = [5, 0, 3000]  # positions far out: angles of thousands of radians
    n = sum(seq_lens)
    tables, k_pool, v_pool = paged_setup([s + l for s, l in zip(starts, seq_lens)], page_size, 1024, kv_heads, head_dim, dtype)
    token_seq = torch.cat([torch.full((l,), i) for i, l in enumerate(seq_lens)]).int()
    positions = torch.cat([torch.arange(s, s + l) for s, l in zip(starts, seq_lens)]).int()
    qkv = torch.randn(n, (heads + 2 * kv_heads) * head_dim)
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2).float() / head_dim))
    buf = dev(qkv, dtype)
    ops.rope_kv_store(buf, heads, kv_heads, head_dim, head_dim, dev(inv_freq), dev(positions), dev(token_seq), tables, k_pool, v_pool, page_size)

    x = rounded(qkv, dtype)
    q = x[:, : heads * head_dim].view(n, heads, head_dim)
    k = x[:, heads * head_dim : (heads + kv_heads) * head_dim].view(n, kv_heads, head_dim)
    v = x[:, (heads + kv_heads) * head_dim :].view(n, kv_heads, head_dim)
    cos, sin = plain.rope_tables(positions.long(), head_dim, theta)
    close(buf[:, : heads * head_dim].reshape(n, heads, head_dim), plain.apply_rope(q, cos, sin), dtype)
    for t in range(n):
        s, p = int(token_seq[t]), int(positions[t])
        page = int(tables[s, p // page_size])
        close(get_key(k_pool, page, p % page_size), plain.apply_rope(k[t : t + 1], cos[t : t + 1], sin[t : t + 1])[0], dtype)
        assert torch.equal(v_pool[page, :, :, p % page_size].cpu().double(), v[t])
    # nothing else was written: every other slot is still NaN
    written = sum(seq_lens) * kv_heads * head_dim
    assert int((~torch.isnan(k_pool.float())).sum()) == written
    assert int((~torch.isnan(v_pool.float())).sum()) == written


def put_key(k_pool, page, slot, k):
    """k [kv_heads, head_dim] into the slabs of a page: [kv_heads, head_dim / slab, page_size, slab]."""
    k_pool[page, :, :, slot, :] = k.to(k_pool.device).view(k_pool.shape[1], k_pool.shape[2], k_pool.shape[4])


def get_key(k_pool, page, slot):
    return k_pool[page, :, :, slot, :].reshape(k_pool.shape[1], -1)


def reference_attention(q, k_pool, v_pool, tables, seq_lens, starts, page_size, window, scale):
    """Gathers each sequence's keys through its table and runs the plain attention."""
    outs = []
    heads = q.shape[1]
    off = 0
    for s, (start, n_new) in enumerate(zip(starts, seq_lens)):
        ctx = start + n_new
        pages = tables[s, : -(-ctx // page_size)].long().cpu()
        # [pages, kv_heads, slabs, page_size, slab] -> [keys, kv_heads, head_dim]
        k = k_pool[pages.to(k_pool.device)].cpu().double().permute(0, 3, 1, 2, 4).reshape(-1, k_pool.shape[1], k_pool.shape[2] * k_pool.shape[4])[:ctx]
        v = v_pool[pages.to(v_pool.device)].cpu().double().permute(0, 3, 1, 2).reshape(-1, v_pool.shape[1], v_pool.shape[2])[:ctx]
        k, v = torch.nan_to_num(k), torch.nan_to_num(v)  # slots outside the window may be poisoned
        d = q.shape[2]
        o = plain.causal_attention(q[off : off + n_new].double() * (scale / d**-0.5), k, v, window, first=start)
        outs.append(o)
        off += n_new
    return torch.cat(outs)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize(
    "heads, kv_heads, head_dim, page_size, window",
    [(14, 2, 64, 16, None), (4, 4, 16, 4, None), (28, 4, 128, 16, None), (6, 3, 48, 8, 20), (5, 1, 80, 64, None), (2, 1, 256, 16, 100)],
)
def test_attention_mixed_batch(ops, dtype, heads, kv_heads, head_dim, page_size, window):
    """Portions with earlier context beside single tokens, context lengths of the
    reference's own decode test (1, 15, 16, 17, 100, 333, 512, 7)."""
    torch.manual_seed(7)
    ctx = [1, 15, 16, 17, 100, 333, 512, 7, 260, 90]
    seq_lens = [1, 1, 1, 1, 1, 1, 1, 1, 200, 90]  # two portions: 200 tokens after 60, 90 from the start
    starts = [c - l for c, l in zip(ctx, seq_lens)]
    num_pages = 2 * sum(-(-c // page_size) for c in ctx) + 3
    tables, k_pool, v_pool = paged_setup(ctx, page_size, num_pages, kv_heads, head_dim, dtype, seed=1)
    for s, c in enumerate(ctx):  # fill each sequence's slots; everything else stays NaN
        for p in range(c):
            page = int(tables[s, p // page_size])
            put_key(k_pool, page, p % page_size, torch.randn(kv_heads, head_dim).to(dtype))
            v_pool[page, :, :, p % page_size] = torch.randn(kv_heads, head_dim).to(dtype)
    n = sum(seq_lens)
    q = torch.randn(n, heads, head_dim).to(dtype)
    token_seq = torch.cat([torch.full((l,), i) for i, l in enumerate(seq_lens)]).int()
    positions = torch.cat([torch.arange(s, s + l) for s, l in zip(starts, seq_lens)]).int()
    out = torch.empty(n, heads * head_dim, device="cuda", dtype=dtype)
    scale = 0.7 * head_dim**-0.5  # not the default: the scale is a parameter
    ops.attention(dev(q).view(n, -1), out, heads, kv_heads, head_dim, dev(positions), dev(token_seq), tables, k_pool, v_pool, page_size, window, scale)
    want = reference_attention(q.double(), k_pool, v_pool, tables, seq_lens, starts, page_size, window, scale)
    assert not torch.isnan(out.float()).any(), "a slot outside the context was read"
    close(out.view(n, heads, head_dim), want, dtype, scale=1.0)


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_finds_one_far_key_among_hundreds(ops, dtype):
    """One key far back is made to stand out; the output must be its value."""
    torch.manual_seed(8)
    heads, kv_heads, head_dim, page_size, ctx = 4, 2, 64, 16, 700
    tables, k_pool, v_pool = paged_setup([ctx], page_size, 64, kv_heads, head_dim, dtype)
    k = torch.randn(ctx, kv_heads, head_dim) * 0.1
    v = torch.randn(ctx, kv_heads, head_dim)
    q = torch.randn(1, heads, head_dim)
    far = 37  # third page, far from the query at position 699
    k[far] = q[0, ::2] * 4.0  # heads 0 and 2 are the first of each group
    for p in range(ctx):
        page = int(tables[0, p // page_size])
        put_key(k_pool, page, p % page_size, k[p].to(dtype))
        v_pool[page, :, :, p % page_size] = v[p].to(dtype)
    out = torch.empty(1, heads * head_dim, device="cuda", dtype=dtype)
    ops.attention(dev(q, dtype).view(1, -1), out, heads, kv_heads, head_dim, torch.tensor([ctx - 1], dtype=torch.int32, device="cuda"),
                  torch.zeros(1, dtype=torch.int32, device="cuda"), tables, k_pool, v_pool, page_size, None, 1.0)
    got = out.view(heads, head_dim).float().cpu()
    for h in (0, 2):
        assert torch.allclose(got[h], v[far, h // 2].to(dtype).float(), atol=2e-2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_window_edge(ops, dtype):
    """The key just outside the window would dominate if it were read."""
    heads = kv_heads = 1
    head_dim, page_size, ctx, window = 32, 8, 100, 24
    tables, k_pool, v_pool = paged_setup([ctx], page_size, 32, kv_heads, head_dim, dtype)
    torch.manual_seed(9)
    q = torch.randn(1, 1, head_dim)
    k = torch.randn(ctx, 1, head_dim) * 0.1
    v = torch.randn(ctx, 1, head_dim)
    edge = ctx - 1 - window  # first key outside
    k[edge] = q[0] * 8.0
    k[edge + 1] = q[0] * 0.5
    for p in range(ctx):
        page = int(tables[0, p // page_size])
        put_key(k_pool, page, p % page_size, k[p].to(dtype))
        v_pool[page, :, :, p % page_size] = v[p].to(dtype)
    args = (heads, kv_heads, head_dim, torch.tensor([ctx - 1], dtype=torch.int32, device="cuda"),
            torch.zeros(1, dtype=torch.int32, device="cuda"), tables, k_pool, v_pool, page_size)
    out = torch.empty(1, head_dim, device="cuda", dtype=dtype)
    ops.attention(dev(q, dtype).view(1, -1), out, *args, window, 1.0)
    kk, vv = rounded(k, dtype), rounded(v, dtype)
    want = plain.causal_attention(rounded(q, dtype).expand(ctx, 1, head_dim) * head_dim**0.5, kk, vv, window)[-1]
    close(out.view(1, head_dim), want, dtype, scale=1.0)
    out_full = torch.empty_like(out)
    ops.attention(dev(q, dtype).view(1, -1), out_full, *args, None, 1.0)
    assert torch.allclose(out_full.float().cpu()[0], v[edge, 0].to(dtype).float(), atol=2e-2)  # without a window the edge key wins


def test_attention_refuses_head_sizes_it_cannot_do(ops):
    from shrike_amd.kernels import KernelError

    with pytest.raises(KernelError, match="head_dim"):
        z = torch.zeros(1, 272, device="cuda")
        k_pool = torch.zeros(2, 1, 1, 4, 272, device="cuda")
        v_pool = torch.zeros(2, 1, 272, 4, device="cuda")
        i = torch.zeros(1, dtype=torch.int32, device="cuda")
        ops.attention(z, torch.empty_like(z), 1, 1, 272, i, i, i.view(1, 1), k_pool, v_pool, 4, None, 1.0)


def test_position_kernel_refuses_more_rows_than_positions(ops):
    """Refused on the host: the kernel would read a position per row of qkv."""
    from shrike_amd.kernels import KernelError

    qkv = torch.zeros(5, 4 * 16, device="cuda")
    i3 = torch.zeros(3, dtype=torch.int32, device="cuda")
    k_pool, v_pool = torch.zeros(2, 1, 1, 4, 16, device="cuda"), torch.zeros(2, 1, 16, 4, device="cuda")
    with pytest.raises(KernelError, match="positions"):
        ops.rope_kv_store(qkv, 2, 1, 16, 0, None, i3, i3, i3.view(3, 1), k_pool, v_pool, 4)


# ------------------------------------------------------------------- sampling


def test_argmax_takes_the_lowest_index_among_equal_maxima(ops):
    torch.manual_seed(10)
    logits = torch.randn(6, 152064)
    logits[0, [5, 99999, 150000]] = 50.0
    logits[1, 152063] = 60.0
    logits[2, 0] = 60.0
    out = torch.empty(6, dtype=torch.int32, device="cuda")
    ops.argmax(dev(logits), out)
    assert out.tolist() == logits.argmax(-1).tolist()
    assert out.tolist()[:3] == [5, 152063, 0]
    # the reference's vectors (tests/test_sampler.py:20-23)
    small = torch.tensor([[0.1, 5.0, 0.2], [9.0, 0.0, 0.0]], device="cuda")
    out2 = torch.empty(2, dtype=torch.int32, device="cuda")
    ops.argmax(small, out2)
    assert out2.tolist() == [1, 0]


def run_sample(ops, logits, temperature, top_p, u, nucleus=True):
    rows, vocab = logits.shape
    out = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
    f = lambda x: torch.tensor(x, dtype=torch.float32, device="cuda")  # noqa: E731
    scratch = torch.full((ops.sample_scratch_floats(rows, vocab),), float("nan"), device="cuda")
    ops.sample(dev(logits), out, f(temperature), f(top_p), f(u), scratch, nucleus=nucleus)
    return out.tolist()


def test_sample_vectors_of_the_reference(ops):
    # tests/test_sampler.py:36-42: a dominant entry and top_p 0.5 -> always that entry
    logits = torch.tensor([[100.0, 0.0, 0.0, 0.0]] * 8)
    us = [0.0, 0.1, 0.3, 0.5, 0.7, 0.9, 0.999, 0.25]
    assert run_sample(ops, logits, [1.0] * 8, [0.5] * 8, us) == [0] * 8
    # :45-51: a greedy row beside a sampled one
    mixed = torch.tensor([[0.0, 0.0, 7.0], [50.0, 0.0, 0.0]])
    assert run_sample(ops, mixed, [0.0, 1.0], [1.0, 0.9], [0.5, 0.5]) == [2, 0]


def test_sample_draws_from_the_kept_weights_in_index_order(ops):
    """The kept set and its weights are the plain rule's; the draw is the
    inverse of the cumulative kept weight in index order."""
    torch.manual_seed(11)
    vocab = 1000
    logits = torch.randn(1, vocab) * 3
    for temperature, top_p in [(1.0, 1.0), (0.7, 0.9), (1.5, 0.3), (0.2, 0.05)]:
        kept, weights = plain.softmax_sample_reference(logits[0], temperature, top_p)
        order = kept.argsort()
        ids, w = kept[order], weights[order]
        cum = (w / w.sum()).cumsum(0)
        us = [i / 64 + 1 / 256 for i in range(64)]
        got = run_sample(ops, logits.expand(64, vocab).contiguous(), [temperature] * 64, [top_p] * 64, us)
        for u, tok in zip(us, got):
            assert tok in ids.tolist(), f"T={temperature} top_p={top_p}: token {tok} is outside the nucleus"
            j = int(torch.searchsorted(cum, torch.tensor(u, dtype=torch.float64), right=True))
            near = {int(ids[min(max(j + d, 0), len(ids) - 1)]) for d in (-1, 0, 1)}  # float32 cumulative sums
            assert tok in near


def test_sample_keeps_as_many_equal_weights_as_the_rule_admits(ops):
    logits = torch.zeros(1, 10)  # ten equal weights of 0.1: top_p 0.35 keeps four
    got = set()
    for u in [i / 40 for i in range(40)]:
        got.update(run_sample(ops, logits, [1.0], [0.35], [u]))
    assert got == {0, 1, 2, 3}


def test_sample_over_the_vocabulary_of_the_7b_model(ops):
    """152,064 logits are 38 chunks of 4096: the kept set is the plain rule's and the
    draw the inverse of the cumulative kept weight in index order, whatever chunk it
    falls in; rows of every kind side by side (greedy, no nucleus, narrow and wide ones)."""
    torch.manual_seed(17)
    vocab = 152064
    base = torch.randn(vocab) * 3
    cases = [(0.0, 1.0), (1.0, 1.0), (0.7, 0.9), (1.5, 0.3), (0.2, 0.05), (1.0, 0.999), (3.0, 0.5)]
    us = [0.003, 0.21, 0.5, 0.77, 0.9991]
    rows = [(t, p, u) for t, p in cases for u in us]
    logits = base.expand(len(rows), vocab).contiguous()
    got = run_sample(ops, logits, [r[0] for r in rows], [r[1] for r in rows], [r[2] for r in rows])
    for (t, p, u), tok in zip(rows, got):
        if t == 0.0:
            assert tok == int(base.argmax())
            continue
        kept, weights = plain.softmax_sample_reference(base, t, p)
        order = kept.argsort()
        ids, w = kept[order], weights[order]
        assert tok in set(ids.tolist()), f"T={t} top_p={p}: token {tok} is outside the nucleus of {len(ids)}"
        cum = (w / w.sum()).cumsum(0)
        j = int(torch.searchsorted(cum, torch.tensor(u, dtype=torch.float64), right=True))
        near = {int(ids[min(max(j + d, 0), len(ids) - 1)]) for d in (-2, -1, 0, 1, 2)}  # 24-bit weights
        assert tok in near, f"T={t} top_p={p} u={u}: token {tok}, the plain rule draws {int(ids[min(j, len(ids) - 1)])}"
    # rows that all keep everything: the short form gives the same tokens
    plain_rows = [(t, 1.0, u) for t in (0.5, 1.0, 0.0) for u in us]
    args = ([r[0] for r in plain_rows], [r[1] for r in plain_rows], [r[2] for r in plain_rows])
    wide = base.expand(len(plain_rows), vocab).contiguous()
    assert run_sample(ops, wide, *args, nucleus=False) == run_sample(ops, wide, *args, nucleus=True)


def test_sample_with_equal_weights_across_chunks_and_with_holes(ops):
    """20,000 equal logits (five chunks, more equal weights than the threshold search
    holds in LDS): top_p 0.35 keeps the 7,000 with the lowest indices, and the draw is
    uniform over them.  -inf and NaN entries are never drawn."""
    vocab = 20000
    us = [i / 50 + 0.004 for i in range(50)]
    got = run_sample(ops, torch.zeros(50, vocab), [1.0] * 50, [0.35] * 50, us)
    assert all(abs(tok - int(u * 7000)) <= 1 for tok, u in zip(got, us)), got
    holes = torch.randn(vocab)
    holes[::3] = float("-inf")
    holes[1::3] = float("nan")
    got = run_sample(ops, holes.expand(50, vocab).contiguous(), [2.0] * 50, [0.95] * 50, us)
    assert all(tok % 3 == 2 for tok in got)
    got = run_sample(ops, holes.expand(50, vocab).contiguous(), [2.0] * 50, [1.0] * 50, us, nucleus=False)
    assert all(tok % 3 == 2 for tok in got)
    # nothing has any weight: the argmax's answer (index 0)
    assert run_sample(ops, torch.full((2, 5000), float("-inf")), [1.0, 1.0], [0.9, 1.0], [0.3, 0.6]) == [0, 0]


def test_sample_random_rows_follow_the_plain_rule(ops):
    """Rows of many widths (one chunk, a chunk's edge, many chunks), spreads (flat to
    peaked), rounded logits with many equal weights, holes of -inf, temperatures and
    nuclei: the token lies in the plain rule's kept set and near the inverse of its
    cumulative kept weight in index order.  Entries whose membership hangs on less than
    1e-5 of the mass may go either way (the engine's weights have 24 bits)."""
    import random

    for seed in range(120):
        rng = random.Random(seed)
        torch.manual_seed(seed)
        vocab = rng.choice([2, 3, 17, 1000, 4095, 4096, 4097, 8191, 20000, 50000, 152064])
        rows = rng.choice([1, 2, 5])
        logits = torch.randn(rows, vocab) * rng.choice([0.0, 0.1, 1.0, 5.0, 20.0])
        if rng.random() < 0.3:
            logits = (logits * 2).round() / 2
        if rng.random() < 0.2 and vocab > 10:
            logits[:, rng.randrange(vocab)] = float("-inf")
        temps = [rng.choice([0.0, 0.05, 0.3, 0.7, 1.0, 2.0, 5.0]) for _ in range(rows)]
        tops = [rng.choice([0.01, 0.1, 0.5, 0.9, 0.95, 0.999, 1.0]) for _ in range(rows)]
        us = [rng.random() for _ in range(rows)]
        nucleus = any(t > 0 and p < 1 for t, p in zip(temps, tops)) or rng.random() < 0.5
        got = run_sample(ops, logits, temps, tops, us, nucleus=nucleus)
        for r, tok in enumerate(got):
            t, p, u = (float(torch.tensor(x, dtype=torch.float32)) for x in (temps[r], tops[r], us[r]))
            case = f"seed {seed} row {r}: vocab {vocab} T {t} top_p {p} u {u}: token {tok}"
            if t == 0.0:
                assert tok == int(logits[r].argmax()), case
                continue
            probs = torch.softmax(logits[r].double() / t, -1)
            sp, si = probs.sort(descending=True, stable=True)
            before = sp.cumsum(0) - sp
            keep, slack = before < p, (before - p).abs() < 1e-5
            either = set(si[slack].tolist())
            assert tok in set(si[keep].tolist()) | either, case + " is outside the nucleus"
            ids = si[keep].sort().values
            cum = probs[ids].cumsum(0) / probs[ids].sum()
            lo = int(torch.searchsorted(cum, torch.tensor(max(u - 1e-4, 0.0), dtype=torch.float64), right=True))
            hi = int(torch.searchsorted(cum, torch.tensor(min(u + 1e-4, 1.0), dtype=torch.float64), right=True))
            near = set(ids[max(lo - 1, 0): min(hi + 2, len(ids))].tolist()) | either
            assert tok in near, case + f", the plain rule draws {int(ids[min(lo, len(ids) - 1)])}"


def test_sample_refuses_a_scratch_that_is_too_small(ops):
    from shrike_amd.kernels import KernelError

    logits = torch.zeros(2, 5000, device="cuda")
    f = lambda x: torch.tensor(x, dtype=torch.float32, device="cuda")  # noqa: E731
    with pytest.raises(KernelError, match="scratch"):
        ops.sample(logits, torch.empty(2, dtype=torch.int32, device="cuda"), f([1.0, 1.0]), f([0.9, 0.9]),
                   f([0.5, 0.5]), torch.empty(2 * 5000, device="cuda"))
    # and a row of more than 1024 chunks of 4096
    wide = torch.zeros(1, 1024 * 4096 + 1, device="cuda")
    with pytest.raises(KernelError, match="beyond"):
        ops.sample(wide, torch.empty(1, dtype=torch.int32, device="cuda"), f([1.0]), f([0.9]), f([0.5]),
                   torch.empty(ops.sample_scratch_floats(1, wide.shape[1]), device="cuda"))


def test_sample_frequencies_follow_the_distribution(ops):
    probs = torch.tensor([0.5, 0.25, 0.125, 0.125])
    logits = probs.log()[None].expand(4096, 4).contiguous()
    from shrike_amd.sampling import uniform

    us = [uniform(123, i) for i in range(4096)]
    got = torch.tensor(run_sample(ops, logits, [1.0] * 4096, [1.0] * 4096, us))
    freq = torch.bincount(got, minlength=4).float() / 4096
    assert torch.allclose(freq, probs, atol=0.03)


# ------------------------------------------------------ bfloat16 MFMA kernels


@pytest.mark.parametrize(
    "n, m, k",
    [(1, 48, 64), (8, 3584, 3584), (7, 503, 128), (16, 100, 172), (17, 130, 96), (33, 200, 333),
     (48, 64, 64), (64, 1000, 520), (5, 37, 50), (65, 128, 64), (130, 200, 333), (300, 503, 128),
     (1000, 172, 96), (257, 130, 172), (2048, 1024, 512), (33, 200, 1600), (3, 48, 4000), (64, 100, 2100),
     (40, 33000, 1000),
     # 17 to 64 aligned rows: the kernel that streams weights per wavefront; whole and partial last
     # stages of 128 of k, shares of k, fewer row blocks than a workgroup has wavefronts
     (64, 3584, 3584), (64, 4608, 3584), (64, 3584, 18944), (17, 3584, 3584), (32, 100, 3584),
     (33, 4608, 3616), (50, 72, 160), (24, 40, 32), (64, 66000, 96)],
)
def test_gemm_tiled_weight(ops, n, m, k):
    """The MFMA kernels over the tiled weight layout (weight-streaming up to 64
    rows, LDS-staged above), at sizes that are no multiple of the tiles and
    rows that are not 16-byte aligned."""
    torch.manual_seed(12)
    dtype = torch.bfloat16
    a, w, b = torch.randn(n, k), torch.randn(m, k) / math.sqrt(k), torch.randn(m)
    want = rounded(a, dtype) @ rounded(w, dtype).t() + b.double()
    wt = ops.retile_weight(dev(w, dtype))
    assert wt.numel() == -(-m // 16) * -(-k // 32) * 512
    out = torch.empty(n, m, device="cuda", dtype=dtype)
    ops.gemm_tiled_weight(dev(a, dtype), wt, m, k, out, bias=dev(b))
    close(out, want, dtype)
    out32 = torch.full((n, m), 2.0, device="cuda")
    ops.gemm_tiled_weight(dev(a, dtype), wt, m, k, out32, accumulate=True)
    close(out32, want - b.double() + 2.0, torch.float32, scale=want.abs().max() * 20)  # float32 sums of bfloat16 products
    # a strided view of the activations (rows of a wider buffer)
    wide = torch.zeros(n, k + 24, device="cuda", dtype=dtype)
    wide[:, :k] = dev(a, dtype)
    out2 = torch.empty(n, m, device="cuda", dtype=dtype)
    ops.gemm_tiled_weight(wide[:, :k], wt, m, k, out2, bias=dev(b))
    assert torch.equal(out2, out)


@pytest.mark.parametrize(
    "n, m, k, gated",
    [(1000, 16384, 288, False),  # tiles of 256 x 256, the last token tile partly empty
     (2048, 3584, 192, False),   # tiles of 256 x 128, stages of 64: three of them
     (2000, 3600, 448, False),   # the same with a partly empty tile on both sides, seven stages
     (1000, 8192, 352, True),    # gated, 256 x 256, eleven stages
     # stages of 64 whose activations arrive as units of 8 tokens x 128 bytes: the last unit of
     # tokens partly empty, the last tile of k partly beyond k (its lanes fetch column 0)
     (1997, 3600, 424, False),
     (500, 2048, 616, False),    # tiles of 128 x 128, eight wavefronts
     # two products: the rows whose 256 x 256 tiles make a whole round of the compute
     # units, then the rest with smaller tiles (gated pairs, a bias, rows that end
     # inside a block of 16)
     (500, 18950, 1024, True),
     (500, 37900, 1024, False)],
)
def test_large_products_that_load_straight_into_lds(ops, n, m, k, gated):
    """The large tiles with aligned rows and whole stages of k: operands go from
    global memory into LDS without passing through registers; every count of
    stages ends the ring of stage buffers at another place."""
    torch.manual_seed(21)
    dtype = torch.bfloat16
    assert ops.gemm_parts(n, m, k, gated) == (2 if m > 18000 else 1)
    a = torch.randn(n, k)
    if gated:
        g, u = torch.randn(m, k) / math.sqrt(k) * 2, torch.randn(m, k) / math.sqrt(k)
        wt = ops.interleave_gate_up(dev(g, dtype), dev(u, dtype))
        gate = rounded(a, dtype) @ rounded(g, dtype).t()
        want = gate * torch.sigmoid(gate) * (rounded(a, dtype) @ rounded(u, dtype).t())
        out = torch.full((n, m), float("nan"), device="cuda", dtype=dtype)
        ops.gemm_tiled_weight(dev(a, dtype), wt, m, k, out, gated=True)
        close(out, want, dtype)
        return
    w, b = torch.randn(m, k) / math.sqrt(k), torch.randn(m)
    want = rounded(a, dtype) @ rounded(w, dtype).t() + b.double()
    wt = ops.retile_weight(dev(w, dtype))
    out = torch.full((n, m), float("nan"), device="cuda", dtype=dtype)
    ops.gemm_tiled_weight(dev(a, dtype), wt, m, k, out, bias=dev(b))
    close(out, want, dtype)
    # a row's result does not depend on the rows around it
    first = min(500, n - 300)
    part = torch.empty(300, m, device="cuda", dtype=dtype)
    ops.gemm_tiled_weight(dev(a, dtype)[first : first + 300], wt, m, k, part, bias=dev(b))
    assert torch.equal(part, out[first : first + 300])


def test_copy_words_between_page_locked_and_device_memory(ops):
    """The kernel that carries a step's index arrays to the device and its tokens
    back, with the tokens of the step before patched in on the way."""
    from shrike_amd.kernels.ops import KernelError

    host = torch.arange(1000, dtype=torch.int32).pin_memory()
    dev_buf = torch.full((1000,), -1, dtype=torch.int32, device="cuda")
    ops.copy_words(host, dev_buf)
    assert torch.equal(dev_buf.cpu(), host)
    patch = torch.tensor([7, 8, 9], dtype=torch.int32, device="cuda")
    ops.copy_words(host, dev_buf, patch=patch, patch_at=997)
    want = host.clone()
    want[997:] = torch.tensor([7, 8, 9], dtype=torch.int32)
    assert torch.equal(dev_buf.cpu(), want)
    back = torch.zeros(1000, dtype=torch.int32).pin_memory()
    ops.copy_words(dev_buf, back)
    torch.cuda.synchronize()
    assert torch.equal(back, want)
    with pytest.raises(KernelError):
        ops.copy_words(host, dev_buf, patch=patch, patch_at=998)  # the patch does not fit
    with pytest.raises(KernelError):
        ops.copy_words(torch.arange(1000, dtype=torch.int32), dev_buf)  # pageable host memory


def test_matrix_units_alone(ops):
    """The measuring kernel behind the benchmark's `mfma_tflops`: it runs, says how
    many flop it did, and refuses operands that would be read out of bounds."""
    from shrike_amd.kernels.ops import KernelError

    operands = torch.randn(32768, device="cuda").to(torch.bfloat16)
    assert ops.mfma_alone(operands, 4, 3) == 2.0 * 64 * 64 * 32 * 4 * 4 * 3
    torch.cuda.synchronize()
    with pytest.raises(KernelError):
        ops.mfma_alone(operands[:1000], 1, 1)


def test_gemm_tiled_weight_rows_do_not_depend_on_the_rest_of_the_batch(ops):
    """Within one kernel (up to 16 rows, 17 to 64, more) a row's result is bit
    for bit the same whatever else is in the call; between kernels the order of
    the float32 sums differs, so only rounding may differ."""
    torch.manual_seed(13)
    a, w = dev(torch.randn(300, 256), torch.bfloat16), dev(torch.randn(96, 256), torch.bfloat16)
    wt = ops.retile_weight(w)

    def rows(lo, hi):
        out = torch.empty(hi - lo, 96, device="cuda")
        ops.gemm_tiled_weight(a[lo:hi], wt, 96, 256, out)
        return out

    assert torch.equal(rows(23, 24)[0], rows(10, 26)[13])      # 1 row and 16 rows
    assert torch.equal(rows(0, 40)[23], rows(20, 37)[3])       # 40 rows and 17 rows
    assert torch.equal(rows(0, 300)[150], rows(100, 165)[50])  # 300 rows and 65 rows
    assert torch.allclose(rows(23, 24)[0], rows(0, 40)[23], rtol=1e-4, atol=1e-4)
    assert torch.allclose(rows(23, 24)[0], rows(0, 300)[23], rtol=1e-4, atol=1e-4)


def fill_pools(tables, k_pool, v_pool, ctx, page_size):
    kv_heads, head_dim = v_pool.shape[1], v_pool.shape[2]
    for s, c in enumerate(ctx):
        for p in range(c):
            page = int(tables[s, p // page_size])
            put_key(k_pool, page, p % page_size, torch.randn(kv_heads, head_dim).to(k_pool.dtype))
            v_pool[page, :, :, p % page_size] = torch.randn(kv_heads, head_dim).to(v_pool.dtype)


@pytest.mark.parametrize(
    "heads, kv_heads, head_dim, page_size, window, nsplit",
    [(14, 2, 64, 16, None, 1), (14, 2, 64, 16, None, 5), (28, 4, 128, 16, None, 8), (6, 3, 96, 32, 40, 3),
     (16, 1, 32, 64, None, 2), (5, 5, 256, 16, 100, 4), (8, 8, 160, 48, None, 64),
     (40, 8, 128, 16, None, 1), (40, 8, 128, 16, None, 4)],  # five query heads per group
)
def test_attention_decode_mfma(ops, heads, kv_heads, head_dim, page_size, window, nsplit):
    """Context lengths of the reference's decode test (tests/test_triton_attention.py:40-42),
    distinct random pages, unused slots poisoned with NaN."""
    torch.manual_seed(14)
    dtype = torch.bfloat16
    assert ops.attention_supports_mfma(heads, kv_heads, head_dim, page_size, heads * head_dim)
    ctx = [1, 15, 16, 17, 100, 333, 512, 7, 31, 32, 33, 129]
    n = len(ctx)
    num_pages = sum(-(-c // page_size) for c in ctx) + 5
    tables, k_pool, v_pool = paged_setup(ctx, page_size, num_pages, kv_heads, head_dim, dtype, seed=2)
    fill_pools(tables, k_pool, v_pool, ctx, page_size)
    q = torch.randn(n, heads, head_dim).to(dtype)
    positions = torch.tensor([c - 1 for c in ctx], dtype=torch.int32)
    out = torch.full((n, heads * head_dim), float("nan"), device="cuda", dtype=dtype)
    partial = torch.full((n * heads * nsplit * (head_dim + 2),), float("nan"), device="cuda")
    scale = 1.3 * head_dim**-0.5
    ops.attention_decode(dev(q).view(n, -1), out, n, heads, kv_heads, head_dim, dev(positions), tables,
                         k_pool, v_pool, page_size, window, scale, partial, nsplit)
    want = reference_attention(q.double(), k_pool, v_pool, tables, [1] * n, [c - 1 for c in ctx], page_size, window, scale)
    assert not torch.isnan(out.float()).any(), "a slot outside the context reached the output"
    close(out.view(n, heads, head_dim), want, dtype, scale=1.0)
    # with non-temporal loads of keys and values: the same bits
    streamed = torch.full_like(out, float("nan"))
    partial.fill_(float("nan"))
    ops.attention_decode(dev(q).view(n, -1), streamed, n, heads, kv_heads, head_dim, dev(positions), tables,
                         k_pool, v_pool, page_size, window, scale, partial, nsplit, streaming=True)
    assert torch.equal(streamed, out)


@pytest.mark.parametrize(
    "heads, kv_heads, head_dim, page_size, window",
    [(14, 2, 64, 16, None), (28, 4, 128, 16, None), (6, 3, 96, 32, 40), (4, 1, 32, 64, 17), (5, 5, 256, 16, None),
     (40, 8, 128, 16, None)],
)
def test_attention_prefill_mfma(ops, heads, kv_heads, head_dim, page_size, window):
    """Portions of 2 to 200 tokens, some with earlier context, tiles with fewer than 16 queries."""
    torch.manual_seed(15)
    dtype = torch.bfloat16
    seq_lens = [2, 200, 16, 17, 90, 33]
    starts = [0, 60, 5, 100, 0, 31]
    ctx = [s + l for s, l in zip(starts, seq_lens)]
    n = sum(seq_lens)
    num_pages = sum(-(-c // page_size) for c in ctx) + 5
    tables, k_pool, v_pool = paged_setup(ctx, page_size, num_pages, kv_heads, head_dim, dtype, seed=3)
    fill_pools(tables, k_pool, v_pool, ctx, page_size)
    q = torch.randn(n, heads, head_dim).to(dtype)
    cu = [0]
    for l in seq_lens:
        cu.append(cu[-1] + l)
    tile_seq, tile_q0 = [], []
    for s, l in enumerate(seq_lens):
        for q0 in range(0, l, 16):
            tile_seq.append(s)
            tile_q0.append(q0)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device="cuda")  # noqa: E731
    out = torch.full((n, heads * head_dim), float("nan"), device="cuda", dtype=dtype)
    scale = head_dim**-0.5
    ops.attention_prefill(dev(q).view(n, -1), out, len(tile_seq), heads, kv_heads, head_dim, i32(cu), i32(ctx),
                          i32(tile_seq), i32(tile_q0), tables, k_pool, v_pool, page_size, window, scale)
    want = reference_attention(q.double(), k_pool, v_pool, tables, seq_lens, starts, page_size, window, scale)
    assert not torch.isnan(out.float()).any()
    close(out.view(n, heads, head_dim), want, dtype, scale=1.0)


def test_attention_mfma_finds_one_far_key_among_thousands(ops):
    """Decode over 3000 keys split 16 ways: one key in an early page is made to stand out."""
    torch.manual_seed(16)
    dtype = torch.bfloat16
    heads, kv_heads, head_dim, page_size, ctx = 14, 2, 128, 16, 3000
    tables, k_pool, v_pool = paged_setup([ctx], page_size, 256, kv_heads, head_dim, dtype, seed=4)
    k = torch.randn(ctx, kv_heads, head_dim) * 0.1
    v = torch.randn(ctx, kv_heads, head_dim)
    q = torch.randn(1, heads, head_dim)
    far = 41
    k[far, 0] = q[0, 3] * 2.0  # head 3 of group 0
    for p in range(ctx):
        page = int(tables[0, p // page_size])
        put_key(k_pool, page, p % page_size, k[p].to(dtype))
        v_pool[page, :, :, p % page_size] = v[p].to(dtype)
    out = torch.empty(1, heads * head_dim, device="cuda", dtype=dtype)
    partial = torch.empty(heads * 16 * (head_dim + 2), device="cuda")
    ops.attention_decode(dev(q, dtype).view(1, -1), out, 1, heads, kv_heads, head_dim,
                         torch.tensor([ctx - 1], dtype=torch.int32, device="cuda"), tables, k_pool, v_pool,
                         page_size, None, 1.0, partial, 16)
    got = out.view(heads, head_dim).float().cpu()
    assert torch.allclose(got[3], v[far, 0].to(dtype).float(), atol=3e-2)
    want = reference_attention(q.to(dtype).double(), k_pool, v_pool, tables, [1], [ctx - 1], page_size, None, 1.0)
    close(out.view(1, heads, head_dim), want, dtype, scale=1.0)


@pytest.mark.parametrize("n, inter, k", [(1, 172, 64), (8, 18944, 256), (20, 100, 96), (40, 352, 128), (64, 48, 50),
                                         (9, 100, 1700), (50, 64, 3000), (40, 16400, 1040),
                                         (64, 18944, 3584), (17, 2000, 416), (32, 66000, 64),
                                         (65, 172, 64), (300, 1000, 520), (1000, 200, 96)])
@pytest.mark.parametrize("activation", ["silu", "gelu_tanh"])
def test_gated_gemm_is_the_activated_gate_times_up(ops, n, inter, k, activation):
    """One product over the interleaved gate/up weight yields act(x g^T) * (x u^T), in
    every kernel that serves gated products (few tokens, 17 to 64, many)."""
    torch.manual_seed(17)
    dtype = torch.bfloat16
    x = torch.randn(n, k)
    g, u = torch.randn(inter, k) / math.sqrt(k) * 2, torch.randn(inter, k) / math.sqrt(k)
    wt = ops.interleave_gate_up(dev(g, dtype), dev(u, dtype))
    out = torch.full((n, inter), float("nan"), device="cuda", dtype=dtype)
    ops.gemm_tiled_weight(dev(x, dtype), wt, inter, k, out, gated=activation)
    gate = rounded(x, dtype) @ rounded(g, dtype).t()
    want = gate_reference(gate, activation) * (rounded(x, dtype) @ rounded(u, dtype).t())
    close(out, want, dtype)
    if activation == "silu":  # True stands for the activation of SwiGLU
        again = torch.empty_like(out)
        ops.gemm_tiled_weight(dev(x, dtype), wt, inter, k, again, gated=True)
        assert torch.equal(again, out)


@pytest.mark.parametrize("n, m, k", [(8, 3584, 3584), (1, 48, 4000), (33, 200, 2400), (64, 100, 2100),
                                     (64, 3584, 3584), (64, 4608, 3584), (64, 3584, 18944), (20, 3584, 18944),
                                     (100, 3584, 3584), (300, 136, 1100), (64, 2100, 16400), (40, 2100, 16400),
                                     (512, 5120, 5120)])  # the last: many tokens, tiles of 256 x 128 in three shares
def test_split_product_and_its_readers(ops, n, m, k):
    """A product split along k leaves partial sums; the norm and the cache-write
    kernel add them up in order and give what the unsplit product gives."""
    torch.manual_seed(18)
    dtype = torch.bfloat16
    splits = ops.gemm_splits(n, m, k)
    assert splits > 1 and ops.gemm_splits(n, 40000, k) == 1 and ops.gemm_splits(4096, 20000, k) == 1
    a, w = torch.randn(n, k), torch.randn(m, k) / math.sqrt(k)
    wt = ops.retile_weight(dev(w, dtype))
    parts = torch.full((splits, n, m), float("nan"), device="cuda")
    ops.gemm_tiled_weight(dev(a, dtype), wt, m, k, parts, splits=splits)
    want = rounded(a, dtype) @ rounded(w, dtype).t()
    close(parts.sum(0), want, torch.float32, scale=want.abs().max() * 50)
    total = parts[0].clone()
    for z in range(1, splits):
        total += parts[z]
    # the norm adds the parts to the residual stream
    if m % 4 == 0:
        resid = torch.randn(n, m, device="cuda")
        before = resid.clone()
        wn = 1 + 0.1 * torch.randn(m, device="cuda")
        out = torch.empty(n, m, device="cuda", dtype=dtype)
        ops.add_rmsnorm(resid, ops.SplitSum(parts), wn, 1e-5, out)
        assert torch.equal(resid, before + total)
        close(out, plain.rms_norm((before + total).double().cpu(), wn.double().cpu(), 1e-5), dtype)


@pytest.mark.parametrize("n, splits", [(5, 3), (70, 3), (66, 9)])  # few tokens: element by element; many: in vectors
def test_rope_kv_store_adds_up_a_split_product(ops, n, splits):
    torch.manual_seed(19)
    dtype = torch.bfloat16
    heads, kv_heads, head_dim, page_size, theta = 6, 2, 64, 16, 1e4
    width = (heads + 2 * kv_heads) * head_dim
    parts = torch.randn(splits, n, width, device="cuda")
    bias = torch.randn(width, device="cuda")
    positions = torch.tensor([3, 17, 100, 0, 31] + list(range(40, 35 + n)), dtype=torch.int32, device="cuda")
    token_seq = torch.arange(n, dtype=torch.int32, device="cuda")
    tables, k_pool, v_pool = paged_setup([p + 1 for p in positions.tolist()], page_size, 512, kv_heads, head_dim, dtype)
    inv_freq = (1.0 / (theta ** (torch.arange(0, head_dim, 2).float() / head_dim))).cuda()
    qkv = torch.full((n, width), float("nan"), device="cuda", dtype=dtype)
    ops.rope_kv_store(qkv, heads, kv_heads, head_dim, head_dim, inv_freq, positions, token_seq, tables,
                      k_pool, v_pool, page_size, split_sum=ops.SplitSum(parts, bias))
    total = parts[0].clone()
    for z in range(1, splits):
        total += parts[z]
    x = (total + bias).double().cpu()
    cos, sin = plain.rope_tables(positions.long().cpu(), head_dim, theta)
    q = plain.apply_rope(x[:, : heads * head_dim].view(n, heads, head_dim), cos, sin)
    close(qkv[:, : heads * head_dim].reshape(n, heads, head_dim), q, dtype)
    k = plain.apply_rope(x[:, heads * head_dim : (heads + kv_heads) * head_dim].view(n, kv_heads, head_dim), cos, sin)
    v = x[:, (heads + kv_heads) * head_dim :].view(n, kv_heads, head_dim)
    for t in range(n):
        p = int(positions[t])
        page = int(tables[t, p // page_size])
        close(get_key(k_pool, page, p % page_size), k[t], dtype)
        close(v_pool[page, :, :, p % page_size], v[t], dtype)


@pytest.mark.parametrize(
    "heads, kv_heads, head_dim, page_size, window",
    [(14, 2, 64, 16, None), (28, 4, 128, 16, None), (6, 3, 96, 32, 40), (4, 1, 32, 64, 17), (5, 5, 128, 16, None),
     (16, 2, 64, 16, 100), (3, 1, 128, 48, None), (16, 1, 32, 16, None), (12, 1, 64, 32, 50),
     (40, 8, 128, 16, None)],
)
@pytest.mark.parametrize("small, nsplit, singles", [(False, 1, 0), (True, 1, 0), (True, 3, 0), (False, 8, 0),
                                                    (True, 3, 5), (False, 8, 5), (False, 1, 3)])
def test_attention_prefill_shared_mfma(ops, heads, kv_heads, head_dim, page_size, window, small, nsplit, singles):
    """The prefill kernel that shares each chunk of keys among the query heads of a
    key/value head: 1 to 16 heads per group, portions of 2 to 200 tokens, in
    workgroups of 16 wavefronts and of 8 (`small`), every entry's keys in one
    workgroup or shared among 3 or 8 (more shares than some entries have chunks
    of keys: the last ones find nothing to do).  `singles`: that many sequences
    with one token each come first in the step, as in a step that mixes decoding
    with prompt portions; the kernel is told where the prompt tokens begin
    (first_token) and must leave the single tokens' rows alone."""
    torch.manual_seed(20)
    dtype = torch.bfloat16
    tiles = ops.attention_prefill_shared_tiles(heads, kv_heads, head_dim, small)
    assert tiles == (8 if small else 16) // (heads // kv_heads)
    if tiles == 0:
        pytest.skip("more query heads per key/value head than the small workgroup has wavefronts")
    seq_lens = [1] * singles + [2, 200, 16, 17, 90, 33, 130]
    starts = [9, 40, 0, 77, 16][:singles] + [0, 60, 5, 100, 0, 31, 7]
    ctx = [s + l for s, l in zip(starts, seq_lens)]
    n = sum(seq_lens)
    num_pages = sum(-(-c // page_size) for c in ctx) + 5
    tables, k_pool, v_pool = paged_setup(ctx, page_size, num_pages, kv_heads, head_dim, dtype, seed=5)
    fill_pools(tables, k_pool, v_pool, ctx, page_size)
    q = torch.randn(n, heads, head_dim).to(dtype)
    cu = [0]
    for l in seq_lens:
        cu.append(cu[-1] + l)
    wg_seq, wg_q0 = [], []
    for s, l in enumerate(seq_lens):
        if s < singles:
            continue  # the decode kernel's rows
        for q0 in range(0, l, 16 * tiles):
            wg_seq.append(s)
            wg_q0.append(q0)
    # the kernel takes the list in any order (the engine sends the heaviest entries first)
    mixed = torch.randperm(len(wg_seq), generator=torch.Generator().manual_seed(3)).tolist()
    wg_seq, wg_q0 = [wg_seq[i] for i in mixed], [wg_q0[i] for i in mixed]
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device="cuda")  # noqa: E731
    out = torch.full((n, heads * head_dim), float("nan"), device="cuda", dtype=dtype)
    scale = head_dim**-0.5
    partial = torch.full(((n - singles) * heads * nsplit * (head_dim + 2),), float("nan"), device="cuda")
    ops.attention_prefill_shared(dev(q).view(n, -1), out, len(wg_seq), heads, kv_heads, head_dim, i32(cu), i32(ctx),
                                 i32(wg_seq), i32(wg_q0), tables, k_pool, v_pool, page_size, window, scale,
                                 small=small, partial=partial, nsplit=nsplit, first_token=singles)
    want = reference_attention(q.double(), k_pool, v_pool, tables, seq_lens, starts, page_size, window, scale)
    assert torch.isnan(out[:singles].float()).all()  # the single tokens' rows were not touched
    assert not torch.isnan(out[singles:].float()).any()
    close(out[singles:].view(n - singles, heads, head_dim), want[singles:], dtype, scale=1.0)


def test_attention_prefill_shared_refuses_wide_groups(ops):
    assert ops.attention_prefill_shared_tiles(34, 2, 64) == 0  # 17 heads per group: the per-tile kernel serves it
    assert ops.attention_prefill_shared_tiles(8, 2, 256) == 0


def fill_pools_from(tables, k_pool, v_pool, seq, keys, values, page_size):
    """Whole sequences of keys/values [ctx, kv_heads, head_dim] into sequence `seq`'s pages."""
    ctx = keys.shape[0]
    for first in range(0, ctx, page_size):
        page = int(tables[seq, first // page_size])
        n = min(page_size, ctx - first)
        k = keys[first : first + n].to(k_pool.dtype).to(k_pool.device)  # [n, kv, d]
        k_pool[page, :, :, :n, :] = k.view(n, k_pool.shape[1], k_pool.shape[2], k_pool.shape[4]).permute(1, 2, 0, 3)
        v_pool[page, :, :, :n] = values[first : first + n].to(v_pool.dtype).to(v_pool.device).permute(1, 2, 0)


@pytest.mark.parametrize("heads, kv_heads", [(28, 4), (40, 8)])
@pytest.mark.parametrize("kernel", ["shared", "tiles"])
def test_attention_prefill_over_two_thousand_keys(ops, heads, kv_heads, kernel):
    """A 2,048-token prompt in one step (64 chunks of keys per query tile at the
    end) beside a 300-token portion that starts at position 1,900.  Among random
    scores near zero, chosen queries each have one key far away (or at a chunk's
    or a page's edge) whose score stands out: a chunk of keys that is skipped,
    read twice or masked wrongly changes those rows beyond the tolerance, where
    uniform attention over thousands of keys would hide it."""
    torch.manual_seed(31)
    dtype = torch.bfloat16
    head_dim, page_size, group = 128, 16, heads // kv_heads
    seq_lens, starts = [2048, 300], [0, 1900]
    ctx = [s + l for s, l in zip(starts, seq_lens)]
    n = sum(seq_lens)
    tables, k_pool, v_pool = paged_setup(ctx, page_size, sum(-(-c // page_size) for c in ctx) + 3, kv_heads,
                                         head_dim, dtype, seed=6)
    q = torch.randn(n, heads, head_dim) * 0.3
    keys = [torch.randn(c, kv_heads, head_dim) * 0.3 for c in ctx]
    values = [torch.randn(c, kv_heads, head_dim) for c in ctx]
    # (sequence, query position, key position): far back, the query's own key, edges of 32-key
    # chunks and of pages, the first key of all
    pairs = [(0, 2047, 0), (0, 2046, 2015), (0, 2040, 1000), (0, 1024, 1023), (0, 1025, 31), (0, 1026, 32),
             (0, 16, 15), (0, 33, 0), (0, 15, 15), (0, 1500, 1471), (0, 777, 16), (0, 2031, 2031),
             (1, 1900, 3), (1, 2199, 1899), (1, 2100, 1900), (1, 1915, 1915), (1, 2000, 63), (1, 2001, 64)]
    amp = 20.0  # score of a pair: amp^2 / sqrt(128) = 35 against scores of a few units
    for i, (s, p, j) in enumerate(pairs):
        u = torch.zeros(head_dim)
        u[(7 * i) % head_dim] = amp
        row = sum(seq_lens[:s]) + p - starts[s]
        head = (3 * i) % heads
        q[row, head] = u
        keys[s][j, head // group] = u
    for s in range(2):
        fill_pools_from(tables, k_pool, v_pool, s, keys[s], values[s], page_size)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device="cuda")  # noqa: E731
    out = torch.full((n, heads * head_dim), float("nan"), device="cuda", dtype=dtype)
    scale = head_dim**-0.5
    qd = dev(q.to(dtype)).view(n, -1)
    run = 16 * (ops.attention_prefill_shared_tiles(heads, kv_heads, head_dim) if kernel == "shared" else 1)
    wg_seq = [s for s, l in enumerate(seq_lens) for _ in range(0, l, run)]
    wg_q0 = [q0 for l in seq_lens for q0 in range(0, l, run)]
    args = (i32([0, 2048, n]), i32(ctx), i32(wg_seq), i32(wg_q0), tables, k_pool, v_pool, page_size, None, scale)
    if kernel == "shared":
        ops.attention_prefill_shared(qd, out, len(wg_seq), heads, kv_heads, head_dim, *args)
    else:
        ops.attention_prefill(qd, out, len(wg_seq), heads, kv_heads, head_dim, *args)
    want = reference_attention(q.to(dtype).double(), k_pool, v_pool, tables, seq_lens, starts, page_size, None, scale)
    assert not torch.isnan(out.float()).any()
    got = out.view(n, heads, head_dim)
    close(got, want, dtype, scale=1.0)
    for i, (s, p, j) in enumerate(pairs):  # each chosen row is its far key's value
        row, head = sum(seq_lens[:s]) + p - starts[s], (3 * i) % heads
        v = values[s][j, head // group].to(dtype).double()
        assert (got[row, head].double().cpu() - v).abs().max() <= 2e-2 * v.abs().max(), (s, p, j)


@pytest.mark.parametrize("kernel", ["shared", "tiles"])
def test_attention_prefill_of_portions_far_into_a_sequence(ops, kernel):
    """Prompt portions that start at positions 30,000 and 16,000 (a long prompt cut
    by the token budget): their queries read thousands of keys written by earlier
    steps; chosen queries have one key that stands out, at the sequence's start, at
    the portion's own start, just before it."""
    torch.manual_seed(33)
    dtype = torch.bfloat16
    heads, kv_heads, head_dim, page_size, group = 28, 4, 128, 16, 7
    seq_lens, starts = [200, 64], [30000, 16000]
    ctx = [s + l for s, l in zip(starts, seq_lens)]
    n = sum(seq_lens)
    tables, k_pool, v_pool = paged_setup(ctx, page_size, sum(-(-c // page_size) for c in ctx) + 3, kv_heads,
                                         head_dim, dtype, seed=8)
    q = torch.randn(n, heads, head_dim) * 0.3
    keys = [torch.randn(c, kv_heads, head_dim) * 0.3 for c in ctx]
    values = [torch.randn(c, kv_heads, head_dim) for c in ctx]
    pairs = [(0, 30000, 0), (0, 30199, 29999), (0, 30100, 30000), (0, 30017, 15000), (0, 30150, 30150),
             (1, 16000, 15999), (1, 16063, 31), (1, 16032, 16000)]
    for i, (s, p, j) in enumerate(pairs):
        u = torch.zeros(head_dim)
        u[(7 * i) % head_dim] = 20.0
        head = (3 * i) % heads
        q[sum(seq_lens[:s]) + p - starts[s], head] = u
        keys[s][j, head // group] = u
    for s in range(2):
        fill_pools_from(tables, k_pool, v_pool, s, keys[s], values[s], page_size)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device="cuda")  # noqa: E731
    out = torch.full((n, heads * head_dim), float("nan"), device="cuda", dtype=dtype)
    scale = head_dim**-0.5
    run = 16 * (ops.attention_prefill_shared_tiles(heads, kv_heads, head_dim, small=True) if kernel == "shared" else 1)
    wg_seq = [s for s, l in enumerate(seq_lens) for _ in range(0, l, run)]
    wg_q0 = [q0 for l in seq_lens for q0 in range(0, l, run)]
    args = (i32([0, 200, n]), i32(ctx), i32(wg_seq), i32(wg_q0), tables, k_pool, v_pool, page_size, None, scale)
    qd = dev(q.to(dtype)).view(n, -1)
    if kernel == "shared":  # as the engine launches such a step: every entry's keys shared among workgroups
        from shrike_amd.parts.attention import portion_splits

        nsplit = portion_splits(len(wg_seq) * kv_heads, 23000)
        assert nsplit > 1
        partial = torch.full((n * heads * nsplit * (head_dim + 2),), float("nan"), device="cuda")
        ops.attention_prefill_shared(qd, out, len(wg_seq), heads, kv_heads, head_dim, *args, small=True,
                                     partial=partial, nsplit=nsplit)
    else:
        ops.attention_prefill(qd, out, len(wg_seq), heads, kv_heads, head_dim, *args)
    want = reference_attention(q.to(dtype).double(), k_pool, v_pool, tables, seq_lens, starts, page_size, None, scale)
    assert not torch.isnan(out.float()).any()
    got = out.view(n, heads, head_dim)
    close(got, want, dtype, scale=1.0)
    for i, (s, p, j) in enumerate(pairs):
        row, head = sum(seq_lens[:s]) + p - starts[s], (3 * i) % heads
        v = values[s][j, head // group].to(dtype).double()
        assert (got[row, head].double().cpu() - v).abs().max() <= 2e-2 * v.abs().max(), (s, p, j)


@pytest.mark.parametrize(
    "ctx, special",
    [([4100, 4096, 2049, 2048, 1025, 300, 4097, 1], [0, 4095, 1023, 2047, 512, 299, 2048, 0]),
     # block tables of 2,500 pages, the most key splits the kernel has
     ([40000, 33001, 16385, 70], [0, 33000, 8192, 69])],
)
def test_attention_decode_finds_far_keys_in_a_long_context(ops, ctx, special):
    """Single tokens at contexts up to 4,100 and up to 40,000 with the key splits
    the engine would choose for them; every sequence has one key whose score
    stands out, at the start, at a split's edge, at the very end."""
    from shrike_amd.parts.attention import decode_splits

    torch.manual_seed(32)
    dtype = torch.bfloat16
    heads, kv_heads, head_dim, page_size, group = 28, 4, 128, 16, 7
    n = len(ctx)
    tables, k_pool, v_pool = paged_setup(ctx, page_size, sum(-(-c // page_size) for c in ctx) + 3, kv_heads,
                                         head_dim, dtype, seed=7)
    q = torch.randn(n, heads, head_dim) * 0.3
    values = []
    for s, c in enumerate(ctx):
        keys, vals = torch.randn(c, kv_heads, head_dim) * 0.3, torch.randn(c, kv_heads, head_dim)
        u = torch.zeros(head_dim)
        u[(11 * s) % head_dim] = 20.0
        q[s, (5 * s) % heads] = u
        keys[special[s], ((5 * s) % heads) // group] = u
        fill_pools_from(tables, k_pool, v_pool, s, keys, vals, page_size)
        values.append(vals)
    positions = torch.tensor([c - 1 for c in ctx], dtype=torch.int32)
    scale = head_dim**-0.5
    for nsplit in sorted({decode_splits(n, kv_heads, max(ctx)), decode_splits(1, kv_heads, max(ctx)), 1}):
        out = torch.full((n, heads * head_dim), float("nan"), device="cuda", dtype=dtype)
        partial = torch.full((n * heads * nsplit * (head_dim + 2),), float("nan"), device="cuda")
        ops.attention_decode(dev(q.to(dtype)).view(n, -1), out, n, heads, kv_heads, head_dim, dev(positions), tables,
                             k_pool, v_pool, page_size, None, scale, partial, nsplit, streaming=nsplit > 1)
        want = reference_attention(q.to(dtype).double(), k_pool, v_pool, tables, [1] * n, [c - 1 for c in ctx],
                                   page_size, None, scale)
        got = out.view(n, heads, head_dim)
        assert not torch.isnan(out.float()).any()
        close(got, want, dtype, scale=1.0)
        for s in range(n):
            head = (5 * s) % heads
            v = values[s][special[s], head // group].to(dtype).double()
            assert (got[s, head].double().cpu() - v).abs().max() <= 2e-2 * v.abs().max(), (nsplit, s)
