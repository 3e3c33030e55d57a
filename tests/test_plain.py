"""Pins the plain implementation by what fixes it beside the reference's text:
library routines it must reduce to, invariants, and vectors the reference's
own tests hold.  Each check is chosen so that a plausible mistake fails it."""

import torch
import torch.nn.functional as F

from .plain import model as plain
from .tiny import make_model_dir

torch.manual_seed(0)


def test_rms_norm_is_the_library_routine_and_eps_is_inside_the_root():
    x, w = torch.randn(5, 48, dtype=torch.float64), torch.randn(48, dtype=torch.float64)
    assert torch.allclose(plain.rms_norm(x, w, 1e-5), F.rms_norm(x, (48,), w, 1e-5), atol=1e-12)
    tiny = torch.full((1, 4), 1e-4, dtype=torch.float64)
    one = torch.ones(4, dtype=torch.float64)
    # mean square 1e-8 against eps 1e-2: eps inside the root gives x / sqrt(eps + ms)
    assert torch.allclose(plain.rms_norm(tiny, one, 1e-2), tiny / (1e-2 + 1e-8) ** 0.5)
    # not a mean-subtracting norm: a constant row stays constant and non-zero
    assert torch.allclose(plain.rms_norm(torch.full((1, 8), 3.0), torch.ones(8), 1e-12), torch.ones(1, 8))


def test_rope_is_a_complex_rotation_on_the_half_split_pairing():
    d, theta = 16, 10000.0
    pos = torch.tensor([0, 1, 5, 77])
    x = torch.randn(4, 3, d, dtype=torch.float64)
    cos, sin = plain.rope_tables(pos, d, theta)
    got = plain.apply_rope(x, cos, sin)
    inv_freq = 1.0 / (theta ** (torch.arange(0, d, 2).float() / d))
    angle = torch.outer(pos.float(), inv_freq).double()
    z = torch.complex(x[..., : d // 2], x[..., d // 2 :]) * torch.polar(torch.ones_like(angle), angle)[:, None]
    assert torch.allclose(got[..., : d // 2], z.real, atol=1e-12)
    assert torch.allclose(got[..., d // 2 :], z.imag, atol=1e-12)
    assert torch.equal(got[0], x[0])  # position 0 is the identity
    # an interleaved pairing (0,1),(2,3).. would not keep these pair norms
    pair = lambda t: t[..., : d // 2] ** 2 + t[..., d // 2 :] ** 2  # noqa: E731
    assert torch.allclose(pair(got), pair(x), atol=1e-12)


def test_rope_frequencies_are_a_geometric_sequence_from_one_down():
    """The rotation rates, written out as numbers rather than recomputed from the
    expression under test (shrike/models/qwen.py:80): pair i turns by
    theta**(-2i/d) per position, so for theta = 10^4 and d = 16 the rates are
    10**(-i/2), and for theta = 10^6 and d = 32 each is 10**-0.375 times the one
    before, the last 10**-5.625.  An exponent of i/d, of 2i/(d-2) or an order
    from slow to fast fails this."""
    cos, sin = plain.rope_tables(torch.tensor([1]), 16, 10000.0)
    rates = torch.atan2(sin[0, :8], cos[0, :8]).double()
    want = torch.tensor([1.0, 0.31622776601683794, 0.1, 0.031622776601683794, 0.01,
                         0.0031622776601683794, 0.001, 0.00031622776601683794], dtype=torch.float64)
    assert torch.allclose(rates, want, rtol=1e-6, atol=0)
    assert torch.equal(cos[0, :8], cos[0, 8:]) and torch.equal(sin[0, :8], sin[0, 8:])  # both halves alike
    cos, sin = plain.rope_tables(torch.tensor([1]), 32, 1e6)
    rates = torch.atan2(sin[0, :16], cos[0, :16]).double()
    assert abs(float(rates[0]) - 1.0) < 1e-6 and abs(float(rates[15]) / 2.3713737056616554e-06 - 1) < 1e-5
    assert torch.allclose(rates[1:] / rates[:-1], torch.full((15,), 0.42169650342858224, dtype=torch.float64),
                          rtol=1e-5)
    # position scales the angle: 1,000 positions turn the slowest pair of the first table by 0.316 rad
    cos, sin = plain.rope_tables(torch.tensor([1000]), 16, 10000.0)
    assert abs(float(torch.atan2(sin[0, 7], cos[0, 7])) - 0.31622776601683794) < 1e-5


def test_rope_scores_depend_only_on_distance():
    d, theta = 32, 1e6
    q, k = torch.randn(1, 1, d, dtype=torch.float64), torch.randn(1, 1, d, dtype=torch.float64)

    def score(m, n):
        cq, sq = plain.rope_tables(torch.tensor([m]), d, theta)
        ck, sk = plain.rope_tables(torch.tensor([n]), d, theta)
        return (plain.apply_rope(q, cq, sq) * plain.apply_rope(k, ck, sk)).sum()

    assert torch.allclose(score(9, 4), score(105, 100), atol=1e-9)
    assert not torch.allclose(score(9, 4), score(4, 9), atol=1e-6)  # a wrong sign would swap these


def test_attention_is_the_library_routine():
    n, h, hkv, d = 9, 6, 2, 16
    q = torch.randn(n, h, d, dtype=torch.float64)
    k, v = torch.randn(n, hkv, d, dtype=torch.float64), torch.randn(n, hkv, d, dtype=torch.float64)
    got = plain.causal_attention(q, k, v)
    # the reference's oracle: SDPA, causal, grouped (shrike/models/qwen.py:240-244)
    want = F.scaled_dot_product_attention(
        q.transpose(0, 1)[None], k.transpose(0, 1)[None], v.transpose(0, 1)[None],
        is_causal=True, enable_gqa=True,
    )[0].transpose(0, 1)
    assert torch.allclose(got, want, atol=1e-12)
    # grouped = every kv head repeated for its group of consecutive query heads
    want2 = plain.causal_attention(q, k.repeat_interleave(h // hkv, 1), v.repeat_interleave(h // hkv, 1))
    assert torch.allclose(got, want2, atol=1e-12)
    assert torch.allclose(got[0], v[0].repeat_interleave(h // hkv, 0))  # one key: the value itself


def test_attention_vectors_of_the_reference_decode_test():
    """The einsum formula of tests/test_triton_attention.py:22-37 (H=14, Hkv=2, D=64)
    on the last query of a sequence."""
    h, hkv, d = 14, 2, 64
    for n in (1, 15, 16, 17, 100):
        q = torch.randn(n, h, d, dtype=torch.float64)
        k, v = torch.randn(n, hkv, d, dtype=torch.float64), torch.randn(n, hkv, d, dtype=torch.float64)
        qg = q[-1].view(hkv, h // hkv, d)
        scores = torch.einsum("kgd,skd->kgs", qg, k) * d**-0.5
        want = torch.einsum("kgs,skd->kgd", scores.softmax(-1), v).reshape(h, d)
        assert torch.allclose(plain.causal_attention(q, k, v)[-1], want, atol=1e-12)


def test_attention_window_keeps_the_last_keys_only():
    n, d = 12, 8
    q, k, v = (torch.randn(n, 1, d, dtype=torch.float64) for _ in range(3))
    got = plain.causal_attention(q, k, v, window=4)
    for p in range(n):
        lo = max(0, p - 3)
        want = plain.causal_attention(q[lo : p + 1], k[lo : p + 1], v[lo : p + 1])[-1]
        assert torch.allclose(got[p], want, atol=1e-12)
    assert torch.allclose(plain.causal_attention(q, k, v, window=n), plain.causal_attention(q, k, v))


def test_swiglu_is_silu_times_up():
    x = torch.randn(3, 10, dtype=torch.float64)
    wg, wu, wd = (torch.randn(*s, dtype=torch.float64) for s in ((7, 10), (7, 10), (10, 7)))
    want = F.linear(F.silu(F.linear(x, wg)) * F.linear(x, wu), wd)
    assert torch.allclose(plain.swiglu(x, wg, wu, wd), want, atol=1e-12)
    assert torch.count_nonzero(plain.swiglu(x, torch.zeros_like(wg), wu, wd)) == 0  # gate 0 -> 0


def test_model_is_causal_and_shift_invariant(tmp_path):
    m = plain.PlainModel(make_model_dir("B", tmp_path))
    ids = torch.randint(0, 503, (20,)).tolist()
    full = m.logits(ids)
    changed = ids[:12] + [(t + 1) % 503 for t in ids[12:]]
    assert torch.allclose(m.logits(changed)[:12], full[:12], atol=1e-12)
    assert not torch.allclose(m.logits(changed)[12:], full[12:], atol=1e-6)
    # only distances between positions count
    shifted = plain.forward(m.cfg, m.weights, ids, first_position=37)
    assert torch.allclose(shifted, full, atol=1e-6)


def test_tied_model_uses_the_embedding_table_as_output_matrix(tmp_path):
    m = plain.PlainModel(make_model_dir("A", tmp_path))
    assert "lm_head.weight" not in m.weights
    ids = [3, 9, 200]
    w = dict(m.weights)
    w["lm_head.weight"] = w["model.embed_tokens.weight"].clone()
    assert torch.equal(plain.forward(m.cfg, w, ids), m.logits(ids))


def test_norm_sits_before_each_part_and_the_residual_skips_it(tmp_path):
    """With the attention and feed-forward outputs forced to zero the model is
    embedding -> final norm -> output matrix: no norm touches the residual."""
    m = plain.PlainModel(make_model_dir("A", tmp_path))
    w = {k: (torch.zeros_like(v) if "o_proj" in k or "down_proj" in k else v) for k, v in m.weights.items()}
    ids = [1, 2, 3]
    e = w["model.embed_tokens.weight"][torch.tensor(ids)]
    want = plain.rms_norm(e, w["model.norm.weight"], m.cfg.rms_norm_eps) @ w["model.embed_tokens.weight"].t()
    assert torch.allclose(plain.forward(m.cfg, w, ids), want, atol=1e-12)


def test_sampler_vectors_of_the_reference():
    # tests/test_sampler.py:36-42: one dominant entry, top_p 0.5 -> only it is kept
    ids, weights = plain.softmax_sample_reference(torch.tensor([100.0, 0.0, 0.0, 0.0]), 1.0, 0.5)
    assert ids.tolist() == [0]
    # top_p 1 keeps everything
    ids, _ = plain.softmax_sample_reference(torch.tensor([1.0, 2.0, 3.0, 0.5]), 1.0, 1.0)
    assert sorted(ids.tolist()) == [0, 1, 2, 3]
    # mass before an entry below top_p: [0.5, 0.3, 0.2], top_p 0.6 keeps two
    ids, _ = plain.softmax_sample_reference(torch.log(torch.tensor([0.2, 0.5, 0.3])), 1.0, 0.6)
    assert ids.tolist() == [1, 2]


def test_attention_of_the_last_queries_alone():
    """`first`: only the queries from that position on, against the rows of the whole."""
    torch.manual_seed(5)
    n, h, hkv, d = 23, 6, 2, 8
    q, k, v = torch.randn(n, h, d).double(), torch.randn(n, hkv, d).double(), torch.randn(n, hkv, d).double()
    for window in (None, 5):
        whole = plain.causal_attention(q, k, v, window)
        for first in (0, 1, 17, 22):
            assert torch.allclose(plain.causal_attention(q[first:], k, v, window, first=first), whole[first:], atol=1e-13)


def test_a_one_token_sequence_written_out_with_library_routines(tmp_path):
    """With one token there is one key: softmax gives weight 1, position 0 rotates
    nothing, and attention returns the value projection (bias included) of the
    token itself, each key/value head repeated for its group of query heads.  The
    whole model is then a few library calls (shrike/models/qwen.py:111-125, 131-136,
    147-150, 190-192), written here without any function of the plain implementation:
    a missing value bias, a bias on the output projection, a norm after instead of
    before a part, or a residual taken from the normed input would all differ."""
    for name in ("A", "B", "C"):
        m = plain.PlainModel(make_model_dir(name, tmp_path, mode="unit"))
        cfg, w = m.cfg, m.weights
        tok = 17
        x = w["model.embed_tokens.weight"][tok].double()
        group = cfg.num_heads // cfg.num_kv_heads
        for i in range(cfg.num_layers):
            pre = f"model.layers.{i}."
            h = F.rms_norm(x, x.shape, w[pre + "input_layernorm.weight"].double(), cfg.rms_norm_eps)
            v = F.linear(h, w[pre + "self_attn.v_proj.weight"].double(), w[pre + "self_attn.v_proj.bias"].double())
            attn = v.view(cfg.num_kv_heads, 1, cfg.head_dim).expand(-1, group, -1).reshape(-1)
            x = x + F.linear(attn, w[pre + "self_attn.o_proj.weight"].double())
            h = F.rms_norm(x, x.shape, w[pre + "post_attention_layernorm.weight"].double(), cfg.rms_norm_eps)
            act = F.silu(F.linear(h, w[pre + "mlp.gate_proj.weight"].double())) * F.linear(
                h, w[pre + "mlp.up_proj.weight"].double())
            x = x + F.linear(act, w[pre + "mlp.down_proj.weight"].double())
        x = F.rms_norm(x, x.shape, w["model.norm.weight"].double(), cfg.rms_norm_eps)
        out = w.get("lm_head.weight", w["model.embed_tokens.weight"]).double()
        want = F.linear(x, out)
        got = m.logits([tok])[0].double()
        assert torch.allclose(got, want, rtol=1e-9, atol=1e-9), name
        assert not any(k.endswith(("o_proj.bias", "gate_proj.bias", "up_proj.bias", "down_proj.bias")) for k in w)
