"""Each part alone against the plain functions, a layer schedule that runs a
block twice and lets a layer read another layer's cache, and a toy mixer with
state of its own that is registered, built and stepped from here without any
change to the framework's files."""

from dataclasses import dataclass, replace
from typing import ClassVar

import pytest
import torch

from .plain import model as plain

pytestmark = pytest.mark.gpu


def make_runner(spec, tensors_cpu, dtype=torch.float32, page_size=8, num_pages=32):
    from shrike_amd.cache import CacheManager
    from shrike_amd.engine.runner import ModelRunner
    from shrike_amd.engine.runtime import Runtime
    from shrike_amd.models import DecoderModel

    rt = Runtime("cuda:0", dtype)
    model = DecoderModel(spec)
    held = {}
    for p in model.params():
        if p.name in tensors_cpu:
            held[p.name] = tensors_cpu[p.name].to("cuda", torch.float32 if p.keep_float32 else dtype)
    model.load(held, rt)
    cache = CacheManager(model.cache_specs(), page_size, num_pages, max_slots=8, enable_prefix_caching=False)
    cache.allocate(rt.dtype, rt.device)
    return ModelRunner(model, cache, rt), model, cache


def small_spec(**changes):
    from shrike_amd.config import AttentionSpec, BlockSpec, ModelSpec, RMSNormSpec, RotarySpec, SwiGLUSpec

    norm = RMSNormSpec(eps=1e-5)
    mixer = AttentionSpec(num_heads=4, num_kv_heads=2, head_dim=16, qkv_bias=True, out_bias=False,
                          scale=16**-0.5, position=RotarySpec(theta=1e4, rotary_dim=16))
    blocks = tuple(
        BlockSpec(name=f"model.layers.{i}", mixer=mixer, ffn=SwiGLUSpec(intermediate_size=88),
                  mixer_norm=norm, ffn_norm=norm) for i in range(2)
    )
    spec = ModelSpec(architecture="toy", hidden_size=48, vocab_size=97, blocks=blocks, final_norm=norm,
                     tie_word_embeddings=False)
    return replace(spec, **changes)


def cpu_weights(spec, seed=0):
    from shrike_amd.models import DecoderModel
    from shrike_amd.weights import random_tensors

    return random_tensors(DecoderModel(spec).params(), seed, torch.float32, "cpu", mode="unit")


def step_whole(runner, cache, ids, cuts=None):
    from shrike_amd.engine.runner import StepEntry

    seq = cache.new_sequence()
    rows, p = [], 0
    for n in cuts or [len(ids)]:
        cache.append(seq, p, n)
        rows.append(runner.step([StepEntry(seq, ids[p : p + n], p, list(range(n)))]).cpu().clone())
        p += n
    cache.free(seq)
    return torch.cat(rows).double()


# ------------------------------------------------------------ parts on their own


def part_context(n_tokens, dtype=torch.float32):
    """A step context for parts that only need buffers."""
    from shrike_amd.engine.context import StepContext, Workspace

    dev = torch.device("cuda:0")
    z = torch.zeros(1, dtype=torch.int32, device=dev)
    return StepContext(dtype=dtype, device=dev, workspace=Workspace(dev), num_tokens=n_tokens, num_seqs=1,
                       num_decode=0, token_ids=z, positions=z, token_seq=z, cu_q=z, ctx_lens=z,
                       state_slots=z, fresh=z, out_rows=z, block_tables=[])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_part(dtype):
    from shrike_amd.config import RMSNormSpec
    from shrike_amd.engine.runtime import Runtime
    from shrike_amd.parts import HiddenState, build_part

    torch.manual_seed(0)
    part = build_part("norm", RMSNormSpec(eps=2e-4), 200, "n")
    assert [(p.name, p.shape, p.keep_float32) for p in part.params()] == [("n.weight", (200,), True)]
    w = 1 + 0.1 * torch.randn(200)
    part.load({"n.weight": w.cuda()}, Runtime("cuda:0", dtype))
    resid, pending = torch.randn(6, 200), torch.randn(6, 200)
    hidden = HiddenState(resid.cuda(), pending.cuda().to(dtype))
    out = part.forward(part_context(6, dtype), hidden)
    total = resid.double() + pending.to(dtype).double()
    assert hidden.pending is None and torch.allclose(hidden.resid.cpu().double(), total, atol=1e-6)
    want = plain.rms_norm(total, w.double(), 2e-4)
    assert (out.cpu().double() - want).abs().max() <= (1e-5 if dtype == torch.float32 else 1.5e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_feed_forward_part(dtype):
    from shrike_amd.config import SwiGLUSpec
    from shrike_amd.engine.runtime import Runtime
    from shrike_amd.parts import build_part

    torch.manual_seed(1)
    part = build_part("ffn", SwiGLUSpec(intermediate_size=100), 72, "mlp")
    assert [p.shape for p in part.params()] == [(100, 72), (100, 72), (72, 100)]
    w = {p.name: (torch.randn(p.shape) / p.shape[1] ** 0.5).to(dtype) for p in part.params()}
    part.load({k: v.cuda() for k, v in w.items()}, Runtime("cuda:0", dtype))
    x = torch.randn(5, 72).to(dtype)
    out = part.forward(part_context(5, dtype), x.cuda())
    want = plain.swiglu(x.double(), w["mlp.gate_proj.weight"].double(), w["mlp.up_proj.weight"].double(),
                        w["mlp.down_proj.weight"].double())
    assert (out.cpu().double() - want).abs().max() <= (1e-5 if dtype == torch.float32 else 1.5e-2) * want.abs().max()


def test_position_part_gives_the_reference_frequencies():
    from shrike_amd.config import RotarySpec
    from shrike_amd.engine.runtime import Runtime
    from shrike_amd.parts import build_part

    part = build_part("position", RotarySpec(theta=1e6, rotary_dim=32), 64, "rope")
    part.load({}, Runtime("cuda:0", torch.float32))
    inv_freq, rot_dim = part.rotary_table()
    want = 1.0 / (1e6 ** (torch.arange(0, 32, 2).float() / 32))
    assert rot_dim == 32 and torch.equal(inv_freq.cpu(), want)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_part_and_block(dtype):
    """One block alone: the mixer's declared tensors, its cache need, and its
    output against the plain attention block and decoder layer."""
    spec = small_spec()
    spec = replace(spec, blocks=spec.blocks[:1], schedule=())
    w = cpu_weights(spec, seed=3)
    if dtype == torch.bfloat16:
        w = {k: v.to(dtype).float() for k, v in w.items()}
    runner, model, cache = make_runner(spec, w, dtype)
    mixer = model.blocks[0].mixer
    names = sorted(p.name.split("self_attn.")[1] for p in mixer.params())
    assert names == ["k_proj.bias", "k_proj.weight", "o_proj.weight", "q_proj.bias", "q_proj.weight",
                     "v_proj.bias", "v_proj.weight"]
    from shrike_amd.parts import kv_cache_spec

    assert mixer.cache_spec() == kv_cache_spec(2, 16, None)
    ids = torch.randint(0, 97, (21,), generator=torch.Generator().manual_seed(1)).tolist()
    got = step_whole(runner, cache, ids, cuts=[9, 1, 11])
    cfg = plain.PlainConfig(48, 88, 1, 4, 2, 16, 97, 1e-5, 1e4, False)
    want = plain.forward(cfg, {k: v.double() for k, v in w.items()}, ids)
    assert plain.rel_err(got, want) <= (1e-5 if dtype == torch.float32 else 1.5e-2)


# ------------------------------------------------------------- the order is data


def plain_scheduled(spec, w, ids, order, cache_of):
    """The plain model with the layers run in `order`; cache_of[i] = j makes run i
    attend over the keys and values that run j computed."""
    cfg = plain.PlainConfig(48, 88, 2, 4, 2, 16, 97, 1e-5, 1e4, False)
    w = {k: v.double() for k, v in w.items()}
    n = len(ids)
    cos, sin = plain.rope_tables(torch.arange(n), 16, 1e4)
    x = w["model.embed_tokens.weight"][torch.tensor(ids)]
    kv = {}
    for run, layer in enumerate(order):
        p = f"model.layers.{layer}"
        h = plain.rms_norm(x, w[f"{p}.input_layernorm.weight"], 1e-5)
        a = f"{p}.self_attn"
        q = plain.apply_rope(plain.linear(h, w[f"{a}.q_proj.weight"], w[f"{a}.q_proj.bias"]).view(n, 4, 16), cos, sin)
        if cache_of[run] is None:
            k = plain.apply_rope(plain.linear(h, w[f"{a}.k_proj.weight"], w[f"{a}.k_proj.bias"]).view(n, 2, 16), cos, sin)
            v = plain.linear(h, w[f"{a}.v_proj.weight"], w[f"{a}.v_proj.bias"]).view(n, 2, 16)
            kv[run] = (k, v)
        else:
            k, v = kv[cache_of[run]]
        o = plain.causal_attention(q, k, v)
        x = x + plain.linear(o.reshape(n, -1), w[f"{a}.o_proj.weight"])
        h = plain.rms_norm(x, w[f"{p}.post_attention_layernorm.weight"], 1e-5)
        x = x + plain.swiglu(h, w[f"{p}.mlp.gate_proj.weight"], w[f"{p}.mlp.up_proj.weight"], w[f"{p}.mlp.down_proj.weight"])
    x = plain.rms_norm(x, w["model.norm.weight"], 1e-5)
    return plain.linear(x, w["lm_head.weight"])


def test_schedule_may_name_a_layer_twice_and_share_a_cache():
    from shrike_amd.config import ScheduleEntry

    schedule = (ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0), ScheduleEntry(1, cache_of=1))
    spec = small_spec(schedule=schedule)
    w = cpu_weights(spec, seed=4)
    runner, model, cache = make_runner(spec, w)
    assert [c is not None for c in model.cache_specs()] == [True, True, True, False]
    assert len(cache.groups) == 1 and cache.groups[0].layers == [0, 1, 2]
    ids = torch.randint(0, 97, (30,), generator=torch.Generator().manual_seed(2)).tolist()
    want = plain_scheduled(spec, w, ids, [0, 1, 0, 1], [None, None, None, 1])
    for cuts in (None, [13, 1, 1, 15], [2] * 15):
        assert plain.rel_err(step_whole(runner, cache, ids, cuts), want) <= 1e-5


# --------------------------------------------------------- a toy mixer with state


@dataclass(frozen=True)
class DecaySpec:
    """y_t = s_t,  s_t = decay * s_{t-1} + W x_t  per sequence."""

    kind: ClassVar[str] = "toy_decay"
    decay: float


def define_toy_mixer():
    from shrike_amd.parts import Mixer, ParamSpec, StateSpec, register_mixer

    class DecayMixer(Mixer):
        def params(self):
            return [ParamSpec(f"{self.name}.in_proj.weight", (self.width, self.width))]

        def cache_spec(self):
            return StateSpec((self.width,), "float32")

        def load(self, tensors, runtime):
            self.w = tensors[f"{self.name}.in_proj.weight"].float()

        def forward(self, ctx, x, cache):
            u = x.float() @ self.w.t()
            out = torch.empty_like(u)
            slots = ctx.state_slots.tolist()
            start = 0
            for s, n in enumerate(ctx.q_lens):
                state = cache.state[slots[s]]
                for t in range(start, start + n):
                    state = self.spec.decay * state + u[t]
                    out[t] = state
                cache.state[slots[s]] = state
                start += n
            return out.to(x.dtype)

    register_mixer("toy_decay", DecayMixer)


def test_toy_mixer_with_state_is_registered_built_and_stepped():
    from shrike_amd.engine.runner import StepEntry
    from shrike_amd.parts import StateSpec

    define_toy_mixer()
    base = small_spec()
    toy_block = replace(base.blocks[1], mixer=DecaySpec(decay=0.8), mixer_name="decay")
    spec = replace(base, blocks=(base.blocks[0], toy_block))
    w = cpu_weights(spec, seed=5)
    assert "model.layers.1.decay.in_proj.weight" in w and "model.layers.1.self_attn.q_proj.weight" not in w
    runner, model, cache = make_runner(spec, w)
    assert model.cache_specs()[1] == StateSpec((48,), "float32")
    assert len(cache.state_groups) == 1 and cache.state_groups[0].tensor.shape == (1, 8, 48)
    assert cache.enable_prefix_caching is False

    def want_for(ids):
        cfg = plain.PlainConfig(48, 88, 2, 4, 2, 16, 97, 1e-5, 1e4, False)
        wd = {k: v.double() for k, v in w.items()}
        n = len(ids)
        cos, sin = plain.rope_tables(torch.arange(n), 16, 1e4)
        x = plain.decoder_layer(cfg, wd, 0, wd["model.embed_tokens.weight"][torch.tensor(ids)], cos, sin)
        p = "model.layers.1"
        u = plain.rms_norm(x, wd[f"{p}.input_layernorm.weight"], 1e-5) @ wd[f"{p}.decay.in_proj.weight"].t()
        state, ys = torch.zeros(48, dtype=torch.float64), []
        for t in range(n):
            state = 0.8 * state + u[t]
            ys.append(state)
        x = x + torch.stack(ys)
        h = plain.rms_norm(x, wd[f"{p}.post_attention_layernorm.weight"], 1e-5)
        x = x + plain.swiglu(h, wd[f"{p}.mlp.gate_proj.weight"], wd[f"{p}.mlp.up_proj.weight"], wd[f"{p}.mlp.down_proj.weight"])
        return plain.linear(plain.rms_norm(x, wd["model.norm.weight"], 1e-5), wd["lm_head.weight"])

    g = torch.Generator().manual_seed(3)
    a = torch.randint(0, 97, (19,), generator=g).tolist()
    b = torch.randint(0, 97, (11,), generator=g).tolist()
    assert plain.rel_err(step_whole(runner, cache, a), want_for(a)) <= 1e-5
    assert plain.rel_err(step_whole(runner, cache, a, [4, 1, 1, 13]), want_for(a)) <= 1e-5
    # two requests side by side, each with its own state slot; the slot of a
    # finished request is handed out again and starts from zero
    sa, sb = cache.new_sequence(), cache.new_sequence()
    cache.append(sa, 0, 19)
    cache.append(sb, 0, 11)
    first = runner.step([StepEntry(sa, a[:7], 0, [6]), StepEntry(sb, b[:1], 0, [0])]).cpu().clone()
    second = runner.step([StepEntry(sb, b[1:], 1, [9]), StepEntry(sa, a[7:], 7, [11])]).cpu().clone()
    wa, wb = want_for(a), want_for(b)
    got = torch.stack([first[0], first[1], second[0], second[1]]).double()
    want = torch.stack([wa[6], wb[0], wb[10], wa[18]])
    assert plain.rel_err(got, want) <= 1e-5
    cache.free(sa)
    cache.free(sb)
    assert plain.rel_err(step_whole(runner, cache, b), wb) <= 1e-5


# ------------------------------------- a toy feed-forward that routes its tokens


@dataclass(frozen=True)
class Top1Spec:
    """y = p_e(x) * W2_e relu(W1_e x), e the expert with the largest router logit,
    p the softmax of the router logits."""

    kind: ClassVar[str] = "toy_top1"
    experts: int
    inner: int


def define_toy_routed_ffn():
    from shrike_amd.parts import FeedForward, ParamSpec, register_ffn

    class Top1Experts(FeedForward):
        graph_safe = False  # the rows of an expert are gathered on the host's say-so

        def params(self):
            e, i, w = self.spec.experts, self.spec.inner, self.width
            out = [ParamSpec(f"{self.name}.router.weight", (e, w), keep_float32=True)]
            for x in range(e):
                out += [ParamSpec(f"{self.name}.experts.{x}.w1.weight", (i, w)),
                        ParamSpec(f"{self.name}.experts.{x}.w2.weight", (w, i))]
            return out

        def load(self, tensors, runtime):
            self.router = tensors[f"{self.name}.router.weight"].float()
            self.w1 = torch.stack([tensors[f"{self.name}.experts.{x}.w1.weight"] for x in range(self.spec.experts)]).float()
            self.w2 = torch.stack([tensors[f"{self.name}.experts.{x}.w2.weight"] for x in range(self.spec.experts)]).float()

        def forward(self, ctx, x):
            xf = x.float()
            probs = torch.softmax(xf @ self.router.t(), dim=-1)  # router logits in float32
            weight, expert = probs.max(dim=-1)
            out = torch.zeros_like(xf)
            for e in range(self.spec.experts):
                rows = (expert == e).nonzero().flatten()
                if rows.numel():
                    h = torch.relu(xf[rows] @ self.w1[e].t())
                    out[rows] = (h @ self.w2[e].t()) * weight[rows, None]
            return out.to(x.dtype)

    register_ffn("toy_top1", Top1Experts)


def test_toy_routed_feed_forward_in_one_layer_of_two():
    """One layer keeps the dense feed-forward, the other routes each token to one of
    three experts: layers of one model choose their parts independently."""
    define_toy_routed_ffn()
    base = small_spec()
    routed = replace(base.blocks[0], ffn=Top1Spec(experts=3, inner=40), ffn_name="moe")
    spec = replace(base, blocks=(routed, base.blocks[1]))
    w = cpu_weights(spec, seed=6)
    assert "model.layers.0.moe.experts.2.w2.weight" in w and "model.layers.0.mlp.gate_proj.weight" not in w
    runner, model, cache = make_runner(spec, w)

    def want_for(ids):
        cfg = plain.PlainConfig(48, 88, 2, 4, 2, 16, 97, 1e-5, 1e4, False)
        wd = {k: v.double() for k, v in w.items()}
        n = len(ids)
        cos, sin = plain.rope_tables(torch.arange(n), 16, 1e4)
        x = wd["model.embed_tokens.weight"][torch.tensor(ids)]
        p = "model.layers.0"
        x = x + plain.attention_block(cfg, wd, f"{p}.self_attn", plain.rms_norm(x, wd[f"{p}.input_layernorm.weight"], 1e-5), cos, sin, None)
        h = plain.rms_norm(x, wd[f"{p}.post_attention_layernorm.weight"], 1e-5)
        probs = torch.softmax(h @ wd[f"{p}.moe.router.weight"].t(), dim=-1)
        ys = []
        for t in range(n):
            e = int(probs[t].argmax())
            inner = torch.relu(wd[f"{p}.moe.experts.{e}.w1.weight"] @ h[t])
            ys.append(probs[t, e] * (wd[f"{p}.moe.experts.{e}.w2.weight"] @ inner))
        x = x + torch.stack(ys)
        x = plain.decoder_layer(cfg, wd, 1, x, cos, sin)
        return plain.linear(plain.rms_norm(x, wd["model.norm.weight"], 1e-5), wd["lm_head.weight"])

    ids = torch.randint(0, 97, (23,), generator=torch.Generator().manual_seed(8)).tolist()
    want = want_for(ids)
    assert plain.rel_err(step_whole(runner, cache, ids), want) <= 1e-5
    assert plain.rel_err(step_whole(runner, cache, ids, [5, 1, 1, 2, 14]), want) <= 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gated_feed_forward_with_a_gelu_gate_in_one_layer_of_two(dtype):
    """The gate's activation is a field of the feed-forward's spec: one layer keeps
    SiLU, the other takes GELU in its tanh form, with nothing but the spec changed."""
    from shrike_amd.config import SwiGLUSpec

    base = small_spec()
    gelu = replace(base.blocks[1], ffn=SwiGLUSpec(intermediate_size=88, activation="gelu_tanh"))
    spec = replace(base, blocks=(base.blocks[0], gelu))
    w = cpu_weights(spec, seed=11)
    if dtype == torch.bfloat16:
        w = {k: v.to(dtype).float() for k, v in w.items()}  # the values the engine holds
    runner, model, cache = make_runner(spec, w, dtype=dtype)
    cfg = plain.PlainConfig(48, 88, 2, 4, 2, 16, 97, 1e-5, 1e4, False)
    wd = {k: v.double() for k, v in w.items()}
    ids = torch.randint(0, 97, (27,), generator=torch.Generator().manual_seed(12)).tolist()
    n = len(ids)
    cos, sin = plain.rope_tables(torch.arange(n), 16, 1e4)
    x = plain.decoder_layer(cfg, wd, 0, wd["model.embed_tokens.weight"][torch.tensor(ids)], cos, sin)
    p = "model.layers.1"
    x = x + plain.attention_block(cfg, wd, f"{p}.self_attn", plain.rms_norm(x, wd[f"{p}.input_layernorm.weight"], 1e-5),
                                  cos, sin, None)
    h = plain.rms_norm(x, wd[f"{p}.post_attention_layernorm.weight"], 1e-5)
    gate = torch.nn.functional.gelu(h @ wd[f"{p}.mlp.gate_proj.weight"].t(), approximate="tanh")
    x = x + (gate * (h @ wd[f"{p}.mlp.up_proj.weight"].t())) @ wd[f"{p}.mlp.down_proj.weight"].t()
    want = plain.linear(plain.rms_norm(x, wd["model.norm.weight"], 1e-5), wd["lm_head.weight"])
    tol = 1e-5 if dtype == torch.float32 else 1.5e-2
    assert plain.rel_err(step_whole(runner, cache, ids), want) <= tol
    assert plain.rel_err(step_whole(runner, cache, ids, [20, 1, 1, 5]), want) <= tol
    # and it is not the same function: the SiLU model gives other logits
    silu_runner, _, silu_cache = make_runner(base, w, dtype=dtype)
    assert plain.rel_err(step_whole(silu_runner, silu_cache, ids), want) > 3e-2


# --------------------------------------------------- another position encoding


@dataclass(frozen=True)
class PairRotarySpec:
    """Rotation of neighbouring pairs (2i, 2i + 1) by the angle pos * theta^(-2i/d)."""

    kind: ClassVar[str] = "toy_pair_rotary"
    theta: float


def define_toy_position():
    from shrike_amd.parts import PositionEncoding, register_position

    class PairRotary(PositionEncoding):
        def load(self, tensors, runtime):
            self.device = runtime.device

        def apply(self, ctx, qkv, heads, kv_heads, head_dim):
            n = qkv.shape[0]
            inv = 1.0 / (self.spec.theta ** (torch.arange(0, head_dim, 2, device=self.device).float() / head_dim))
            angle = ctx.positions[:n].float()[:, None] * inv[None, :]
            cos, sin = angle.cos()[:, None, :], angle.sin()[:, None, :]
            qk = qkv[:, : (heads + kv_heads) * head_dim].view(n, heads + kv_heads, head_dim // 2, 2).float()
            a, b = qk[..., 0], qk[..., 1]
            rotated = torch.stack([a * cos - b * sin, b * cos + a * sin], dim=-1)
            qkv[:, : (heads + kv_heads) * head_dim] = rotated.view(n, -1).to(qkv.dtype)

    register_position("toy_pair_rotary", PairRotary)


def test_toy_position_encoding_through_the_unfused_path():
    """A position encoding without a fused kernel encodes q and k in place before
    the keys go into the cache; decoding one by one gives what the whole prompt gives."""
    define_toy_position()
    base = small_spec()
    blocks = tuple(replace(b, mixer=replace(b.mixer, position=PairRotarySpec(theta=500.0))) for b in base.blocks)
    spec = replace(base, blocks=blocks)
    w = cpu_weights(spec, seed=7)
    runner, model, cache = make_runner(spec, w)

    def pair_rope(x, positions):
        d = x.shape[-1]
        inv = 1.0 / (500.0 ** (torch.arange(0, d, 2).double() / d))
        ang = positions.double()[:, None] * inv[None, :]
        cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
        a, b = x[..., 0::2], x[..., 1::2]
        return torch.stack([a * cos - b * sin, b * cos + a * sin], dim=-1).flatten(-2)

    def want_for(ids):
        wd = {k: v.double() for k, v in w.items()}
        n = len(ids)
        pos = torch.arange(n)
        x = wd["model.embed_tokens.weight"][torch.tensor(ids)]
        for i in range(2):
            p = f"model.layers.{i}"
            h = plain.rms_norm(x, wd[f"{p}.input_layernorm.weight"], 1e-5)
            q = plain.linear(h, wd[f"{p}.self_attn.q_proj.weight"], wd[f"{p}.self_attn.q_proj.bias"]).view(n, 4, 16)
            k = plain.linear(h, wd[f"{p}.self_attn.k_proj.weight"], wd[f"{p}.self_attn.k_proj.bias"]).view(n, 2, 16)
            v = plain.linear(h, wd[f"{p}.self_attn.v_proj.weight"], wd[f"{p}.self_attn.v_proj.bias"]).view(n, 2, 16)
            att = plain.causal_attention(pair_rope(q, pos), pair_rope(k, pos), v)
            x = x + plain.linear(att.reshape(n, -1), wd[f"{p}.self_attn.o_proj.weight"])
            h = plain.rms_norm(x, wd[f"{p}.post_attention_layernorm.weight"], 1e-5)
            x = x + plain.swiglu(h, wd[f"{p}.mlp.gate_proj.weight"], wd[f"{p}.mlp.up_proj.weight"], wd[f"{p}.mlp.down_proj.weight"])
        return plain.linear(plain.rms_norm(x, wd["model.norm.weight"], 1e-5), wd["lm_head.weight"])

    ids = torch.randint(0, 97, (21,), generator=torch.Generator().manual_seed(9)).tolist()
    want = want_for(ids)
    assert plain.rel_err(step_whole(runner, cache, ids), want) <= 1e-5
    assert plain.rel_err(step_whole(runner, cache, ids, [9] + [1] * 12), want) <= 1e-5


# ---------------------- a toy state mixer that HIP graphs may record, with a prepare()


@dataclass(frozen=True)
class DeviceDecaySpec:
    """The decay mixer again (s_t = decay * s_{t-1} + W x_t), computed on the device
    from the step's own index arrays, so that decode steps replay from a graph."""

    kind: ClassVar[str] = "toy_decay_device"
    decay: float


def define_graph_safe_state_mixer():
    import numpy as np

    from shrike_amd.parts import Mixer, ParamSpec, StateSpec, register_mixer

    class DeviceDecayMixer(Mixer):
        state_graph_safe = True  # the state is reached through ctx.state_slots on the device

        def params(self):
            return [ParamSpec(f"{self.name}.in_proj.weight", (self.width, self.width))]

        def cache_spec(self):
            return StateSpec((self.width,), "float32")

        def load(self, tensors, runtime):
            self.w = tensors[f"{self.name}.in_proj.weight"].float()

        def prepare(self, shape):
            """What forward needs beyond the step's common arrays: each token's
            offset within its portion, and the last row of each sequence."""
            if "decay_offset" in shape.extras:
                return  # another layer of this kind has added them
            first = np.cumsum(shape.q_lens) - shape.q_lens
            shape.add("decay_offset", np.arange(shape.num_tokens) - np.repeat(first, shape.q_lens))
            shape.add("decay_last_row", first + shape.q_lens - 1)
            shape.notes["decay_prepared"] = shape.notes.get("decay_prepared", 0) + 1

        def forward(self, ctx, x, cache):
            u = x.float() @ self.w.t()  # [N, width]
            n = u.shape[0]
            seq, off = ctx.token_seq[:n].long(), ctx.extras["decay_offset"][:n].long()
            slots = ctx.state_slots.long()
            state = cache.state_padded  # padding rows of a graph batch use the spare slot
            before = state[slots]  # [S, width], zero for a fresh slot
            rows = torch.arange(n, device=u.device)
            # y_t = sum_{j <= t, same sequence} decay^(t-j) u_j + decay^(offset+1) s_before
            same = (seq[:, None] == seq[None, :]) & (rows[None, :] <= rows[:, None])
            power = (rows[:, None] - rows[None, :]).clamp_min(0).float()
            mix = torch.where(same, self.spec.decay ** power, torch.zeros_like(power))
            y = mix @ u + (self.spec.decay ** (off.float() + 1))[:, None] * before[seq]
            state.index_copy_(0, slots, y[ctx.extras["decay_last_row"].long()])
            return y.to(x.dtype)

    register_mixer("toy_decay_device", DeviceDecayMixer)


def test_toy_state_mixer_with_prepare_is_replayed_from_graphs():
    """A mixer with state of its own declares itself safe for graphs and adds its
    own index arrays in prepare(): decode steps are captured and replayed, two
    requests keep apart, and everything matches the recurrence computed plainly."""
    from shrike_amd.engine.runner import StepEntry

    define_graph_safe_state_mixer()
    base = small_spec()
    toy_block = replace(base.blocks[1], mixer=DeviceDecaySpec(decay=0.7), mixer_name="decay")
    spec = replace(base, blocks=(base.blocks[0], toy_block))
    w = cpu_weights(spec, seed=12)
    runner, model, cache = make_runner(spec, w)
    assert runner.use_graphs and model.graph_safe()

    def want_for(ids):
        cfg = plain.PlainConfig(48, 88, 2, 4, 2, 16, 97, 1e-5, 1e4, False)
        wd = {k: v.double() for k, v in w.items()}
        n = len(ids)
        cos, sin = plain.rope_tables(torch.arange(n), 16, 1e4)
        x = plain.decoder_layer(cfg, wd, 0, wd["model.embed_tokens.weight"][torch.tensor(ids)], cos, sin)
        p = "model.layers.1"
        u = plain.rms_norm(x, wd[f"{p}.input_layernorm.weight"], 1e-5) @ wd[f"{p}.decay.in_proj.weight"].t()
        state, ys = torch.zeros(48, dtype=torch.float64), []
        for t in range(n):
            state = 0.7 * state + u[t]
            ys.append(state)
        x = x + torch.stack(ys)
        h = plain.rms_norm(x, wd[f"{p}.post_attention_layernorm.weight"], 1e-5)
        x = x + plain.swiglu(h, wd[f"{p}.mlp.gate_proj.weight"], wd[f"{p}.mlp.up_proj.weight"], wd[f"{p}.mlp.down_proj.weight"])
        return plain.linear(plain.rms_norm(x, wd["model.norm.weight"], 1e-5), wd["lm_head.weight"])

    g = torch.Generator().manual_seed(13)
    a = torch.randint(0, 97, (40,), generator=g).tolist()
    b = torch.randint(0, 97, (33,), generator=g).tolist()
    wa, wb = want_for(a), want_for(b)
    assert plain.rel_err(step_whole(runner, cache, a, [7, 2, 5] + [1] * 26), wa) <= 1e-5
    replays = runner.graph_replays
    assert replays == 26
    # three requests decode side by side from one graph of four rows, each from its
    # own slot; the fourth row is padding and writes to the spare slot only
    sa, sb, sc = cache.new_sequence(), cache.new_sequence(), cache.new_sequence()
    cache.append(sa, 0, 40)
    cache.append(sb, 0, 33)
    cache.append(sc, 0, 33)
    runner.step([StepEntry(sa, a[:12], 0, []), StepEntry(sb, b[:5], 0, []), StepEntry(sc, b[:2], 0, [])])
    for k in range(28):
        out = runner.step([StepEntry(sa, [a[12 + k]], 12 + k, [0]), StepEntry(sb, [b[5 + k]], 5 + k, [0]),
                           StepEntry(sc, [b[2 + k]], 2 + k, [0])]).cpu().double()
        assert plain.rel_err(out, torch.stack([wa[12 + k], wb[5 + k], wb[2 + k]])) <= 1e-5
    assert runner.graph_replays == replays + 28
    for s in (sa, sb, sc):
        cache.free(s)


# ------------------------------------ a toy embedding and a toy head as parts of a model


@dataclass(frozen=True)
class ScaledEmbeddingSpec:
    """x = multiplier * table[token] + position_table[position]."""

    kind: ClassVar[str] = "toy_scaled_embedding"
    vocab_size: int
    multiplier: float
    max_positions: int


@dataclass(frozen=True)
class CappedHeadSpec:
    """logits = cap * tanh((x @ W.T) / cap)."""

    kind: ClassVar[str] = "toy_capped_head"
    vocab_size: int
    cap: float


def define_toy_embedding_and_head():
    from shrike_amd.parts import Embedding, Head, ParamSpec, register_embedding, register_head

    class ScaledEmbedding(Embedding):
        def params(self):
            return [ParamSpec(f"{self.name}.weight", (self.spec.vocab_size, self.width), init="embedding"),
                    ParamSpec(f"{self.name}.positions", (self.spec.max_positions, self.width), init="embedding")]

        def load(self, tensors, runtime):
            self.table, self.positions = tensors[f"{self.name}.weight"], tensors[f"{self.name}.positions"]

        def forward(self, ctx):
            n = ctx.num_tokens
            rows = self.table[ctx.token_ids[:n].long()].float() * self.spec.multiplier
            return (rows + self.positions[ctx.positions[:n].long()].float()).contiguous()

    class CappedHead(Head):
        def tie(self, embedding):
            self.tied_to = embedding

        def params(self):
            return [ParamSpec(f"{self.name}.weight", (self.spec.vocab_size, self.width), optional=True)]

        def load(self, tensors, runtime):
            w = tensors.get(f"{self.name}.weight")
            self.w = (self.tied_to.table if w is None else w).float()

        def forward(self, ctx, x):
            return self.spec.cap * torch.tanh((x.float() @ self.w.t()) / self.spec.cap)

    register_embedding("toy_scaled_embedding", ScaledEmbedding)
    register_head("toy_capped_head", CappedHead)


def test_toy_embedding_and_head_are_parts_like_the_others():
    """An embedding with a multiplier and a learned position table, and a head that
    caps its logits and shares the embedding's table: both come from the spec."""
    define_toy_embedding_and_head()
    base = small_spec()
    spec = replace(base, embedding=ScaledEmbeddingSpec(97, 3.0, 64), head=CappedHeadSpec(97, 5.0),
                   tie_word_embeddings=True)
    w = cpu_weights(spec, seed=14)
    assert "model.embed_tokens.positions" in w and "lm_head.weight" not in w
    runner, model, cache = make_runner(spec, w)

    def want_for(ids):
        cfg = plain.PlainConfig(48, 88, 2, 4, 2, 16, 97, 1e-5, 1e4, True)
        wd = {k: v.double() for k, v in w.items()}
        n = len(ids)
        cos, sin = plain.rope_tables(torch.arange(n), 16, 1e4)
        x = 3.0 * wd["model.embed_tokens.weight"][torch.tensor(ids)] + wd["model.embed_tokens.positions"][:n]
        for i in range(2):
            x = plain.decoder_layer(cfg, wd, i, x, cos, sin)
        x = plain.rms_norm(x, wd["model.norm.weight"], 1e-5)
        return 5.0 * torch.tanh(plain.linear(x, wd["model.embed_tokens.weight"]) / 5.0)

    ids = torch.randint(0, 97, (29,), generator=torch.Generator().manual_seed(15)).tolist()
    want = want_for(ids)
    assert plain.rel_err(step_whole(runner, cache, ids), want) <= 1e-5
    assert plain.rel_err(step_whole(runner, cache, ids, [6, 1, 1, 2, 19]), want) <= 1e-5


# ------------------- a toy paged mixer whose cache is one latent vector per token


@dataclass(frozen=True)
class LatentSpec:
    """Attention over one shared latent per token: c_t = W_c x_t is all that is
    cached; y_t = W_o sum_j softmax_j(q_t . c_j / sqrt(r)) c_j over the tokens j
    up to t (the last `window` of them), q_t = W_q x_t."""

    kind: ClassVar[str] = "toy_latent"
    latent: int
    window: int | None = None


def define_toy_latent_mixer():
    from shrike_amd.parts import PAGE, Mixer, PagedSpec, PageTensor, ParamSpec, register_mixer

    class LatentMixer(Mixer):
        graph_safe = False  # its forward walks the sequences on the host

        def params(self):
            r, h = self.spec.latent, self.width
            return [ParamSpec(f"{self.name}.q_proj.weight", (r, h)), ParamSpec(f"{self.name}.c_proj.weight", (r, h)),
                    ParamSpec(f"{self.name}.o_proj.weight", (h, r))]

        def cache_spec(self):
            # one tensor per page, in float32 whatever the compute dtype: a layout of its own
            return PagedSpec((PageTensor("latent", (PAGE, self.spec.latent), "float32"),), self.spec.window)

        def load(self, tensors, runtime):
            self.wq, self.wc, self.wo = (tensors[f"{self.name}.{n}_proj.weight"].float() for n in "qco")

        def forward(self, ctx, x, cache):
            pool, ps = cache.pools["latent"], cache.page_size  # [pages + 1, page_size, latent]
            tables = ctx.block_tables[cache.group].long()
            pos, seq = ctx.positions.long(), ctx.token_seq.long()
            q, c = x.float() @ self.wq.t(), x.float() @ self.wc.t()
            if cache.owned:
                pool[tables[seq, pos // ps], pos % ps] = c
            out = torch.empty_like(q)
            start = 0
            for s, (n, length) in enumerate(zip(ctx.q_lens, ctx.ctx_lens_host)):
                first = 0 if self.spec.window is None else max(0, length - n - self.spec.window + 1)
                lo = first // ps  # pages before it may have been given back (table entry -1)
                pages = tables[s, lo : -(-length // ps)]
                keys = pool[pages].reshape(-1, self.spec.latent)[: length - lo * ps]
                j = torch.arange(lo * ps, length, device=x.device)[None, :]
                p = pos[start : start + n, None]
                seen = (j <= p) if self.spec.window is None else (j <= p) & (j > p - self.spec.window)
                scores = (q[start : start + n] @ keys.t()) * self.spec.latent**-0.5
                out[start : start + n] = scores.masked_fill(~seen, float("-inf")).softmax(-1) @ keys
                start += n
            return (out @ self.wo.t()).to(x.dtype)

    register_mixer("toy_latent", LatentMixer)


@pytest.mark.parametrize("window", [None, 11])
def test_toy_paged_mixer_with_one_latent_per_token_keeps_its_own_layout(window):
    """A mixer whose pages hold a single tensor of its own shape and dtype is
    registered, given pages, stepped in several cuttings beside ordinary attention
    layers, and survives the poisoning of every page that no request holds, without
    a change to the cache manager, the step function or the poisoner."""
    from shrike_amd.engine.runner import StepEntry
    from shrike_amd.parts import PAGE, PagedSpec, PageTensor
    from shrike_amd.replay.poison import PagePoisoner

    define_toy_latent_mixer()
    base = small_spec()
    toy_block = replace(base.blocks[1], mixer=LatentSpec(latent=24, window=window), mixer_name="latent")
    spec = replace(base, blocks=(base.blocks[0], toy_block))
    w = cpu_weights(spec, seed=6)
    runner, model, cache = make_runner(spec, w, page_size=4, num_pages=24)
    assert model.cache_specs()[1] == PagedSpec((PageTensor("latent", (PAGE, 24), "float32"),), window)
    assert len(cache.groups) == 2  # attention's keys and values; the toy's latents
    latents = cache.groups[1].tensors
    assert list(latents) == ["latent"] and latents["latent"].shape == (1, 25, 4, 24)
    assert latents["latent"].dtype == torch.float32
    kv_bytes = 2 * 4 * 2 * 16 * 4  # keys and values of a page: 4 tokens, 2 heads of 16, float32
    assert cache.bytes_per_page(4) == kv_bytes + 4 * 24 * 4
    assert runner.use_graphs is False

    def want_for(ids):
        cfg = plain.PlainConfig(48, 88, 2, 4, 2, 16, 97, 1e-5, 1e4, False)
        wd = {k: v.double() for k, v in w.items()}
        n = len(ids)
        cos, sin = plain.rope_tables(torch.arange(n), 16, 1e4)
        x = plain.decoder_layer(cfg, wd, 0, wd["model.embed_tokens.weight"][torch.tensor(ids)], cos, sin)
        p = "model.layers.1"
        h = plain.rms_norm(x, wd[f"{p}.input_layernorm.weight"], 1e-5)
        q, c = h @ wd[f"{p}.latent.q_proj.weight"].t(), h @ wd[f"{p}.latent.c_proj.weight"].t()
        # plain attention with one head whose keys and values are the same vectors
        att = plain.causal_attention(q[:, None], c[:, None], c[:, None], window)
        x = x + att[:, 0] @ wd[f"{p}.latent.o_proj.weight"].t()
        h = plain.rms_norm(x, wd[f"{p}.post_attention_layernorm.weight"], 1e-5)
        x = x + plain.swiglu(h, wd[f"{p}.mlp.gate_proj.weight"], wd[f"{p}.mlp.up_proj.weight"], wd[f"{p}.mlp.down_proj.weight"])
        return plain.linear(plain.rms_norm(x, wd["model.norm.weight"], 1e-5), wd["lm_head.weight"])

    poisoner = PagePoisoner(cache)
    poisoner.poison_everything()
    assert torch.isnan(latents["latent"]).all()
    g = torch.Generator().manual_seed(4)
    a = torch.randint(0, 97, (41,), generator=g).tolist()
    b = torch.randint(0, 97, (23,), generator=g).tolist()
    wa, wb = want_for(a), want_for(b)
    assert plain.rel_err(step_whole(runner, cache, a), wa) <= 1e-5
    poisoner.poison_everything()  # the request is gone: all its pages are poisoned again
    assert plain.rel_err(step_whole(runner, cache, a, [7, 2, 1, 1, 19, 11]), wa) <= 1e-5
    poisoner.poison_everything()
    # two requests side by side, a portion of one beside single tokens of the other; the
    # windowed group gives pages back on the way, and they are poisoned at once
    sa, sb = cache.new_sequence(), cache.new_sequence()
    rows = {}
    pa = pb = 0
    for na, nb in [(9, 1), (1, 1), (20, 2), (1, 13), (10, 6)]:
        entries = []
        for seq, ids, p, n, name in ((sa, a, pa, na, "a"), (sb, b, pb, nb, "b")):
            cache.append(seq, p, n)
            entries.append(StepEntry(seq, ids[p : p + n], p, list(range(n))))
        before = [poisoner.held(sa), poisoner.held(sb)]
        out = runner.step(entries).cpu().double()
        assert torch.isfinite(out).all()
        for i in range(na):
            rows[("a", pa + i)] = out[i]
        for i in range(nb):
            rows[("b", pb + i)] = out[na + i]
        pa, pb = pa + na, pb + nb
        for seq, p, held in ((sa, pa, before[0]), (sb, pb, before[1])):
            cache.trim(seq, p)
            poisoner.poison_released(held, seq)
    assert pa == 41 and pb == 23
    assert plain.rel_err(torch.stack([rows[("a", i)] for i in range(41)]), wa) <= 1e-5
    assert plain.rel_err(torch.stack([rows[("b", i)] for i in range(23)]), wb) <= 1e-5
    if window:
        assert -1 in sa.tables[1] and -1 not in sa.tables[0]  # only the toy's group has a window
    cache.free(sa)
    cache.free(sb)
    cache.check([])
