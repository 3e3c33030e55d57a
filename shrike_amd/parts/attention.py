"""Causal grouped-query attention over the paged key/value cache."""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch

from ..kernels import ops
from .base import PAGE, Mixer, PagedSpec, PageTensor, ParamSpec, build_part, register_mixer

QUERY_TILE = 16  # queries per tile of the MFMA kernels for prompt portions
COMPUTE_UNITS = 256  # of an MI355X; compute_units() asks the device that is there
KEYS_PER_WORKGROUP = 256  # a decode workgroup's four wavefronts want at least this many keys
MAX_KEY_SPLITS = 64
# decode attention fetches keys and values with non-temporal loads from this many bytes
# of them per launch on (counted with the batch and the context rounded up to powers of two)
STREAMING_FROM_BYTES = 96 << 20
_UNITS: int | None = None


def compute_units() -> int:
    """Compute units of the GPU the process runs on (read once; COMPUTE_UNITS where no
    GPU is visible, so that launch plans can be computed and tested without one)."""
    global _UNITS
    if _UNITS is None:
        _UNITS = (torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count
                  if torch.cuda.is_available() else COMPUTE_UNITS)
    return _UNITS


def kv_cache_spec(num_kv_heads: int, head_dim: int, window: int | None = None) -> PagedSpec:
    """The cache of grouped-query attention, laid out for this file's kernels: per
    page and key/value head the keys in slabs of 32 elements, [head_dim / 32,
    page_size, 32] (a wavefront's operand load for the matrix instruction then
    touches whole cache lines: 64 bytes from each of four consecutive keys; one
    slab of head_dim elements where head_dim is no multiple of 32), and the values
    transposed, [head_dim, page_size] (the keys of a page side by side for every
    element, which is the operand layout of V^T)."""
    slab = ops.key_slab(head_dim)
    return PagedSpec(
        tensors=(PageTensor("k", (num_kv_heads, head_dim // slab, PAGE, slab)),
                 PageTensor("v", (num_kv_heads, head_dim, PAGE))),
        window=window,
    )


def _pow2(n: int, floor: int = 1) -> int:
    b = floor
    while b < n:
        b *= 2
    return b


def decode_splits(num_seqs: int, kv_heads: int, max_ctx: int) -> int:
    """Workgroups per (sequence, key/value head) of decode attention: enough to
    put one on every compute unit, each with at least KEYS_PER_WORKGROUP keys
    for its four wavefronts.  Both inputs are rounded up to powers of two first,
    so a step gives the same result whether it runs kernel by kernel or as a
    graph captured for a padded batch."""
    want = -(-compute_units() // (_pow2(num_seqs) * kv_heads))
    most = max(1, _pow2(max_ctx, KEYS_PER_WORKGROUP) // KEYS_PER_WORKGROUP)
    return max(1, min(want, most, MAX_KEY_SPLITS))


def decode_streams(num_seqs: int, kv_heads: int, head_dim: int, max_ctx: int, window: int | None = None) -> bool:
    """Whether a decode launch reads so many keys and values that non-temporal
    loads pay (measured with 4 key/value heads of 128: a tenth faster from 64
    sequences of 2,200 keys or 8 of 16,000, 2 % at 8 of 4,000, 1 to 4 % slower
    below).  The result is the same either way; batch and context are rounded up
    as in decode_splits(), so that a graph's steps all decide alike."""
    keys = _pow2(max_ctx, KEYS_PER_WORKGROUP)
    if window:
        keys = min(keys, window)
    return _pow2(num_seqs) * keys * kv_heads * head_dim * 4 >= STREAMING_FROM_BYTES


@dataclass
class AttentionPlan:
    """How one step's attention is launched for a (heads, kv heads, head size)."""

    mfma: bool = False
    nsplit: int = 1  # key splits of the single-token rows
    streaming: bool = False  # single-token rows: non-temporal loads of keys and values
    kernel: str = ""  # for prompt portions: "shared", "tiles" or "" (none in the step)
    small: bool = False  # "shared" with half as many wavefronts per workgroup
    portion_splits: int = 1  # "shared": workgroups that share an entry's keys
    first_token: int = 0  # index of the step's first prompt token
    count: int = 0  # workgroups ("shared") or tiles ("tiles")
    seq_name: str = ""  # names of the launch lists among the step's extras
    q0_name: str = ""


def portion_runs(q_lens, first_seq: int, run: int):
    """Prompt portions cut into runs of `run` queries: (sequence of each run, its
    first query within the portion)."""
    counts = -(-np.asarray(q_lens, dtype=np.int64) // run)
    seqs = np.repeat(np.arange(first_seq, first_seq + counts.size), counts)
    first = np.zeros(counts.size + 1, dtype=np.int64)
    np.cumsum(counts, out=first[1:])
    q0 = (np.arange(int(counts.sum())) - first[seqs - first_seq]) * run
    return seqs, q0


def portion_splits(workgroups: int, mean_keys: int) -> int:
    """Among how many workgroups each entry of a step's prompt portions shares
    its keys.  A few hundred queries far into a sequence (a long prompt cut by
    the token budget) make few workgroups with thousands of keys each; shared,
    they fill the chip.  Measured at 28 heads over 4, 512 queries (128
    workgroups): at position 1,536 64 us a layer unshared, 47 / 40 / 48 in 2 / 4
    / 8 shares; at 31,000 900 us against 464 / 337 / 345; from position 0 (264
    keys on average) 21 us against 25 in 2.  Hence as many shares as bring the
    launch to twice the compute units, each worth 256 keys or more on average."""
    if workgroups <= 0:
        return 1
    return max(1, min(2 * compute_units() // workgroups, mean_keys // KEYS_PER_WORKGROUP, MAX_KEY_SPLITS))


def heavy_first(work):
    """The order in which workgroups of unequal `work` are launched: the
    heaviest first (a causal prompt's last queries read every key, its first
    ones few), so that the light ones fill the compute units that the heavy
    ones leave last."""
    return np.argsort(-np.asarray(work, dtype=np.int64), kind="stable")


class PagedAttention(Mixer):
    """q/k/v projections (with or without bias), position encoding of q and k,
    cache write, attention over the sequence's pages, output projection
    (reference: shrike/models/qwen.py:111-125, shrike/engine/model_runner.py:63-151).

    The three projections are stacked into one [(H + 2 Hkv) D, h] matrix at
    load time; head j of q is rows j*D..(j+1)*D-1 of the q part, as in the
    reference's view (qwen.py:120-122).
    """

    @property
    def launches_follow_shape(self):
        # the plan of a step's launches is a function of the step's shape and goes into its
        # launch key (prepare); a position encoding of its own kind must say the same of itself
        return self.position is None or self.position.launches_follow_shape

    def __init__(self, spec, width, name):
        super().__init__(spec, width, name)
        self.position = (
            build_part("position", spec.position, width, name) if spec.position is not None else None
        )

    def params(self):
        s, h = self.spec, self.width
        q, kv = s.num_heads * s.head_dim, s.num_kv_heads * s.head_dim
        out = [
            ParamSpec(f"{self.name}.q_proj.weight", (q, h)),
            ParamSpec(f"{self.name}.k_proj.weight", (kv, h)),
            ParamSpec(f"{self.name}.v_proj.weight", (kv, h)),
            ParamSpec(f"{self.name}.o_proj.weight", (h, q)),
        ]
        if s.qkv_bias:
            out += [
                ParamSpec(f"{self.name}.q_proj.bias", (q,), init="bias", keep_float32=True),
                ParamSpec(f"{self.name}.k_proj.bias", (kv,), init="bias", keep_float32=True),
                ParamSpec(f"{self.name}.v_proj.bias", (kv,), init="bias", keep_float32=True),
            ]
        if s.out_bias:
            out.append(ParamSpec(f"{self.name}.o_proj.bias", (h,), init="bias", keep_float32=True))
        return out

    def cache_spec(self):
        s = self.spec
        return kv_cache_spec(s.num_kv_heads, s.head_dim, s.window)

    def check(self, runtime):
        s = self.spec
        if s.num_heads % s.num_kv_heads:
            raise ValueError(
                f"{self.name}: {s.num_heads} query heads are not a multiple of "
                f"{s.num_kv_heads} key/value heads"
            )
        if not 1 <= s.head_dim <= 256:
            raise ValueError(f"{self.name}: head_dim {s.head_dim} is outside 1..256")
        if s.window is not None and s.window < 1:
            raise ValueError(f"{self.name}: window must be positive, got {s.window}")

    def load(self, tensors, runtime):
        s, n = self.spec, self.name
        self.w_qkv = runtime.weight(torch.cat(
            [tensors[f"{n}.q_proj.weight"], tensors[f"{n}.k_proj.weight"], tensors[f"{n}.v_proj.weight"]],
            dim=0,
        ))
        self.b_qkv = (
            torch.cat([tensors[f"{n}.q_proj.bias"], tensors[f"{n}.k_proj.bias"], tensors[f"{n}.v_proj.bias"]])
            .contiguous()
            if s.qkv_bias
            else None
        )
        self.w_o = runtime.weight(tensors[f"{n}.o_proj.weight"])
        self.b_o = tensors[f"{n}.o_proj.bias"] if s.out_bias else None
        if self.position is not None:
            self.position.load(tensors, runtime)
        self.linear = runtime.linear
        self.linear_deferred = runtime.linear_deferred
        self.dtype = runtime.dtype

    # ------------------------------------------------------------ launch plans

    @property
    def plan_key(self):
        s = self.spec
        return ("paged_attention", s.num_heads, s.num_kv_heads, s.head_dim, s.window)

    def prepare(self, shape) -> None:
        """Decides once per step and head geometry how attention is launched:
        the key splits of single-token rows, and for prompt portions the kernel
        and its list of workgroups, which goes up with the step's metadata."""
        key = self.plan_key
        if key in shape.notes:
            return  # a layer with the same geometry has prepared this step
        s = self.spec
        h, hkv, d = s.num_heads, s.num_kv_heads, s.head_dim
        plan = shape.notes[key] = AttentionPlan()
        plan.mfma = self.dtype == torch.bfloat16 and ops.attention_supports_mfma(
            h, hkv, d, shape.page_size, (h + 2 * hkv) * d)
        if not plan.mfma:
            return  # the general kernel takes every token alike
        if shape.num_decode:
            plan.nsplit = decode_splits(shape.num_decode, hkv, shape.max_decode_ctx)
            plan.streaming = decode_streams(shape.num_decode, hkv, d, shape.max_decode_ctx, s.window)
            shape.launch_key.append((key, plan.nsplit, plan.streaming))
        portions = shape.q_lens[shape.num_decode:]
        if portions.size == 0:
            return
        tiles = ops.attention_prefill_shared_tiles(h, hkv, d)
        if tiles:
            plan.kernel = "shared"
            small_tiles = ops.attention_prefill_shared_tiles(h, hkv, d, small=True)
            if small_tiles:
                # Workgroups of half the size while all of them find room on the chip at
                # once (two on a compute unit): the step then takes as long as the
                # heaviest of them, which has half the queries.  Measured at 28 heads
                # over 4: 2,048 queries in 67 to 77 us against 92, 4,096 the same either way;
                # at 40 over 8: 1,024 in 37 against 48, 2,048 in 118 against 98.
                small_count = int((-(-portions // (QUERY_TILE * small_tiles))).sum())
                # (two workgroups of 8 wavefronts fit on a compute unit)
                if small_count * hkv <= 2 * compute_units():
                    plan.small, tiles = True, small_tiles
            seqs, q0 = portion_runs(portions, shape.num_decode, QUERY_TILE * tiles)
            # the keys an entry's last query reads: where its portion starts plus its queries
            keys = shape.starts[seqs] + q0 + QUERY_TILE * tiles
            if s.window:
                keys = np.minimum(keys, s.window + QUERY_TILE * tiles)
            order = heavy_first(keys)
            seqs, q0 = seqs[order], q0[order]
            plan.portion_splits = portion_splits(int(seqs.size) * hkv, int(keys.mean()))
            plan.first_token = shape.num_decode
        else:
            plan.kernel = "tiles"
            seqs, q0 = portion_runs(portions, shape.num_decode, QUERY_TILE)
        plan.count = int(seqs.size)
        # what the launches of the portions depend on beyond the step's sizes
        shape.launch_key.append((key, plan.kernel, plan.small, plan.portion_splits, plan.first_token, plan.count))
        tag = f"{h}:{hkv}:{d}:{s.window or 0}"
        plan.seq_name, plan.q0_name = f"attention_seq:{tag}", f"attention_q0:{tag}"
        shape.add(plan.seq_name, seqs)
        shape.add(plan.q0_name, q0)

    def attend(self, ctx, qkv, out, tables, cache) -> None:
        """Attention of every token of the step over its sequence's cache."""
        s = self.spec
        h, hkv, d = s.num_heads, s.num_kv_heads, s.head_dim
        plan = ctx.notes.get(self.plan_key)
        if plan is None:
            raise RuntimeError(f"{self.name}: the step was not prepared for this mixer "
                               "(the step function calls prepare() on every part)")
        q = qkv[:, : h * d]
        if not plan.mfma:
            ops.attention(q, out, h, hkv, d, ctx.positions, ctx.token_seq, tables, cache.pools["k"],
                          cache.pools["v"], cache.page_size, s.window, s.scale)
            return
        if ctx.num_decode:
            partial = ctx.buffer("attn_partial", (ctx.num_decode * h * plan.nsplit * (d + 2),),
                                 torch.float32)
            ops.attention_decode(q, out, ctx.num_decode, h, hkv, d, ctx.positions, tables,
                                 cache.pools["k"], cache.pools["v"], cache.page_size, s.window, s.scale,
                                 partial, plan.nsplit, plan.streaming)
        if plan.kernel == "shared":
            partial = None
            if plan.portion_splits > 1:
                prompt_tokens = ctx.num_tokens - plan.first_token
                partial = ctx.buffer("attn_portion_partial",
                                     (prompt_tokens * h * plan.portion_splits * (d + 2),), torch.float32)
            ops.attention_prefill_shared(q, out, plan.count, h, hkv, d, ctx.cu_q, ctx.ctx_lens,
                                         ctx.extras[plan.seq_name], ctx.extras[plan.q0_name], tables,
                                         cache.pools["k"], cache.pools["v"], cache.page_size, s.window,
                                         s.scale, small=plan.small, partial=partial,
                                         nsplit=plan.portion_splits, first_token=plan.first_token)
        elif plan.kernel == "tiles":
            ops.attention_prefill(q, out, plan.count, h, hkv, d, ctx.cu_q, ctx.ctx_lens,
                                  ctx.extras[plan.seq_name], ctx.extras[plan.q0_name], tables,
                                  cache.pools["k"], cache.pools["v"], cache.page_size, s.window, s.scale)

    def forward(self, ctx, x: torch.Tensor, cache) -> torch.Tensor:
        s = self.spec
        n = x.shape[0]
        qkv_width = (s.num_heads + 2 * s.num_kv_heads) * s.head_dim
        table = self.position.rotary_table() if self.position is not None else None
        fused_position = self.position is None or table is not None
        split_sum = None
        if fused_position:
            # the cache-write kernel can take the projections as partial sums
            qkv = self.linear_deferred(ctx, "attn_qkv_sum", x, self.w_qkv, bias=self.b_qkv,
                                       reader="position")
            if isinstance(qkv, ops.SplitSum):
                split_sum, qkv = qkv, ctx.buffer("attn_qkv", (n, qkv_width), ctx.dtype)
        else:
            qkv = ctx.buffer("attn_qkv", (n, qkv_width), ctx.dtype)
            self.linear(x, self.w_qkv, qkv, bias=self.b_qkv)
            self.position.apply(ctx, qkv, s.num_heads, s.num_kv_heads, s.head_dim)
        inv_freq, rot_dim = table if table is not None else (None, 0)
        tables = ctx.block_tables[cache.group]
        ops.rope_kv_store(
            qkv, s.num_heads, s.num_kv_heads, s.head_dim, rot_dim, inv_freq, ctx.positions,
            ctx.token_seq, tables, cache.pools["k"], cache.pools["v"], cache.page_size,
            write_kv=cache.owned, split_sum=split_sum,
        )
        attn = ctx.buffer("attn_out", (n, s.num_heads * s.head_dim), ctx.dtype)
        self.attend(ctx, qkv, attn, tables, cache)
        # the norm that follows adds the output to the residual stream and can add up parts
        return self.linear_deferred(ctx, "attn_proj", attn, self.w_o, bias=self.b_o)


register_mixer("paged_attention", PagedAttention)
