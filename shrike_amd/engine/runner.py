"""The step function: one flat batch of (sequence, its next tokens), portions
of prompts beside single decoded tokens, run from the cache; logits come back
for the wanted places only.

Reference: shrike/engine/model_runner.py:183-250.  Differences by design: the
entries carry their tokens and wanted rows explicitly (so replay can ask for
any row), all metadata goes to the device in one copy, nothing is computed on
the host per token, and steps that hold only single tokens are replayed from
HIP graphs (one per batch-size bucket), because such a step is a few hundred
short kernels whose launches would otherwise cost more than they run.
"""

from __future__ import annotations

from collections import OrderedDict
from dataclasses import dataclass

import numpy as np
import torch

from ..cache.manager import CacheManager, SequenceCache
from ..kernels import lib as kernel_lib
from ..kernels import ops
from .context import StepContext, StepShape, Workspace

GRAPH_BATCH_BUCKETS = (1, 2, 4, 8, 16, 32, 64, 128, 256)
GRAPH_TABLE_QUANTUM = 64  # block-table widths of graphs are multiples of this
MAX_GRAPHS = 24  # captured decode steps kept; the least recently used one goes first
MAX_CALL_LISTS = 64  # recorded launch lists of other steps kept, by shape


@dataclass
class StepEntry:
    """`tokens` are the sequence's next tokens, the first at position `start`
    (= tokens already in its cache); `want` are offsets into `tokens`."""

    cache: SequenceCache
    tokens: list
    start: int
    want: list


class StepError(ValueError):
    """A step was refused before anything ran."""


class _Meta:
    """The int32 metadata of a step, laid out in one buffer."""

    FIELDS = ("token_ids", "positions", "token_seq", "cu_q", "ctx_lens", "state_slots", "fresh",
              "out_rows")

    def __init__(self, arrays: dict, tables: list[np.ndarray], shape: StepShape):
        self.arrays = arrays
        self.tables = tables
        self.shape = shape
        self.extra_names = sorted(shape.extras)  # what the parts added in prepare()
        self.names = list(self.FIELDS) + self.extra_names
        self.parts = ([arrays[f] for f in self.FIELDS] + [shape.extras[n] for n in self.extra_names]
                      + [t.reshape(-1) for t in tables])
        self.sizes = [int(p.size) for p in self.parts]
        self.total = int(sum(self.sizes))

    def views(self, dev: torch.Tensor, num_seqs: int) -> dict:
        out, off = {}, 0
        for name, size in zip(self.names, self.sizes):
            out[name] = dev[off : off + size]
            off += size
        tables = []
        for t in self.tables:
            tables.append(dev[off : off + t.size].view(num_seqs, t.shape[1]))
            off += t.size
        out["block_tables"] = tables
        out["extras"] = {n: out[n] for n in self.extra_names}
        return out


class _DecodeGraph:
    """A captured decode step for one (batch bucket, table widths, launch key)."""

    def __init__(self, workspace: Workspace):
        self.workspace = workspace  # shared by the graphs of one batch bucket
        self.graph = None
        self.meta_dev = None
        self.logits = None
        self.ctx = None
        # host copy of the metadata, updated in place from step to step
        self.pinned = None
        self.host = None  # numpy view of `pinned`
        self.copied = None  # event: the last copy out of `pinned` is done
        self.offsets = None  # field -> offset in the buffer; tables -> list of offsets
        self.rows = None  # the sequences of the last step, in row order
        self.table_lens = None  # per group, pages of each row already written to `host`


class ModelRunner:
    def __init__(self, model, cache: CacheManager, runtime, graphs: bool = True):
        self.model = model
        self.cache = cache
        self.runtime = runtime
        self.workspace = Workspace(runtime.device)
        self.vocab_size = model.spec.vocab_size
        self.layer_caches = []
        for pos, entry in enumerate(model.spec.schedule):
            owner = pos if entry.cache_of is None else entry.cache_of
            if cache.owns_cache(owner):
                self.layer_caches.append(cache.layer_cache(owner, reader=entry.cache_of is not None))
            else:
                self.layer_caches.append(None)
        self._pinned = None
        self._pinned_free = None  # event: the last copy out of the pinned buffer is done
        # Graphs replay fixed kernel arguments: the model's parts say whether
        # their launches can be recorded.
        self.use_graphs = bool(graphs) and model.graph_safe()
        self._graphs: OrderedDict[tuple, _DecodeGraph] = OrderedDict()
        # one workspace per batch bucket, shared by its graphs: their buffers have
        # the same shapes, and a buffer that one of them outgrows is kept
        self._graph_workspaces: dict[int, Workspace] = {}
        self.graph_replays = 0
        self.graph_captures = 0
        # Steps that are no graph (they hold prompt portions, or do not want every row)
        # run their forward from a recorded list of launches when a step of the same
        # shape has run before: one call into the library instead of one per kernel.
        self.use_call_lists = bool(graphs) and model.launches_follow_shape()
        self._call_lists: OrderedDict[tuple, tuple] = OrderedDict()  # shape key -> (list, logits)
        self._call_lists_generation = -1
        self.list_replays = 0
        self.list_records = 0

    # ---------------------------------------------------------------- metadata

    def _check(self, entries: list[StepEntry]) -> None:
        ps = self.cache.page_size
        seen = set()
        for e in entries:
            if id(e.cache) in seen:
                raise StepError("a sequence appears twice in one step")
            seen.add(id(e.cache))
            n = len(e.tokens)
            if n < 1:
                raise StepError("an entry of a step needs at least one token")
            if e.start < 0:
                raise StepError(f"negative start {e.start}")
            if any(not 0 <= w < n for w in e.want):
                raise StepError(f"wanted offsets {list(e.want)} lie outside the entry's {n} tokens")
            last_page = (e.start + n - 1) // ps
            for g, table in zip(self.cache.groups, e.cache.tables):
                if len(table) <= last_page:
                    raise StepError(
                        f"block table has {len(table)} pages but the step reaches page {last_page}"
                    )
                # the pages this step writes, and the oldest page it reads
                w = g.spec.window
                first = 0 if w is None else max(0, e.start - w + 1) // ps
                touched = table[e.start // ps : last_page + 1]
                if min(touched) < 0 or max(touched) >= self.cache.num_pages or table[first] < 0:
                    raise StepError("block table names a page outside the pool")

    def _meta(self, entries: list[StepEntry], order: list[int], pad_to: int = 0,
              table_widths: list[int] | None = None) -> _Meta:
        """Arrays of the step.  With pad_to, rows are added up to that many
        sequences: one token each at position 0 whose page is the spare page
        that no request ever holds."""
        n_real = len(order)
        q_lens = np.array([len(entries[i].tokens) for i in order], dtype=np.int64)
        starts = np.array([entries[i].start for i in order], dtype=np.int64)
        pads = max(0, pad_to - n_real)
        if pads:
            q_lens = np.concatenate([q_lens, np.ones(pads, dtype=np.int64)])
            starts = np.concatenate([starts, np.zeros(pads, dtype=np.int64)])
        shape = StepShape(q_lens, starts, self.cache.page_size, padded_rows=pads)
        self.model.prepare(shape)
        num_seqs, num_tokens, num_decode = shape.num_seqs, shape.num_tokens, shape.num_decode
        cu_q = np.zeros(num_seqs + 1, dtype=np.int64)
        np.cumsum(q_lens, out=cu_q[1:])
        token_seq = np.repeat(np.arange(num_seqs), q_lens)
        positions = np.arange(num_tokens) - cu_q[token_seq] + starts[token_seq]
        token_ids = np.concatenate(
            [np.asarray(entries[i].tokens, dtype=np.int64) for i in order]
            + [np.zeros(pads, dtype=np.int64)]
        )
        if token_ids.min() < 0 or token_ids.max() >= self.vocab_size:
            raise StepError(f"token ids must lie in [0, {self.vocab_size})")
        ctx_lens = starts + q_lens
        slot_of = {i: k for k, i in enumerate(order)}
        if pad_to:
            out_rows = np.arange(num_seqs, dtype=np.int64)  # one row per sequence, pads included
        else:
            out_rows = np.asarray(
                [cu_q[slot_of[i]] + w for i, e in enumerate(entries) for w in e.want], dtype=np.int64
            )
        # padding rows carry the spare slot, as they carry the spare page
        state_slots = np.array([entries[i].cache.state_slot for i in order]
                               + [self.cache.slots.num_slots] * pads, dtype=np.int64)
        fresh = np.array([int(entries[i].cache.fresh_state) for i in order] + [0] * pads,
                         dtype=np.int64)
        tables = []
        for gi in range(len(self.cache.groups)):
            need = max(1, max(len(entries[i].cache.tables[gi]) for i in order))
            # in steps of GRAPH_TABLE_QUANTUM pages for every step: the width is part of a
            # step's shape, and shapes that come back are run from recorded launches
            width = table_widths[gi] if table_widths else -(-need // GRAPH_TABLE_QUANTUM) * GRAPH_TABLE_QUANTUM
            t = np.zeros((num_seqs, width), dtype=np.int64)
            for k, i in enumerate(order):
                row = entries[i].cache.tables[gi]
                t[k, : len(row)] = row
            t[n_real:, :] = self.cache.num_pages  # the spare page
            tables.append(t)
        arrays = dict(token_ids=token_ids, positions=positions, token_seq=token_seq, cu_q=cu_q,
                      ctx_lens=ctx_lens, state_slots=state_slots, fresh=fresh, out_rows=out_rows)
        meta = _Meta(arrays, tables, shape)
        meta.q_lens, meta.ctx_lens = q_lens, ctx_lens
        meta.num_seqs, meta.num_tokens, meta.num_decode = num_seqs, num_tokens, num_decode
        return meta

    def _upload(self, meta: _Meta, dev: torch.Tensor) -> None:
        if self._pinned_free is not None:
            self._pinned_free.synchronize()
        if self._pinned is None or self._pinned.numel() < meta.total:
            self._pinned = torch.empty(max(2 * meta.total, 4096), dtype=torch.int32, pin_memory=True)
            self._pinned_free = torch.cuda.Event()
        host = self._pinned[: meta.total]
        np.concatenate(meta.parts, out=host.numpy(), casting="unsafe")
        dev.copy_(host, non_blocking=True)
        self._pinned_free.record()

    def _context(self, meta: _Meta, dev: torch.Tensor, workspace: Workspace) -> StepContext:
        v = meta.views(dev, meta.num_seqs)
        nd = meta.num_decode
        return StepContext(
            dtype=self.runtime.dtype, device=self.runtime.device, workspace=workspace,
            num_tokens=meta.num_tokens, num_seqs=meta.num_seqs, num_decode=nd,
            token_ids=v["token_ids"], positions=v["positions"], token_seq=v["token_seq"],
            cu_q=v["cu_q"], ctx_lens=v["ctx_lens"], state_slots=v["state_slots"], fresh=v["fresh"],
            out_rows=v["out_rows"], block_tables=v["block_tables"],
            q_lens=meta.q_lens.tolist(), ctx_lens_host=meta.ctx_lens.tolist(),
            max_q_len=int(meta.q_lens.max()), max_ctx_len=int(meta.ctx_lens.max()),
            max_decode_ctx=int(meta.ctx_lens[:nd].max()) if nd else 0,
            extras=v["extras"], notes=meta.shape.notes,
        )

    def build_context(self, entries: list[StepEntry]) -> StepContext:
        self._check(entries)
        order = sorted(range(len(entries)), key=lambda i: 0 if len(entries[i].tokens) == 1 else 1)
        meta = self._meta(entries, order)
        dev = self.workspace.get("step_meta", (meta.total,), torch.int32)
        self._upload(meta, dev)
        ctx = self._context(meta, dev, self.workspace)
        ctx.shape_key = (meta.num_tokens, meta.num_seqs, meta.num_decode, int(meta.arrays["out_rows"].size),
                         tuple(t.shape[1] for t in meta.tables),
                         tuple((n, int(meta.shape.extras[n].size)) for n in meta.extra_names),
                         tuple(meta.shape.launch_key))
        return ctx

    def _forward(self, ctx: StepContext) -> torch.Tensor:
        """The model's forward for a step that is no graph: from the recorded launches
        of an earlier step of the same shape where there is one, else kernel by kernel
        (and recorded).  The step's metadata is already on its way to the device; the
        launches name the same buffers step after step, so a list stands as long as no
        buffer of the workspace has been replaced by a larger one."""
        if not self.use_call_lists:
            return self.model.forward(ctx, self.layer_caches)
        generation = self.workspace.generation
        if self._call_lists_generation != generation:
            self._call_lists.clear()
            self._call_lists_generation = generation
        key = ctx.shape_key
        held = self._call_lists.get(key)
        if held is not None:
            self._call_lists.move_to_end(key)
            calls, logits = held
            calls.run(ops.current_stream())
            self.list_replays += 1
            return logits
        kernel_lib.begin_recording()
        try:
            logits = self.model.forward(ctx, self.layer_caches)
        except BaseException:
            kernel_lib.end_recording(keep=False)
            raise
        calls = kernel_lib.end_recording()
        self.list_records += 1
        if self.workspace.generation != generation:
            # this step grew a buffer: lists recorded before it may name the one that went
            self._call_lists.clear()
            self._call_lists_generation = self.workspace.generation
        if len(self._call_lists) >= MAX_CALL_LISTS:
            self._call_lists.popitem(last=False)
        self._call_lists[key] = (calls, logits)
        return logits

    # ------------------------------------------------------------------ graphs

    def _graph_key(self, entries: list[StepEntry]):
        """Bucket of a step that holds only single tokens which all want their
        logits, or None when the step does not qualify."""
        if not self.use_graphs or len(entries) > GRAPH_BATCH_BUCKETS[-1]:
            return None
        for e in entries:
            if len(e.tokens) != 1 or list(e.want) != [0]:
                return None
        batch = next(b for b in GRAPH_BATCH_BUCKETS if b >= len(entries))
        widths = []
        for gi in range(len(self.cache.groups)):
            need = max(len(e.cache.tables[gi]) for e in entries)
            widths.append(-(-need // GRAPH_TABLE_QUANTUM) * GRAPH_TABLE_QUANTUM)
        # what the parts' launches depend on beyond the number of rows (a mixer's
        # split of long contexts, say): steps share a graph only if it is equal
        starts = np.zeros(batch, dtype=np.int64)
        starts[: len(entries)] = [e.start for e in entries]
        shape = StepShape(np.ones(batch, dtype=np.int64), starts, self.cache.page_size,
                          padded_rows=batch - len(entries))
        self.model.prepare(shape)
        return batch, tuple(widths), tuple(shape.launch_key)

    def _graph_step(self, entries: list[StepEntry], key) -> torch.Tensor:
        batch, widths, _launch_key = key
        g = self._graphs.get(key)
        if g is not None:
            self._graphs.move_to_end(key)
        if g is None or not self._refresh(g, entries, widths):
            self._check(entries)
            order = list(range(len(entries)))
            meta = self._meta(entries, order, pad_to=batch, table_widths=list(widths))
            if g is None:
                if len(self._graphs) >= MAX_GRAPHS:
                    # the device may still be replaying the graph that goes
                    torch.cuda.synchronize(self.runtime.device)
                    self._graphs.popitem(last=False)
                workspace = self._graph_workspaces.get(batch)
                if workspace is None:
                    workspace = Workspace(self.runtime.device, keep_outgrown=True)
                    self._graph_workspaces[batch] = workspace
                g = _DecodeGraph(workspace)
                g.meta_dev = torch.zeros(meta.total, dtype=torch.int32, device=self.runtime.device)
                g.pinned = torch.empty(meta.total, dtype=torch.int32, pin_memory=True)
                g.host = g.pinned.numpy()
                g.copied = torch.cuda.Event()
                offsets, off = {}, 0
                for name, size in zip(meta.names, meta.sizes):
                    offsets[name] = off
                    off += size
                offsets["tables"] = []
                for t in meta.tables:
                    offsets["tables"].append(off)
                    off += t.size
                g.offsets = offsets
                self._fill(g, entries, meta)
                ops.copy_words(g.pinned, g.meta_dev)  # the eager run below reads it
                g.copied.record()
                g.ctx = self._context(meta, g.meta_dev, g.workspace)
                # This step itself runs kernel by kernel: every workspace buffer exists
                # before the capture starts.  Recording executes nothing, so this
                # run's logits are the step's result and the graph is not replayed
                # now: a part that advances a state of its own must see each step once.
                eager_logits = self.model.forward(g.ctx, self.layer_caches)
                torch.cuda.synchronize(self.runtime.device)
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph):
                    g.logits = self.model.forward(g.ctx, self.layer_caches)
                # The recording wrote nothing: eager_logits, be it the workspace buffer
                # that the recorded run names too or a tensor that a part allocated for
                # itself, still holds what the kernel-by-kernel run put there.
                g.graph = graph
                self._graphs[key] = g
                self.graph_captures += 1
                self.graph_replays += 1  # counted with the steps that the graph path served
                return eager_logits[: len(entries)]
            else:
                self._fill(g, entries, meta)
        ops.copy_words(g.pinned, g.meta_dev)
        g.copied.record()
        g.graph.replay()
        self.graph_replays += 1
        return g.logits[: len(entries)]

    def _fill(self, g: _DecodeGraph, entries: list[StepEntry], meta: _Meta) -> None:
        """Writes a step's whole metadata into the graph's host buffer."""
        g.copied.synchronize()
        np.concatenate(meta.parts, out=g.host, casting="unsafe")
        g.rows = [e.cache for e in entries]  # the objects, so that their identity cannot be reused
        g.table_lens = [[len(e.cache.tables[gi]) for e in entries]
                        for gi in range(len(self.cache.groups))]

    def _refresh(self, g: _DecodeGraph, entries: list[StepEntry], widths) -> bool:
        """The common case of decoding: the same sequences as in the graph's last
        step, each one token further.  Only what changed is written into the host
        buffer: tokens, positions, lengths and the pages that were appended.
        False: the rows differ, and the caller rebuilds the buffer."""
        if g.rows is None or len(g.rows) != len(entries):
            return False
        for e, row in zip(entries, g.rows):
            if e.cache is not row:
                return False
        n = len(entries)
        tokens = [e.tokens[0] for e in entries]
        starts = [e.start for e in entries]
        if min(tokens) < 0 or max(tokens) >= self.vocab_size or min(starts) < 0:
            return False  # let the full path raise the proper error
        ps, num_pages = self.cache.page_size, self.cache.num_pages
        g.copied.synchronize()
        host, off = g.host, g.offsets
        # (entries of pages that a window has passed stay as they were: no kernel reads them)
        for gi in range(len(self.cache.groups)):
            lens, width, base = g.table_lens[gi], widths[gi], off["tables"][gi]
            for k, e in enumerate(entries):
                table = e.cache.tables[gi]
                have = len(table)
                if have <= e.start // ps or have > width or have < lens[k]:
                    return False
                if have != lens[k]:
                    new = table[lens[k]:have]
                    if min(new) < 0 or max(new) >= num_pages:
                        return False
                    host[base + k * width + lens[k] : base + k * width + have] = new
                    lens[k] = have
        host[off["token_ids"] : off["token_ids"] + n] = tokens
        host[off["positions"] : off["positions"] + n] = starts
        ctx = off["ctx_lens"]
        host[ctx : ctx + n] = starts
        host[ctx : ctx + n] += 1
        host[off["fresh"] : off["fresh"] + n] = 0
        return True

    # ------------------------------------------------------ a step in two halves

    def prepare_decode(self, caches: list, starts: list[int]):
        """The host's share of a decode step whose tokens are not known yet: one
        token for each sequence, at position starts[i], logits wanted.  Returns a
        handle for launch_decode, or None when the step cannot be prepared (no
        captured graph fits, or its rows changed): step() then does everything."""
        entries = [StepEntry(c, [0], s, [0]) for c, s in zip(caches, starts)]
        key = self._graph_key(entries)
        g = self._graphs.get(key) if key is not None else None
        if g is None or not self._refresh(g, entries, key[1]):
            return None
        return g, entries

    def launch_decode(self, prepared, tokens: list[int]) -> torch.Tensor:
        """Runs a step that prepare_decode() laid out, now that its tokens are known."""
        g, entries = prepared
        n = len(entries)
        if len(tokens) != n or min(tokens) < 0 or max(tokens) >= self.vocab_size:
            for e, t in zip(entries, tokens):
                e.tokens = [t]
            return self.step(entries)  # raises what an ordinary step raises
        off = g.offsets["token_ids"]
        g.host[off : off + n] = tokens
        ops.copy_words(g.pinned, g.meta_dev)
        g.copied.record()
        g.graph.replay()
        self.graph_replays += 1
        for e in entries:
            e.cache.fresh_state = False
        return g.logits[:n]

    def launch_decode_from(self, prepared, tokens: torch.Tensor) -> torch.Tensor:
        """launch_decode() with the tokens still on the device (int32, one per entry,
        as the sampler of the step before left them): they are copied into the
        step's metadata there, and the host need not know them to launch."""
        g, entries = prepared
        n = len(entries)
        if tokens.dtype != torch.int32 or tokens.shape != (n,) or tokens.device != g.meta_dev.device:
            raise ValueError("launch_decode_from: one int32 token per entry, on the model's device")
        off = g.offsets["token_ids"]
        ops.copy_words(g.pinned, g.meta_dev, patch=tokens, patch_at=off)
        g.copied.record()
        g.graph.replay()
        self.graph_replays += 1
        for e in entries:
            e.cache.fresh_state = False
        return g.logits[:n]

    def dry_run(self, singles: int, portion: int) -> None:
        """Runs the model once on made-up tokens so that every buffer of such a
        step exists: `singles` rows of one token, or else one sequence of
        `portion` tokens.  The single-token rows are padding rows beside one
        real row; the cache must be otherwise unused (its first pages are
        written)."""
        seq = self.cache.new_sequence()
        try:
            n = portion if not singles else 1
            self.cache.append(seq, 0, n)
            entries = [StepEntry(seq, [0] * n, 0, [n - 1])]
            meta = self._meta(entries, [0], pad_to=singles)
            dev = self.workspace.get("step_meta", (meta.total,), torch.int32)
            self._upload(meta, dev)
            self.model.forward(self._context(meta, dev, self.workspace), self.layer_caches)
            torch.cuda.synchronize(self.runtime.device)
        finally:
            self.cache.free(seq)

    # -------------------------------------------------------------------- step

    def step(self, entries: list[StepEntry]) -> torch.Tensor:
        """Runs the entries' tokens as one batch; returns float32 logits
        [wanted, vocab] in the order of the entries and of their `want`.
        The tensor is a view of a buffer that a later step overwrites."""
        if not entries:
            return torch.empty(0, self.vocab_size, dtype=torch.float32, device=self.runtime.device)
        key = self._graph_key(entries)
        if key is not None:
            logits = self._graph_step(entries, key)
        else:
            ctx = self.build_context(entries)
            logits = self._forward(ctx)
        for e in entries:
            e.cache.fresh_state = False
        return logits
