"""LLMEngine ties the step function, the scheduler and the sampler into a loop:
step() = schedule -> one batched forward -> sample -> append / finish.

Reference: shrike/engine/engine.py (same public names: add_request, has_work,
step, generate, metrics, StepOutput).
"""

from __future__ import annotations

import time
from dataclasses import dataclass, field

import torch

from ..cache import CacheManager
from ..config.engine_config import EngineConfig
from ..sampling import Sampler
from .loading import load_model
from .request import Request, SamplingParams, Status
from .runner import ModelRunner, StepEntry
from .scheduler import Scheduler


@dataclass
class StepOutput:
    req_id: int
    token_id: int
    finished: bool
    finish_reason: str | None


@dataclass
class EngineStats:
    steps: int = 0
    tokens_generated: int = 0
    started_at: float = field(default_factory=time.perf_counter)


class LLMEngine:
    """LLMEngine(model_dir, block_size=16, gpu_mem_util=0.85,
    max_tokens_per_step=512, max_running=256, enable_prefix_caching=True,
    num_kv_blocks=None, dtype=None, seed=0)."""

    def __init__(self, model_dir: str, config: EngineConfig | None = None, *, model=None,
                 runtime=None, **options) -> None:
        self.config = config if config is not None else EngineConfig(**options)
        cfg = self.config
        self.model_dir = model_dir
        if model is None:
            model, runtime, _ = load_model(model_dir, cfg.dtype, cfg.device)
        self.model, self.runtime = model, runtime
        self.tokenizer = _load_tokenizer(model_dir) if model_dir is not None else None

        specs = model.cache_specs()
        elem = torch.empty(0, dtype=runtime.dtype).element_size()
        probe = CacheManager(specs, cfg.block_size, 1, max_slots=1)
        if cfg.num_kv_blocks is not None:
            num_blocks = cfg.num_kv_blocks
        else:
            # shrike/engine/model_runner.py:165-174: a share of the free device memory
            # ... less what the step function's own buffers will take, which do not
            # exist yet: the pool must leave them room
            reserve = workspace_reserve(model, runtime, cfg)
            free, _total = torch.cuda.mem_get_info(runtime.device)
            per_page = max(1, probe.bytes_per_page(elem))
            num_blocks = max(1, int(max(0, free - reserve) * cfg.gpu_mem_util) // per_page)
        self.cache = CacheManager(specs, cfg.block_size, num_blocks, max_slots=cfg.max_running,
                                  enable_prefix_caching=cfg.enable_prefix_caching)
        self.cache.allocate(runtime.dtype, runtime.device)
        self.runner = ModelRunner(model, self.cache, runtime, graphs=cfg.graphs)
        self.scheduler = Scheduler(self.cache, cfg.max_tokens_per_step, cfg.max_running)
        self.sampler = Sampler(runtime.device, cfg.seed)
        self.eos_ids = set(model.spec.eos_token_ids)
        self.requests: dict[int, Request] = {}
        self._next_req_id = 0
        self.stats = EngineStats()
        # (batch, prepared step) of the next step, laid out while the device ran the last
        # one; dropped whenever a request arrives, ends or is aborted
        self._planned = None
        # (batch, logits) of a decode step that is already running on the device: it was
        # launched, fed with the last step's tokens on the device, before the host read them
        self._inflight = None
        self._row_list = self._row_list_read = None  # page-locked row indices for _rows_of

    # reference name for the cache manager
    @property
    def block_manager(self) -> CacheManager:
        return self.cache

    def add_request(self, prompt, sampling: SamplingParams, chat: bool = True) -> int:
        if isinstance(prompt, str):
            token_ids = _encode(self.tokenizer, self.model_dir, prompt, chat)
        else:
            token_ids = [int(t) for t in prompt]
        if len(token_ids) == 0:
            raise ValueError("a request with an empty prompt cannot be served: there is no token "
                             "to compute a next one from")
        vocab = self.model.spec.vocab_size
        if min(token_ids) < 0 or max(token_ids) >= vocab:
            raise ValueError(f"prompt token ids must lie in [0, {vocab})")
        page = self.cache.page_size
        longest = len(token_ids) + sampling.max_new_tokens
        pages_at_most = -(-longest // page)
        if pages_at_most > self.cache.num_pages:
            raise ValueError(
                f"this request could never be scheduled: {len(token_ids)} prompt tokens and up to "
                f"{sampling.max_new_tokens} new ones fill {pages_at_most} pages of {page} tokens, and "
                f"the whole pool is {self.cache.num_pages} pages.  A shorter prompt, a smaller "
                "max_new_tokens or a larger pool (num_kv_blocks, gpu_mem_util) would let it in"
            )
        req = Request(token_ids=token_ids, sampling=sampling, req_id=self._next_req_id)
        self._next_req_id += 1
        self.requests[req.req_id] = req
        self.scheduler.add(req)
        self._planned = None
        return req.req_id

    @property
    def has_work(self) -> bool:
        return self.scheduler.has_work

    def step(self) -> list[StepOutput]:
        batch = logits = None
        inflight, self._inflight = self._inflight, None
        if inflight is not None:
            # The step is already running.  Rows of requests that ended meanwhile
            # (the end-of-sequence token, an abort) computed something nobody needs;
            # what they wrote went into pages and slots that were theirs to write.
            launched, all_logits = inflight
            live = [i for i, (req, _) in enumerate(launched)
                    if req.status is Status.RUNNING and self.requests.get(req.req_id) is req]
            if live:
                batch = [launched[i] for i in live]
                logits = all_logits if len(live) == len(launched) else self._rows_of(all_logits, live)
                sampled = [req for req, _ in batch]
        if batch is None:
            planned, self._planned = self._planned, None
            running = self.scheduler.running
            if planned is not None and (self.scheduler.waiting or len(planned[0]) != len(running)
                                        or any(p[0] is not r for p, r in zip(planned[0], running))):
                planned = None  # the queues were changed behind the engine's back
            if planned is not None:
                batch, prepared = planned
            else:
                batch, prepared = self.scheduler.schedule(), None
            if not batch:
                return []
            entries, sampled = [], []
            for req, n_new in batch:
                start = req.num_computed_tokens
                reaches_end = start + n_new >= req.num_tokens
                entries.append(
                    StepEntry(req.cache, req.token_ids[start : start + n_new], start,
                              [n_new - 1] if reaches_end else [])
                )
                if reaches_end:
                    sampled.append(req)
            if prepared is not None:
                logits = self.runner.launch_decode(prepared, [e.tokens[0] for e in entries])
            else:
                logits = self.runner.step(entries)
        chosen = self.sampler.launch(logits, sampled)

        # While the device works: what does not depend on the tokens it will choose.
        self.scheduler.postprocess(batch)  # before finishing: finish() gives the pages back
        ahead = self.scheduler.plan_decode_step() if len(sampled) == len(batch) else None
        if ahead is not None:
            prepared = self.runner.prepare_decode(
                [req.cache for req, _ in ahead], [req.num_computed_tokens for req, _ in ahead])
            if (prepared is not None and self.config.overlap_steps and len(ahead) == len(sampled)
                    and all(a[0] is r for a, r in zip(ahead, sampled))):
                # the next step starts behind this one without waiting for the host
                self._inflight = (ahead, self.runner.launch_decode_from(prepared, chosen.device))
            else:
                self._planned = (ahead, prepared)

        tokens = [] if chosen is None else chosen.tolist()  # waits for the device
        outputs: list[StepOutput] = []
        for req, token in zip(sampled, tokens):
            req.token_ids.append(token)
            self.stats.tokens_generated += 1
            finished, reason = False, None
            if token in self.eos_ids and not req.sampling.ignore_eos:
                finished, reason = True, "stop"
            elif req.num_generated >= req.sampling.max_new_tokens:
                finished, reason = True, "length"
            outputs.append(StepOutput(req.req_id, token, finished, reason))
            if finished:
                self.scheduler.finish(req, reason)
                del self.requests[req.req_id]
                self._planned = None  # the next step is not the one that was planned
        self.stats.steps += 1
        return outputs

    def _rows_of(self, logits: torch.Tensor, rows: list[int]) -> torch.Tensor:
        """The given rows of `logits`, gathered by a kernel whose row list lies in
        page-locked memory (no copy of it to the device, no library indexing)."""
        from ..kernels import ops

        if self._row_list is None or self._row_list.numel() < len(rows):
            self._row_list = torch.empty(max(256, len(rows)), dtype=torch.int32, pin_memory=True)
            self._row_list_read = torch.cuda.Event()
        else:
            self._row_list_read.synchronize()  # the last gather has read the list
        index = self._row_list[: len(rows)]
        index.numpy()[:] = rows
        out = self.runner.workspace.get("live_logits", (len(rows), logits.shape[1]), logits.dtype)
        ops.gather_rows(logits, index, out)
        self._row_list_read.record()
        return out

    def generate(self, prompts, sampling, chat: bool = True) -> list[list[int]]:
        """Runs the prompts to their ends; the tokens generated for each, in the
        order of `prompts` (an end-of-sequence token that ended one is its last)."""
        prompts = list(prompts)
        per_prompt = [sampling] * len(prompts) if isinstance(sampling, SamplingParams) else list(sampling)
        if len(per_prompt) != len(prompts):
            raise ValueError("one SamplingParams per prompt, or one for all")
        generated: dict[int, list[int]] = {}
        for prompt, params in zip(prompts, per_prompt):
            generated[self.add_request(prompt, params, chat)] = []
        while self.scheduler.has_work:
            for out in self.step():
                if out.req_id in generated:  # a request added by someone else runs along unrecorded
                    generated[out.req_id].append(out.token_id)
        return list(generated.values())

    def abort(self, req_id: int) -> None:
        req = self.requests.pop(req_id, None)
        if req is not None:
            self.scheduler.abort(req)
            self._planned = None

    def metrics(self) -> dict:
        sched, cache = self.scheduler, self.cache
        elapsed = time.perf_counter() - self.stats.started_at
        return {
            "steps": self.stats.steps,
            "tokens_generated": self.stats.tokens_generated,
            "avg_tokens_per_sec": round(self.stats.tokens_generated / max(elapsed, 1e-9), 1),
            "running": len(sched.running),
            "waiting": len(sched.waiting),
            "kv_blocks_total": cache.num_pages,
            "kv_blocks_free": cache.num_free,
            "preemptions": sched.num_preemptions,
            "prefix_cache_hit_rate": round(
                cache.cache_hit_blocks / max(1, cache.cache_query_blocks), 3
            ),
        }


def workspace_reserve(model, runtime, cfg: EngineConfig) -> int:
    """Bytes of device memory that the step function's buffers take once serving
    is under way, measured on a throwaway cache of a few pages: one step of the
    largest batch of single tokens (all of them padding rows) and one of the
    largest prompt portion.  Every batch bucket of the decode graphs has buffers
    of its own, each half the next one's size, so the largest counts twice."""
    from .runner import GRAPH_BATCH_BUCKETS, Workspace

    from ..kernels import ops

    pages = -(-cfg.max_tokens_per_step // cfg.block_size) + 1
    cache = CacheManager(model.cache_specs(), cfg.block_size, pages, max_slots=2,
                         enable_prefix_caching=False)
    cache.allocate(runtime.dtype, runtime.device)
    runner = ModelRunner(model, cache, runtime, graphs=False)
    rows = min(cfg.max_running, cfg.max_tokens_per_step, GRAPH_BATCH_BUCKETS[-1])
    rows = next(b for b in GRAPH_BATCH_BUCKETS if b >= rows)
    sizes = []
    for singles, portion in ((rows, 0), (0, cfg.max_tokens_per_step)):
        runner.workspace = Workspace(runtime.device)
        runner.dry_run(singles, portion)
        sizes.append(runner.workspace.nbytes())
    torch.cuda.synchronize(runtime.device)
    # What the probe allocated goes back to the device, not only to torch's own pool of
    # freed blocks: the caller reads the free memory next, and would otherwise count the
    # probe's buffers twice, once as memory that is gone and once in this reserve.
    del runner, cache
    torch.cuda.empty_cache()
    # the sampler's scratch for the largest batch that can want a token in one step
    sampler = 4 * ops.sample_scratch_floats(min(cfg.max_running, cfg.max_tokens_per_step),
                                            model.spec.vocab_size)
    slack = 64 << 20  # graph objects, page-locked staging
    return 2 * sizes[0] + sizes[1] + sampler + slack


class LLM:
    """Python entry point: LLM(model_dir, **engine options).generate(prompts, sampling_params)."""

    def __init__(self, model: str, **options):
        self.engine = LLMEngine(model, **options)

    def generate(self, prompts, sampling_params: SamplingParams | list | None = None,
                 chat: bool = False) -> list[list[int]]:
        if sampling_params is None:
            sampling_params = SamplingParams()
        if prompts and isinstance(prompts[0], int):
            prompts = [prompts]
        return self.engine.generate(list(prompts), sampling_params, chat=chat)


# ------------------------------------------------------------------- tokenizer


def _load_tokenizer(model_dir):
    """The `tokenizers` library's tokenizer from tokenizer.json, if the folder has one."""
    import os

    path = os.path.join(str(model_dir), "tokenizer.json")
    if not os.path.isfile(path):
        return None
    from tokenizers import Tokenizer

    return Tokenizer.from_file(path)


def _chat_template(model_dir) -> str | None:
    import json
    import os

    path = os.path.join(str(model_dir), "tokenizer_config.json")
    if not os.path.isfile(path):
        return None
    with open(path) as f:
        return json.load(f).get("chat_template")


def apply_chat_template(model_dir, messages: list[dict]) -> str:
    """Render messages with the folder's own chat template (tokenizer_config.json)."""
    template = _chat_template(model_dir)
    if template is None:
        raise ValueError(f"{model_dir!r} has no chat template; pass chat=False or token ids")
    try:
        import jinja2
    except ImportError:
        raise ValueError("rendering a chat template needs jinja2; pass chat=False or token ids") from None
    env = jinja2.Environment(trim_blocks=True, lstrip_blocks=True)
    return env.from_string(template).render(messages=messages, add_generation_prompt=True)


def _encode(tokenizer, model_dir, prompt: str, chat: bool) -> list[int]:
    if tokenizer is None:
        raise ValueError(
            f"{model_dir!r} has no tokenizer.json: text prompts need one; pass token ids instead"
        )
    if chat:
        prompt = apply_chat_template(model_dir, [{"role": "user", "content": prompt}])
    return list(tokenizer.encode(prompt, add_special_tokens=False).ids)
