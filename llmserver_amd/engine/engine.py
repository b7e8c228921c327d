"""The engine: requests come in, steps run, tokens come out.

Its options, the names of what a caller uses (``add_request``, ``step``, ``run``, ``cancel_request``,
``active_requests``, ``completed_requests``, ``step_profile``) and what they do follow the reference's ``Engine``
(utils/engine.py:46-475 there): a bounded history of finished requests (230-248), stop rules (299-314), recompute
preemption when pages run out (412-435), complete pages of prompts shared between requests (193-208, 383-401),
a loop that yields to other tasks between steps (445-475).  What differs is the shape of a step: the reference runs
a decode pass and then padded prefill passes; here the scheduler's plan becomes one flat batch through
:class:`~llmserver_amd.engine.step.ModelRunner`.

A step goes through these hands: :meth:`Engine.schedule_step` (offer cached prefixes to the requests that may be
admitted, plan, make room if the plan is short of pages, commit) and :meth:`Engine.run_scheduled` (entries, the
model's step, sampling, the host's share of the next step while the GPU works, then every request moves on).
Requests that wait hold nothing between steps: neither pages nor a state slot.
"""
from __future__ import annotations

import asyncio
import dataclasses
import json
import os
import time
import uuid
from collections import OrderedDict
from datetime import datetime, timedelta
from typing import Dict, List, Optional

from ..cache import CacheExhaustedError, CacheManager
from ..sampling import Sampler, request_uniform
from .batch import StepEntry
from .request import CompletedRequest, Request, RequestFinishReason, RequestStatus, SamplingParams
from .scheduler import Scheduler, StepPlan
from .step import ModelRunner, padded_rows
from .stream import STREAM_END, ByteLevelText, ByteLevelVocabulary, TokenStream


@dataclasses.dataclass
class EngineConfig:
    """The engine's options, typed and checked in one place.  The names are the reference's where it has the option
    (utils/engine.py:47 there); ``temperature``, ``seed``, ``enable_prefix_caching`` and ``launch_ahead`` are this
    engine's own."""
    max_new_tokens: int = 128
    max_batch_size: int = 8
    max_num_batched_tokens: int = 2048
    max_completed_requests: int = 1000
    completed_request_ttl_seconds: float = 3600
    prefill_chunk_size: Optional[int] = None
    kv_cache_num_blocks: int = 500
    kv_cache_block_size: int = 500
    stream_text: bool = True
    ignore_eos: bool = False
    temperature: float = 0.0
    seed: int = 0
    enable_prefix_caching: bool = True
    launch_ahead: bool = True         # decoding steps may start before the host has seen the tokens they bring

    def validate(self) -> "EngineConfig":
        for name in ("max_new_tokens", "max_num_batched_tokens", "kv_cache_num_blocks", "kv_cache_block_size"):
            if getattr(self, name) <= 0:
                raise ValueError(f"{name} must be positive, got {getattr(self, name)}")
        for name in ("max_completed_requests", "completed_request_ttl_seconds", "temperature"):
            if getattr(self, name) < 0:
                raise ValueError(f"{name} cannot be negative, got {getattr(self, name)}")
        return self


class CompletedHistory:
    """Finished and cancelled requests, oldest first, kept up to a number and an age."""

    def __init__(self, most: int, ttl_seconds: float):
        self.most, self.ttl = most, timedelta(seconds=ttl_seconds)
        self.records: "OrderedDict[str, CompletedRequest]" = OrderedDict()

    def prune(self, now: Optional[datetime] = None) -> None:
        deadline = (now or datetime.now()) - self.ttl
        expired = 0
        for record in self.records.values():          # in the order they finished: stop at the first that is young enough
            if record.finished_at > deadline:
                break
            expired += 1
        for _ in range(max(expired, len(self.records) - self.most)):
            self.records.popitem(last=False)

    def add(self, request: Request) -> None:
        if self.most == 0:
            return
        self.records.pop(request.request_id, None)
        self.records[request.request_id] = CompletedRequest.from_request(request)
        self.prune()


def _generation_config(model) -> dict:
    folder = getattr(model, "name", None)
    path = os.path.join(folder, "generation_config.json") if isinstance(folder, str) else None
    if path and os.path.isfile(path):
        with open(path) as handle:
            return json.load(handle)
    return {}


class Engine:
    def __init__(self, model, tokenizer=None, config: Optional[EngineConfig] = None, *, ops=None, **options):
        if config is not None and options:
            raise TypeError("pass an EngineConfig or keyword options, not both")
        self.config = (config or EngineConfig(**options)).validate()
        config = self.config
        self.model, self.tokenizer = model, tokenizer
        self.device, self.dtype = model.device, model.dtype
        self.max_new_tokens, self.max_num_batched_tokens = config.max_new_tokens, config.max_num_batched_tokens
        self.stream_text, self.ignore_eos = config.stream_text, config.ignore_eos
        self.temperature, self.seed = float(config.temperature), int(config.seed)
        self.launch_ahead = bool(config.launch_ahead)
        self.num_blocks, self.block_size = config.kv_cache_num_blocks, config.kv_cache_block_size
        self.scheduler = Scheduler(config.max_batch_size, config.max_num_batched_tokens, config.prefill_chunk_size)
        self.history = CompletedHistory(config.max_completed_requests, config.completed_request_ttl_seconds)
        self.active_requests: Dict[str, Request] = {}
        self.step_profile = {"steps": 0, "decode_steps": 0, "prefill_steps": 0, "schedule_s": 0.0, "step_s": 0.0,
                             "yield_s": 0.0, "tokens": 0, "prefix_hit_tokens": 0, "preemptions": 0,
                             "decode_by_rows": {}}       # decoding rows of a step -> [steps, seconds] (utils/engine.py:69, 468-471)
        ops = ops if ops is not None else self._default_ops()
        # what the kernels cannot take is refused here, not at the first step
        ops.check_cache_geometry(model.cache_specs(), config.kv_cache_block_size, config.kv_cache_num_blocks)
        self._warn_of_slow_page_size(ops, model, config.kv_cache_block_size)
        self.kv_cache = CacheManager(model.cache_specs(), config.kv_cache_block_size, config.kv_cache_num_blocks,
                                     num_state_slots=config.max_batch_size, device=self.device, dtype=self.dtype,
                                     model_identity=str(getattr(model, "name", "model")))
        self.enable_prefix_caching = config.enable_prefix_caching and self.kv_cache.prefix_caching_possible
        self.runner = ModelRunner(model, self.kv_cache, ops)
        self.sampler = Sampler(self.runner.ops, self.device)
        self._requests_added = 0
        self._text: Dict[str, ByteLevelText] = {}
        self._byte_level = ByteLevelVocabulary.of(tokenizer) if tokenizer is not None and config.stream_text else None
        self._read_special_tokens()

    @staticmethod
    def _default_ops():
        from ..kernels import default_ops
        return default_ops()

    def _read_special_tokens(self) -> None:
        """bos, pad and the set of end-of-sequence ids: the generation configuration first, then the model's
        configuration, then the tokenizer (utils/engine.py:88-117 in the reference)."""
        sources = (_generation_config(self.model), self.model.config, self.tokenizer)

        def first(name):
            for source in sources:
                value = source.get(name) if isinstance(source, dict) else getattr(source, name, None)
                if value is not None:
                    return value
            return None

        self.bos_token_id, self.pad_token_id = first("bos_token_id"), first("pad_token_id")
        eos = first("eos_token_id")
        self.eos_token_ids = set() if eos is None else {eos} if isinstance(eos, int) else set(eos)

    @property
    def completed_requests(self) -> "OrderedDict[str, CompletedRequest]":
        return self.history.records

    def prune_completed_requests(self, now=None) -> None:
        self.history.prune(now)

    # -- requests come in ----------------------------------------------------------------------
    def _encode(self, prompt: str) -> List[int]:
        if self.tokenizer is None:
            raise ValueError("a text prompt needs a tokenizer; pass prompt_token_ids instead")
        encoded = self.tokenizer(prompt) if callable(self.tokenizer) else self.tokenizer.encode(prompt)
        if isinstance(encoded, dict) or hasattr(encoded, "keys"):
            return list(encoded["input_ids"])
        return list(getattr(encoded, "ids", encoded))

    def _prompt_ids(self, prompt, prompt_token_ids) -> List[int]:
        if prompt_token_ids is not None:
            ids = [int(token) for token in prompt_token_ids]
            if not ids:
                raise ValueError("prompt_token_ids must not be empty")
        elif prompt is None or not prompt.strip():      # nothing to say: the sequence starts with the bos token alone
            if self.bos_token_id is None:
                raise ValueError("an empty prompt needs a bos_token_id, and the model folder gives none")
            ids = [self.bos_token_id]
        else:
            ids = self._encode(prompt)
        outside = [token for token in ids if not 0 <= token < self.runner.vocab]
        if outside:
            raise ValueError(f"token id {outside[0]} is outside the vocabulary of {self.runner.vocab}")
        return ids

    def add_request(self, prompt=None, prompt_token_ids=None, max_new_tokens=None, temperature=None, seed=None) -> Request:
        """Queue a request; returns it (tokens appear in ``generated_token_ids`` and on ``output_queue``)."""
        self.history.prune()
        ids = self._prompt_ids(prompt, prompt_token_ids)
        sampling = SamplingParams(self.temperature if temperature is None else float(temperature),
                                  self.seed + self._requests_added if seed is None else int(seed))
        self._requests_added += 1
        request = Request(f"req-{uuid.uuid4()}", prompt, ids, max_new_tokens or self.max_new_tokens, TokenStream(), sampling)
        self.active_requests[request.request_id] = request
        if self._byte_level is not None:
            self._text[request.request_id] = ByteLevelText(self._byte_level)
        self.scheduler.waiting.append(request)
        return request

    # -- requests go out -----------------------------------------------------------------------
    def _release(self, request: Request) -> None:
        if self.kv_cache.has(request.request_id):
            self.kv_cache.close(request.request_id)

    def _retire(self, request: Request) -> None:
        """The request is over (finished or cancelled): close its stream, free what it holds, keep a record."""
        text = self._text.pop(request.request_id, None)
        if text is not None and request.status == RequestStatus.FINISHED:
            self._emit_text(request, text.finish())
        request.output_queue.put_nowait(STREAM_END)
        self._release(request)
        self.active_requests.pop(request.request_id, None)
        self.history.add(request)

    def cancel_request(self, request_id) -> bool:
        """Take a live request out, wherever it is; False if there is no such live request."""
        self.history.prune()
        request = self.active_requests.get(request_id)
        if request is None or not request.is_alive:
            return False
        for queue in (self.scheduler.waiting, self.scheduler.running):
            if request in queue:
                queue.remove(request)
        request.cancel()
        request.output_queue.drain()             # what nobody has read yet is dropped; the end marker follows
        self._retire(request)
        return True

    def _emit_text(self, request: Request, piece: str) -> None:
        if piece:
            request.output_queue.put_nowait(piece)
            request.emitted_text += piece

    def _emit(self, request: Request, token_id: int) -> None:
        """Put the new token on the request's stream: as text if there is a tokenizer, as its id otherwise."""
        text = self._text.get(request.request_id)
        if text is not None:                              # byte-level vocabulary: one token at a time
            self._emit_text(request, text.push(token_id))
        elif self.tokenizer is not None and hasattr(self.tokenizer, "decode"):
            # any other tokenizer: decode everything and emit what is new, holding back a character still split across tokens
            whole = self.tokenizer.decode(request.generated_token_ids, skip_special_tokens=True).rstrip("�")
            self._emit_text(request, whole[len(request.emitted_text):])
        else:
            request.output_queue.put_nowait(token_id)

    def _take_token(self, request: Request, token_id: int) -> None:
        request.accept(token_id)
        if self.stream_text:
            self._emit(request, token_id)
        if token_id in self.eos_token_ids and not self.ignore_eos:
            request.finish(RequestFinishReason.EOS)
        elif len(request.generated_token_ids) >= request.max_new_tokens:
            request.finish(RequestFinishReason.LENGTH)
        if not request.is_alive:
            self._retire(request)

    # -- scheduling ----------------------------------------------------------------------------
    def _offer_prefixes(self) -> None:
        """The requests that the next plan may admit look up cached pages of their prompts.  Done here and not when a
        request arrives: requests that arrived together find what the first of them has computed meanwhile, a
        request that comes back after a preemption finds its own prompt again, and nobody holds pages while waiting."""
        if not self.enable_prefix_caching:
            return
        places = self.scheduler.places(self.kv_cache)
        for request, _ in zip(self.scheduler.waiting, range(places)):
            if request.prefix_digests is None:
                request.prefix_digests = self.kv_cache.prefix_digests(request.prompt_token_ids)
            if not request.prefix_digests or request.num_computed_tokens >= len(request.prefix_digests) * self.block_size:
                continue
            if not self.kv_cache.has(request.request_id):
                self.kv_cache.open(request.request_id, state=False)
            covered = self.kv_cache.share_prefix(request.request_id, request.prompt_token_ids, request.prefix_digests)
            if covered:
                request.reuse(covered)

    def _withdraw_offers(self) -> int:
        """Requests that still wait give back the cached pages they were offered (a held page cannot be recycled).
        The pages stay cached for as long as nobody needs the room.  Returns how many pages were let go."""
        let_go = 0
        for request in self.scheduler.waiting:
            if self.kv_cache.has(request.request_id):
                let_go += sum(len(table) for table in self.kv_cache.record(request.request_id).tables)
                self.kv_cache.close(request.request_id)
                request.forget_reused()
        return let_go

    def _choose_victim(self) -> Request:
        """Who gives its cache up when the running requests need more pages than there are: among those that hold
        anything, the one preempted least often, then the one that waited least, then the one admitted last
        (utils/engine.py:430-434 in the reference; its tests/test_engine.py:525-545 hold the cases)."""
        running = self.scheduler.running
        holders = [request for request in running if self.kv_cache.holds_anything(request.request_id)]
        if len(running) <= 1 or not holders:
            raise CacheExhaustedError("the running request needs more pages than the cache has, and nobody else can give any up")
        order = {id(request): position for position, request in enumerate(running)}
        return min(holders, key=lambda request: (request.preemption_count, request.waiting_steps, -order[id(request)]))

    def _preempt(self, request: Request) -> None:
        """Recompute preemption: everything the request holds goes back (pages and state slot), the request goes to
        the end of the waiting queue and will be computed again from its first token."""
        self._release(request)
        self.scheduler.running.remove(request)
        request.preempt()
        self.scheduler.waiting.append(request)
        self.step_profile["preemptions"] += 1

    def schedule_step(self) -> StepPlan:
        offers = True
        while True:
            if offers:
                self._offer_prefixes()
            plan = self.scheduler.plan(self.kv_cache)
            if plan.fits:
                break
            if offers and self._withdraw_offers():
                offers = False          # first the pages that waiting requests were offered, then a running request
                continue
            offers = False
            self._preempt(self._choose_victim())
        for request in self.scheduler.commit(plan):
            if not self.kv_cache.has(request.request_id):
                self.kv_cache.open(request.request_id, state=False)
            self.kv_cache.acquire_state(request.request_id)
            self.step_profile["prefix_hit_tokens"] += request.num_computed_tokens
        self._withdraw_offers()         # offered but not admitted: nothing is held over a step
        return plan

    def _warn_of_slow_page_size(self, ops, model, page_size: int) -> None:
        """Say so once if these pages keep prompt portions out of the kernel that shares a workgroup's keys between its
        tiles (the step's plan then gives every tile a wavefront of its own, which reads its keys itself: correct,
        and about half as fast on long prompts)."""
        import warnings
        for head_dim in sorted({spec.head_dim for spec in model.cache_specs().values() if hasattr(spec, "head_dim")}):
            if ops.attention_workgroup_tiles(self.dtype, head_dim) and not ops.attention_workgroup_tiles(self.dtype, head_dim, page_size):
                warnings.warn(f"kv_cache_block_size={page_size}: the attention kernel for prompt portions takes pages of a multiple of 8 keys "
                              f"in {str(self.dtype).split('.')[-1]}; with this page size prompts run through the slower per-tile kernel "
                              "(a multiple of 16, such as 496 or 512, keeps them on the fast one)", stacklevel=3)
                return

    # -- one step ------------------------------------------------------------------------------
    def warmup_graphs(self, batch_sizes=None, max_context=None) -> int:
        """Capture the decode graphs of these numbers of rows (default: every size that decoding steps of up to
        ``max_batch_size`` rows are filled up to) before serving, so that the first steps of those sizes do not pay for
        it; an idle engine only.  Returns how many graphs are held afterwards (utils/engine.py:150-161 in the
        reference).  The graphs serve contexts up to the first width of the block table, or, with ``max_context``,
        every width up to that context (the pool has to hold that many tokens for every row meanwhile; sizes it
        cannot hold are left to be captured when they are met)."""
        from .step import TABLE_WIDTH_STEP
        if not self.runner.use_graphs or self.active_requests:
            return 0
        most = self.scheduler.max_batch_size
        if batch_sizes is None:
            batch_sizes = sorted({min(most, padded_rows(rows)) for rows in range(1, most + 1)})
        tokens_per_width = TABLE_WIDTH_STEP * self.block_size
        # one token, the first context beyond each edge at which a mixer's captured work changes its shape, then every width of the table
        edges = sorted({edge + 1 for block in self.runner.model.blocks for edge in block.mixer.graph_shape_edges()})
        contexts = [1] + edges + [width * tokens_per_width + 1 for width in range(1, -(-(max_context or 1) // tokens_per_width))]
        try:
            for context in contexts:
                pages_per_row = -(-context // self.block_size)
                for rows in batch_sizes:
                    if not 0 < rows <= most or rows * pages_per_row > min(self.kv_cache.available_pages()):
                        continue
                    names = [f"warmup-{i}" for i in range(rows)]
                    try:
                        for name in names:
                            self.kv_cache.open(name)
                            self.kv_cache.ensure(name, context)       # pages of zeros stand for a context of this length
                            self.kv_cache.advance(name, context - 1)
                        self.runner.step([StepEntry(name, [0], [0]) for name in names])  # one token each: the captured kind of step
                    finally:
                        for name in names:
                            if name in self.kv_cache.requests:
                                self.kv_cache.close(name)
        except Exception as error:               # as the reference: serving goes on, graphs are captured on first use
            import warnings
            warnings.warn(f"graph warm-up failed ({error!r}); graphs will be captured on first use")
            self.runner.drop_graphs()
            return 0
        return self.runner.graph_count()

    def calibrate(self, save_to: Optional[str] = None, portions=(24, 32, 48, 64, 96, 128, 192, 256, 384, 512, 640, 768, 896, 1024)) -> int:
        """Measure, for this model's shapes, which products go through a hand-written kernel and which through the
        library, for every number of decoding rows up to ``max_batch_size`` and for prompt portions of the given sizes;
        an idle engine only, never part of serving.  The findings join the kernel namespace's table of choices (and the
        file ``save_to``, if given, which ``LLMSERVER_AMD_CHOICES`` can name in later runs).  Returns how many shapes
        were measured.  Graphs captured before are dropped: they may hold the other choice."""
        if self.active_requests:
            return 0
        measuring = self.runner.ops.measuring
        most = self.scheduler.max_batch_size
        sizes = [(rows, 1) for rows in range(1, most + 1)]
        sizes += [(1, tokens) for tokens in portions if tokens <= self.max_num_batched_tokens]
        graphs, self.runner.use_graphs = self.runner.use_graphs, False
        try:
            with measuring() as choices:
                if choices is None:                  # a kernel namespace that keeps no table of choices
                    return 0
                before = len(choices.measured)
                for rows, tokens in sizes:
                    if rows * -(-tokens // self.block_size) > min(self.kv_cache.available_pages() or [1 << 30]):
                        continue
                    names = [f"calibrate-{i}" for i in range(rows)]
                    try:
                        for name in names:
                            self.kv_cache.open(name)
                        self.runner.step([StepEntry(name, [0] * tokens, [tokens - 1]) for name in names])
                    finally:
                        for name in names:
                            if name in self.kv_cache.requests:
                                self.kv_cache.close(name)
                measured = len(choices.measured) - before
                if save_to:
                    choices.save(save_to)
        finally:
            self.runner.use_graphs = graphs
            self.runner.drop_graphs()
        return measured

    def prepare_next_step(self, sampled, pending=None) -> bool:
        """If the next step can only be a decoding step of known requests (nobody can join, nobody is still behind
        its sequence), let the runner lay it out before this step's tokens are back; and if it brings exactly the
        requests that were sampled just now, in their order, start it at once with the tokens ``pending`` that are still
        on the device, so that the GPU does not wait for the host between the steps.  A request that stops at this step
        for a reason the host cannot foresee (an end-of-sequence token, a cancellation) makes the next step another one
        than the one prepared or started, which is then dropped and run again without that request."""
        following, someone_leaves = [], False
        for request in self.scheduler.running:
            if request.status != RequestStatus.DECODING:
                return False                     # still behind its sequence: the next step brings a portion of it
            if len(request.generated_token_ids) + 1 < request.max_new_tokens:
                following.append(request)
            else:
                someone_leaves = True
        # Requests that wait can only join when a place is free: with every place taken and nobody about to leave,
        # the next step is a decoding step of the same requests all the same.
        if self.scheduler.waiting and (someone_leaves or self.scheduler.places(self.kv_cache) > 0):
            return False
        if not following or not self.runner.prepare_ahead([request.request_id for request in following]):
            return False
        if self.launch_ahead and pending is not None and len(following) == len(sampled) \
                and all(a is b for a, b in zip(following, sampled)):
            self.runner.launch_ahead(pending.device)
        return True

    def run_scheduled(self, plan: StepPlan) -> None:
        """Turn the plan into one flat batch, run it, sample, and move every request on."""
        work = [(request, 1) for request in plan.decodes]
        work += [(request, count) for request, count in plan.portions if request.status == RequestStatus.PREFILL]
        if not work:
            return
        entries, sampled = [], []
        for request, count in work:
            reaches_end = count == request.tokens_ahead       # then the last of these tokens gives the next token's logits
            entries.append(StepEntry(request.request_id, request.next_tokens(count), [count - 1] if reaches_end else []))
            if reaches_end:
                sampled.append(request)
        logits = self.runner.step(entries)
        computed_before = [request.num_computed_tokens for request, _ in work]
        for request, count in work:
            request.computed(count)
        token_ids: List[int] = []
        if sampled:
            temperatures = [request.sampling.temperature for request in sampled]
            uniforms = [request_uniform(request.sampling.seed, request.num_samples_drawn) if request.sampling.temperature > 0 else 0.0
                        for request in sampled]
            pending = self.sampler.launch(logits, temperatures, uniforms)
            self.prepare_next_step(sampled, pending)      # the host's share of the next step, while the GPU works on this one
            token_ids = pending.tolist()
        self.step_profile["tokens"] += sum(count for _, count in work)
        if self.enable_prefix_caching:
            for (request, _), before in zip(work, computed_before):
                if before < len(request.prompt_token_ids):
                    self.kv_cache.register_prefix(request.request_id, request.prompt_token_ids, before, request.num_computed_tokens)
        for request, token_id in zip(sampled, token_ids):
            request.num_samples_drawn += 1
            self._take_token(request, token_id)
        self.scheduler.running[:] = [request for request in self.scheduler.running if request.is_alive]

    def _timed_step(self):
        clock, profile = time.perf_counter, self.step_profile
        t0 = clock()
        plan = self.schedule_step()
        t1 = clock()
        self.run_scheduled(plan)
        t2 = clock()
        profile["steps"] += 1
        profile["schedule_s"] += t1 - t0
        profile["step_s"] += t2 - t1
        profile["prefill_steps"] += bool(plan.portions)
        if plan.decodes:
            profile["decode_steps"] += 1
            if not plan.portions:                      # a pure decoding step: its time belongs to its number of rows
                bucket = profile["decode_by_rows"].setdefault(len(plan.decodes), [0, 0.0])
                bucket[0] += 1
                bucket[1] += t2 - t1
        return t2

    def has_work(self) -> bool:
        return bool(self.scheduler.waiting or self.scheduler.running)

    def step(self) -> bool:
        """One step; True while requests are left (utils/engine.py:437-443 in the reference)."""
        self._timed_step()
        return self.has_work()

    async def run(self) -> None:
        """Step until nothing is left, letting other tasks (readers of the streams) run between steps."""
        while self.has_work():
            done = self._timed_step()
            await asyncio.sleep(0)
            self.step_profile["yield_s"] += time.perf_counter() - done

    def generate(self, prompts_token_ids, max_new_tokens=None, temperature=None, seed=None) -> List[List[int]]:
        """Add the prompts, run to the end, return the generated token ids in the prompts' order."""
        requests = [self.add_request(None, prompt_token_ids=ids, max_new_tokens=max_new_tokens, temperature=temperature,
                                     seed=None if seed is None else seed + i) for i, ids in enumerate(prompts_token_ids)]
        while self.step():
            pass
        return [list(request.generated_token_ids) for request in requests]
