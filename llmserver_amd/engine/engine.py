"""The engine loop: admission, scheduling, one mixed step, sampling, streaming, finishing.

Constructor options, method names and behaviour follow the reference's ``Engine``
(/root/reference/utils/engine.py:46-475): ``add_request`` (210-228), ``step`` (437-443),
``run`` (445-475), ``cancel_request`` (260-277), stop rules (299-314), recompute preemption when
pages run out (412-435), complete-page prefix caching (193-208, 383-401), bounded history of
completed requests (230-248).  The difference is the shape of a step: the reference runs a decode
pass and then padded prefill passes; here the scheduler's plan becomes one flat batch through
:class:`~llmserver_amd.engine.step.ModelRunner`.
"""
from __future__ import annotations

import asyncio
import json
import math
import os
import time
import uuid
from collections import OrderedDict
from datetime import datetime, timedelta
from typing import List, Optional

import torch

from ..cache import CacheExhaustedError, CacheManager
from ..sampling import Sampler, request_uniform
from .batch import StepEntry
from .request import (STREAM_END, CompletedRequest, Request, RequestFinishReason, RequestStatus, SamplingParams,
                      TokenStream)
from .scheduler import Scheduler
from .step import ModelRunner, padded_rows


def _read_generation_config(model) -> dict:
    folder = getattr(model, "name", None)
    if isinstance(folder, str):
        path = os.path.join(folder, "generation_config.json")
        if os.path.isfile(path):
            with open(path) as handle:
                return json.load(handle)
    return {}


class Engine:
    def __init__(self, model, tokenizer=None, max_new_tokens=128, max_batch_size=8, max_num_batched_tokens=2048,
                 max_completed_requests=1000, completed_request_ttl_seconds=3600, prefill_chunk_size=None,
                 kv_cache_num_blocks=500, kv_cache_block_size=500, stream_text=True, ignore_eos=False,
                 temperature=0.0, seed=0, enable_prefix_caching=True, ops=None, launch_ahead=True):
        if max_new_tokens <= 0:
            raise ValueError(f"max_new_tokens is <= 0: {max_new_tokens}")
        if max_num_batched_tokens <= 0:
            raise ValueError(f"max_num_batched_tokens is <= 0: {max_num_batched_tokens}")
        if max_completed_requests < 0:
            raise ValueError(f"max_completed_requests cannot be negative: {max_completed_requests}")
        if completed_request_ttl_seconds < 0:
            raise ValueError(f"completed_request_ttl_seconds cannot be negative: {completed_request_ttl_seconds}")
        if temperature < 0:
            raise ValueError(f"temperature cannot be negative: {temperature}")
        self.model, self.tokenizer = model, tokenizer
        self.device, self.dtype = model.device, model.dtype
        self.max_new_tokens = max_new_tokens
        self.stream_text = stream_text
        self.ignore_eos = ignore_eos
        self.temperature, self.seed = float(temperature), int(seed)
        self.launch_ahead = bool(launch_ahead)      # decoding steps may start before the host has seen the tokens they bring
        self.max_num_batched_tokens = max_num_batched_tokens
        self.max_completed_requests = max_completed_requests
        self.completed_request_ttl = timedelta(seconds=completed_request_ttl_seconds)
        self.scheduler = Scheduler(max_batch_size, max_num_batched_tokens, prefill_chunk_size)
        self.step_profile = {"steps": 0, "decode_steps": 0, "prefill_steps": 0, "schedule_s": 0.0, "step_s": 0.0,
                             "yield_s": 0.0, "tokens": 0, "prefix_hit_tokens": 0, "preemptions": 0}
        self.active_requests = {}
        self.completed_requests = OrderedDict()
        self.num_blocks, self.block_size = kv_cache_num_blocks, kv_cache_block_size
        self.kv_cache = CacheManager(model.cache_specs(), kv_cache_block_size, kv_cache_num_blocks,
                                     num_state_slots=max_batch_size, device=self.device, dtype=self.dtype,
                                     model_identity=str(getattr(model, "name", "model")))
        self.enable_prefix_caching = enable_prefix_caching and self.kv_cache.prefix_caching_possible
        self.runner = ModelRunner(model, self.kv_cache, ops)
        self.sampler = Sampler(self.runner.ops, self.device)
        self._requests_added = 0
        generation = _read_generation_config(model)
        config = model.config

        def token_id(name):
            for source in (generation.get(name), getattr(config, name, None), getattr(tokenizer, name, None)):
                if source is not None:
                    return source
            return None

        self.bos_token_id = token_id("bos_token_id")
        self.pad_token_id = token_id("pad_token_id")
        eos = token_id("eos_token_id")
        self.eos_token_ids = set() if eos is None else ({eos} if isinstance(eos, int) else set(eos))

    # -- admission ---------------------------------------------------------------------------
    def _tokenize(self, prompt: str) -> List[int]:
        if self.tokenizer is None:
            raise ValueError("a text prompt needs a tokenizer; pass prompt_token_ids instead")
        encoded = self.tokenizer(prompt) if callable(self.tokenizer) else self.tokenizer.encode(prompt)
        if isinstance(encoded, dict) or hasattr(encoded, "keys"):
            return list(encoded["input_ids"])
        return list(getattr(encoded, "ids", encoded))

    def add_request(self, prompt=None, prompt_token_ids=None, max_new_tokens=None, temperature=None, seed=None) -> Request:
        self.prune_completed_requests()
        if prompt_token_ids is not None:
            prompt_token_ids = list(prompt_token_ids)
            if not prompt_token_ids:
                raise ValueError("prompt_token_ids must not be empty")
        elif not prompt or prompt.strip() == "":
            if self.bos_token_id is None:
                raise ValueError("an empty prompt needs a bos_token_id, and the model folder gives none")
            prompt_token_ids = [self.bos_token_id]
        else:
            prompt_token_ids = self._tokenize(prompt)
        for token in prompt_token_ids:
            if not 0 <= token < self.runner.vocab:
                raise ValueError(f"token id {token} is outside the vocabulary of {self.runner.vocab}")
        sampling = SamplingParams(self.temperature if temperature is None else float(temperature),
                                  self.seed + self._requests_added if seed is None else int(seed))
        self._requests_added += 1
        request = Request(f"req-{uuid.uuid4()}", prompt, prompt_token_ids, max_new_tokens or self.max_new_tokens,
                          TokenStream(), sampling)
        self.active_requests[request.request_id] = request
        self._open_cache(request)
        self.scheduler.waiting.append(request)
        return request

    def _open_cache(self, request: Request, share: bool = True) -> None:
        """Give the request its block tables and state slot and attach cached prefix pages
        (/root/reference/utils/engine.py:197-208)."""
        record = self.kv_cache.open(request.request_id)
        request.block_table = record.tables[0] if record.tables else []
        if share:
            self._share_prefix(request)

    def release_waiting_prefixes(self) -> int:
        """Take back the cached prefix pages that waiting requests hold (they have computed nothing themselves).  A
        page that a waiting request holds cannot be evicted, and enough of them leave the running requests without
        room to grow; given back, the pages stay cached for as long as nobody needs the room, and a request looks
        its prefix up again when it is up for admission.  Returns the number of pages let go."""
        let_go = 0
        for request in self.scheduler.waiting:
            if request.block_table and self.kv_cache.has(request.request_id):
                let_go += len(request.block_table)
                self.step_profile["prefix_hit_tokens"] -= request.num_computed_tokens
                self.kv_cache.close(request.request_id)
                request.num_computed_tokens = 0
                self._open_cache(request, share=False)
        return let_go

    def _share_prefix(self, request: Request) -> None:
        """Attach cached pages of the prompt's prefix.  Done when the request arrives, as in the
        reference, and again each time it is up for admission, because requests that arrived
        together may by then find what an earlier one of them has computed."""
        if not self.enable_prefix_caching:
            return
        if request.prefix_digests is None:
            request.prefix_digests = self.kv_cache.prefix_digests(request.prompt_token_ids)
        covered = self.kv_cache.share_prefix(request.request_id, request.prompt_token_ids, request.prefix_digests)
        request.num_computed_tokens += covered
        self.step_profile["prefix_hit_tokens"] += covered

    # -- history -----------------------------------------------------------------------------
    def prune_completed_requests(self, now=None):
        now = now or datetime.now()
        while self.completed_requests:
            oldest = next(iter(self.completed_requests.values()))
            if now - oldest.finished_at < self.completed_request_ttl:
                break
            self.completed_requests.popitem(last=False)
        while len(self.completed_requests) > self.max_completed_requests:
            self.completed_requests.popitem(last=False)

    def archive_request(self, request):
        self.active_requests.pop(request.request_id, None)
        if self.max_completed_requests == 0:
            return
        self.completed_requests[request.request_id] = CompletedRequest.from_request(request)
        self.completed_requests.move_to_end(request.request_id)
        self.prune_completed_requests()

    def release_request_resources(self, request):
        if self.kv_cache.has(request.request_id):
            self.kv_cache.close(request.request_id)
        request.block_table = []

    def cancel_request(self, request_id) -> bool:
        self.prune_completed_requests()
        request = self.active_requests.get(request_id)
        if request is None or request.status in (RequestStatus.FINISHED, RequestStatus.CANCELLED):
            return False
        if request in self.scheduler.waiting:
            self.scheduler.waiting.remove(request)
        if request in self.scheduler.running:
            self.scheduler.running.remove(request)
        request.cancel()
        request.output_queue.drain()
        request.output_queue.put_nowait(STREAM_END)
        self.release_request_resources(request)
        self.archive_request(request)
        return True

    # -- output ------------------------------------------------------------------------------
    def check_stopping(self, request, token_id):
        if token_id in self.eos_token_ids and not self.ignore_eos:
            request.finish(RequestFinishReason.EOS)
        elif len(request.generated_token_ids) >= request.max_new_tokens:
            request.finish(RequestFinishReason.LENGTH)
        else:
            return
        request.output_queue.put_nowait(STREAM_END)
        self.release_request_resources(request)
        self.archive_request(request)

    def stream_output(self, request):
        if self.tokenizer is None or not hasattr(self.tokenizer, "decode"):
            request.output_queue.put_nowait(request.generated_token_ids[-1])
            return
        text = self.tokenizer.decode(request.generated_token_ids, skip_special_tokens=True)
        while text.endswith("�"):        # a character still split across tokens: hold it back
            text = text[:-1]
        new_text = text[len(request.emitted_text):]
        if new_text:
            request.output_queue.put_nowait(new_text)
            request.emitted_text = text

    def accept_generated_token(self, request, token_id):
        request.append_generated_token(token_id)
        if self.stream_text:
            self.stream_output(request)
        self.check_stopping(request, token_id)

    # -- scheduling --------------------------------------------------------------------------
    def remove_finished_and_cancelled_requests(self):
        self.scheduler.running[:] = [r for r in self.scheduler.running if r.status not in (RequestStatus.FINISHED, RequestStatus.CANCELLED)]

    def preempt_request(self, request):
        """Recompute preemption: give everything back, go to the back of the waiting queue
        (/root/reference/utils/engine.py:412-416)."""
        self.release_request_resources(request)
        self.scheduler.running.remove(request)
        request.preempt_for_compute()
        self.scheduler.waiting.append(request)
        self.step_profile["preemptions"] += 1

    def available_blocks(self) -> int:
        return min(self.kv_cache.available_pages()) if self.kv_cache.groups else 1 << 30

    def schedule_step(self):
        share = True
        while True:
            # A preempted request gets a fresh table back; the requests that a free place may admit now also look
            # their prefix up (again): what arrived together with them may have computed it meanwhile.
            places = self.scheduler.max_batch_size - len(self.scheduler.running)
            for index, request in enumerate(self.scheduler.waiting):
                admissible = share and index < places
                if not self.kv_cache.has(request.request_id):
                    self._open_cache(request, share=admissible)
                elif admissible and request.num_computed_tokens < len(request.prefix_digests or ()) * self.block_size:
                    self._share_prefix(request)
            available = self.available_blocks()
            out = self.scheduler.plan(available, self.block_size)
            needed = sum(max(0, math.ceil((r.num_computed_tokens + n) / self.block_size) - len(r.block_table))
                         for r, n in zip(out.prefill_requests, out.prefill_token_counts))
            needed += sum(max(0, math.ceil((r.num_computed_tokens + 1) / self.block_size) - len(r.block_table))
                          for r in out.decode_requests)
            if needed <= available:
                self.scheduler.commit(out)
                return out
            if share and self.release_waiting_prefixes():
                share = False             # pages that waiting requests held come first; then running requests are preempted
                continue
            if len(self.scheduler.running) == 1:
                raise CacheExhaustedError(f"Required blocks {needed} in KV cache exceeds currently free blocks")
            candidates = [r for r in reversed(self.scheduler.running) if r.block_table]
            if not candidates:
                raise CacheExhaustedError(f"Required blocks {needed} in KV cache exceeds currently free blocks")
            victim = sorted(candidates, key=lambda r: (r.preemption_count, r.waiting_steps))[0]
            self.preempt_request(victim)

    # -- one step ----------------------------------------------------------------------------
    def warmup_graphs(self, batch_sizes=None, max_context=None) -> int:
        """Capture the decode graphs of these numbers of rows (default: every size that decoding steps of up to
        ``max_batch_size`` rows are filled up to) before serving, so that the first steps of those sizes do not pay for
        it, nor for the measurements by which kernels are chosen; an idle engine only.  Returns how many graphs are held
        afterwards (/root/reference/utils/engine.py:150-161).  The graphs serve contexts up to the first width of the
        block table, or, with ``max_context``, every width up to that context (the pool has to hold that many tokens
        for every row meanwhile; sizes it cannot hold are left to be captured when they are met)."""
        from .step import SHORT_CONTEXT, TABLE_WIDTH_STEP
        if not self.runner.use_graphs or self.active_requests:
            return 0
        most = self.scheduler.max_batch_size
        if batch_sizes is None:
            batch_sizes = sorted({min(most, padded_rows(rows)) for rows in range(1, most + 1)})
        tokens_per_width = TABLE_WIDTH_STEP * self.block_size
        # one token (the shape of short contexts), the first context that is not short, then every width of the table
        contexts = [1, SHORT_CONTEXT + 1] + [width * tokens_per_width + 1 for width in range(1, -(-(max_context or 1) // tokens_per_width))]
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

    def prepare_next_step(self, sampled, pending=None) -> bool:
        """If the next step can only be a decoding step of known requests (nobody can join, nobody is still in its
        prompt), let the runner lay it out before this step's tokens are back; and if it brings exactly the requests
        that were sampled just now, in their order, start it at once with the tokens ``pending`` that are still on the
        device, so that the GPU does not wait for the host between the steps.  A request that stops at this step for
        a reason the host cannot foresee (an end-of-sequence token, a cancellation) makes the next step another one
        than the one prepared or started, which is then dropped and run again without that request."""
        following, someone_leaves = [], False
        for request in self.scheduler.running:
            if request.status == RequestStatus.DECODING:
                if len(request.generated_token_ids) + 1 < request.max_new_tokens:
                    following.append(request.request_id)
                else:
                    someone_leaves = True
            elif request.status == RequestStatus.PREFILL:
                return False
        # Requests that wait can only join when a place is free: with every place taken and nobody about to leave,
        # the next step is a decoding step of the same requests all the same.
        if self.scheduler.waiting and (someone_leaves or len(self.scheduler.running) < self.scheduler.max_batch_size):
            return False
        if not following or not self.runner.prepare_ahead(following):
            return False
        if self.launch_ahead and pending is not None and following == [request.request_id for request in sampled]:
            self.runner.launch_ahead(pending.device)
        return True

    def run_scheduled(self, out) -> None:
        """Turn the plan into one flat batch, run it, sample, and move every request on."""
        entries, sampled = [], []
        for request in out.decode_requests:
            entries.append(StepEntry(request.request_id, [request.generated_token_ids[-1]], [0]))
            sampled.append(request)
        prefill = [(r, n) for r, n in zip(out.prefill_requests, out.prefill_token_counts) if r.status == RequestStatus.PREFILL]
        for request, chunk_len in prefill:
            start = request.num_computed_tokens
            tokens = request.prefill_token_ids[start:start + chunk_len]
            final = start + chunk_len == len(request.prefill_token_ids) and not request.needs_decode_resume
            entries.append(StepEntry(request.request_id, tokens, [chunk_len - 1] if final else []))
            if final:
                sampled.append(request)
        if not entries:
            return
        logits = self.runner.step(entries)
        temperatures = [r.sampling.temperature for r in sampled]
        uniforms = [request_uniform(r.sampling.seed, r.num_samples_drawn) if r.sampling.temperature > 0 else 0.0 for r in sampled]
        if sampled:
            pending = self.sampler.launch(logits, temperatures, uniforms)
            self.prepare_next_step(sampled, pending)  # the host's share of the next step, while the GPU works on this one
            token_ids = pending.tolist()
        else:
            token_ids = []
        self.step_profile["tokens"] += sum(len(e.tokens) for e in entries)
        for request in out.decode_requests:
            request.complete_decode()
        for request, chunk_len in prefill:
            old = request.num_computed_tokens
            request.advance_prefill(chunk_len)
            if self.enable_prefix_caching:
                self.kv_cache.register_prefix(request.request_id, request.prompt_token_ids, old, request.num_computed_tokens)
            if request.num_computed_tokens == len(request.prefill_token_ids):
                request.complete_prefill()
        for request, token_id in zip(sampled, token_ids):
            request.num_samples_drawn += 1
            self.accept_generated_token(request, token_id)
        self.remove_finished_and_cancelled_requests()

    def step(self) -> bool:
        clock, profile = time.perf_counter, self.step_profile
        t0 = clock()
        out = self.schedule_step()
        t1 = clock()
        self.run_scheduled(out)
        profile["steps"] += 1
        profile["schedule_s"] += t1 - t0
        profile["step_s"] += clock() - t1
        profile["decode_steps"] += bool(out.decode_requests)
        profile["prefill_steps"] += bool(out.prefill_requests)
        return bool(self.scheduler.waiting or self.scheduler.running)

    async def run(self):
        profile, clock = self.step_profile, time.perf_counter
        while self.scheduler.waiting or self.scheduler.running:
            t0 = clock()
            out = self.schedule_step()
            t1 = clock()
            self.run_scheduled(out)
            t2 = clock()
            await asyncio.sleep(0)          # let other tasks (stream readers) run between steps
            t3 = clock()
            profile["steps"] += 1
            profile["schedule_s"] += t1 - t0
            profile["step_s"] += t2 - t1
            profile["yield_s"] += t3 - t2
            profile["decode_steps"] += bool(out.decode_requests)
            profile["prefill_steps"] += bool(out.prefill_requests)

    def generate(self, prompts_token_ids, max_new_tokens=None, temperature=None, seed=None) -> List[List[int]]:
        """Add the prompts, run to the end, return the generated token ids in the prompts' order."""
        requests = [self.add_request(None, prompt_token_ids=ids, max_new_tokens=max_new_tokens, temperature=temperature,
                                     seed=None if seed is None else seed + i) for i, ids in enumerate(prompts_token_ids)]
        while self.step():
            pass
        return [list(r.generated_token_ids) for r in requests]
