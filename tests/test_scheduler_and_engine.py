"""The scheduler's decisions and the engine's loop on the host (CPU).  The model's forward is
replaced by a script that returns one-hot logits, the reference's own way of testing its engine
(tests/test_engine.py:11-55 there); cache, step builder and sampler are the real ones
(with the torch twins of the kernels).  Decision vectors marked "reference" are the outcomes the
reference's tests hold for the same situations."""
import asyncio

import pytest
import torch

from llmserver_amd.cache import CacheExhaustedError
from llmserver_amd.engine import (STREAM_END, Engine, EngineConfig, Request, RequestFinishReason, RequestStateError, RequestStatus,
                                  Scheduler, load_model)
from helpers import model_folder
from torch_ops import TorchOps


def request(name, prompt=None):
    return Request(name, "Hello", prompt or [9707], 20)


def decoding(name, prompt=None, generated=7):
    """A request that has been through its prompt and holds its first generated token."""
    r = request(name, prompt)
    r.admit()
    assert r.computed(len(r.prompt_token_ids))
    r.accept(generated)
    return r


class Pages:
    """What the scheduler asks of a cache manager, for one group of pages of ``page`` tokens: ``free`` pages are
    available, ``held`` says how many pages a request has already."""

    def __init__(self, free, page, held=None, slots=None):
        self.free, self.page, self.held, self.slots = free, page, dict(held or {}), slots

    def available_pages(self):
        return [self.free]

    def pages_needed(self, request_id, num_tokens):
        return [max(0, -(-num_tokens // self.page) - self.held.get(request_id, 0))]

    def token_room(self, request_id, spare):
        return (self.held.get(request_id, 0) + max(0, spare[0])) * self.page

    def state_slots_free(self):
        return self.slots


# ---------------------------------------------------------------- request state machine
def test_request_walks_through_its_states():
    r = request("a", [1, 2, 3])
    with pytest.raises(RequestStateError):
        r.computed(1)                       # it has not been admitted
    r.admit()
    with pytest.raises(RequestStateError):
        r.admit()
    with pytest.raises(ValueError):
        r.computed(4)
    assert r.next_tokens(2) == [1, 2] and not r.computed(2)
    assert (r.status, r.tokens_ahead) == (RequestStatus.PREFILL, 1)
    with pytest.raises(RequestStateError):
        r.accept(7)                         # the end of the sequence has not been reached: there are no logits to sample
    assert r.computed(1) and r.status == RequestStatus.DECODING
    r.accept(7)
    assert r.next_tokens(1) == [7] and r.computed(1)
    assert (r.status, r.num_computed_tokens, r.sequence_length) == (RequestStatus.DECODING, 4, 4)
    r.finish("length")
    assert r.finish_reason == RequestFinishReason.LENGTH and not r.is_alive
    for event in (lambda: r.finish("eos"), r.cancel, r.preempt, r.admit):
        with pytest.raises(RequestStateError):
            event()


def test_a_preempted_request_is_computed_again_over_all_it_has_and_emits_nothing_twice():
    r = decoding("a", [20], generated=60)
    r.computed(1)
    r.accept(51)
    r.preempt()
    assert (r.status, r.num_computed_tokens, r.preemption_count, r.tokens_ahead) == (RequestStatus.WAITING, 0, 1, 3)
    r.admit()
    assert r.next_tokens(2) == [20, 60] and not r.computed(2)     # the reference's re-prefill: tests/test_engine.py:507
    assert r.next_tokens(1) == [51] and r.computed(1)             # ... and its decode step, which gives the next token
    assert r.status == RequestStatus.DECODING and r.generated_token_ids == [60, 51]
    r.preempt()
    r.admit()
    assert r.next_tokens(3) == [20, 60, 51] and r.computed(3)     # or all of it in one portion
    r.accept(52)
    assert r.generated_token_ids == [60, 51, 52]


def test_cached_tokens_move_the_mark_of_a_waiting_request_only():
    r = request("a", [1, 2, 3, 4, 5])
    with pytest.raises(ValueError):
        r.reuse(5)                          # one token at least must be computed
    r.reuse(4)
    assert r.tokens_ahead == 1 and r.next_tokens(1) == [5]
    r.forget_reused()
    assert r.tokens_ahead == 5
    r.admit()
    with pytest.raises(RequestStateError):
        r.reuse(2)


# ---------------------------------------------------------------- scheduler decisions
def plan_commit(scheduler, free=100, page=2, held=None):
    plan = scheduler.plan(Pages(free, page, held))
    scheduler.commit(plan)
    return plan


def counts(plan):
    return [count for _, count in plan.portions]


def who(plan):
    return [r for r, _ in plan.portions]


def test_budget_is_shared_by_decodes_and_portions():
    s = Scheduler(max_batch_size=3, max_num_batched_tokens=5)
    d, first, second = decoding("d"), request("first", [10, 11, 12]), request("second", [20, 21])
    s.running.append(d)
    s.waiting.extend([first, second])
    plan = plan_commit(s)
    assert plan.decodes == [d] and who(plan) == [first, second]
    assert counts(plan) == [3, 1] and plan.tokens == 5                                      # reference [3, 1]
    assert s.running == [d, first, second] and not s.waiting


def test_prompt_longer_than_the_budget_is_cut_and_computed_tokens_are_not_counted():
    s = Scheduler(max_batch_size=1, max_num_batched_tokens=3)
    r = request("long", [10, 11, 12, 13])
    s.waiting.append(r)
    assert counts(plan_commit(s)) == [3]
    r.computed(3)
    assert counts(plan_commit(s)) == [1]                                                    # reference [3] then [1]
    s = Scheduler(max_batch_size=2, max_num_batched_tokens=4)
    partial = request("partial", [10, 11, 12, 13, 14])
    partial.reuse(2)                                                                        # a cached prefix
    s.running.append(decoding("d"))
    s.waiting.append(partial)
    assert counts(plan_commit(s, held={"partial": 1})) == [3]


def test_chunk_size_caps_each_portion_and_running_prefills_keep_their_slot():
    s = Scheduler(max_batch_size=2, max_num_batched_tokens=4, prefill_chunk_size=2)
    a, b = request("a", [1, 2, 3, 4, 5]), request("b", [6, 7, 8, 9, 10])
    s.waiting.extend([a, b])
    assert counts(plan_commit(s)) == [2, 2]
    a.computed(2)
    b.computed(2)
    plan = plan_commit(s)
    assert who(plan) == [a, b] and counts(plan) == [2, 2] and s.running == [a, b]


def test_plan_changes_nothing_and_waiting_steps_count_committed_steps():
    s = Scheduler(max_batch_size=1, max_num_batched_tokens=1)
    rs = [request(f"r{i}") for i in range(3)]
    s.waiting.extend(rs)
    plan = s.plan(Pages(10, 2))
    assert list(s.waiting) == rs and not s.running and [r.waiting_steps for r in rs] == [0, 0, 0]
    assert s.commit(plan) == [rs[0]]
    assert [r.waiting_steps for r in rs] == [0, 1, 1]
    plan_commit(s, 10)
    s.running.remove(rs[0])
    plan_commit(s, 10)
    assert [r.waiting_steps for r in rs] == [0, 2, 3] and s.running == [rs[1]]            # reference [0, 2, 3]


def test_admission_keeps_one_spare_page_per_running_request():
    for free, admitted in ((2, 0), (3, 1)):                                               # reference: headroom cases
        s = Scheduler(max_batch_size=2, max_num_batched_tokens=2)
        d = decoding("d", [10, 11])                                                       # two tokens in one page; the third needs another
        w = request("w", [20])
        s.running.append(d)
        s.waiting.append(w)
        plan = s.plan(Pages(free, 2, held={"d": 1}))
        assert plan.decodes == [d] and plan.admitted == admitted and plan.fits
    s = Scheduler(max_batch_size=1, max_num_batched_tokens=5)
    s.waiting.append(request("long", [1, 2, 3, 4, 5]))
    assert counts(s.plan(Pages(1, 2))) == [2]                                             # shrunk to the free page


def test_a_plan_that_overdraws_the_pages_says_by_how_much():
    s = Scheduler(max_batch_size=2, max_num_batched_tokens=4)
    a, b = decoding("a", [1, 2]), decoding("b", [3, 4])
    s.running.extend([a, b])
    s.waiting.append(request("w"))
    plan = s.plan(Pages(1, 2, held={"a": 1, "b": 1}))          # both need a second page, one is free
    assert plan.short == [1] and not plan.fits and plan.admitted == 0 and plan.decodes == [a, b]
    assert s.plan(Pages(2, 2, held={"a": 1, "b": 1})).fits


def test_state_slots_are_places_too():
    s = Scheduler(max_batch_size=4, max_num_batched_tokens=8)
    s.waiting.extend(request(f"r{i}") for i in range(3))
    assert s.plan(Pages(100, 2, slots=2)).admitted == 2 and s.plan(Pages(100, 2, slots=None)).admitted == 3


def test_a_preempted_request_comes_back_only_when_all_of_it_fits():
    s = Scheduler(max_batch_size=2, max_num_batched_tokens=8, prefill_chunk_size=2)
    back = request("back", [1, 2, 3, 4, 5, 6])
    back.preemption_count = 1
    s.running.append(decoding("d", [9]))
    s.waiting.append(back)
    assert s.plan(Pages(3, 2, held={"d": 1})).admitted == 0          # 3 free, one kept for d: two pages hold four of its six tokens
    assert s.plan(Pages(4, 2, held={"d": 1})).admitted == 1
    back.preemption_count = 0
    assert counts(s.plan(Pages(3, 2, held={"d": 1}))) == [2]          # a new request starts on whatever portion fits


def test_nothing_fits_raises_and_bad_limits_are_refused():
    s = Scheduler(max_batch_size=1, max_num_batched_tokens=1)
    s.waiting.append(request("w"))
    with pytest.raises(CacheExhaustedError):
        s.plan(Pages(0, 2))
    assert s.plan(Pages(1, 2)).admitted == 1
    empty = Scheduler(max_batch_size=1, max_num_batched_tokens=1).plan(Pages(1, 2))
    assert empty.tokens == 0 and not empty.requests
    for args in ((0, 2), (2, 0), (3, 2)):
        with pytest.raises(ValueError):
            Scheduler(*args)
    with pytest.raises(ValueError):
        Scheduler(1, 2, prefill_chunk_size=0)


# ---------------------------------------------------------------- the engine with a scripted model
class Script:
    """Replaces the model's forward: one-hot logits from a list of token ids per call; records the calls."""

    def __init__(self, model, token_ids_by_call):
        self.tokens, self.calls, self.vocab = list(token_ids_by_call), [], model.head.out_features
        model.forward = self

    def __call__(self, ctx, caches):
        self.calls.append({"requests": list(ctx.request_ids), "tokens": [ctx.h_token_ids[s:s + n].tolist() for s, n in zip(ctx.h_row_start, ctx.h_row_len)],
                           "start": [int(c - n) for c, n in zip(ctx.h_row_ctx, ctx.h_row_len)], "n_out": ctx.n_out})
        ids = self.tokens.pop(0) if self.tokens else [0] * ctx.n_out
        assert len(ids) == ctx.n_out, (ids, ctx.n_out)
        logits = torch.zeros(ctx.n_out, self.vocab)
        for row, token in enumerate(ids):
            logits[row, token] = 1.0
        return logits


def scripted_engine(script, **options):
    model = load_model(model_folder("A"), "cpu", torch.float32)
    defaults = dict(max_new_tokens=3, max_batch_size=2, max_num_batched_tokens=2, kv_cache_num_blocks=2, kv_cache_block_size=2,
                    ignore_eos=True, ops=TorchOps())
    defaults.update(options)
    engine = Engine(model, None, **defaults)
    return engine, Script(model, script)


def test_recompute_preemption_resumes_without_duplicate_output():
    """Two one-token prompts, two pages of two tokens: the third step needs a third page.
    The reference's trace for this situation is tests/test_engine.py:494-523."""
    engine, script = scripted_engine([[50, 60], [51, 51], [51], [], [51]])
    first, second = engine.add_request(None, [10]), engine.add_request(None, [20])
    assert engine.step() and engine.step()
    assert second.generated_token_ids == [60, 51] and min(engine.kv_cache.available_pages()) == 0
    assert second.output_queue.drain() == [60, 51]
    assert engine.step()                                # the later request is the victim; the first decodes and finishes
    assert first.status == RequestStatus.FINISHED and first.generated_token_ids == [50, 51, 51]
    assert second.status == RequestStatus.WAITING and second.tokens_ahead == 3 and not engine.kv_cache.has(second.request_id)
    assert engine.step()                                # computed again: the budget of two tokens takes [20, 60], nothing to sample yet
    assert second.status == RequestStatus.PREFILL and second.num_computed_tokens == 2
    assert second.generated_token_ids == [60, 51] and second.output_queue.empty()
    assert script.calls[3]["tokens"] == [[20, 60]] and script.calls[3]["n_out"] == 0
    assert not engine.step()
    assert second.generated_token_ids == [60, 51, 51] and second.status == RequestStatus.FINISHED
    assert script.calls[4]["tokens"] == [[51]] and script.calls[4]["start"] == [2]
    assert [c["requests"] for c in script.calls] == [[first.request_id, second.request_id]] * 2 + [[first.request_id]] + [[second.request_id]] * 2
    assert engine.step_profile["preemptions"] == 1
    engine.kv_cache.check_invariants()
    assert min(engine.kv_cache.available_pages()) == 2


@pytest.mark.parametrize("first, second, victim", [((0, 0), (0, 0), 1), ((0, 0), (1, 0), 0), ((1, 1), (1, 3), 0), ((1, 3), (1, 1), 1)])
def test_victim_is_least_preempted_then_least_waited_then_latest_admitted(first, second, victim):
    """reference: tests/test_engine.py:525-545"""
    engine, _ = scripted_engine([[50, 60], [51, 51]])
    requests = [engine.add_request(None, [10]), engine.add_request(None, [20])]
    engine.step()
    engine.step()
    for r, (count, steps) in zip(requests, (first, second)):
        r.preemption_count, r.waiting_steps = count, steps
    out = engine.schedule_step()
    assert out.decodes == [requests[1 - victim]] and list(engine.scheduler.waiting) == [requests[victim]]
    assert requests[victim].preemption_count == (first, second)[victim][0] + 1 and not engine.kv_cache.has(requests[victim].request_id)


def test_a_single_request_that_cannot_grow_raises():
    engine, _ = scripted_engine([[50], [51], [52], [53], [54]], max_new_tokens=8, max_batch_size=1, max_num_batched_tokens=4)
    engine.add_request(None, [10, 11])
    engine.step()
    engine.step()
    with pytest.raises(CacheExhaustedError):
        for _ in range(4):
            engine.step()


@pytest.mark.parametrize("length, complete", [(3, 0), (4, 1), (6, 1), (8, 2)])
def test_only_complete_pages_of_prompt_tokens_become_shareable(length, complete):
    """reference: tests/test_engine.py:186-194"""
    engine, _ = scripted_engine([[50]], max_batch_size=1, max_num_batched_tokens=8, kv_cache_num_blocks=4, kv_cache_block_size=4)
    r = engine.add_request(None, list(range(10, 10 + length)))
    engine.step()
    assert engine.kv_cache.groups[0].pool.published_pages() == set(engine.kv_cache.record(r.request_id).tables[0][:complete])


@pytest.mark.parametrize("length, shared", [(4, 0), (8, 1), (10, 2)])
def test_second_request_reuses_the_longest_cached_prefix(length, shared):
    """reference: tests/test_engine.py:230-250"""
    prompt = list(range(10, 10 + length))
    engine, script = scripted_engine([[50], [51, 60]], max_num_batched_tokens=12, kv_cache_num_blocks=6, kv_cache_block_size=4)
    first = engine.add_request(None, prompt)
    engine.step()
    second = engine.add_request(None, prompt)
    assert not engine.kv_cache.has(second.request_id)       # a request that waits holds nothing; it looks when it is admitted
    engine.step()                       # one mixed step: the first request's decode token beside the second's portion
    tables = [engine.kv_cache.record(r.request_id).tables[0] for r in (first, second)]
    assert tables[1][:shared] == tables[0][:shared] and not set(tables[1][shared:]) & set(tables[0])
    assert all(engine.kv_cache.groups[0].pool.holders[p] == 2 for p in tables[1][:shared])
    call = script.calls[-1]
    assert call["requests"] == [first.request_id, second.request_id]
    index = call["requests"].index(second.request_id)
    assert call["tokens"][index] == prompt[shared * 4:] and call["start"][index] == shared * 4
    assert second.generated_token_ids == [60]
    assert engine.step_profile["prefix_hit_tokens"] == shared * 4


def test_stop_rules_stream_and_history():
    engine, _ = scripted_engine([[7], [9], [9]], max_batch_size=1, max_num_batched_tokens=4, kv_cache_num_blocks=4, ignore_eos=False)
    engine.eos_token_ids = {9}
    r = engine.add_request(None, [1, 2, 3])
    assert engine.step() and not engine.step()
    assert r.generated_token_ids == [7, 9] and r.finish_reason == RequestFinishReason.EOS
    assert r.output_queue.drain() == [7, 9, STREAM_END]
    assert r.request_id in engine.completed_requests and r.request_id not in engine.active_requests
    assert min(engine.kv_cache.available_pages()) == 4
    with pytest.raises(ValueError):
        engine.add_request(None, [])
    with pytest.raises(ValueError):
        engine.add_request(None, [10 ** 6])
    with pytest.raises(ValueError):
        engine.add_request("text without a tokenizer")


def test_cancel_frees_pages_and_ends_the_stream():
    engine, _ = scripted_engine([[50, 60]], kv_cache_num_blocks=4)
    a, b = engine.add_request(None, [10]), engine.add_request(None, [20])
    engine.step()
    assert engine.cancel_request(b.request_id) and not engine.cancel_request(b.request_id)
    assert b.status == RequestStatus.CANCELLED and b.output_queue.drain() == [STREAM_END]
    assert engine.scheduler.running == [a]
    engine.kv_cache.check_invariants()


def test_run_yields_between_steps():
    engine, _ = scripted_engine([[50, 60], [51, 61], [52, 62]], kv_cache_num_blocks=8)
    a, b = engine.add_request(None, [10]), engine.add_request(None, [20])
    ticks = []

    async def watcher():
        while engine.scheduler.waiting or engine.scheduler.running:
            ticks.append(len(a.generated_token_ids))
            await asyncio.sleep(0)

    async def both():
        await asyncio.gather(engine.run(), watcher())

    asyncio.run(both())
    assert a.generated_token_ids == [50, 51, 52] and b.generated_token_ids == [60, 61, 62]
    assert ticks == [1, 2] and engine.step_profile["steps"] == 3      # the watcher ran after the first and second step


def test_real_model_under_a_small_budget_and_few_pages_generates_the_same_tokens():
    """Chunked prefill beside decodes under a token budget of 32, and a pool so small that requests
    are preempted and recomputed, must not change greedy output (CPU, torch twins of the kernels)."""
    import plain_qwen3 as plain
    from helpers import plain_model, random_tokens
    config, tensors = plain_model("B")
    prompts = [random_tokens(config["vocab_size"], n, 60 + i) for i, n in enumerate((1, 40, 64, 100))]
    expected = [plain.greedy_generate(config, tensors, prompt, 12) for prompt in prompts]
    model = load_model(model_folder("B"), "cpu", torch.float32)
    for pages in (64, 27):
        engine = Engine(model, None, max_new_tokens=12, max_batch_size=4, max_num_batched_tokens=32, kv_cache_num_blocks=pages,
                        kv_cache_block_size=8, ignore_eos=True, ops=TorchOps())
        assert engine.generate(prompts) == expected
        engine.kv_cache.check_invariants()
        assert min(engine.kv_cache.available_pages()) == pages
    assert engine.step_profile["preemptions"] > 0


def test_requests_that_arrive_together_share_what_the_first_of_them_computed():
    """Both arrive before any step; only one fits into the first step; when the second is admitted it
    finds the first one's complete prompt pages and computes the rest only."""
    prompt = list(range(10, 20))
    engine, script = scripted_engine([[50], [51, 60]], max_batch_size=2, max_num_batched_tokens=10, kv_cache_num_blocks=8,
                                     kv_cache_block_size=4)
    first, second = engine.add_request(None, prompt), engine.add_request(None, prompt)
    assert second.num_computed_tokens == 0
    engine.step()
    assert script.calls[0]["requests"] == [first.request_id]
    engine.step()
    call = script.calls[1]
    assert call["requests"] == [first.request_id, second.request_id]
    assert call["tokens"][1] == prompt[8:] and call["start"][1] == 8
    assert engine.kv_cache.record(second.request_id).tables[0][:2] == engine.kv_cache.record(first.request_id).tables[0][:2]
    assert engine.step_profile["prefix_hit_tokens"] == 8
    engine.kv_cache.check_invariants()


@pytest.mark.parametrize("seed", range(8))
def test_so_few_pages_that_requests_take_turns_still_ends(seed):
    """Eight requests, three places, a pool that holds one or two of them: requests are preempted over and over.
    Waiting requests must not keep the cached pages of their prefixes from the running ones (held pages cannot be
    evicted), and two requests that do not fit together must not throw each other out for ever: a preempted request
    comes back when all it has to compute again fits at once.  Everybody finishes with all tokens, in few steps."""
    import random
    rng = random.Random(seed)
    pages = rng.choice((9, 10, 12, 14))
    engine, script = scripted_engine([], max_new_tokens=8, max_batch_size=3, max_num_batched_tokens=8, kv_cache_num_blocks=pages,
                                     kv_cache_block_size=2)
    requests = [engine.add_request(None, [rng.randrange(5, 60) for _ in range(rng.randint(3, 9))]) for _ in range(8)]
    steps = 0
    while engine.step():
        steps += 1
        engine.kv_cache.check_invariants()
        assert steps < 200, "requests take turns without getting anywhere"
    assert all(r.status == RequestStatus.FINISHED and len(r.generated_token_ids) == 8 for r in requests)
    assert engine.step_profile["preemptions"] > 0
    assert min(engine.kv_cache.available_pages()) == pages and not engine.kv_cache.requests


def test_waiting_requests_hold_no_pages_so_cached_prefixes_never_starve_a_running_request():
    """One place, five pages.  A finished request leaves two cached pages; a waiting request with the same prefix
    would like them, while the running request grows to need all five pages.  A request that waits holds nothing (it
    looks its prefix up when a place is free), so the cached pages are recycled for the running request instead of
    the engine giving up, and the waiting one computes its prompt itself when its turn comes."""
    engine, script = scripted_engine([], max_new_tokens=6, max_batch_size=1, max_num_batched_tokens=8, kv_cache_num_blocks=5,
                                     kv_cache_block_size=2)
    first = engine.add_request(None, [7, 8, 9, 10, 11], max_new_tokens=1)
    assert not engine.step() and first.status == RequestStatus.FINISHED      # its two complete pages stay cached
    assert engine.kv_cache.groups[0].pool.num_idle == 2
    running = engine.add_request(None, [20, 21, 22, 23, 24])
    waiting = engine.add_request(None, [7, 8, 9, 10, 12])
    while running.status != RequestStatus.FINISHED:        # ten tokens in the cache: five pages, two of them were the cached ones
        assert engine.step()
        engine.kv_cache.check_invariants()
        assert waiting.status != RequestStatus.WAITING or not engine.kv_cache.has(waiting.request_id)
    assert running.generated_token_ids == [0] * 6 and engine.step_profile["preemptions"] == 0
    while engine.step():
        pass
    assert waiting.status == RequestStatus.FINISHED and len(waiting.generated_token_ids) == 6
    assert engine.step_profile["prefix_hit_tokens"] == 0
    assert min(engine.kv_cache.available_pages()) == 5 and not engine.kv_cache.requests


def test_an_offered_prefix_is_given_back_if_the_request_is_not_admitted_after_all():
    """Two places; the budget of a step is used up by the first waiting request, so the second, which was offered the
    cached pages of its prefix, is not admitted: it gives them back and holds nothing over the step."""
    engine, script = scripted_engine([], max_new_tokens=2, max_batch_size=2, max_num_batched_tokens=4, kv_cache_num_blocks=8,
                                     kv_cache_block_size=2)
    seed = engine.add_request(None, [7, 8, 9, 10, 11], max_new_tokens=1)
    while engine.step():
        pass
    assert seed.status == RequestStatus.FINISHED and engine.kv_cache.groups[0].pool.num_idle == 2
    long, follower = engine.add_request(None, [30, 31, 32, 33, 34, 35]), engine.add_request(None, [7, 8, 9, 10, 12])
    engine.step()                                           # four tokens of `long`; nothing is left for `follower`
    assert follower.status == RequestStatus.WAITING and follower.num_computed_tokens == 0
    assert not engine.kv_cache.has(follower.request_id) and engine.kv_cache.groups[0].pool.num_idle == 2
    engine.step()                                           # two tokens of `long`, and `follower` joins behind its cached prefix
    assert script.calls[-1]["requests"] == [long.request_id, follower.request_id]
    assert script.calls[-1]["tokens"][1] == [12] and script.calls[-1]["start"][1] == 4
    assert engine.step_profile["prefix_hit_tokens"] == 4
    while engine.step():
        pass
    engine.kv_cache.check_invariants()
    assert not engine.kv_cache.requests


def test_a_preempted_request_at_the_head_of_the_queue_stalls_admissions_only_until_it_fits():
    """This engine's own rule (a preempted request is admitted again only when all of it fits beside the running ones)
    holds back whoever queued behind it meanwhile.  Under steady arrivals, with one long request that is preempted:
    the stall ends when the running requests have finished (each is bounded by its own length limit), and everybody
    finishes."""
    engine, _ = scripted_engine([], max_new_tokens=6, max_batch_size=3, max_num_batched_tokens=16, kv_cache_num_blocks=16,
                                kv_cache_block_size=2)
    long = engine.add_request(None, list(range(5, 19)), max_new_tokens=12)           # 14 + 12 tokens: 13 of the 16 pages
    others = [engine.add_request(None, [30 + i, 40 + i, 50 + i]) for i in range(2)]
    finished, preempted_at, stalled, steps = [], None, 0, 0
    arrivals = 0
    while engine.has_work() or arrivals < 10:
        if arrivals < 10 and steps % 2 == 0:                                         # a short request every other step
            others.append(engine.add_request(None, [60 + arrivals, 70 + arrivals], max_new_tokens=4))
            arrivals += 1
        waiting_before = len(engine.scheduler.waiting)
        running_before = len(engine.scheduler.running)
        engine.step()
        steps += 1
        engine.kv_cache.check_invariants()
        if preempted_at is None and long.preemption_count:
            preempted_at = steps
        head = engine.scheduler.waiting[0] if engine.scheduler.waiting else None
        if head is long and waiting_before > 1 and running_before < 3:
            stalled += 1                                                             # a place was free, somebody waited behind the long one
        finished += [r for r in [long] + others if r.status == RequestStatus.FINISHED and r not in finished]
        assert steps < 300
    assert preempted_at is not None and long.preemption_count >= 1, "the pool was meant to be too small for all of them"
    assert long.status == RequestStatus.FINISHED and len(long.generated_token_ids) == 12
    assert all(r.status == RequestStatus.FINISHED for r in others)
    # the stall is bounded by what the running requests still had to generate (at most 6 tokens each) plus the plan's own step
    assert stalled <= 8, stalled
    assert min(engine.kv_cache.available_pages()) == 16 and not engine.kv_cache.requests
