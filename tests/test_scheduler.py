"""The scheduler's decisions, on the CPU: the policy functions alone, and the engine's
ticks over a fake step function that keeps real page accounting.  The vectors are those
the reference's scheduler tests pin (/root/reference/tests/test_continuous_batching.py)."""
from types import SimpleNamespace

import pytest
import torch

from pylon_amd.cache import CacheManager, OutOfPages
from pylon_amd.config import PylonConfig
from pylon_amd.engine.engine import Engine, EngineClosedError, QueueFullError
from pylon_amd.engine.scheduler import (AdmissionPolicy, PromptWork, Waiter, WAIT_LIMIT_SECONDS,
                                        cut_prompts, hold_prompts)
from pylon_amd.parts.base import KVRequirement
from pylon_amd.sampling import Sampling

PAGE = 256


class FakeRunner:
    """Real cache bookkeeping, no model: a step records what it was given and returns the
    request ids of the rows that want logits (the fake sampler's 'logits')."""

    def __init__(self, pages, max_requests=8, vocab=64, page_size=PAGE, max_positions=1 << 20):
        self.manager = CacheManager([KVRequirement(1, 16)], page_size=page_size, num_pages=pages,
                                    max_requests=max_requests, dtype=torch.float32, device="cpu")
        self.model = SimpleNamespace(spec=SimpleNamespace(vocab_size=vocab, max_positions=max_positions),
                                     device="cpu")
        self.steps = []
        self.fail_next = None

    def open(self, request_id, capacity=None):
        return self.manager.open(request_id, capacity)

    def close(self, seq):
        self.manager.close(seq)

    def step(self, entries):
        if self.fail_next is not None:
            error, self.fail_next = self.fail_next, None
            raise error
        pairs = [(e.seq, len(e.tokens)) for e in entries]
        self.manager.reserve(pairs)
        self.manager.commit(pairs)
        self.steps.append([(e.seq.request_id[0], list(e.tokens), list(e.want)) for e in entries])
        ready = [e.seq.request_id[0] for e in entries if e.want]
        return ready or None


class ScriptedSampler:
    """Hands each request the next token of its script (default token 7)."""

    def __init__(self):
        self.scripts = {}
        self.calls = []

    def sample(self, logits, rows):
        self.calls.append([(s.temperature, index) for s, index in rows])
        out = []
        for rid in logits:
            script = self.scripts.get(rid)
            out.append(script.pop(0) if script else 7)
        return out


class Clock:
    def __init__(self):
        self.now = 1000.0

    def __call__(self):
        return self.now


def make_engine(pages=8, slots=8, chunk=2048, admit_skip=4, queue=32, runner_slots=None, **kw):
    runner = FakeRunner(pages, max_requests=runner_slots or slots, **kw)
    clock = Clock()
    config = PylonConfig(max_batch_size=slots, prefill_chunk_size=chunk, admit_skip=admit_skip,
                         max_queue_size=queue, page_size=PAGE)
    engine = Engine(config, runner=runner, sampler=ScriptedSampler(), clock=clock)
    return engine, runner, clock


def enqueue(engine, rid, prompt, max_new, eos=None):
    return engine.enqueue(prompt, eos, Sampling(max_new_tokens=max_new, temperature=0.0), rid)


def ids(engine, which):
    return engine.snapshot()[which]


# ---- the policy functions alone --------------------------------------------------------

def test_cut_prompts_portions():
    # a 10-token prompt at a budget of 4 runs as 4, 4, 2
    # (/root/reference/tests/test_continuous_batching.py:252-267)
    sizes, left = [], 10
    while left:
        (key, count), = cut_prompts([PromptWork("p", left, 0.0)], 4, 0.0)
        sizes.append(count)
        left -= count
    assert sizes == [4, 4, 2]
    # one step packs every prompt that fits (:526-537); the budget is shared in order
    work = [PromptWork("a", 4, 0.0), PromptWork("b", 4, 0.0)]
    assert cut_prompts(work, 2048, 0.0) == [("a", 4), ("b", 4)]
    # a prompt that finishes inside the budget goes before a longer one that came first
    work = [PromptWork("long", 100, 0.0), PromptWork("short", 8, 0.0)]
    assert cut_prompts(work, 16, 0.05) == [("short", 8), ("long", 8)]
    # but one that has waited 100 ms goes first, oldest first (:501-524)
    work = [PromptWork("long", 100, 0.0), PromptWork("short", 8, 0.05), PromptWork("older", 50, -1.0)]
    assert cut_prompts(work, 16, 0.1) == [("older", 16)]
    assert cut_prompts(work, 0, 0.1) == [] and cut_prompts([], 16, 0.0) == []
    assert cut_prompts([PromptWork("done", 0, 0.0)], 16, 0.0) == []


def test_hold_prompts_only_with_a_full_decode_batch_and_young_work():
    work = [PromptWork("p", 5, 0.0)]
    assert hold_prompts(4, 4, work, 0.05)
    assert not hold_prompts(4, 4, work, WAIT_LIMIT_SECONDS)
    assert not hold_prompts(3, 4, work, 0.05)
    assert not hold_prompts(4, 4, [], 0.05)


def test_admission_policy_rules():
    policy = AdmissionPolicy(page_budget=4, page_size=PAGE, admit_skip=4)
    assert policy.pages(64 + 200) == 2 and policy.pages(256) == 1 and policy.pages(257) == 2
    # reservations within the pool and a free page per decoding request
    assert policy.fits(256, reserved_pages=3, decoding=0)
    assert not policy.fits(256, reserved_pages=3, decoding=1)  # the free-page floor
    assert not policy.fits(257, reserved_pages=3, decoding=0)
    now = 50.0
    head = Waiter("long", 3 * PAGE, now)
    short = Waiter("short", 72, now)
    v = policy.next([head, short], reserved_pages=1, decoding=1, now=now)
    assert (v.key, v.admit, v.skipped_head, v.pages) == ("short", True, True, 1)
    # a head that has waited 100 ms is not overtaken
    aged = Waiter("long", 3 * PAGE, now - WAIT_LIMIT_SECONDS)
    assert policy.next([aged, short], reserved_pages=1, decoding=1, now=now) is None
    # nor is an aged waiter behind the head
    assert policy.next([head, aged, short], reserved_pages=1, decoding=1, now=now) is None
    # admit_skip = 0 never looks past the head
    strict = AdmissionPolicy(page_budget=4, page_size=PAGE, admit_skip=0)
    assert strict.next([head, short], reserved_pages=1, decoding=1, now=now) is None
    # four non-fitting waiters behind the head may be passed, a fifth stops the scan
    blocks = [Waiter(f"b{i}", 3 * PAGE, now) for i in range(5)]
    assert policy.next(blocks + [short], reserved_pages=1, decoding=1, now=now).key == "short"
    blocks.append(Waiter("b5", 3 * PAGE, now))
    assert policy.next(blocks + [short], reserved_pages=1, decoding=1, now=now) is None
    # a request that can never fit is rejected, not waited for
    v = policy.next([Waiter("huge", 5 * PAGE, now)], reserved_pages=0, decoding=0, now=now)
    assert not v.admit and "cannot fit in the KV-cache budget" in v.reason
    assert policy.next([], reserved_pages=0, decoding=0, now=now) is None


# ---- ticks over the fake step function ------------------------------------------------------

def test_prompt_portions_first_token_and_length_finish():
    engine, runner, _ = make_engine(chunk=4)
    future = enqueue(engine, "a", list(range(10)), 2)
    engine.run_until_idle()
    chunks = [step[0] for step in runner.steps]
    assert [len(tokens) for _, tokens, _ in chunks[:3]] == [4, 4, 2]
    # non-final portions skip the vocabulary head; the final one samples from its last row
    assert [want for _, _, want in chunks[:3]] == [[], [], [1]]
    assert chunks[3] == ("a", [7], [0])  # then one decode step with the sampled token
    result = future.result(timeout=0)
    assert result.output_ids == [7, 7] and result.finish_reason == "length"
    assert runner.manager.free_pages == 8 and not runner.manager.live_sequences()
    # the sampler was told which draw each token is
    assert [call[0][1] for call in engine.sampler.calls] == [0, 1]


def test_eos_frees_the_slot_and_the_stop_token_is_not_emitted():
    # /root/reference/tests/test_continuous_batching.py:299-310
    engine, runner, _ = make_engine()
    engine.sampler.scripts["a"] = [9]
    future = enqueue(engine, "a", [1, 2, 3], 5, eos=9)
    engine.run_until_idle()
    result = future.result(timeout=0)
    assert result.output_ids == [] and result.finish_reason == "eos"
    engine.sampler.scripts["b"] = [3, 4, 9, 5]
    future = enqueue(engine, "b", [1, 2, 3], 8, eos=[9, 11])
    engine.run_until_idle()
    assert future.result(timeout=0).output_ids == [3, 4]
    assert runner.manager.free_pages == 8


def test_decode_rows_come_first_and_do_not_shrink_the_portion():
    # /root/reference/tests/test_continuous_batching.py:557-578
    engine, runner, _ = make_engine(chunk=4)
    enqueue(engine, "d", [1, 2], 8)
    engine.tick()
    enqueue(engine, "p", [5, 6, 7, 8, 9, 10], 4)
    engine.tick()
    step = runner.steps[-1]
    assert step[0] == ("d", [7], [0])
    assert step[1] == ("p", [5, 6, 7, 8], [])  # a full portion of 4 beside the decode row
    assert engine.last_step == (["d"], [("p", 4)])


def test_one_step_packs_every_prompt_that_fits_and_two_waves_when_not():
    engine, runner, _ = make_engine()
    enqueue(engine, "a", [1, 2, 3, 4], 2)
    enqueue(engine, "b", [5, 6, 7, 8], 2)
    engine.tick()
    assert runner.steps[0] == [("a", [1, 2, 3, 4], [3]), ("b", [5, 6, 7, 8], [3])]
    # 8 prompts of 512 tokens at a budget of 2048 take two steps of four (:539-549)
    engine, runner, _ = make_engine(pages=64)
    for i in range(8):
        enqueue(engine, f"r{i}", [1] * 512, 1)
    engine.tick()
    engine.tick()
    assert [len(step) for step in runner.steps[:2]] == [4, 4]
    assert all(len(tokens) == 512 for step in runner.steps[:2] for _, tokens, _ in step)


def test_full_decode_batch_holds_young_prompt_work_back():
    # /root/reference/tests/test_continuous_batching.py:604-645
    engine, runner, clock = make_engine(slots=2, pages=16, runner_slots=3)
    enqueue(engine, "a", [1], 64)
    enqueue(engine, "b", [2], 64)
    engine.tick()  # both prefilled and decoding
    engine._max_batch_size = 3  # let a third in, then close the door again
    enqueue(engine, "c", [3, 4, 5], 4)
    engine._admit()
    engine._max_batch_size = 2
    engine.tick()
    assert [rid for rid, _, _ in runner.steps[-1]] == ["a", "b"]  # decode-only: c is young
    clock.now += WAIT_LIMIT_SECONDS
    engine.tick()
    assert [rid for rid, _, _ in runner.steps[-1]] == ["a", "b", "c"]


def engine_with_one_decode(pages, admit_skip=4):
    engine, runner, clock = make_engine(pages=pages, slots=8, admit_skip=admit_skip)
    enqueue(engine, "decode", [1, 2, 3, 4], 32)
    engine.tick()
    assert ids(engine, "active") == ["decode"] and engine._active[0].pending_token_id is not None
    return engine, runner, clock


def test_short_job_starts_while_the_longer_head_keeps_its_place():
    # /root/reference/tests/test_continuous_batching.py:722-735
    engine, runner, _ = engine_with_one_decode(4)
    long = enqueue(engine, "long", [2] * (3 * PAGE - 1), 1)
    enqueue(engine, "short", [3] * 64, 8)
    engine.tick()
    assert ids(engine, "waiting") == ["long"] and ids(engine, "active") == ["decode", "short"]
    assert engine.head_skips == 1 and not long.done()
    assert engine._active[1].reserved_pages == 1


def test_admit_skip_zero_and_aged_head_keep_the_order():
    engine, _, _ = engine_with_one_decode(4, admit_skip=0)
    enqueue(engine, "long", [2] * (3 * PAGE - 1), 1)
    short = enqueue(engine, "short", [3] * 64, 8)
    engine.tick()
    assert ids(engine, "waiting") == ["long", "short"] and engine.head_skips == 0 and not short.done()
    engine, _, clock = engine_with_one_decode(4)
    enqueue(engine, "long", [2] * (3 * PAGE - 1), 1)
    enqueue(engine, "short", [3] * 64, 8)
    clock.now += WAIT_LIMIT_SECONDS
    engine.tick()
    assert ids(engine, "waiting") == ["long", "short"] and ids(engine, "active") == ["decode"]


def test_each_admission_behind_the_head_counts_once_and_order_is_kept():
    engine, _, _ = engine_with_one_decode(4)
    enqueue(engine, "first-block", [2] * (3 * PAGE - 1), 1)
    enqueue(engine, "second-block", [4] * (3 * PAGE - 1), 1)
    enqueue(engine, "short-a", [3] * 64, 8)
    enqueue(engine, "short-b", [4] * 64, 8)
    engine.tick()
    assert ids(engine, "waiting") == ["first-block", "second-block"]
    assert ids(engine, "active") == ["decode", "short-a", "short-b"] and engine.head_skips == 2


def test_reservation_and_free_page_floor():
    # reservation = rounded prompt + max_new (:836-846)
    engine, _, _ = make_engine(pages=4, chunk=8)
    enqueue(engine, "job", [4] * 64, 200)
    engine.tick()
    assert engine._active[0].prompt_offset == 8 and engine._active[0].reserved_pages == 2
    # a reservation that would leave no free page for the decoding request waits (:848-859)
    engine, _, _ = engine_with_one_decode(2)
    job = enqueue(engine, "fills", [3] * 64, 8)
    engine.tick()
    assert ids(engine, "waiting") == ["fills"] and not job.done()
    # a prefilling request does not count against the floor (:861-873)
    engine, _, _ = make_engine(pages=2, chunk=4)
    enqueue(engine, "prefill", [1] * 200, 1)
    engine.tick()
    enqueue(engine, "next", [3] * 40, 8)
    engine.tick()
    assert ids(engine, "active") == ["prefill", "next"]


def test_never_fitting_request_fails_alone_and_validation_errors():
    engine, runner, _ = make_engine(pages=2)
    ok = enqueue(engine, "ok", [1, 2], 2)
    with pytest.raises(ValueError, match="KV-cache tokens"):
        enqueue(engine, "huge", [1] * (2 * PAGE), 1)
    with pytest.raises(ValueError, match="at least one token"):
        enqueue(engine, "empty", [], 1)
    with pytest.raises(ValueError, match="Token IDs must be between 0 and 63"):
        enqueue(engine, "bad", [64], 1)
    with pytest.raises(ValueError, match="Token IDs"):
        enqueue(engine, "badstop", [1], 1, eos=99)
    engine.run_until_idle()
    assert ok.result(timeout=0).output_ids == [7, 7]
    small = FakeRunner(2, max_positions=16)
    eng = Engine(PylonConfig(page_size=PAGE), runner=small, sampler=ScriptedSampler())
    with pytest.raises(ValueError, match="cache positions"):
        eng.enqueue([1] * 10, None, Sampling(max_new_tokens=10), "x")


def test_queue_bound_cancellation_and_close():
    engine, runner, _ = make_engine(queue=2, slots=1)
    a = enqueue(engine, "a", [1], 4)
    b = enqueue(engine, "b", [2], 4)
    with pytest.raises(QueueFullError):
        enqueue(engine, "c", [3], 4)
    assert b.cancel()
    c = enqueue(engine, "c", [3], 4)  # the cancelled one was swept
    engine.tick()
    assert ids(engine, "active") == ["a"] and ids(engine, "waiting") == ["c"]
    assert a.cancel() is False  # running
    engine.close()
    with pytest.raises(EngineClosedError):
        a.result(timeout=0)
    with pytest.raises(EngineClosedError):
        c.result(timeout=0)
    with pytest.raises(EngineClosedError):
        enqueue(engine, "d", [1], 1)
    assert runner.manager.free_pages == 8 and not runner.manager.live_sequences()


def test_when_pages_run_out_the_running_requests_fail_and_free_their_pages():
    # Whole-life reservations keep this from happening; if a step is refused for pages all
    # the same, every running request fails and gives its pages back, and waiting requests
    # stay queued (/root/reference/src/pylon/engine.py:260-264,716-722).
    engine, runner, _ = make_engine(pages=4, slots=2, runner_slots=4)
    a = enqueue(engine, "a", [1] * PAGE, 4)  # its first decoded token opens a second page
    b = enqueue(engine, "b", [4, 5], 4)
    engine.tick()
    assert runner.manager.free_pages == 2
    thief = runner.manager.open("thief")  # takes the free pages behind the scheduler's back
    runner.manager.reserve([(thief, 2 * PAGE)])
    later = enqueue(engine, "later", [9], 2)
    engine.tick()
    for future in (a, b):
        with pytest.raises(OutOfPages):
            future.result(timeout=0)
    assert not later.done() and ids(engine, "active") == ["later"]
    assert {s.request_id for s in runner.manager.live_sequences() if s.request_id != "thief"} == {("later", 3)}
    assert runner.manager.free_pages == 2  # a's and b's pages came back
    runner.manager.check()
    runner.manager.close(thief)
    engine.run_until_idle()
    assert later.result(timeout=0).output_ids == [7, 7]


def test_a_step_that_raises_fails_active_requests_only():
    engine, runner, _ = make_engine(slots=1)
    a = enqueue(engine, "a", [1, 2, 3], 4)
    b = enqueue(engine, "b", [4], 2)
    runner.fail_next = RuntimeError("kernel refused")
    engine.tick()
    with pytest.raises(RuntimeError, match="kernel refused"):
        a.result(timeout=0)
    engine.run_until_idle()
    assert b.result(timeout=0).output_ids == [7, 7]
    assert runner.manager.free_pages == 8


def test_threaded_engine_serves_requests():
    runner = FakeRunner(8)
    engine = Engine(PylonConfig(page_size=PAGE, batch_wait_ms=1.0), runner=runner,
                    sampler=ScriptedSampler(), threaded=True)
    try:
        futures = [engine.enqueue([1, 2, 3], None, Sampling(max_new_tokens=3, temperature=0.0), f"r{i}")
                   for i in range(5)]
        assert [f.result(timeout=10).output_ids for f in futures] == [[7, 7, 7]] * 5
        results = engine.generate([[1, 2], [3]], Sampling(max_new_tokens=2, temperature=0.0))
        assert [r.finish_reason for r in results] == ["length", "length"]
    finally:
        engine.close()


# ---- running ahead: the next step is queued before the last one's tokens are read -----------

class DeviceTableRunner(FakeRunner):
    """A fake step function that also keeps the 'device' table of last sampled tokens: a
    token given as PENDING is looked up there, as the embedding kernel does."""

    def __init__(self, *args, **kw):
        super().__init__(*args, **kw)
        self.chosen = {}
        self.logit_slots = None

    def step(self, entries):
        from pylon_amd.engine.batch import PENDING

        ready = super().step(entries)
        seen = []
        for e, record in zip(entries, self.steps[-1]):
            seen.append((record[0], [self.chosen[e.seq.slot] if t == PENDING else t for t in e.tokens],
                         record[2], [t == PENDING for t in e.tokens]))
        self.steps[-1] = seen
        self.logit_slots = [e.seq.slot for e in entries if e.want]
        return ready


class LaggedSampler(ScriptedSampler):
    """Writes the device table at once (stream order) but counts how often the host reads."""

    def __init__(self):
        super().__init__()
        self.reads = 0

    def launch(self, logits, rows, *, chosen, place):
        ids = self.sample(logits, rows)
        for slot, token in zip(place, ids):
            chosen[slot] = token
        sampler = self

        class Draw:
            def result(self):
                sampler.reads += 1
                return ids

        return Draw()


def make_ahead_engine(pages=8, slots=8, chunk=2048, **kw):
    runner = DeviceTableRunner(pages, max_requests=slots, **kw)
    clock = Clock()
    config = PylonConfig(max_batch_size=slots, prefill_chunk_size=chunk, page_size=PAGE)
    engine = Engine(config, runner=runner, sampler=LaggedSampler(), clock=clock)
    assert engine._run_ahead
    return engine, runner, clock


def test_run_ahead_feeds_tokens_from_the_device_and_length_costs_no_extra_step():
    engine, runner, _ = make_ahead_engine(chunk=4)
    engine.sampler.scripts["a"] = [3, 4, 5]
    future = enqueue(engine, "a", list(range(6)), 3)
    engine.tick()  # portion of 4: nothing sampled
    engine.tick()  # portion of 2, first token sampled, not read yet
    assert engine.sampler.reads == 0 and len(runner.steps) == 2
    engine.tick()  # decode step queued with the token still "on the device"; then token 0 read
    assert runner.steps[2] == [("a", [3], [0], [True])]
    assert engine.sampler.reads == 1
    engine.run_until_idle()
    # prompt in two portions + two decode steps: the third token ends the request by length,
    # which is known beforehand, so no further step was queued
    assert len(runner.steps) == 4
    assert runner.steps[3] == [("a", [4], [0], [True])]
    result = future.result(timeout=0)
    assert result.output_ids == [3, 4, 5] and result.finish_reason == "length"
    assert [call[0][1] for call in engine.sampler.calls] == [0, 1, 2]  # the draws' numbers
    assert runner.manager.free_pages == 8 and not runner.manager.live_sequences()
    runner.manager.check()


def test_run_ahead_sees_a_stop_token_one_step_late_and_drops_that_step():
    engine, runner, _ = make_ahead_engine()
    engine.sampler.scripts["a"] = [3, 9, 6, 6]
    engine.sampler.scripts["b"] = [1, 2, 3, 4]
    fa = enqueue(engine, "a", [1, 2, 3], 8, eos=9)
    fb = enqueue(engine, "b", [4, 5], 4)
    engine.run_until_idle()
    assert fa.result(timeout=0).output_ids == [3] and fa.result(timeout=0).finish_reason == "eos"
    assert fb.result(timeout=0).output_ids == [1, 2, 3, 4]
    # a was given exactly one step after the one that sampled its stop token
    a_steps = [row for step in runner.steps for row in step if row[0] == "a"]
    assert [tokens for _, tokens, _, _ in a_steps] == [[1, 2, 3], [3], [9]]
    b_steps = [row for step in runner.steps for row in step if row[0] == "b"]
    assert [tokens for _, tokens, _, _ in b_steps] == [[4, 5], [1], [2], [3]]
    assert runner.manager.free_pages == 8 and not runner.manager.live_sequences()
    runner.manager.check()


def test_run_ahead_matches_the_tick_by_tick_engine():
    scripts = {"a": [5, 6, 7, 9, 1], "b": [2, 2, 2, 2, 2, 2], "c": [9]}
    outputs = []
    for ahead in (False, True):
        engine, runner, _ = (make_ahead_engine if ahead else make_engine)(chunk=4)
        engine.sampler.scripts.update({k: list(v) for k, v in scripts.items()})
        futures = [enqueue(engine, "a", list(range(9)), 6, eos=9), enqueue(engine, "b", [1], 5),
                   enqueue(engine, "c", [3, 3], 3, eos=9)]
        engine.run_until_idle()
        outputs.append([(f.result(timeout=0).output_ids, f.result(timeout=0).finish_reason) for f in futures])
        assert runner.manager.free_pages == 8
    assert outputs[0] == outputs[1] == [([5, 6, 7], "eos"), ([2, 2, 2, 2, 2], "length"), ([], "eos")]


def test_run_ahead_cancellation_and_failure_with_a_step_in_flight():
    engine, runner, _ = make_ahead_engine()
    fa = enqueue(engine, "a", [1, 2], 8)
    fb = enqueue(engine, "b", [3], 8)
    engine.tick()
    engine.tick()  # a decode step is in flight
    # cancel is refused for a running future; the engine's own cancellation path is the flag
    fa.cancel()
    runner.fail_next = OutOfPages("no free page")
    engine.tick()
    with pytest.raises(OutOfPages):
        fb.result(timeout=0)
    assert fa.done()
    assert engine._flight is None and not ids(engine, "active")
    assert runner.manager.free_pages == 8 and not runner.manager.live_sequences()
    runner.manager.check()
    # and the engine goes on
    fc = enqueue(engine, "c", [1], 2)
    engine.run_until_idle()
    assert fc.result(timeout=0).output_ids == [7, 7]


def test_a_request_without_a_seed_gets_one_of_its_own_and_a_given_seed_is_kept():
    engine, runner, clock = make_engine()
    seen = {}

    class Recording(ScriptedSampler):
        def sample(self, logits, rows):
            for rid, (sampling, _index) in zip(logits, rows):
                seen.setdefault(rid, set()).add(sampling.seed)
            return super().sample(logits, rows)

    engine.sampler = Recording()
    hot = Sampling(max_new_tokens=3, temperature=0.8)
    futures = [engine.enqueue([1, 2, 3], None, hot, "a"), engine.enqueue([1, 2, 3], None, hot, "b"),
               engine.enqueue([1, 2, 3], None, Sampling(max_new_tokens=3, temperature=0.8, seed=5), "c"),
               engine.enqueue([1, 2, 3], None, Sampling(max_new_tokens=3, temperature=0.8, seed=5), "d")]
    engine.run_until_idle()
    assert all(f.done() for f in futures)
    (a,), (b,) = seen["a"], seen["b"]  # one seed for the whole of a request
    assert a != b and a is not None and b is not None  # two unseeded equal prompts differ
    assert seen["c"] == {5} and seen["d"] == {5}  # a given seed is kept, so it repeats
    with pytest.raises(ValueError):
        Sampling(seed=-1)


def test_results_carry_the_reference_timing_fields():
    # /root/reference/src/pylon/engine.py:59-74, 598-618: first_token_at on the engine's clock,
    # token_intervals between emitted tokens (one fewer than the tokens)
    engine, runner, clock = make_engine()
    future = enqueue(engine, "a", [1, 2, 3], 4)
    while engine.tick():
        clock.now += 0.25
    result = future.result()
    assert len(result.output_ids) == 4 and len(result.token_intervals) == 3
    assert result.first_token_at == pytest.approx(1000.0 + result.first_token_seconds)
    assert all(abs(dt - 0.25) < 1e-9 for dt in result.token_intervals)


def test_enqueue_and_snapshot_do_not_wait_for_a_step():
    """A tick waits for the device only while it reads a step's tokens, and it holds no lock
    then: a request arrives, and the engine's state can be read, while that wait lasts."""
    import threading

    release, waiting = threading.Event(), threading.Event()

    class SlowSampler(ScriptedSampler):
        def launch(self, logits, rows, **_):
            ids = self.sample(logits, rows)

            class Draw:
                def result(self):
                    waiting.set()
                    assert release.wait(10)
                    return ids

            return Draw()

    config = PylonConfig(max_batch_size=4, page_size=PAGE, run_ahead=False)
    engine = Engine(config, runner=FakeRunner(8), sampler=SlowSampler(), clock=Clock())
    first = enqueue(engine, "first", [1, 2, 3], 2)
    ticker = threading.Thread(target=engine.tick)
    ticker.start()
    try:
        assert waiting.wait(10)  # the tick is inside its wait for the device
        done = threading.Event()
        box = {}

        def arrive():
            box["future"] = enqueue(engine, "second", [4, 5], 1)
            box["snapshot"] = engine.snapshot()
            done.set()

        threading.Thread(target=arrive).start()
        assert done.wait(2), "enqueue waited for the step"
        assert box["snapshot"]["waiting"] == ["second"] and box["snapshot"]["active"] == ["first"]
    finally:
        release.set()
        ticker.join(10)
    engine.run_until_idle()
    assert first.result(timeout=1).output_ids == [7, 7] and box["future"].result(timeout=1).output_ids == [7]
