"""The scheduler's decisions, with a step function that needs no GPU: the
next token is a fixed function of all tokens before it, so any mistake in
cutting, ordering, setting back or finishing changes the output."""

import pytest

from rvllm_amd.cache import CacheManager, OutOfPages
from rvllm_amd.engine.scheduler import Request, RequestState, Scheduler, SchedulerError
from rvllm_amd.parts.base import KVNeed
from rvllm_amd.sampling.params import SamplingParams

VOCAB = 97


def next_token(tokens):
    h = 7
    for t in tokens:
        h = (h * 31 + t + 1) % 1000003
    return h % VOCAB


def expected_output(prompt, n, eos=()):
    seq, out = list(prompt), []
    for _ in range(n):
        t = next_token(seq)
        out.append(t)
        seq.append(t)
        if t in eos:
            break
    return out


class FakeRunner:
    """Keeps the cache's books as the real step does and checks that every
    request's tokens arrive once, in order."""

    def __init__(self, cache):
        self.cache = cache
        self.seen = {}
        self.steps = []

    def step(self, plan):
        entries = [(p.request.id, p.request.tokens[p.start:p.start + p.count], p.wants_token) for p in plan.portions]
        self.cache.require([(rid, self.cache.length(rid) + len(toks)) for rid, toks, _ in entries])
        out = {}
        for rid, toks, wants in entries:
            start = self.cache.length(rid)
            if start == 0:
                self.seen[rid] = []
            assert start == len(self.seen[rid]), "tokens must continue where the cache ends"
            self.cache.extend(rid, start + len(toks))
            self.seen[rid] += toks
            self.cache.commit(rid, start + len(toks))
            if wants:
                out[rid] = next_token(self.seen[rid])
        self.steps.append([(rid, len(toks)) for rid, toks, _ in entries])
        self.cache.check()
        return out


def build(num_pages=64, page_size=4, window=8, max_num_seqs=4, budget=16, chunk=8, max_model_len=256):
    cache = CacheManager([KVNeed(1, 8, window), KVNeed(1, 8, None)], page_size, num_pages, max_num_seqs)
    sched = Scheduler(cache, max_num_seqs, budget, chunk, max_model_len)
    return sched, FakeRunner(cache)


def run(sched, runner, limit=2000):
    done = {}
    for _ in range(limit):
        if not sched.has_work():
            break
        plan = sched.schedule()
        for r in plan.ended:
            done[r.id] = r
        if plan.portions:
            for r in sched.commit(plan, runner.step(plan)):
                done[r.id] = r
    assert not sched.has_work(), "the scheduler did not finish"
    return done


def test_prompt_is_cut_into_portions_under_the_budget():
    sched, runner = build(budget=16, chunk=8)
    sched.add(Request("a", list(range(1, 21)), max_new_tokens=3))
    done = run(sched, runner)
    assert runner.steps[:3] == [[("a", 8)], [("a", 8)], [("a", 4)]]
    assert runner.steps[3:] == [[("a", 1)], [("a", 1)]]  # the last token chosen is never run
    assert done["a"].output == expected_output(range(1, 21), 3) and done["a"].finish_reason == "length"


def test_decodes_come_first_and_prompts_fill_the_rest():
    sched, runner = build(budget=10, chunk=8)
    sched.add(Request("a", [1, 2, 3], max_new_tokens=6))
    plan = sched.schedule()
    sched.commit(plan, runner.step(plan))
    sched.add(Request("b", list(range(1, 30)), max_new_tokens=2))
    plan = sched.schedule()
    # a decodes one token, b gets a portion beside it, within the budget
    assert [(p.request.id, p.count, p.wants_token) for p in plan.portions] == [("a", 1, True), ("b", 8, False)]
    assert plan.num_tokens <= 10
    sched.commit(plan, runner.step(plan))
    done = run(sched, runner)
    assert done["a"].output == expected_output([1, 2, 3], 6)
    assert done["b"].output == expected_output(range(1, 30), 2)


def test_budget_is_shared_between_prompts():
    sched, runner = build(budget=12, chunk=8)
    sched.add(Request("a", list(range(1, 11)), max_new_tokens=1))
    sched.add(Request("b", list(range(1, 11)), max_new_tokens=1))
    plan = sched.schedule()
    assert [(p.request.id, p.count) for p in plan.portions] == [("a", 8), ("b", 4)]


def test_max_num_seqs_limits_admission():
    sched, runner = build(max_num_seqs=2)
    for name in "abc":
        sched.add(Request(name, [1, 2], max_new_tokens=2))
    plan = sched.schedule()
    assert [p.request.id for p in plan.portions] == ["a", "b"] and len(sched.waiting) == 1
    sched.commit(plan, runner.step(plan))
    done = run(sched, runner)
    assert set(done) == {"a", "b", "c"}


def test_eos_stops_and_ignore_eos_does_not():
    prompt = [5, 6, 7]
    full = expected_output(prompt, 12)
    eos = full[4]
    first = full.index(eos)
    sched, runner = build()
    sched.add(Request("a", prompt, max_new_tokens=12, eos_ids=frozenset([eos])))
    sched.add(Request("b", prompt, max_new_tokens=12, eos_ids=frozenset([eos]), ignore_eos=True))
    done = run(sched, runner)
    assert done["a"].output == full[:first + 1] and done["a"].finish_reason == "stop"
    assert done["b"].output == full and done["b"].finish_reason == "length"


def test_a_step_that_finds_no_token_ends_its_request_with_an_error():
    """The device's choice is -1 where a row of logits holds no number: the request ends with what it has and
    gives its pages back; the others go on."""
    prompt = [5, 6, 7]
    sched, runner = build()
    sched.add(Request("a", prompt, max_new_tokens=6))
    sched.add(Request("b", prompt, max_new_tokens=6))
    done = {}
    steps = 0
    while sched.has_work():
        plan = sched.schedule()
        if plan.portions:
            chosen = runner.step(plan)
            steps += 1
            if steps == 3 and "a" in chosen:
                chosen["a"] = -1
            for r in sched.commit(plan, chosen):
                done[r.id] = r
    assert done["a"].finish_reason == "error" and done["a"].output == expected_output(prompt, 6)[:len(done["a"].output)]
    assert 0 < len(done["a"].output) < 6 and all(t >= 0 for t in done["a"].output)
    assert done["b"].output == expected_output(prompt, 6) and done["b"].finish_reason == "length"
    assert not sched.cache.has_request("a")


def test_context_limit_bounds_new_tokens():
    sched, runner = build(max_model_len=12)
    sched.add(Request("a", list(range(1, 10)), max_new_tokens=50))
    done = run(sched, runner)
    assert len(done["a"].output) == 3  # 9 + 3 = 12 (worker.rs:1067-1080)
    with pytest.raises(SchedulerError, match="max_model_len"):
        sched.add(Request("b", list(range(12)), max_new_tokens=1))


def test_bad_requests_are_refused():
    sched, _ = build()
    sched.add(Request("a", [1], max_new_tokens=1))
    with pytest.raises(SchedulerError, match="duplicate"):
        sched.add(Request("a", [1], max_new_tokens=1))
    with pytest.raises(SchedulerError, match="empty"):
        sched.add(Request("b", [], max_new_tokens=1))
    with pytest.raises(SchedulerError, match="max_new_tokens"):
        sched.add(Request("c", [1], max_new_tokens=0))
    with pytest.raises(ValueError):
        sched.add(Request("d", [1], SamplingParams(temperature=-1.0)))


def test_pages_run_out_latest_request_is_set_back_and_output_is_unchanged():
    # 10 pages of 4 tokens; three requests that need 5 + 5 + 5 pages in the full group by their end
    prompts = {"a": list(range(1, 9)), "b": list(range(11, 19)), "c": list(range(21, 29))}
    sched, runner = build(num_pages=10, page_size=4, budget=32, chunk=8, max_num_seqs=3)
    for name, p in prompts.items():
        sched.add(Request(name, p, max_new_tokens=12))
    done = run(sched, runner)
    for name, p in prompts.items():
        assert done[name].output == expected_output(p, 12), name
    assert sum(r.set_backs for r in done.values()) >= 1
    # the oldest request is never the one set back
    assert done["a"].set_backs == 0
    assert runner.cache.free_pages() == {"window8": 10, "full": 10}


def test_set_back_request_resumes_its_random_stream():
    prompts = {"a": list(range(1, 9)), "b": list(range(11, 19))}
    sched, runner = build(num_pages=6, page_size=4, budget=32, chunk=8, max_num_seqs=2)
    reqs = {n: Request(n, p, SamplingParams(0.8, 10, 1.0, seed=3), max_new_tokens=10) for n, p in prompts.items()}
    for r in reqs.values():
        sched.add(r)
    done = run(sched, runner)
    assert done["b"].set_backs >= 1
    assert reqs["b"].rng.state == 3  # the fake step draws nothing: the stream was neither reset nor replaced
    assert done["b"].output == expected_output(prompts["b"], 10)


def test_a_request_too_large_for_the_pool_ends_with_capacity():
    sched, runner = build(num_pages=3, page_size=4, budget=32, chunk=8)
    sched.add(Request("a", list(range(1, 9)), max_new_tokens=20))  # 8 + 20 tokens need 7 pages
    sched.add(Request("b", [1, 2], max_new_tokens=2))
    done = run(sched, runner)
    assert done["a"].finish_reason == "capacity" and len(done["a"].output) < 20
    assert done["a"].output == expected_output(range(1, 9), len(done["a"].output))
    assert done["b"].output == expected_output([1, 2], 2) and done["b"].finish_reason == "length"
    assert runner.cache.free_pages() == {"window8": 3, "full": 3}
    small, _ = build(num_pages=1, page_size=4, chunk=8)
    with pytest.raises(SchedulerError, match="does not fit"):
        small.add(Request("c", list(range(1, 40)), max_new_tokens=1))  # its first portion alone needs two pages


def test_state_changes_only_after_the_step():
    sched, runner = build()
    req = Request("a", [1, 2, 3], max_new_tokens=2)
    sched.add(req)
    plan = sched.schedule()
    assert req.state is RequestState.RUNNING and req.computed == 0 and req.output == []
    sched.commit(plan, runner.step(plan))
    assert req.computed == 3 and len(req.output) == 1


def test_a_requests_tokens_from_a_place_on():
    from rvllm_amd.engine.scheduler import Request

    req = Request("r", [1, 2, 3, 4], output=[5, 6, 7])
    for start in range(7):
        for count in range(1, 8 - start):
            assert req.tokens_at(start, count) == req.tokens[start:start + count], (start, count)


# ---- the engine's loop around a step that fails -----------------------------------------------------------
class FailingRunner:
    """What ``LLMEngine`` asks of a runner, without a GPU: the cache's books are kept as the real step keeps
    them; a step that holds a token of ``poison`` extends the cache and then raises, as a kernel error or a
    sampler that meets logits that are no numbers would.  Its 'logits' are the next tokens themselves."""

    def __init__(self, cache, config, poison):
        import types

        self.cache, self.config, self.poison, self.device = cache, config, poison, "cpu"
        self.model = types.SimpleNamespace(spec=types.SimpleNamespace(vocab_size=VOCAB))
        self.storage = types.SimpleNamespace(clear_slot=lambda slot: None)
        self.seen = {}

    def step(self, entries, starts=None):
        self.cache.extend_all([(rid, self.cache.length(rid) + len(toks)) for rid, toks, _ in entries])
        if any(self.poison in toks for _, toks, _ in entries):
            raise RuntimeError("the step failed")
        out = []
        for rid, toks, want in entries:
            start = self.cache.length(rid)
            self.seen[rid] = (self.seen[rid] if start else []) + list(toks)
            self.cache.commit(rid, start + len(toks))
            if want:
                out.append(next_token(self.seen[rid]))
        return out


    def decode_ahead(self, entries, steps, choose=None):
        """Several decode steps from one plan: pages for all of them are taken first, as the real runner does."""
        self.cache.extend_all([(rid, self.cache.length(rid) + steps) for rid, _ in entries])
        if any(token == self.poison for _, token in entries):
            raise RuntimeError("the steps ahead failed")
        rows = []
        tokens = [token for _, token in entries]
        for _ in range(steps):
            for (rid, _), token in zip(entries, tokens):
                self.seen[rid].append(token)
            tokens = [next_token(self.seen[rid]) for rid, _ in entries]
            rows.append(tokens)
        for rid, _ in entries:
            self.cache.commit(rid, self.cache.length(rid) + steps)
        return rows


class PassThroughSampler:
    vocab_size = VOCAB

    def sample(self, logits, params, rngs):
        return list(logits)


def test_a_step_that_fails_ends_its_requests_and_the_others_go_on():
    import types

    from rvllm_amd.config.engine_config import EngineConfig
    from rvllm_amd.engine.engine import LLMEngine

    cache = CacheManager([KVNeed(1, 8, 8), KVNeed(1, 8, None)], 4, 64, 4)
    config = EngineConfig(max_model_len=256, max_num_seqs=2, max_num_batched_tokens=16, max_prefill_chunk=8,
                          greedy_steps_ahead=1, page_size=16)
    free_at_first = dict(cache.free_pages())
    engine = LLMEngine(FailingRunner(cache, config, poison=90))
    engine.sampler = PassThroughSampler()
    good, bad, late = [1, 2, 3], [4, 5, 90, 6], [7, 8, 9, 10, 11]
    engine.add_request("good", good, max_new_tokens=1)
    engine.add_request("bad", bad, max_new_tokens=4)
    engine.add_request("late", late, max_new_tokens=3)  # waits: two places only
    # the first step holds both prompts; "good" would end in it (one new token), "bad" makes it fail
    with pytest.raises(RuntimeError, match="the step failed"):
        engine.step()
    assert not cache.has_request("good") and not cache.has_request("bad")  # their pages are back
    assert cache.free_pages() == free_at_first
    done = {}
    while engine.has_work():
        for res in engine.step():
            done[res.request_id] = res
    assert done["good"].finish_reason == "error" and done["bad"].finish_reason == "error"
    assert done["good"].tokens == [] and done["bad"].tokens == []
    assert done["late"].finish_reason == "length" and done["late"].tokens == expected_output(late, 3)
    assert cache.free_pages() == free_at_first
    cache.check()
    # nothing is handed out twice
    assert engine.step() == []


def test_steps_ahead_that_fail_end_their_requests_too():
    from rvllm_amd.config.engine_config import EngineConfig
    from rvllm_amd.engine.engine import LLMEngine

    cache = CacheManager([KVNeed(1, 8, 8), KVNeed(1, 8, None)], 4, 64, 4)
    config = EngineConfig(max_model_len=256, max_num_seqs=2, max_num_batched_tokens=16, max_prefill_chunk=8,
                          greedy_steps_ahead=4, page_size=16)
    free_at_first = dict(cache.free_pages())
    prompt, other = [2, 5, 6], [9, 8, 7, 6]
    poison = expected_output(prompt, 6)[4]  # the fifth new token, which the second plan of steps ahead starts from
    assert poison not in expected_output(prompt, 4) and poison not in expected_output(other, 12) + prompt + other
    engine = LLMEngine(FailingRunner(cache, config, poison))
    engine.sampler = PassThroughSampler()
    engine.add_request("a", prompt, max_new_tokens=12)
    engine.add_request("late", other, max_new_tokens=3)
    engine.scheduler.max_num_seqs = 1  # "late" waits until "a" is gone; nobody waits for a place that is free
    with pytest.raises(RuntimeError, match="the steps ahead failed"):
        while engine.has_work():
            assert engine.step() == []
    assert engine.plans < engine.steps  # steps ahead did run before
    assert not cache.has_request("a") and cache.free_pages() == free_at_first
    engine.scheduler.max_num_seqs = 2
    done = {}
    while engine.has_work():
        for res in engine.step():
            done[res.request_id] = res
    assert done["a"].finish_reason == "error" and done["a"].tokens == expected_output(prompt, 5)
    assert done["late"].tokens == expected_output(other, 3)
    cache.check()
