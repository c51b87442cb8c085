"""The engine: scheduler, model runner and sampler in one loop.

    engine = LLMEngine.from_model_dir(folder, EngineConfig(...))
    engine.add_request("a", prompt_ids, SamplingParams(), max_new_tokens=32)
    while engine.has_work():
        for finished in engine.step():
            ...

Each step: plan (scheduler), run the planned tokens as one batch (runner.step),
choose the next tokens (sampler), commit (scheduler).  The request's state
changes only after its step has run, as in the reference's engine shell
(v3/crates/rvllm-runtime/src/engine.rs:93-143).
"""

from __future__ import annotations

import dataclasses
import os
import time
from typing import Hashable, Iterable, Optional, Sequence

import torch

from ..config.engine_config import EngineConfig
from ..sampling.params import SamplingParams
from ..sampling.sampler import DeviceDraws, Sampler
from .runner import ModelRunner
from .scheduler import PlannedPortion, Request, RequestState, Scheduler, StepPlan


@dataclasses.dataclass
class GenerationResult:
    request_id: Hashable
    prompt: list[int]
    tokens: list[int]
    finish_reason: str  # "stop" (an end-of-sequence id), "length", "capacity", or "error" (its step failed)
    set_backs: int = 0


class LLMEngine:
    def __init__(self, runner: ModelRunner):
        self.runner = runner
        cfg = runner.config
        self.scheduler = Scheduler(runner.cache, cfg.max_num_seqs, cfg.max_num_batched_tokens, cfg.max_prefill_chunk,
                                   cfg.max_model_len, on_admit=self._on_admit)
        self.sampler = Sampler(runner.model.spec.vocab_size)
        if cfg.tune_products and cfg.dtype == "bfloat16":
            runner.tune_products()
        self._held_back: list[GenerationResult] = []  # results of a step that failed, handed out by the next one
        self.steps = 0
        self.plans = 0  # plans that ran something; fewer than steps when greedy steps followed one another
        self.tokens_run = 0

    @classmethod
    def from_model_dir(cls, model_dir: str | os.PathLike, config: Optional[EngineConfig] = None) -> "LLMEngine":
        return cls(ModelRunner.from_model_dir(model_dir, config or EngineConfig()))

    @classmethod
    def from_random(cls, model_config, seed: int, config: Optional[EngineConfig] = None) -> "LLMEngine":
        return cls(ModelRunner.from_random(model_config, seed, config or EngineConfig()))

    def _on_admit(self, request_id: Hashable) -> None:
        self.runner.storage.clear_slot(self.runner.cache.slot(request_id))

    # ---- requests ----------------------------------------------------
    def add_request(self, request_id: Hashable, prompt: Sequence[int], params: Optional[SamplingParams] = None,
                    max_new_tokens: int = 16, eos_ids: Iterable[int] = (), ignore_eos: bool = False) -> Request:
        vocab = self.runner.model.spec.vocab_size
        prompt = [int(t) for t in prompt]
        for t in prompt:
            if not 0 <= t < vocab:
                raise ValueError(f"token id {t} outside the vocabulary of {vocab}")
        params = (params or SamplingParams()).validate()
        if not params.is_greedy():
            params.kernel_k(vocab)  # a draw over a large vocabulary needs an explicit top_k
        req = Request(request_id, prompt, params, int(max_new_tokens), frozenset(int(e) for e in eos_ids), ignore_eos)
        self.scheduler.add(req)
        return req

    def has_work(self) -> bool:
        return self.scheduler.has_work()

    # ---- one step --------------------------------------------------------
    def step(self) -> list[GenerationResult]:
        """Plans and runs one step; returns the requests that ended in it.  If the step fails (the model, the
        sampler) the exception goes to the caller after the plan's requests have ended with the reason
        ``error`` and given their pages back; their results, and those of requests that had ended in this step
        before, come with the next call, and the requests that were not in the plan go on."""
        plan = self.scheduler.schedule()
        results, self._held_back = self._held_back + [self._result(r) for r in plan.ended], []
        if not plan.portions:
            return results
        entries = []
        wanting = []
        for p in plan.portions:
            tokens = p.request.tokens_at(p.start, p.count)
            entries.append((p.request.id, tokens, [p.count - 1] if p.wants_token else []))
            if p.wants_token:
                wanting.append(p.request)
        self.plans += 1
        try:
            ahead = self._steps_ahead(plan)
            if ahead > 1:
                return results + self._decode_ahead(plan, ahead)
            logits = self.runner.step(entries, starts=[p.start for p in plan.portions])
            self.steps += 1
            self.tokens_run += plan.num_tokens
            chosen = self.sampler.sample(logits, [r.params for r in wanting], [r.rng for r in wanting])
        except Exception:
            # The cache may hold this step's tokens while the requests do not count them (the sampler refuses
            # logits that are not finite, for one; steps run ahead have taken pages for tokens that were never
            # chosen): the plan's requests end here, so that nothing is run twice or a portion further on.
            self._held_back = results
            for p in plan.portions:
                if p.request.state is not RequestState.FINISHED:
                    self.scheduler.abort(p.request, "error")
                    self._held_back.append(self._result(p.request))
            raise
        next_tokens = {r.id: t for r, t in zip(wanting, chosen)}
        finished = self.scheduler.commit(plan, next_tokens)
        return results + [self._result(r) for r in finished]

    # ---- several decode steps from one plan ------------------------------
    def _steps_ahead(self, plan: StepPlan) -> int:
        """How many decode steps may follow one another from this plan: more
        than one only if every request in it decodes one token and gets its
        next one chosen on the device (the arg-max, or a draw as the host
        draws), none could end by its length or the model's on the
        way, nothing was set back, and no request waits for which there is a
        place (it would be admitted that much later; with every place taken,
        the most a waiting request can lose is the few steps by which an end
        id is noticed late).  A request that meets an end id on the way stops
        there; what was run for it after that is dropped, its stream of
        numbers stands after its last token's draw, and it costs the others
        nothing."""
        ahead = self.runner.config.greedy_steps_ahead
        if ahead <= 1 or plan.set_back:
            return 1
        if self.scheduler.waiting and len(self.scheduler.running) < self.scheduler.max_num_seqs:
            return 1
        for p in plan.portions:
            req = p.request
            if p.count != 1 or not p.wants_token:
                return 1
            ahead = min(ahead, req.max_new_tokens - len(req.output), self.scheduler.max_model_len - req.total)
        # requests that sample are drawn for on the device (not with parameters that the host's draw refuses too)
        params = [p.request.params for p in plan.portions]
        if not all(sp.is_greedy() for sp in params) and not DeviceDraws.usable(self.sampler.vocab_size, params):
            return 1
        return max(1, ahead)

    def _decode_ahead(self, plan: StepPlan, ahead: int) -> list[GenerationResult]:
        requests = [p.request for p in plan.portions]
        choose = None
        if not all(r.params.is_greedy() for r in requests):
            choose = DeviceDraws(self.sampler.vocab_size, [r.params for r in requests], [r.rng for r in requests],
                                 self.runner.device)
        rows = self.runner.decode_ahead([(p.request.id, p.request.tokens_at(p.start, 1)[0]) for p in plan.portions],
                                        ahead, choose)
        finished: list[Request] = []
        for i, row in enumerate(rows):
            live = [(p, token) for p, token in zip(plan.portions, row) if p.request.state is RequestState.RUNNING]
            if not live:
                break
            self.steps += 1
            self.tokens_run += len(live)
            step_plan = StepPlan([PlannedPortion(p.request, p.start + i, 1, True) for p, _ in live], [], [])
            for p, token in live:
                if token >= 0 and not p.request.params.is_greedy():
                    p.request.rng.next_u64()  # the draw that the device made for this token
            finished += self.scheduler.commit(step_plan, {p.request.id: token for p, token in live})
        return [self._result(r) for r in finished]

    @staticmethod
    def _result(req: Request) -> GenerationResult:
        return GenerationResult(req.id, list(req.prompt), list(req.output), req.finish_reason or "length",
                                req.set_backs)

    # ---- whole requests ----------------------------------------------------
    def generate(self, prompts: Sequence[Sequence[int]], params=None, max_new_tokens: int = 16,
                 eos_ids: Iterable[int] = (), ignore_eos: bool = False) -> list[GenerationResult]:
        """Runs all prompts to their end; results in the order of the prompts.
        ``params`` is one SamplingParams for all, or one per prompt."""
        if params is None or isinstance(params, SamplingParams):
            params = [params] * len(prompts)
        base = f"gen{id(prompts):x}-"
        for i, (prompt, sp) in enumerate(zip(prompts, params)):
            self.add_request(f"{base}{i}", prompt, sp, max_new_tokens, eos_ids, ignore_eos)
        done: dict = {}
        while self.has_work():
            for res in self.step():
                done[res.request_id] = res
        return [done[f"{base}{i}"] for i in range(len(prompts))]
