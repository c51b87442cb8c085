"""The scheduler: admits requests, cuts prompts into portions under a token
budget, decodes, finishes and frees.

States and the rule that a request's state changes only after the step that
was planned for it has run come from the reference's scheduler shell
(v3/crates/rvllm-runtime/src/sched_state.rs:9-81, scheduler.rs:154-198,
engine.rs:93-143).  Unlike the reference (scheduler.rs:3-5) a step here mixes
decoded tokens and portions of prompts: every step first takes one token from
each request that is decoding, then fills what is left of the budget with
portions of prompts, oldest request first.

When pages run out (the reference declares ``KvExhausted`` and a recompute
mode, error.rs:243, config/runtime.rs:7-10, and uses neither): the request
admitted last is set back — its pages are given back and it waits at the head
of the queue; when it is admitted again it runs its prompt and the tokens it
had produced as one new prompt, and goes on where it was.  A request that
runs alone and still does not fit ends with the reason ``capacity``.
"""

from __future__ import annotations

import collections
import dataclasses
import enum
import itertools
from typing import Callable, Hashable, Optional, Sequence

from ..cache.manager import CacheManager
from ..sampling.params import SamplingParams
from ..sampling.sampler import SplitMix64


class RequestState(enum.Enum):
    WAITING = "waiting"
    RUNNING = "running"
    FINISHED = "finished"


class SchedulerError(ValueError):
    pass


@dataclasses.dataclass
class Request:
    id: Hashable
    prompt: list[int]
    params: SamplingParams = dataclasses.field(default_factory=SamplingParams)
    max_new_tokens: int = 16
    eos_ids: frozenset = frozenset()
    ignore_eos: bool = False
    output: list[int] = dataclasses.field(default_factory=list)
    state: RequestState = RequestState.WAITING
    finish_reason: Optional[str] = None
    computed: int = 0  # tokens of prompt + output whose keys are in the cache
    set_backs: int = 0
    rng: SplitMix64 = None  # type: ignore[assignment]

    def __post_init__(self):
        if self.rng is None:
            self.rng = SplitMix64(self.params.seed)

    @property
    def tokens(self) -> list[int]:
        return self.prompt + self.output

    def tokens_at(self, start: int, count: int) -> list[int]:
        """``tokens[start : start + count]`` without joining the lists (a step asks every request for its next
        tokens, and a long request's whole list is long)."""
        n = len(self.prompt)
        if start >= n:
            return self.output[start - n : start - n + count]
        if start + count <= n:
            return self.prompt[start : start + count]
        return self.prompt[start:] + self.output[: start + count - n]

    @property
    def total(self) -> int:
        return len(self.prompt) + len(self.output)


@dataclasses.dataclass
class PlannedPortion:
    request: Request
    start: int
    count: int
    wants_token: bool  # the portion ends at the request's last token: its logits choose the next one


@dataclasses.dataclass
class StepPlan:
    portions: list[PlannedPortion]
    set_back: list[Request]  # requests that lost their pages while this step was planned
    ended: list[Request]  # requests that ended with reason "capacity"

    @property
    def num_tokens(self) -> int:
        return sum(p.count for p in self.portions)


class Scheduler:
    MAX_REQUESTS = 256  # v3/crates/rvllm-runtime/src/scheduler.rs:53-65

    def __init__(self, cache: CacheManager, max_num_seqs: int, max_num_batched_tokens: int, max_prefill_chunk: int,
                 max_model_len: int, on_admit: Optional[Callable[[Hashable], None]] = None):
        self.cache = cache
        self.max_num_seqs = max_num_seqs
        self.max_num_batched_tokens = max_num_batched_tokens
        self.max_prefill_chunk = max_prefill_chunk
        self.max_model_len = max_model_len
        self.on_admit = on_admit
        self.waiting: collections.deque[Request] = collections.deque()
        self.running: list[Request] = []  # in order of admission
        self.known: dict[Hashable, Request] = {}

    # ---- admission -----------------------------------------------------
    def add(self, request: Request) -> None:
        if request.id in self.known:
            raise SchedulerError(f"duplicate request id {request.id!r}")
        if len(self.waiting) + len(self.running) >= self.MAX_REQUESTS:
            raise SchedulerError(f"more than {self.MAX_REQUESTS} requests in flight")
        if not request.prompt:
            raise SchedulerError("prompt must not be empty")
        if request.max_new_tokens < 1:
            raise SchedulerError("max_new_tokens must be >= 1")
        if len(request.prompt) >= self.max_model_len:
            raise SchedulerError(f"prompt of {len(request.prompt)} tokens does not fit max_model_len "
                                 f"{self.max_model_len}")
        request.params.validate()
        # never more new tokens than the context allows (worker.rs:1067-1080)
        request.max_new_tokens = min(request.max_new_tokens, self.max_model_len - len(request.prompt))
        for name, g in self.cache.groups.items():
            if g.pages_to_add([], min(len(request.prompt), self.max_prefill_chunk)) > g.pool.num_pages:
                raise SchedulerError(f"the first portion of the prompt does not fit page group {name!r}")
        self.known[request.id] = request
        self.waiting.append(request)

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    # ---- planning --------------------------------------------------------
    def schedule(self) -> StepPlan:
        budget = self.max_num_batched_tokens
        portions: list[PlannedPortion] = []
        reserved = self.cache.reservation()  # the pages that the portions planned so far will take
        set_back: list[Request] = []
        ended: list[Request] = []

        def fits(req: Request, new_len: int) -> bool:
            return reserved.fits(req.id, new_len)

        def take(req: Request, count: int) -> None:
            nonlocal budget
            portions.append(PlannedPortion(req, req.computed, count, req.computed + count == req.total))
            reserved.add(req.id, req.computed + count)
            budget -= count

        # Requests that are decoding come first, then prompts under way; both
        # in order of admission.
        order = [r for r in self.running if r.total - r.computed == 1] + \
                [r for r in self.running if r.total - r.computed > 1]
        for req in order:
            if req.state is not RequestState.RUNNING or budget <= 0:
                continue  # set back while an earlier request was planned, or no budget left
            left = req.total - req.computed
            count = min(left, self.max_prefill_chunk if left > 1 else 1, budget)
            room = fits(req, req.computed + count)
            while not room:
                victim = self._latest_running(exclude_planned={p.request.id for p in portions})
                if victim is None or victim is req:
                    break
                self._set_back(victim)
                set_back.append(victim)
                room = fits(req, req.computed + count)
            if room:
                take(req, count)
            elif self._runs_alone(req, portions):
                # nothing else holds pages and it still does not fit
                self._finish(req, "capacity")
                ended.append(req)
            else:
                # others planned in this step hold the pages; wait a step
                continue

        # Admit waiting requests while there is room, oldest first.
        while self.waiting and budget > 0 and len(self.running) < self.max_num_seqs:
            req = self.waiting[0]
            count = min(req.total, self.max_prefill_chunk, budget)
            if not fits(req, count):
                if not self.running and not portions:
                    # alone and still too large for the pool
                    self.waiting.popleft()
                    self._finish(req, "capacity")
                    ended.append(req)
                    continue
                break
            self.waiting.popleft()
            self.cache.add_request(req.id)
            if self.on_admit is not None:
                self.on_admit(req.id)
            req.state = RequestState.RUNNING
            req.computed = 0
            self.running.append(req)
            take(req, count)
        return StepPlan(portions, set_back, ended)

    def _latest_running(self, exclude_planned: set) -> Optional[Request]:
        for req in reversed(self.running):
            if req.id not in exclude_planned:
                return req
        return None

    def _runs_alone(self, req: Request, portions: list[PlannedPortion]) -> bool:
        return all(r is req for r in self.running) and not portions

    def _set_back(self, req: Request) -> None:
        """Recompute later: give everything back and wait at the head of the queue."""
        self.cache.release(req.id)
        self.running.remove(req)
        req.state = RequestState.WAITING
        req.computed = 0
        req.set_backs += 1
        self.waiting.appendleft(req)

    def _finish(self, req: Request, reason: str) -> None:
        if self.cache.has_request(req.id):
            self.cache.release(req.id)
        if req in self.running:
            self.running.remove(req)
        req.state = RequestState.FINISHED
        req.finish_reason = reason
        self.known.pop(req.id, None)

    def abort(self, req: Request, reason: str = "abort") -> None:
        """Ends a request wherever it stands and gives back what it holds."""
        if req.state is RequestState.FINISHED:
            return
        if req in self.waiting:
            self.waiting.remove(req)
        self._finish(req, reason)

    # ---- after the step ----------------------------------------------------
    def commit(self, plan: StepPlan, next_tokens: dict) -> list[Request]:
        """The planned step has run.  ``next_tokens[request id]`` is the token
        chosen for every portion that wanted one.  Returns the requests that
        finished."""
        finished = []
        for p in plan.portions:
            req = p.request
            req.computed = p.start + p.count
            if not p.wants_token:
                continue
            token = int(next_tokens[req.id])
            if token < 0:
                # the device found no token (a row of logits that are not numbers): the request ends here, with
                # what it has, rather than with an id that is none in its output
                self._finish(req, "error")
                finished.append(req)
                continue
            req.output.append(token)
            if not req.ignore_eos and token in req.eos_ids:
                self._finish(req, "stop")
            elif len(req.output) >= req.max_new_tokens or req.total >= self.max_model_len:
                self._finish(req, "length")
            if req.state is RequestState.FINISHED:
                finished.append(req)
        return finished
