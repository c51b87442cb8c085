"""The model runner: one model, its cache, and the step function.

``step`` takes a batch of (request, its next tokens) — portions of prompts
beside single decoded tokens, cut anywhere — runs exactly those tokens as one
batch against the cache, and returns 32-bit logits at the wanted places.  It
is the only way tokens reach the model: generation, the command line and
trace replay all go through it.
"""

from __future__ import annotations

import collections
import dataclasses
import gc
import os
import warnings
from typing import Hashable, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheManager, group_name, window_pages_bound
from ..cache.storage import CacheStorage
from ..config.engine_config import EngineConfig
from ..kernels import ops
from ..models.model import DecoderModel
from ..models.registry import Architecture, get_architecture, load_config
from ..parts.base import KVNeed
from ..weights.loader import load_tensors, open_model_files, tensor_names
from ..weights.random_init import random_tensors
from .batch import BatchBuilder, Portion, StepBatch

_frozen = False


def _freeze_what_exists_once() -> None:
    """What exists when the first engine of a process is built (the interpreter's modules, the libraries' objects)
    lives as long as the process: taken out of the garbage collector's sight, so that a full collection between two
    steps, which would walk all of it (some 100 ms with the libraries loaded here), has little to walk.  Once only:
    what is frozen is never collected, and an engine built and dropped later must still be."""
    global _frozen
    if not _frozen:
        _frozen = True
        gc.collect()
        gc.freeze()


class ModelRunner:
    def __init__(self, model: DecoderModel, engine_config: EngineConfig):
        """``model`` has its weights bound already."""
        self.model = model
        self.config = engine_config.validate()
        self.device = model.device
        self.dtype = model.dtype
        if self.config.max_model_len > model.spec.max_position:
            # the reference caps a request the same way: prompt + new tokens <= min(cache, max_position_embeddings)
            # (v3/crates/rvllm-runtime/src/gemma4_bring_up.rs:271-294)
            warnings.warn(f"max_model_len {self.config.max_model_len} is more than the model's "
                          f"{model.spec.max_position} positions; requests are held to {model.spec.max_position}")
            self.config = dataclasses.replace(self.config, max_model_len=model.spec.max_position)
        cfg = self.config
        ps = cfg.page_size
        needs = model.cache_needs()
        full_pages = max(1, -(-cfg.cache_tokens() // ps))
        num_pages = {}
        for need in needs:
            if isinstance(need, KVNeed):
                name = group_name(need.window)
                if need.window is None:
                    num_pages[name] = full_pages
                else:
                    per_request = window_pages_bound(need.window, ps, cfg.max_num_batched_tokens)
                    num_pages[name] = min(full_pages, cfg.max_num_seqs * per_request)
        self.cache = CacheManager(needs, ps, num_pages, cfg.max_num_seqs)
        self.weight_bytes = model.weight_bytes()
        self.storage = CacheStorage(self.cache, self.device, self.dtype, held_by_weights=self.weight_bytes)
        width = -(-cfg.max_model_len // ps)
        self.builder = BatchBuilder(self.device, cfg.max_num_batched_tokens, cfg.max_num_seqs,
                                    {name: width for name in self.cache.groups})
        # Captured decode steps, by (requests, context bucket).
        self._graphs: collections.OrderedDict[tuple[int, int], tuple] = collections.OrderedDict()
        self._graph_pool = None
        self.graph_replays = 0
        # Whether steps whose products go to the library may come from graphs: only for models that keep nothing
        # but keys and values between steps (replaying such a step writes the same keys and values again, so the
        # check below may replay it; a state that a mixer moves on would be moved on with every replay), and
        # until a recording fails its check.
        self._library_steps_from_graphs = all(need is None or isinstance(need, KVNeed) for need in needs)
        _freeze_what_exists_once()

    # ---- decode steps from captured graphs -------------------------------
    GRAPH_CONTEXT_BUCKET = 1024
    GRAPH_MAX_KEPT = 128     # shapes whose graphs are kept; the one unused for longest goes first
    # Steps of more requests than the few-row product takes hand their products to the library.  A recording of
    # library calls is trusted only after it has shown itself right: it is replayed this many times against the
    # logits of the same step run kernel by kernel (nodes that a library records have given wrong results on
    # replays after the first on this hardware), and if one replay differs no step with library products is
    # taken from a graph again.
    GRAPH_LIBRARY_CHECKS = 3
    GRAPH_LIBRARY_TOLERANCE = 1e-3  # of the largest logit: the library may add in another order, not more

    def _graph_key(self, batch: StepBatch):
        """The key of the captured graph that can run this batch, or None.

        A graph replays launches with fixed grids, so it covers steps of one
        shape: B requests with one token each, logits wanted for all of them,
        contexts up to a bucket's upper end (the attention kernel's split plan
        is made for that end; splits past a request's own context are empty).
        The reference captures its decode step the same way, once per batch
        size (v3/crates/rvllm-runtime/src/gemma4_serve.rs:594-694)."""
        if not batch.decode_only or batch.num_logit_rows != batch.num_tokens:
            return None
        return self._decode_graph_key(batch.num_requests, batch.max_context)

    def _decode_graph_key(self, num_requests: int, max_context: int):
        """The key for a step of ``num_requests`` decoded tokens, all wanted, at contexts up to ``max_context``."""
        if not (self.config.use_graphs and self.dtype == torch.bfloat16):
            return None
        if not self.model.capturable:  # a part waits for the device or launches by its data
            return None
        if num_requests > ops.SKINNY_MAX_ROWS and not self._library_steps_from_graphs:
            return None
        return num_requests, self.context_bucket(max_context)

    @classmethod
    def context_bucket(cls, max_context: int) -> int:
        """The upper end of the bucket of contexts that one captured graph serves.  Buckets are
        GRAPH_CONTEXT_BUCKET wide up to sixteen of them and then double with the context, so that a graph's
        plan is made for at most an eighth more keys than there are, and a batch that decodes from a long
        context to a longer one records a graph every few thousand steps rather than every thousand."""
        width = cls.GRAPH_CONTEXT_BUCKET
        while max_context > 16 * width:
            width *= 2
        return -(-max_context // width) * width

    def _forward(self, batch: StepBatch) -> torch.Tensor:
        key = self._graph_key(batch)
        if key is None:
            return self.model.forward(batch, self.storage.views)
        entry = self._graphs.get(key)
        if entry is None:
            # The first step of a shape runs eagerly and is then recorded
            # (recording runs nothing) for the steps that follow.
            logits = self.model.forward(batch, self.storage.views)
            shaped = dataclasses.replace(batch, max_context=key[1], shared={})  # nothing made outside the recording
            graph = torch.cuda.CUDAGraph()
            torch.cuda.synchronize()
            # No garbage collection while the stream records: an engine dropped earlier in the process may lie
            # in a cycle with its graphs and their memory, and freeing those is not allowed during a recording
            # (the process aborts).  What is garbage now goes before; the collector rests until the recording ends.
            gc.collect()
            collecting = gc.isenabled()
            gc.disable()
            try:
                with torch.cuda.graph(graph, pool=self._graph_pool):
                    static_logits = self.model.forward(shaped, self.storage.views)
            finally:
                if collecting:
                    gc.enable()
            if key[0] > ops.SKINNY_MAX_ROWS and not self._recording_is_right(graph, static_logits, logits):
                # (the graph goes, and with it its memory; it has not lent its pool to the others yet)
                self._library_steps_from_graphs = False
                warnings.warn("a recorded decode step with library products did not reproduce the step run kernel "
                              "by kernel; such steps are no longer taken from graphs")
                return logits
            if self._graph_pool is None:
                self._graph_pool = graph.pool()
            self._graphs[key] = (graph, static_logits)
            while len(self._graphs) > self.GRAPH_MAX_KEPT:
                self._graphs.popitem(last=False)
            return logits
        self._graphs.move_to_end(key)
        graph, static_logits = entry
        graph.replay()
        self.graph_replays += 1
        return static_logits

    def _recording_is_right(self, graph, static_logits: torch.Tensor, logits: torch.Tensor) -> bool:
        """Replays a fresh recording several times, with a wait for the device between the replays, and holds
        every result against the logits of the same step run kernel by kernel."""
        scale = float(logits.abs().max())
        for _ in range(self.GRAPH_LIBRARY_CHECKS):
            graph.replay()
            torch.cuda.synchronize()
            worst = float((static_logits - logits).abs().max())
            if not worst <= self.GRAPH_LIBRARY_TOLERANCE * scale:  # NaN fails too
                return False
        return True

    # ---- construction --------------------------------------------------
    @classmethod
    def from_model_dir(cls, model_dir: str | os.PathLike, engine_config: EngineConfig) -> "ModelRunner":
        """Model class by config.json, weights by name from the folder's safetensors."""
        engine_config.validate()
        ops.library()  # fail now, and loudly, if the kernels cannot be built or loaded
        arch, config = load_config(model_dir)
        files = open_model_files(model_dir)
        try:
            # where the tensors lie in this checkpoint is the architecture's knowledge
            model = DecoderModel(arch.build_spec(config, **arch.locate_tensors(tensor_names(files))))
            tensors = load_tensors(files, model.param_specs(), engine_config.torch_dtype, source=str(model_dir),
                                   ignore=arch.ignored_prefixes)
            model.bind(tensors, engine_config.device, engine_config.torch_dtype, engine_config.tiled_weights)
        finally:
            for f in files:
                f.close()
        return cls(model, engine_config)

    @classmethod
    def from_random(cls, config, seed: int, engine_config: EngineConfig) -> "ModelRunner":
        """Random weights made on the device (no folder is written)."""
        engine_config.validate()
        ops.library()
        arch = get_architecture(config.architecture)
        model = DecoderModel(arch.build_spec(config))
        tensors = random_tensors(model.param_specs(), seed, engine_config.device, engine_config.torch_dtype)
        model.bind(tensors, engine_config.device, engine_config.torch_dtype, engine_config.tiled_weights)
        return cls(model, engine_config)

    # ---- warm-up ------------------------------------------------------
    def warm_up(self, portion_lengths: Sequence[int] = ()) -> None:
        """Runs a throw-away prompt portion of each given length so that what
        is chosen or built at first use is ready before requests arrive.  For
        bf16 the library's matrix products (portions of more than 64 tokens)
        are tuned meanwhile: every algorithm the library has for a shape is
        timed once and the fastest kept (``ops.set_library_tuning``);
        afterwards tuning is switched off again, so a shape met later costs
        no pause and runs on the library's first suggestion.  If the
        environment names a file (``ops.LIBRARY_PLANS_ENV``), the plans in it
        are taken first, and what is tuned now is written there."""
        tune = self.dtype == torch.bfloat16 and any(n > ops.SKINNY_MAX_ROWS for n in portion_lengths)
        plans_file = os.environ.get(ops.LIBRARY_PLANS_ENV) if tune else None
        if plans_file:
            ops.library_plans_load(plans_file, self.device)
        ops.set_library_tuning(tune)
        try:
            for n in portion_lengths:
                n = min(int(n), self.config.max_num_batched_tokens, self.config.max_model_len)
                if n < 1 or not self.cache.can_extend([("__warm_up__", n)]):
                    continue
                self.add_request("__warm_up__")
                try:
                    # as many rows as requests may decode together want their logits, as such a decode step does:
                    # the head's product of that many rows is then met (and tuned) too
                    wanted = list(range(n)) if n <= self.config.max_num_seqs else [n - 1]
                    self.step([("__warm_up__", [0] * n, wanted)])
                finally:
                    self.release("__warm_up__")
            torch.cuda.synchronize(self.device)
        finally:
            ops.set_library_tuning(False)
        if plans_file:
            try:
                ops.library_plans_save(plans_file, self.device)
            except OSError as e:  # a place that cannot be written costs the next start its tuning, not this one its work
                warnings.warn(f"the tuned plans were not written to {plans_file}: {e}")

    def tune_products(self) -> list[int]:
        """Tunes the library's products (``warm_up``) for a ladder of row counts that the steps of this engine
        can bring: from just above the few-row kernel's 64 up to ``max_num_batched_tokens``, each one and a half
        times the one before, and the longest portion of a prompt.  Returns the row counts."""
        top = min(self.config.max_num_batched_tokens, self.config.max_model_len)
        rows, n = set(), 96
        while n < top:
            rows.add(n)
            n = n * 3 // 2
        rows.update(r for r in (top, min(self.config.max_prefill_chunk, top)) if r > ops.SKINNY_MAX_ROWS)
        ladder = sorted(rows)
        self.warm_up(ladder)
        return ladder

    # ---- requests ----------------------------------------------------
    def add_request(self, request: Hashable) -> None:
        rc = self.cache.add_request(request)
        self.storage.clear_slot(rc.slot)

    def release(self, request: Hashable) -> None:
        self.cache.release(request)

    def length(self, request: Hashable) -> int:
        return self.cache.length(request)

    # ---- the step ------------------------------------------------------
    def step(self, entries: Sequence[tuple[Hashable, Sequence[int], Sequence[int]]],
             starts: Optional[Sequence[int]] = None) -> torch.Tensor:
        """``entries``: (request, next tokens, wanted places among them).

        Runs only these tokens, as one batch, from the cache that earlier
        steps left; returns float32 logits ``[number of wanted places, vocab]``
        in the order of the entries and of their wanted places.  Raises
        ``OutOfPages`` before anything ran if the cache cannot hold the
        tokens.  The tokens of a request go where its cache ends; a caller
        that keeps its own count gives it as ``starts`` and gets an error,
        before anything ran, if the two disagree.

        The logits of a decode step that was replayed from a captured graph
        lie in that graph's own output buffer: they are valid until the next
        step of the same shape, so a caller that keeps them longer copies them."""
        if not entries:
            return torch.empty((0, self.model.spec.vocab_size), dtype=torch.float32, device=self.device)
        portions = self._portions(entries)
        if starts is not None:
            for p, start in zip(portions, starts):
                if p.start != int(start):
                    raise ValueError(f"request {p.request!r}: the caller places its tokens at {start}, "
                                     f"its cache ends at {p.start}")
        self.cache.extend_all([(p.request, p.start + len(p.tokens)) for p in portions])
        logits = self._forward(self._batch(portions))
        for p in portions:
            self.cache.commit(p.request, p.start + len(p.tokens))
        return logits

    def _portions(self, entries) -> list[Portion]:
        """The step's entries, checked, as portions at their requests' present lengths."""
        vocab = self.model.spec.vocab_size
        portions = []
        seen = set()
        for request, tokens, want in entries:
            if request in seen:
                raise ValueError(f"request {request!r} appears twice in one step")
            seen.add(request)
            start = self.cache.length(request)
            if start + len(tokens) > self.config.max_model_len:
                raise ValueError(f"request {request!r} would hold {start + len(tokens)} tokens, "
                                 f"max_model_len is {self.config.max_model_len}")
            ids = np.asarray(tokens, dtype=np.int64)
            if ids.ndim != 1 or ids.size == 0:
                raise ValueError(f"request {request!r}: a portion must hold at least one token")
            low, high = (int(ids[0]),) * 2 if ids.size == 1 else (int(ids.min()), int(ids.max()))
            if low < 0 or high >= vocab:
                raise ValueError(f"request {request!r}: token id outside the vocabulary of {vocab}")
            portions.append(Portion(request, ids, start, want))
        return portions

    def _batch(self, portions: Sequence[Portion]) -> StepBatch:
        tables = {name: [self.cache.table(p.request, name) for p in portions] for name in self.cache.groups}
        return self.builder.build(portions, tables, [self.cache.slot(p.request) for p in portions])

    # ---- several greedy decode steps without the host in between ---------
    def decode_greedy(self, entries: Sequence[tuple[Hashable, int]], steps: int) -> list[list[int]]:
        """``decode_ahead`` with the arg-max as the choice."""
        return self.decode_ahead(entries, steps)

    def decode_ahead(self, entries: Sequence[tuple[Hashable, int]], steps: int, choose=None) -> list[list[int]]:
        """``entries``: (request, its next token), one decoded token each.
        Runs up to ``steps`` decode steps one after the other, each request's
        chosen token becoming its next token on the device, and returns the
        chosen tokens step by step, ``[steps run][request]``: the same tokens
        as as many calls of ``step`` with a choice each, with one wait for
        the device instead of one a step.  ``choose(logits, out)`` writes a
        token id for every row of the 32-bit logits into ``out`` on the device
        (``sampling.sampler.DeviceDraws``); without it, the arg-max.

        The steps after the first replay the graph captured for the shape, so
        fewer than ``steps`` are run (at least one) where there is none yet,
        where the contexts would leave the graph's bucket, or where the cache
        has no pages for all of them."""
        if not entries:
            return []
        portions = self._portions([(request, [token], [0]) for request, token in entries])
        longest = max(p.start + 1 for p in portions)
        run = max(1, min(int(steps), self.config.max_model_len - longest + 1))
        key = None
        if run > 1:
            key = self._decode_graph_key(len(portions), longest)
            if key is None or key not in self._graphs:
                run = 1
            else:
                run = min(run, key[1] - longest + 1)  # the last step's contexts still inside the bucket
        if run > 1 and not self.cache.can_extend([(p.request, p.start + run) for p in portions]):
            run = 1
        self.cache.extend_all([(p.request, p.start + run) for p in portions])
        batch = self._batch(portions)
        chosen = torch.empty((run, len(portions)), dtype=torch.int32, device=self.device)
        for i in range(run):
            if i > 0:
                ops.advance_decode(batch, chosen[i - 1])
            logits = self._forward(batch) if i == 0 else self._replay(key)
            if choose is None:
                ops.argmax(logits, out=chosen[i])
            else:
                choose(logits, chosen[i])
        for p in portions:
            self.cache.commit(p.request, p.start + run)
        return chosen.cpu().tolist()

    def _replay(self, key) -> torch.Tensor:
        graph, static_logits = self._graphs[key]
        self._graphs.move_to_end(key)
        graph.replay()
        self.graph_replays += 1
        return static_logits
