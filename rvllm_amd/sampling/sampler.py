"""Choice of the next token from a step's logits.

Greedy rows: arg-max on the device (NaN skipped, equal maxima give the lowest
id: kernels/argmax.cu:16-25).  Sampled rows: the device selects the K largest
logits and scales them by 1/T; the host sorts them (value descending, id
ascending), cuts to ``top_k``, weighs them by exp(v - max) in 64-bit, cuts the
nucleus (the smallest prefix whose mass reaches ``top_p`` times the total, at
least one token) and draws with one number from the request's SplitMix64
stream (v3/crates/rvllm-sampling/src/sampler.rs:17-135).  The same candidates
and seed give the same token whatever else is in the batch.
"""

from __future__ import annotations

import math
from typing import Optional, Sequence

import torch

from ..kernels import ops
from .params import SamplingError, SamplingParams

_MASK64 = (1 << 64) - 1


class SplitMix64:
    """v3/crates/rvllm-sampling/src/sampler.rs:17-36."""

    def __init__(self, seed: int):
        self.state = seed & _MASK64

    def next_u64(self) -> int:
        self.state = (self.state + 0x9E3779B97F4A7C15) & _MASK64
        z = self.state
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK64
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK64
        return z ^ (z >> 31)

    def next_f64(self) -> float:
        """Uniform in [0, 1) with 53 random bits."""
        return (self.next_u64() >> 11) * (1.0 / (1 << 53))


def sample_from_candidates(cands: Sequence[tuple[float, int]], top_k: int, top_p: float, rng: SplitMix64,
                           vocab: Optional[int] = None) -> int:
    """``cands``: (logit / T, token id) in any order
    (v3/crates/rvllm-sampling/src/sampler.rs:71-135)."""
    if not cands:
        raise SamplingError("candidates: must be non-empty")
    if any(not math.isfinite(v) for v, _ in cands):
        raise SamplingError("candidates: logits must be finite")
    if not math.isfinite(top_p) or not 0.0 <= top_p <= 1.0:
        raise SamplingError("top_p: must be finite and in 0..=1")
    if top_k > 0 and top_k > len(cands):
        raise SamplingError("top_k: must not exceed candidate count")
    if vocab is not None and any(not 0 <= t < vocab for _, t in cands):
        raise SamplingError("candidates: token ID must be below vocab")
    pool = sorted(cands, key=lambda c: (-c[0], c[1]))
    n = min(len(pool), top_k) if top_k > 0 else len(pool)
    pool = pool[:n]
    mx = pool[0][0]
    weights = [math.exp(v - mx) for v, _ in pool]
    total = sum(weights)  # left to right, as the reference sums
    cut = n
    if top_p < 1.0:
        target = max(top_p, 0.0) * total
        cum = 0.0
        for i, w in enumerate(weights):
            cum += w
            if cum >= target:
                cut = i + 1
                break
    z = sum(weights[:cut])
    u = rng.next_f64() * z
    for i in range(cut):
        u -= weights[i]
        if u <= 0.0:
            return pool[i][1]
    return pool[cut - 1][1]


class Sampler:
    """Next tokens for the rows of a step's logits."""

    def __init__(self, vocab_size: int):
        self.vocab_size = vocab_size

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams], rngs: Sequence[SplitMix64]) -> list[int]:
        """``logits`` [R, vocab] float32 on the device; row r belongs to the
        request with ``params[r]`` and ``rngs[r]``."""
        rows = logits.shape[0]
        if rows == 0:
            return []
        if len(params) != rows or len(rngs) != rows:
            raise SamplingError("one set of parameters and one stream per row expected")
        out: list[Optional[int]] = [None] * rows
        greedy = [r for r in range(rows) if params[r].is_greedy()]
        sampled = [r for r in range(rows) if not params[r].is_greedy()]
        greedy_ids = None
        if greedy:
            # arg-max of every row; rows that sample ignore theirs
            greedy_ids = ops.argmax(logits)
        if sampled:
            by_k: dict[int, list[int]] = {}
            for r in sampled:
                by_k.setdefault(params[r].kernel_k(self.vocab_size), []).append(r)
            for k, group in by_k.items():
                idx = torch.tensor(group, dtype=torch.int64, device=logits.device)
                sub = logits.index_select(0, idx) if len(group) != rows else logits
                inv_t = torch.tensor([1.0 / params[r].temperature for r in group], dtype=torch.float32,
                                     device=logits.device)
                vals, ids = ops.topk_select(sub.contiguous(), k, inv_t)
                vals, ids = vals.cpu().tolist(), ids.cpu().tolist()
                for j, r in enumerate(group):
                    out[r] = sample_from_candidates(list(zip(vals[j], ids[j])), params[r].top_k, params[r].top_p,
                                                    rngs[r], self.vocab_size)
        if greedy:
            host = greedy_ids.cpu().tolist()
            for r in greedy:
                out[r] = host[r]
        return out  # type: ignore[return-value]
