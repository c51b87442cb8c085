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

import numpy as np
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


def sample_rows(vals: np.ndarray, ids: np.ndarray, top_k: Sequence[int], top_p: Sequence[float],
                rngs: Sequence[SplitMix64], vocab: Optional[int] = None) -> list[int]:
    """``sample_from_candidates`` for many rows at once: row r has the candidates
    (vals[r, j], ids[r, j]) and its own ``top_k``, ``top_p`` and stream.  The
    same arithmetic in the same order, so the same tokens bit for bit, with the
    sorting, the running sums and the walk along the weights done for all rows
    together (a row at a time in Python costs more than the device's selection)."""
    vals = np.asarray(vals, dtype=np.float64)
    ids = np.asarray(ids, dtype=np.int64)
    rows, k = vals.shape
    if rows == 0:
        return []
    if k == 0:
        raise SamplingError("candidates: must be non-empty")
    if not np.isfinite(vals).all():
        raise SamplingError("candidates: logits must be finite")
    if any(not math.isfinite(p) or not 0.0 <= p <= 1.0 for p in top_p):
        raise SamplingError("top_p: must be finite and in 0..=1")
    if any(t > k for t in top_k):
        raise SamplingError("top_k: must not exceed candidate count")
    if vocab is not None and ((ids < 0) | (ids >= vocab)).any():
        raise SamplingError("candidates: token ID must be below vocab")
    order = np.lexsort((ids, -vals), axis=1)  # value descending, then id ascending
    v = np.take_along_axis(vals, order, axis=1)
    pool = np.take_along_axis(ids, order, axis=1)
    n = np.array([min(k, t) if t > 0 else k for t in top_k], dtype=np.int64)
    cols = np.arange(k)
    inside = cols[None, :] < n[:, None]
    # exp of the C library, as math.exp, not numpy's own (which differs in the last bit now and then)
    diff = (v - v[:, :1])[inside]
    w = np.zeros((rows, k), dtype=np.float64)
    w[inside] = np.fromiter(map(math.exp, diff.tolist()), dtype=np.float64, count=diff.size)
    cum = np.cumsum(w, axis=1)  # left to right, as the reference sums
    total = cum[np.arange(rows), n - 1]
    p = np.asarray(top_p, dtype=np.float64)
    reached = (cum >= (np.maximum(p, 0.0) * total)[:, None]) & inside
    cut = np.where(p < 1.0, reached.argmax(axis=1) + 1, n)
    z = cum[np.arange(rows), cut - 1]
    u = np.array([rng.next_f64() for rng in rngs], dtype=np.float64) * z
    # u - w0 - w1 - ..., one subtraction after the other, as the reference walks
    left = np.subtract.accumulate(np.concatenate([u[:, None], w], axis=1), axis=1)[:, 1:]
    stops = (left <= 0.0) & (cols[None, :] < cut[:, None])
    chosen = np.where(stops.any(axis=1), stops.argmax(axis=1), cut - 1)
    return pool[np.arange(rows), chosen].tolist()


class DeviceDraws:
    """The next tokens of a fixed set of requests, chosen on the device step after step without the host:
    ``topk_select`` and then ``ops.draw``, which does what ``sample_rows`` does with each request's stream of
    numbers kept on the device.  The device selects as many candidates for every row as the row that asks for
    most; a row keeps its own ``top_k`` of them after the sort, which are the ones it would have had selected
    (equal values go by the lower id both times).  A row that samples gets -1 if one of its own ``top_k``
    largest logits is no finite number, as the host's draw refuses it; what was selected beyond them for another
    row's sake is not looked at.  A row that decodes greedily takes the largest candidate that is a number, as
    the arg-max does (``top_k`` -1 tells the kernel so), and draws no number from its stream."""

    def __init__(self, vocab_size: int, params: Sequence[SamplingParams], rngs: Sequence[SplitMix64], device):
        ks = [p.kernel_k(vocab_size) for p in params if not p.is_greedy()]
        if not ks:
            raise SamplingError("no row samples")
        self.k = max(ks)
        greedy = [p.is_greedy() for p in params]
        self.inv_temp = torch.tensor([1.0 if g else 1.0 / p.temperature for p, g in zip(params, greedy)],
                                     dtype=torch.float32, device=device)
        self.top_k = torch.tensor([-1 if g else p.top_k for p, g in zip(params, greedy)], dtype=torch.int32,
                                  device=device)
        self.top_p = torch.tensor([1.0 if g else p.top_p for p, g in zip(params, greedy)], dtype=torch.float64,
                                  device=device)
        # the streams' states as signed 64-bit numbers, which is what the tensor holds
        self.state = torch.tensor([r.state - (1 << 64) if r.state >= (1 << 63) else r.state for r in rngs],
                                  dtype=torch.int64, device=device)

    @staticmethod
    def usable(vocab_size: int, params: Sequence[SamplingParams]) -> bool:
        """Whether some row samples and every such row's parameters are ones the device selects for."""
        try:
            return len([p.kernel_k(vocab_size) for p in params if not p.is_greedy()]) > 0
        except SamplingError:
            return False

    def __call__(self, logits: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        vals, ids = ops.topk_select(logits, self.k, self.inv_temp)
        return ops.draw(vals, ids, self.top_k, self.top_p, self.state, out)


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
                tokens = sample_rows(vals.cpu().numpy(), ids.cpu().numpy(), [params[r].top_k for r in group],
                                     [params[r].top_p for r in group], [rngs[r] for r in group], self.vocab_size)
                for r, token in zip(group, tokens):
                    out[r] = token
        if greedy:
            host = greedy_ids.cpu().tolist()
            for r in greedy:
                out[r] = host[r]
        return out  # type: ignore[return-value]
