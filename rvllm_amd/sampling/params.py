"""Per-request sampling parameters, with the reference's names, defaults and
limits (v3/crates/rvllm-sampling/src/params.rs:10-78): temperature 0 (or below
1e-3) is greedy; ``top_k`` 0 asks for a draw over the whole vocabulary, which
is allowed only when the vocabulary fits the device's candidate capacity of
1024; ``top_p`` 1 disables the nucleus cut.
"""

from __future__ import annotations

import dataclasses
import math

MIN_TEMPERATURE = 1e-3
DEFAULT_TOP_K = 50
KERNEL_K_CAP = 1024


class SamplingError(ValueError):
    pass


@dataclasses.dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.0
    top_k: int = 0
    top_p: float = 1.0
    seed: int = 0

    @classmethod
    def greedy(cls) -> "SamplingParams":
        return cls()

    @classmethod
    def sampled(cls, temperature: float, top_p: float = 1.0, seed: int = 0) -> "SamplingParams":
        return cls(temperature, DEFAULT_TOP_K, top_p, seed)

    def is_greedy(self) -> bool:
        return math.isfinite(self.temperature) and 0.0 <= self.temperature < MIN_TEMPERATURE

    def validate(self) -> "SamplingParams":
        if not math.isfinite(self.temperature) or self.temperature < 0.0:
            raise SamplingError("temperature: must be finite and >= 0")
        if not math.isfinite(self.top_p) or not 0.0 <= self.top_p <= 1.0:
            raise SamplingError("top_p: must be finite and in 0..=1")
        if not 0 <= self.top_k <= KERNEL_K_CAP:
            raise SamplingError("top_k: must be 0 or <= 1024")
        if not 0 <= self.seed < (1 << 64):
            raise SamplingError("seed: must fit 64 bits")
        return self

    def kernel_k(self, vocab: int) -> int:
        """How many candidates the device selects for this request."""
        self.validate()
        if vocab <= 0:
            raise SamplingError("vocab: must be > 0")
        if self.top_k == 0:
            if vocab <= KERNEL_K_CAP:
                return vocab
            raise SamplingError("top_k: set an explicit top_k <= 1024 for this vocabulary")
        if self.top_k <= vocab:
            return self.top_k
        raise SamplingError("top_k: must be <= vocab")
