"""Run-time settings of the engine (not of the model).

Names and defaults follow the reference's server flags
(v3/crates/rvllm-serve/src/lib.rs:61-79: max_model_len 8192,
max_num_batched_tokens 2048, max_prefill_chunk 128) and its runtime limits
(v3/crates/rvllm-core/src/config/builder.rs:61-133: block size in {16, 32, 64},
at most 256 sequences); like the reference's builder, validation reports every
bad field at once.  The reference serves one sequence at a time
(lib.rs:134-136); here ``max_num_seqs`` is a real limit.
"""

from __future__ import annotations

import dataclasses
from typing import Optional

import torch

from .errors import ConfigError

DTYPES = {
    "bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
    "float32": torch.float32, "fp32": torch.float32, "f32": torch.float32,
}
PAGE_SIZES = (16, 32, 64)


@dataclasses.dataclass
class EngineConfig:
    dtype: str = "bfloat16"
    device: str = "cuda:0"
    page_size: int = 16
    max_model_len: int = 8192
    max_num_seqs: int = 8
    max_num_batched_tokens: int = 2048
    max_prefill_chunk: int = 128
    # Tokens the cache pool is made for; None = max_num_seqs * max_model_len.
    max_cache_tokens: Optional[int] = None
    # Replay decode-only steps from captured HIP graphs (bf16 only).
    use_graphs: bool = True
    # Greedy decode steps that may follow one another without the host in between, while nothing waits to be
    # admitted and no request can end by its length on the way (1 = every step is planned by itself).
    greedy_steps_ahead: int = 4
    # Keep the bf16 matrices a second time, in tiles, for the products of decode steps (up to 64 rows): they then
    # read a matrix as contiguous streams and take a tenth to a quarter less time; the weights take twice the memory.
    tiled_weights: bool = True
    # At start-up, time the library's algorithms for the products of prompt portions (more than 64 rows) at a ladder
    # of row counts up to max_num_batched_tokens and keep the fastest (``ModelRunner.tune_products``; some seconds).
    # Row counts in between run on their tuned neighbour's algorithm.  Off: the library's first suggestion, which
    # is often a fifth slower.
    tune_products: bool = False

    @property
    def torch_dtype(self) -> torch.dtype:
        return DTYPES[self.dtype]

    def validate(self) -> "EngineConfig":
        problems = []
        if self.dtype not in DTYPES:
            problems.append(f"dtype {self.dtype!r} must be one of {sorted(set(DTYPES))}")
        if self.page_size not in PAGE_SIZES:
            problems.append(f"page_size {self.page_size} must be one of {PAGE_SIZES}")
        if not 1 <= self.max_num_seqs <= 256:
            problems.append(f"max_num_seqs {self.max_num_seqs} must be in 1..=256")
        if self.max_model_len < 1:
            problems.append("max_model_len must be >= 1")
        if self.max_num_batched_tokens < 1:
            problems.append("max_num_batched_tokens must be >= 1")
        if self.max_prefill_chunk < 1:
            problems.append("max_prefill_chunk must be >= 1")
        if self.max_prefill_chunk > self.max_num_batched_tokens:
            problems.append("max_prefill_chunk must not exceed max_num_batched_tokens")
        if not 1 <= self.greedy_steps_ahead <= 64:
            problems.append(f"greedy_steps_ahead {self.greedy_steps_ahead} must be in 1..=64")
        if self.max_cache_tokens is not None and self.max_cache_tokens < self.page_size:
            problems.append("max_cache_tokens must hold at least one page")
        if problems:
            raise ConfigError("engine configuration", problems)
        return self

    def cache_tokens(self) -> int:
        if self.max_cache_tokens is not None:
            return self.max_cache_tokens
        return self.max_num_seqs * self.max_model_len
