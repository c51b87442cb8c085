"""rvllm_amd: a single-GPU inference engine for the Gemma dense text decoder on
AMD MI355X (gfx950).

    import rvllm_amd
    out = rvllm_amd.generate("path/to/model", [[2, 17, 5]], max_tokens=32)

The reference has no Python entry point; the arguments carry the names its
HTTP API gives them (``max_tokens``, ``temperature``, ``top_p``, ``top_k``,
``seed``, ``ignore_eos``: v3/crates/rvllm-serve/src/openai.rs:32-70,411-443),
with its defaults: temperature 0 (greedy), top_p 1, top_k 0 when greedy and 50
when sampling.
"""

from __future__ import annotations

from typing import Iterable, Optional, Sequence

__version__ = "0.1.0"


def generate(model: str, prompts: Sequence[Sequence[int]], max_tokens: int = 16, temperature: float = 0.0,
             top_p: float = 1.0, top_k: Optional[int] = None, seed: int = 0, ignore_eos: bool = False,
             eos_ids: Iterable[int] = (), dtype: str = "bfloat16", **engine_options) -> list[list[int]]:
    """Generated token ids for every prompt (lists of token ids).

    ``model`` is a folder with config.json and safetensors.  Request i draws
    from the stream seeded ``seed + i``.  ``engine_options`` are fields of
    ``EngineConfig`` (max_model_len, max_num_seqs, max_num_batched_tokens,
    max_prefill_chunk, page_size, max_cache_tokens)."""
    llm = LLM(model, dtype=dtype, **engine_options)
    return llm.generate(prompts, max_tokens=max_tokens, temperature=temperature, top_p=top_p, top_k=top_k, seed=seed,
                        ignore_eos=ignore_eos, eos_ids=eos_ids)


class LLM:
    """A loaded model that answers ``generate`` calls."""

    def __init__(self, model: str, dtype: str = "bfloat16", **engine_options):
        from .config.engine_config import EngineConfig
        from .engine.engine import LLMEngine

        self.engine = LLMEngine.from_model_dir(model, EngineConfig(dtype=dtype, **engine_options))

    def generate(self, prompts: Sequence[Sequence[int]], max_tokens: int = 16, temperature: float = 0.0,
                 top_p: float = 1.0, top_k: Optional[int] = None, seed: int = 0, ignore_eos: bool = False,
                 eos_ids: Iterable[int] = ()) -> list[list[int]]:
        from .sampling.params import DEFAULT_TOP_K, MIN_TEMPERATURE, SamplingParams

        greedy = 0.0 <= temperature < MIN_TEMPERATURE
        if top_k is None:
            top_k = 0 if greedy else DEFAULT_TOP_K
        params = [SamplingParams(temperature, top_k, top_p, seed + i) for i in range(len(prompts))]
        results = self.engine.generate(prompts, params, max_tokens, eos_ids, ignore_eos)
        return [r.tokens for r in results]
