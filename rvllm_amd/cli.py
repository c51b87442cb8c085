"""Command line: a model folder and prompts in, generated tokens out.

The options that the reference's ``rvllm-server`` has keep their names,
meanings and defaults (v3/crates/rvllm-serve/src/lib.rs:61-131): ``--model``,
``--max-model-len`` (8192), ``--max-num-seqs``, ``--max-inflight-requests``,
``--max-num-batched-tokens`` (2048), ``--max-prefill-chunk`` (128),
``--dry-run``; both ``--flag value`` and ``--flag=value`` are read, an unknown
argument or an unknown ``RVLLM_*`` variable is an error (lib.rs:58-60,131).
There is no HTTP server here, so ``--host`` and ``--port`` are refused with a
message.  Prompts and sampling come the way the reference's ``rvllm-bench
--generate`` takes them: ``RVLLM_GEN_PROMPT_FILE`` (whitespace-separated token
ids), ``RVLLM_GEN_PROMPT`` (length of a synthetic prompt), ``RVLLM_GEN_TOKENS``,
``RVLLM_GEN_DUMP``, ``RVLLM_SAMPLE_T/TOPK/TOPP/SEED``, ``RVLLM_EOS``
(v3/crates/rvllm-bench/src/main.rs:911-978,1014-1021;
v3/crates/rvllm-runtime/src/gemma4_bring_up.rs:5594-5611;
v3/crates/rvllm-serve/src/worker.rs:1171-1181), each also as a flag.
``--tune-products`` and ``RVLLM_AMD_LIBRARY_PLANS`` (a file of tuned choices, read and written) stand where the
reference has its autotuned ``RVLLM_POLICY`` file (v3/crates/rvllm-serve/src/main.rs:41): which of the library's
algorithms a product of a given shape runs on.
One JSON line per request goes to standard output.
"""

from __future__ import annotations

import json
import os
import sys
import time
from pathlib import Path

ENV_WHITELIST = {
    "RVLLM_MODEL_DIR", "RVLLM_GEN_PROMPT_FILE", "RVLLM_GEN_PROMPT", "RVLLM_GEN_TOKENS", "RVLLM_GEN_DUMP",
    "RVLLM_SAMPLE_T", "RVLLM_SAMPLE_TOPK", "RVLLM_SAMPLE_TOPP", "RVLLM_SAMPLE_SEED", "RVLLM_EOS",
    "RVLLM_DEFAULT_MAX_TOKENS", "RVLLM_DRY_RUN", "RVLLM_MAX_INFLIGHT_REQUESTS", "RVLLM_DTYPE",
    "RVLLM_AMD_BUILD_DIR", "RVLLM_GRAPHS", "RVLLM_AMD_LIBRARY_PLANS", "RVLLM_TUNE_PRODUCTS",
}

USAGE = """usage: rvllm-amd --model DIR [options]
  --model DIR                    model folder (config.json + safetensors); else $RVLLM_MODEL_DIR
  --dtype bfloat16|float32       compute type (default bfloat16)
  --max-model-len N              longest sequence, prompt plus output (default 8192)
  --max-num-seqs N               requests that run together (default 8)
  --max-inflight-requests N      requests accepted at once (default 4 * max-num-seqs)
  --max-num-batched-tokens N     tokens per step (default 2048)
  --max-prefill-chunk N          longest portion of a prompt in one step (default 128)
  --page-size N                  tokens per cache page: 16, 32 or 64 (default 16)
  --max-cache-tokens N           tokens the cache pool holds (default max-num-seqs * max-model-len)
  --prompt-file FILE             one prompt per line, whitespace-separated token ids  [$RVLLM_GEN_PROMPT_FILE]
  --prompt-ids "1 2 3"           one prompt on the command line (may be repeated)
  --prompt-len N                 synthetic prompt of N tokens                          [$RVLLM_GEN_PROMPT]
  --max-tokens N                 new tokens per request (default 200)                  [$RVLLM_GEN_TOKENS]
  --temperature T --top-k K --top-p P --seed S                                         [$RVLLM_SAMPLE_*]
  --eos 1,107                    ids that end a request                                [$RVLLM_EOS]
  --ignore-eos                   keep going past an end id
  --dump FILE                    write the generated ids, one request per line         [$RVLLM_GEN_DUMP]
  --random-weights CONFIG.json   no folder: random weights for this configuration (with --weights-seed S)
  --no-graphs                    do not replay decode steps from captured HIP graphs   [$RVLLM_GRAPHS=0]
  --greedy-steps-ahead N         greedy decode steps that may follow one another without the host (default 4, 1 = off)
  --tune-products                at start-up time the library's algorithms for the products of prompt portions
                                 and keep the fastest (some seconds)                   [$RVLLM_TUNE_PRODUCTS=1]
                                 with $RVLLM_AMD_LIBRARY_PLANS=FILE the choices are kept in FILE and read from it
  --dry-run                      check the configuration and the arguments, load nothing
"""


class UsageError(Exception):
    pass


def _synthetic_prompt(length: int, vocab: int) -> list[int]:
    """The reference's synthetic prompt (v3/crates/rvllm-bench/src/main.rs:970-977)."""
    prompt = [min(2, vocab - 1)]
    s = 0x12345678
    while len(prompt) < length:
        s = (s * 1103515245 + 12345) & 0xFFFFFFFF
        prompt.append(100 + (s >> 16) % max(vocab - 100, 1) if vocab > 100 else (s >> 16) % vocab)
    return prompt


def parse(argv: list[str], env: dict) -> dict:
    for name in env:
        if name.startswith("RVLLM_") and name not in ENV_WHITELIST:
            raise UsageError(f"unknown environment variable: {name}")
    o = {
        "model": env.get("RVLLM_MODEL_DIR"),
        "dtype": env.get("RVLLM_DTYPE", "bfloat16"),
        "max_model_len": 8192, "max_num_seqs": 8, "max_inflight_requests": None,
        "max_num_batched_tokens": 2048, "max_prefill_chunk": 128, "page_size": 16, "max_cache_tokens": None,
        "prompt_file": env.get("RVLLM_GEN_PROMPT_FILE"), "prompt_ids": [],
        "prompt_len": int(env["RVLLM_GEN_PROMPT"]) if "RVLLM_GEN_PROMPT" in env else None,
        "max_tokens": int(env.get("RVLLM_GEN_TOKENS", env.get("RVLLM_DEFAULT_MAX_TOKENS", 200))),
        "temperature": float(env.get("RVLLM_SAMPLE_T", 0.0)),
        "top_k": int(env["RVLLM_SAMPLE_TOPK"]) if "RVLLM_SAMPLE_TOPK" in env else None,
        "top_p": float(env.get("RVLLM_SAMPLE_TOPP", 1.0)),
        "seed": int(env.get("RVLLM_SAMPLE_SEED", 0)),
        "eos": env.get("RVLLM_EOS", ""), "ignore_eos": False, "dump": env.get("RVLLM_GEN_DUMP"),
        "random_weights": None, "weights_seed": 0,
        "dry_run": env.get("RVLLM_DRY_RUN", "") not in ("", "0", "false"),
        "graphs": env.get("RVLLM_GRAPHS", "1") not in ("0", "false"),
        "greedy_steps_ahead": 4,
        "tune_products": env.get("RVLLM_TUNE_PRODUCTS", "") not in ("", "0", "false"),
    }
    ints = {"--max-model-len", "--max-num-seqs", "--max-inflight-requests", "--max-num-batched-tokens",
            "--max-prefill-chunk", "--page-size", "--max-cache-tokens", "--prompt-len", "--max-tokens", "--top-k",
            "--seed", "--weights-seed", "--greedy-steps-ahead"}
    floats = {"--temperature", "--top-p"}
    strings = {"--model", "--dtype", "--prompt-file", "--eos", "--dump", "--random-weights"}
    it = iter(argv)
    for arg in it:
        key, _, inline = arg.partition("=")
        has_inline = "=" in arg
        if key in ("-h", "--help"):
            raise UsageError(USAGE)
        if key in ("--host", "--port", "--backend", "--served-model-name", "--system-prompt", "--system-prompt-file"):
            raise UsageError(f"{key}: this build has no HTTP server; prompts come from --prompt-file or --prompt-ids")
        if key in ("--dry-run", "--ignore-eos", "--graphs", "--tune-products"):
            o[key[2:].replace("-", "_")] = True
            continue
        if key == "--no-graphs":
            o["graphs"] = False
            continue
        if key not in ints | floats | strings | {"--prompt-ids"}:
            raise UsageError(f"unknown argument: {key}")
        if has_inline:
            value = inline
        else:
            try:
                value = next(it)
            except StopIteration:
                raise UsageError(f"{key} needs a value") from None
        name = key[2:].replace("-", "_")
        try:
            if key in ints:
                o[name] = int(value)
            elif key in floats:
                o[name] = float(value)
            elif key == "--prompt-ids":
                o["prompt_ids"].append([int(t) for t in value.replace(",", " ").split()])
            else:
                o[name] = value
        except ValueError:
            raise UsageError(f"{key}: invalid value {value!r}") from None
    if o["max_inflight_requests"] is None:
        o["max_inflight_requests"] = int(env.get("RVLLM_MAX_INFLIGHT_REQUESTS", 4 * o["max_num_seqs"]))
    if o["max_inflight_requests"] < 1:
        raise UsageError("max_inflight_requests must be >= 1")
    if min(o["max_model_len"], o["max_num_batched_tokens"], o["max_prefill_chunk"]) < 1:
        raise UsageError("model, batching, and prefill limits must be >= 1")
    if o["max_prefill_chunk"] > o["max_num_batched_tokens"]:
        raise UsageError("max_prefill_chunk must not exceed max_num_batched_tokens")
    if not o["model"] and not o["random_weights"]:
        raise UsageError("no model: give --model DIR, $RVLLM_MODEL_DIR or --random-weights CONFIG.json\n" + USAGE)
    return o


def _read_prompts(o: dict, vocab: int) -> list[list[int]]:
    prompts = [list(p) for p in o["prompt_ids"]]
    if o["prompt_file"]:
        text = Path(o["prompt_file"]).read_text()
        for n, line in enumerate(text.splitlines(), 1):
            if line.strip():
                try:
                    prompts.append([int(t) for t in line.split()])
                except ValueError:
                    raise UsageError(f"{o['prompt_file']}:{n}: invalid token id") from None
    if not prompts:
        prompts.append(_synthetic_prompt(o["prompt_len"] or 32, vocab))
    for p in prompts:
        if not p:
            raise UsageError("an empty prompt")
        for t in p:
            if not 0 <= t < vocab:
                raise UsageError(f"token {t} exceeds vocabulary {vocab}")
    return prompts


def main(argv=None, env=None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    env = dict(os.environ if env is None else env)
    try:
        o = parse(argv, env)
        from .config.engine_config import EngineConfig
        from .models.registry import architecture_of, load_config
        from .sampling.params import DEFAULT_TOP_K, SamplingParams

        cfg = EngineConfig(dtype=o["dtype"], page_size=o["page_size"], max_model_len=o["max_model_len"],
                           max_num_seqs=o["max_num_seqs"], max_num_batched_tokens=o["max_num_batched_tokens"],
                           max_prefill_chunk=o["max_prefill_chunk"], max_cache_tokens=o["max_cache_tokens"],
                           use_graphs=o["graphs"], greedy_steps_ahead=o["greedy_steps_ahead"],
                           tune_products=o["tune_products"]).validate()
        if o["random_weights"]:
            doc = json.loads(Path(o["random_weights"]).read_text())
            arch = architecture_of(doc, o["random_weights"])
            model_config = arch.read_config(doc, o["random_weights"])
        else:
            arch, model_config = load_config(o["model"])
        vocab = arch.build_spec(model_config).vocab_size
        prompts = _read_prompts(o, vocab)
        if len(prompts) > o["max_inflight_requests"]:
            raise UsageError(f"{len(prompts)} prompts exceed --max-inflight-requests {o['max_inflight_requests']}")
        greedy = 0.0 <= o["temperature"] < 1e-3
        top_k = o["top_k"] if o["top_k"] is not None else (0 if greedy else DEFAULT_TOP_K)
        params = [SamplingParams(o["temperature"], top_k, o["top_p"], o["seed"] + i).validate()
                  for i in range(len(prompts))]
        eos = [int(t) for t in o["eos"].split(",") if t.strip()]
    except UsageError as e:
        print(str(e), file=sys.stderr)
        return 2
    except ValueError as e:  # configuration, sampling parameters
        print(f"error: {e}", file=sys.stderr)
        return 2
    if o["dry_run"]:
        print(json.dumps({"dry_run": True, "architecture": arch.name, "prompts": len(prompts), "dtype": cfg.dtype}))
        return 0

    from .engine.engine import LLMEngine

    t0 = time.time()
    if o["random_weights"]:
        engine = LLMEngine.from_random(model_config, o["weights_seed"], cfg)
    else:
        engine = LLMEngine.from_model_dir(o["model"], cfg)
    print(f"[rvllm-amd] model ready in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    t0 = time.time()
    results = engine.generate(prompts, params, o["max_tokens"], eos, o["ignore_eos"])
    wall = time.time() - t0
    n = sum(len(r.tokens) for r in results)
    for i, r in enumerate(results):
        print(json.dumps({"index": i, "prompt_tokens": len(r.prompt), "completion_tokens": len(r.tokens),
                          "finish_reason": r.finish_reason, "token_ids": r.tokens}), flush=True)
    print(f"generate: {n} tokens, wall={wall:.3f}s, e2e={n / wall if wall > 0 else 0.0:.1f} tok/s, "
          f"steps={engine.steps}", file=sys.stderr)
    if o["dump"]:
        Path(o["dump"]).write_text("".join(" ".join(map(str, r.tokens)) + "\n" for r in results))
    return 0


if __name__ == "__main__":
    sys.exit(main())
