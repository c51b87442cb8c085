#!/usr/bin/env python3
"""Decode and prefill throughput of the engine at Gemma-3-4B layer sizes.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--context 8192] [--layers L]
    python bench.py --workload 12b|27b [--requests N] [--layers L]     (another measurement, see WORKLOADS)

Default run: the layer sizes of the 4B-sized configuration (34 layers, 5
sliding : 1 global, hidden 2560, 8 query / 4 key-value heads of 256, GeGLU
10240, vocabulary 262 208), random weights N(0, 0.02), bf16, 8 requests with
8 192 tokens of context each.  One "step" is one decode step of the whole
batch through the engine's own step function and sampler (greedy): every
request gets one new token.  The caches are filled with random keys and values
for the contexts (a decode step's work does not depend on their values); the
prefill figure is measured on a real prompt of 2 048 tokens run through the
same step function.

One JSON line goes to standard output.  ``value`` is decoded tokens a second.
``roofline`` prices the decode step against 8 TB/s: the bytes it must read
(every weight it uses once, and the keys and values of the live requests that
a token may see) over its time.  ``prefill.frac`` prices the prompt's flops
against 2.5 PFLOP/s (dense bf16 MFMA).  Beside the vendor's peaks stand
measured ones (``measured_peak``): what a kernel that only reads gets from the
memory (the engine's own probe kernel over 4 GiB), and what the library's bf16
product of 8192 x 8192 x 8192 reaches (hipBLASLt, called as the engine calls it).

The timed decode steps end at the named context: the caches are filled so that
the last timed step sees exactly ``--context`` tokens, and every step runs
under the attention plan (and graph) of that context's bucket.
"""

from __future__ import annotations

import argparse
import json
import sys
import time

PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

GEMMA3_4B = {
    "architectures": ["Gemma3ForCausalLM"],
    "num_hidden_layers": 34,
    "sliding_window_pattern": 6,
    "hidden_size": 2560,
    "num_attention_heads": 8,
    "num_key_value_heads": 4,
    "head_dim": 256,
    "intermediate_size": 10240,
    "vocab_size": 262208,
    "rms_norm_eps": 1e-6,
    "max_position_embeddings": 131072,
    "sliding_window": 1024,
    "rope_theta": 1000000.0,
    "rope_local_base_freq": 10000.0,
    "rope_scaling": {"rope_type": "linear", "factor": 8.0},
    "query_pre_attn_scalar": 256,
    "hidden_activation": "gelu_pytorch_tanh",
    "tie_word_embeddings": True,
    "final_logit_softcapping": None,
}
FULL_LAYERS = GEMMA3_4B["num_hidden_layers"]


def log(msg: str) -> None:
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def model_numbers(cfg, elem_bytes: int):
    """Bytes of the weights a step reads, and flops per token of the matrix products."""
    H, I, V = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    per_layer = (cfg.q_size + 2 * cfg.kv_size) * H + H * cfg.q_size + 3 * H * I
    norms = 4 * H + 2 * cfg.head_dim
    layer_params = cfg.num_hidden_layers * (per_layer + norms) + H
    weight_bytes = (layer_params + V * H) * elem_bytes  # the head reads the (tied) table once
    return weight_bytes, 2 * cfg.num_hidden_layers * per_layer, 2 * V * H


def kv_bytes_per_request(cfg, context: int, elem_bytes: int) -> int:
    per_token = 2 * cfg.kv_size * elem_bytes
    total = 0
    for l in range(cfg.num_hidden_layers):
        seen = min(context, cfg.sliding_window) if cfg.is_sliding(l) else context
        total += seen * per_token
    return total


def attention_flops(cfg, start: int, count: int) -> int:
    """Flops of QK^T and PV for tokens start .. start+count-1 of one request."""
    def visible(window):  # the number of visible keys, summed over the positions start .. start+count-1
        total = count * start + count * (count + 1) // 2  # position p sees p + 1 keys
        if window is not None:
            # positions from window - 1 on see `window` keys: take off what the others would see beyond it
            first = max(start, window - 1)
            n = start + count - first
            if n > 0:
                total -= n * first + n * (n + 1) // 2 - n * window
        return total
    sliding = sum(1 for l in range(cfg.num_hidden_layers) if cfg.is_sliding(l))
    keys = sliding * visible(cfg.sliding_window) + (cfg.num_hidden_layers - sliding) * visible(None)
    return 4 * cfg.num_attention_heads * cfg.head_dim * keys


def fill_cache(runner, batch: int, context: int, torch):
    """Live requests with ``context`` tokens each, their pages filled with random keys and values."""
    ids = []
    for b in range(batch):
        rid = f"bench-{b}"
        runner.add_request(rid)
        runner.cache.adopt_length_for_measurement(rid, context)
        ids.append(rid)
    gen = torch.Generator(device=runner.device)
    gen.manual_seed(1)
    for view in runner.storage.views:
        if view is not None and hasattr(view, "k_pages"):
            view.k_pages.normal_(0.0, 1.0, generator=gen)
            view.v_pages.normal_(0.0, 1.0, generator=gen)
    return ids


def release_all(runner, ids):
    for rid in ids:
        runner.release(rid)


def time_decode(engine_parts, batch: int, context: int, steps: int, warmup: int, sampled: bool = False):
    torch, runner, sampler, SamplingParams, SplitMix64 = engine_parts
    ids = fill_cache(runner, batch, max(1, context - steps - warmup), torch)  # the last timed step sees `context`
    # sampled: temperature 0.8 among the 50 largest logits, as the reference's server samples by default
    params = [SamplingParams.sampled(0.8, seed=b) if sampled else SamplingParams() for b in range(len(ids))]
    rngs = [SplitMix64(p.seed) for p in params]
    draws = None
    if sampled:
        from rvllm_amd.sampling.sampler import DeviceDraws
        draws = DeviceDraws(runner.model.spec.vocab_size, params, rngs, runner.device)
    tokens = [(17 * b + 5) % runner.model.spec.vocab_size for b in range(batch)]

    ahead = runner.config.greedy_steps_ahead

    def decode(count, tokens):
        """Exactly ``count`` decode steps, as the engine runs greedy requests: up to ``ahead`` steps follow one
        another with the chosen tokens handed on on the device, then the ids come back to the host."""
        while count > 0:
            if ahead > 1:
                rows = runner.decode_ahead(list(zip(ids, tokens)), min(ahead, count), draws)
                tokens, count = rows[-1], count - len(rows)
            else:
                logits = runner.step([(rid, [tok], [0]) for rid, tok in zip(ids, tokens)])
                tokens, count = sampler.sample(logits, params, rngs), count - 1
        return tokens

    tokens = decode(warmup, tokens)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    tokens = decode(steps, tokens)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    release_all(runner, ids)
    return elapsed / steps


def time_prefill(engine_parts, length: int, repeats: int, start: int = 0):
    """A prompt portion of ``length`` tokens through the step function; with ``start`` the portion continues a
    request that already holds ``start`` tokens (their keys and values random)."""
    torch, runner, sampler, SamplingParams, SplitMix64 = engine_parts
    vocab = runner.model.spec.vocab_size
    g = torch.Generator().manual_seed(2)
    prompt = torch.randint(0, vocab, (length,), generator=g).tolist()
    runner.warm_up([length])  # first-use work, and the library's products tuned for this shape
    times = []
    for i in range(repeats + 1):
        rid = f"prefill-{i}"
        runner.add_request(rid)
        if start > 0:
            runner.cache.adopt_length_for_measurement(rid, start)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        logits = runner.step([(rid, prompt, [length - 1])])
        sampler.sample(logits, [SamplingParams()], [SplitMix64(0)])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        runner.release(rid)
        if i > 0:  # the first run warms up
            times.append(dt)
    return sum(times) / len(times), min(times)


def measure_peaks(torch, device, short: str) -> dict:
    """What this machine gives a kernel that only reads, and the library's best product: the peaks one can
    reach, beside the vendor's.  Both take the best of several runs."""
    from rvllm_amd.kernels import ops

    out = {}
    buf = torch.empty(4 << 30, dtype=torch.uint8, device=device)  # far more than the caches hold
    buf.zero_()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best = None
    for i in range(6):
        start.record()
        ops.probe_read(buf, blocks=4096)
        stop.record()
        stop.synchronize()
        ms = start.elapsed_time(stop)
        if i > 0:
            best = ms if best is None else min(best, ms)
    out["hbm_read_GBs"] = round(buf.numel() / (best * 1e-3) / 1e9, 1)
    del buf
    if short == "bf16":
        n = 8192
        a = torch.randn((n, n), device=device, dtype=torch.bfloat16)
        b = torch.randn((n, n), device=device, dtype=torch.bfloat16)
        c = torch.empty((n, n), device=device, dtype=torch.bfloat16)
        best = None
        for i in range(6):
            start.record()
            ops.library_gemm(a, b, c)
            stop.record()
            stop.synchronize()
            ms = start.elapsed_time(stop)
            if i > 0:
                best = ms if best is None else min(best, ms)
        out["gemm_bf16_TFLOPs"] = round(2 * n ** 3 / (best * 1e-3) / 1e12, 1)
        del a, b, c
    torch.cuda.empty_cache()
    return out


# The engine workloads of the larger configurations: requests through the scheduler, prompts cut into portions
# and mixed with decoding.  (requests, prompt lengths from .. to, new tokens, portion)
WORKLOADS = {
    "12b": (dict(num_hidden_layers=48, hidden_size=3840, num_attention_heads=16, num_key_value_heads=8, head_dim=256,
                 intermediate_size=15360, query_pre_attn_scalar=256), 64, (512, 4096), 256, 2048),
    "27b": (dict(num_hidden_layers=62, hidden_size=5376, num_attention_heads=32, num_key_value_heads=16, head_dim=128,
                 intermediate_size=21504, query_pre_attn_scalar=168), 32, (16384, 16384), 128, 2048),
}


def run_workload(name: str, requests, layers) -> int:
    """Generates through the whole engine (scheduler, portions, decoding) and prints one JSON line."""
    import torch

    from rvllm_amd.config.engine_config import EngineConfig
    from rvllm_amd.config.gemma3 import Gemma3Config
    from rvllm_amd.engine.engine import LLMEngine
    from rvllm_amd.sampling.params import SamplingParams
    import rvllm_amd.models  # noqa: F401

    sizes, n_req, (lo, hi), new, portion = WORKLOADS[name]
    n_req = requests or n_req
    doc = dict(GEMMA3_4B, **sizes)
    full_layers = doc["num_hidden_layers"]
    if layers:
        doc["num_hidden_layers"] = layers
    cfg = Gemma3Config.from_dict(doc, "workload configuration")
    g = torch.Generator().manual_seed(3)
    lengths = [int(torch.randint(lo, hi + 1, (1,), generator=g)) for _ in range(n_req)]
    prompts = [torch.randint(0, cfg.vocab_size, (n,), generator=g).tolist() for n in lengths]
    engine_cfg = EngineConfig(dtype="bfloat16", page_size=16, max_model_len=max(lengths) + new + 16, max_num_seqs=n_req,
                              max_num_batched_tokens=portion + n_req, max_prefill_chunk=portion,
                              max_cache_tokens=sum(lengths) + n_req * (new + 32), use_graphs=True)
    log(f"building the {name}-sized model ({cfg.num_hidden_layers} layers) with random weights")
    engine = LLMEngine.from_random(cfg, 0, engine_cfg)
    t_tune = time.time()
    ladder = engine.runner.tune_products()  # the library's products tuned at a ladder of row counts up to a step's most
    log(f"the library's products tuned for {ladder} rows in {time.time() - t_tune:.1f} s")

    # What every step of the model must at least do, from the plans the scheduler commits: the bytes it reads
    # (all weights once, the keys and values its tokens may see) and its flops (products, attention, head).
    weight_bytes, layer_flops_per_token, head_flops_per_row = model_numbers(cfg, 2)
    kv_token_bytes = 2 * cfg.kv_size * 2
    planned = []  # every committed step's portions as (start, count, wants a token): priced after the run
    commit = engine.scheduler.commit

    def counting_commit(plan, next_tokens):
        planned.append([(p.start, p.count, p.wants_token) for p in plan.portions])
        return commit(plan, next_tokens)

    def price(planned):
        sliding = sum(1 for l in range(cfg.num_hidden_layers) if cfg.is_sliding(l))
        full = cfg.num_hidden_layers - sliding
        tally = {"steps": 0, "bytes": 0, "flops": 0, "ideal_s": 0.0}
        for portions in planned:
            step_bytes, step_flops = weight_bytes, 0
            for start, count, wants in portions:
                seen = start + count
                step_bytes += (full * seen + sliding * min(seen, cfg.sliding_window - 1 + count)) * kv_token_bytes
                step_flops += count * layer_flops_per_token + attention_flops(cfg, start, count)
                step_flops += head_flops_per_row if wants else 0
            tally["steps"] += 1
            tally["bytes"] += step_bytes
            tally["flops"] += step_flops
            tally["ideal_s"] += max(step_bytes / (PEAK_HBM_GBS * 1e9), step_flops / PEAK_FLOPS["bf16"])
        return tally

    engine.scheduler.commit = counting_commit
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    results = engine.generate(prompts, [SamplingParams() for _ in prompts], new, (), True)
    torch.cuda.synchronize()
    sec = time.perf_counter() - t0
    made = sum(len(r.tokens) for r in results)
    tally = price(planned)
    print(json.dumps({
        "metric": f"tokens/s through the engine, {name}-sized workload", "value": round((sum(lengths) + made) / sec, 1),
        "unit": "tok/s", "n_gpus": 1, "seconds": round(sec, 2), "higher_is_better": True, "dtype": "bf16",
        "data": "synthetic: random weights, uniform token ids, greedy",
        # every step priced at the slower of its bytes at 8 TB/s and its flops at 2.5 PFLOP/s; `frac` is the
        # sum of these times over the run's time
        "roofline": {"bound": "per step: max(hbm, mfma)", "steps": tally["steps"],
                     "bytes_TB": round(tally["bytes"] / 1e12, 3), "flops_PFLOP": round(tally["flops"] / 1e15, 3),
                     "ideal_seconds": round(tally["ideal_s"], 3), "frac": round(tally["ideal_s"] / sec, 4),
                     "achieved_GBs": round(tally["bytes"] / sec / 1e9, 1),
                     "achieved_TFLOPs": round(tally["flops"] / sec / 1e12, 1)},
        "config": {"model": f"gemma3-{name}-sized dense decoder", "requests": n_req, "prompt_tokens": sum(lengths),
                   "new_tokens": made, "portion": portion, "layers": cfg.num_hidden_layers,
                   "layers_of_named_config": full_layers, "hidden_size": cfg.hidden_size, "head_dim": cfg.head_dim,
                   "num_attention_heads": cfg.num_attention_heads, "num_key_value_heads": cfg.num_key_value_heads},
    }), flush=True)
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=8192)
    ap.add_argument("--layers", type=int, default=FULL_LAYERS, help="fewer layers of the same size (named in config)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--prefill-at", type=int, default=0,
                    help="the prompt portion continues a request that already holds this many tokens")
    ap.add_argument("--no-points", action="store_true", help="skip the batch-1 and batch-64 points")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--no-probes", action="store_true", help="skip the measured peaks (read rate, library product)")
    ap.add_argument("--page-size", type=int, default=16, choices=[16, 32, 64], help="tokens a page of the cache holds")
    ap.add_argument("--sampled", action="store_true", help="the decode steps draw their tokens (temperature 0.8 among "
                    "the 50 largest logits) instead of taking the arg-max; the metric then says so")
    ap.add_argument("--graphs", type=int, default=1, help="replay decode steps from captured HIP graphs (0 = off)")
    ap.add_argument("--steps-ahead", type=int, default=None,
                    help="greedy decode steps that follow one another without the host (1 = off; default: the engine's)")
    ap.add_argument("--workload", choices=sorted(WORKLOADS), help="instead of the default run: an engine workload of a "
                    "larger configuration (requests through the scheduler); --requests and --layers shrink it")
    ap.add_argument("--requests", type=int, default=0)
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this single-GPU engine", flush=True)
        return 2
    if args.workload:
        return run_workload(args.workload, args.requests, args.layers if args.layers != FULL_LAYERS else 0)

    import torch

    from rvllm_amd.config.engine_config import EngineConfig
    from rvllm_amd.config.gemma3 import Gemma3Config
    from rvllm_amd.engine.runner import ModelRunner
    from rvllm_amd.sampling.params import SamplingParams
    from rvllm_amd.sampling.sampler import Sampler, SplitMix64
    import rvllm_amd.models  # noqa: F401

    doc = dict(GEMMA3_4B, num_hidden_layers=args.layers)
    cfg = Gemma3Config.from_dict(doc, "bench configuration")
    short = "bf16" if args.dtype == "bfloat16" else "fp32"
    elem = 2 if short == "bf16" else 4
    max_batch = max(args.batch, 1 if args.no_points else 64)
    steps_total = args.steps + args.warmup + 8
    engine_cfg = EngineConfig(
        dtype=args.dtype, page_size=args.page_size, max_model_len=max(args.context + steps_total, args.prefill_at + args.prefill_tokens),
        max_num_seqs=max_batch, max_num_batched_tokens=max(args.prefill_tokens, max_batch),
        max_prefill_chunk=max(args.prefill_tokens, 1), max_cache_tokens=max(max_batch * (args.context + steps_total + 16), args.prefill_at + args.prefill_tokens + 64),
        use_graphs=bool(args.graphs),
        **({} if args.steps_ahead is None else {"greedy_steps_ahead": args.steps_ahead}))
    log(f"building {args.layers}-layer model with random weights ({short})")
    t0 = time.time()
    runner = ModelRunner.from_random(cfg, 0, engine_cfg)
    torch.cuda.synchronize()
    log(f"model ready in {time.time() - t0:.1f} s; weights {runner.weight_bytes / 2**30:.1f} GiB, "
        f"cache {runner.storage.bytes / 2**30:.1f} GiB")
    parts = (torch, runner, Sampler(cfg.vocab_size), SamplingParams, SplitMix64)

    weight_bytes, layer_flops_per_token, head_flops_per_row = model_numbers(cfg, elem)

    def decode_point(batch, steps, warmup):
        if batch > 64 and short == "bf16":
            runner.warm_up([batch])  # beyond 64 rows the products are the library's: tuned for this many rows
        sec = time_decode(parts, batch, args.context, steps, warmup, args.sampled)
        log(f"decode batch {batch}{' (sampled)' if args.sampled else ''}: {sec * 1e3:.3f} ms/step, {batch / sec:.1f} tok/s")
        return sec

    peaks = {} if args.no_probes else measure_peaks(torch, runner.device, short)
    if peaks:
        log(f"measured peaks: {peaks}")
    sec = decode_point(args.batch, args.steps, args.warmup)
    value = args.batch / sec
    # the timed steps see context - steps + 1 .. context tokens: priced at their mean
    mean_context = max(1, args.context - (args.steps - 1) // 2)
    step_bytes = weight_bytes + args.batch * kv_bytes_per_request(cfg, mean_context, elem)
    achieved = step_bytes / sec / 1e9
    result = {
        "metric": f"decode tok/s at batch {args.batch}, context {args.context} (Gemma-3-4B sizes)"
                  + (", sampled" if args.sampled else ""),
        "value": round(value, 2),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(sec * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": short,
        "data": "synthetic: random weights N(0,0.02), caches filled with random keys and values, uniform token ids",
        "config": {
            "model": "gemma3-4b-sized dense decoder",
            "global_batch": args.batch,
            "seq_len": args.context,
            "parallelism": "single GPU",
            "layers": args.layers,
            "layers_of_named_config": FULL_LAYERS,
            "hidden_size": cfg.hidden_size,
            "num_attention_heads": cfg.num_attention_heads,
            "num_key_value_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim,
            "intermediate_size": cfg.intermediate_size,
            "vocab_size": cfg.vocab_size,
            "sliding_window": cfg.sliding_window,
            "sliding_to_global": "5:1",
            "rope_local_global_factor": "1e4/1e6/8",
            "page_size": engine_cfg.page_size,
            "hip_graphs": bool(args.graphs), "greedy_steps_ahead": engine_cfg.greedy_steps_ahead,
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4)},
    }
    if "hbm_read_GBs" in peaks:
        result["roofline"]["measured_peak"] = peaks["hbm_read_GBs"]
        result["roofline"]["frac_of_measured"] = round(achieved / peaks["hbm_read_GBs"], 4)
    if not args.no_prefill:
        T = args.prefill_tokens
        if args.prefill_at > 0:  # the cache's pages hold random keys and values, as for the decode points
            gen = torch.Generator(device=runner.device)
            gen.manual_seed(3)
            for view in runner.storage.views:
                if view is not None and hasattr(view, "k_pages"):
                    view.k_pages.normal_(0.0, 1.0, generator=gen)
                    view.v_pages.normal_(0.0, 1.0, generator=gen)
        psec, pmin = time_prefill(parts, T, repeats=5, start=args.prefill_at)
        flops = T * layer_flops_per_token + attention_flops(cfg, args.prefill_at, T) + head_flops_per_row
        result["prefill"] = {"value": round(T / psec, 1), "tokens": T, "ms": round(psec * 1e3, 3),
                             "frac": round(flops / psec / PEAK_FLOPS[short], 4), "ms_min": round(pmin * 1e3, 3)}
        if args.prefill_at > 0:
            result["prefill"]["at"] = args.prefill_at
        if "gemm_bf16_TFLOPs" in peaks:
            result["prefill"]["measured_peak_TFLOPs"] = peaks["gemm_bf16_TFLOPs"]
            result["prefill"]["frac_of_measured"] = round(flops / psec / (peaks["gemm_bf16_TFLOPs"] * 1e12), 4)
        log(f"prefill {T} tokens: {psec * 1e3:.2f} ms mean ({pmin * 1e3:.2f} min), {T / psec:.0f} tok/s")
    if not args.no_points:
        points = {}
        for b in (1, 64):
            s = decode_point(b, max(8, args.steps // 2), max(2, args.warmup // 2))
            points[f"decode_b{b}"] = round(b / s, 2)
        result["points"] = points
    print(json.dumps(result), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
