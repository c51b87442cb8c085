"""Configurations drawn at random, every size and option at once (1 to 4 layers of either kind in any order, widths
that are no power of two, 1 to 4 key/value heads with 1 to 17 query heads each, head sizes from 16 to 272, windows
from 3 to 200, pages of 16, 32 and 64 tokens, soft-cap or none), with sequences of 7 to 333 tokens replayed whole,
with a decoded tail, in portions of changing size and mixed, in 32-bit and in bfloat16, against the plain model.
The committed tests' own configurations are few and chosen by hand; these are neither.  The draw is fixed by its
seed, so a failure names a configuration that can be built again."""

import json
import random

import pytest
import torch

import plain_gemma
import trace_tools as tt

pytestmark = pytest.mark.gpu

HEAD_SIZES = [16, 32, 48, 64, 80, 96, 128, 160, 256, 272]
GROUPS = [1, 2, 2, 3, 4, 5, 8, 17]
LENGTHS = [7, 20, 33, 64, 65, 97, 130, 200, 333]
PORTIONS = [(2, 3, 5, 9, 16, 31), (1, 2, 64, 65, 100), (7, 33, 70, 128, 150), (2, 17, 200)]


def drawn_config(rng: random.Random) -> dict:
    nkv = rng.choice([1, 2, 3, 4])
    group = rng.choice(GROUPS)
    hd = rng.choice(HEAD_SIZES)
    if nkv * group * hd > 4096:
        group = max(1, 4096 // (nkv * hd))
    layers = rng.randint(1, 4)
    return {
        "architectures": ["Gemma3ForCausalLM"], "num_hidden_layers": layers,
        "layer_types": [rng.choice(["sliding_attention", "full_attention"]) for _ in range(layers)],
        "hidden_size": rng.choice([48, 64, 72, 96, 136, 264]), "num_attention_heads": nkv * group,
        "num_key_value_heads": nkv, "head_dim": hd, "intermediate_size": rng.choice([64, 88, 160, 264]),
        "vocab_size": rng.randint(100, 700), "rms_norm_eps": rng.choice([1e-6, 1e-5]), "max_position_embeddings": 2048,
        "sliding_window": rng.choice([3, 5, 8, 17, 33, 70, 200]), "rope_theta": rng.choice([1e6, 5e5]),
        "rope_local_base_freq": 10000.0,
        "rope_scaling": rng.choice([None, {"rope_type": "linear", "factor": rng.choice([2.0, 4.0, 8.0])}]),
        "query_pre_attn_scalar": rng.choice([hd, 48, 168]), "hidden_activation": "gelu_pytorch_tanh",
        "tie_word_embeddings": True, "final_logit_softcapping": rng.choice([None, None, 30.0]),
    }


@pytest.mark.parametrize("seed", range(12))
def test_a_configuration_drawn_at_random_in_every_cutting(tmp_path, seed):
    from rvllm_amd.config.engine_config import EngineConfig
    from rvllm_amd.engine.runner import ModelRunner
    from rvllm_amd.models.registry import architecture_of
    import rvllm_amd.models.gemma3  # noqa: F401  (registers the architecture)
    from rvllm_amd.weights.random_init import write_random_model

    rng = random.Random(seed)
    doc = drawn_config(rng)
    config = architecture_of(doc).read_config(doc, f"drawn configuration {seed}")
    folder = write_random_model(tmp_path / "model", config, seed, torch.bfloat16)
    (folder / "config.json").write_text(json.dumps(doc))
    weights, cfg = plain_gemma.load_weights(folder), plain_gemma.read_config(folder)
    lengths = [rng.choice(LENGTHS) for _ in range(rng.randint(3, 5))]
    seqs = tt.make_sequences(cfg["vocab"], lengths, seed=seed)
    want = {name: plain_gemma.forward(weights, cfg, ids, torch.float64) for name, ids in seqs.items()}
    sizes = rng.choice(PORTIONS)
    traces = {"whole": tt.trace_whole(seqs), "tail": tt.trace_tail(seqs, tail=rng.choice([5, 32])),
              "portions": tt.trace_portions(seqs, seed=seed, sizes=sizes),
              "mixed": tt.trace_mixed(seqs, seed=seed, sizes=sizes, decode_tail=rng.choice([3, 12]))}
    page = rng.choice([16, 16, 32, 64])
    what = f"seed {seed}: {doc}, pages of {page}, lengths {lengths}, portions {sizes}"
    for dtype in ("float32", "bfloat16"):
        for name, steps in traces.items():
            most_a_step = max(sum(len(e["tokens"]) for e in st["entries"]) for st in steps)
            runner = ModelRunner.from_model_dir(folder, EngineConfig(
                dtype=dtype, page_size=page, max_model_len=max(lengths) + 8, max_num_seqs=4,
                max_num_batched_tokens=most_a_step, max_prefill_chunk=most_a_step,
                max_cache_tokens=max(tt.required_tokens(steps, round_to=64), 64)))  # so few pages that they are used again
            got = tt.collect(steps, tt.run_in_process(runner, steps), cfg["vocab"])
            assert len(got) == len(seqs), what
            for rid, logits in got.items():
                tt.compare(logits, want[rid.split("-", 1)[1]], dtype, f"{what}: {dtype}, {name}, {rid}")
            del runner


@pytest.mark.parametrize("seed", range(10))
def test_generation_with_engine_settings_drawn_at_random(tmp_path, seed):
    """A drawn configuration under drawn engine settings (2 to 6 requests at once, 16 to 200 tokens a step, portions
    of 7 to 128, pages of 16 to 64, a cache from one request's worth, which sets requests back, to all of them,
    graphs or none, 1 to 4 greedy steps a plan): 3 to 10 prompts of 1 to 150 tokens, every generated token the plain
    model's choice, in both dtypes, and no page lost on the way."""
    from rvllm_amd.config.engine_config import EngineConfig
    from rvllm_amd.engine.engine import LLMEngine
    from rvllm_amd.models.registry import architecture_of
    import rvllm_amd.models.gemma3  # noqa: F401
    from rvllm_amd.sampling.params import SamplingParams
    from rvllm_amd.weights.random_init import write_random_model

    rng = random.Random(seed)
    doc = drawn_config(rng)
    config = architecture_of(doc).read_config(doc, f"drawn configuration {seed}")
    folder = write_random_model(tmp_path / "model", config, seed, torch.bfloat16)
    (folder / "config.json").write_text(json.dumps(doc))
    weights, cfg = plain_gemma.load_weights(folder), plain_gemma.read_config(folder)
    lengths = [rng.choice([1, 2, 5, 17, 33, 64, 65, 100, 150]) for _ in range(rng.randint(3, 10))]
    new = rng.choice([4, 9, 20])
    prompts = list(tt.make_sequences(cfg["vocab"], lengths, seed=seed).values())
    seqs = rng.randint(2, 6)
    budget = rng.choice([16, 33, 64, 100, 200])
    chunk = min(budget, rng.choice([7, 16, 64, 128]))
    page = rng.choice([16, 32, 64])
    longest = max(lengths) + new
    one_request = -(-(longest + 1) // page) * page
    cache_tokens = rng.choice([one_request + page, 2 * one_request, seqs * one_request])
    ahead = rng.choice([1, 2, 4])
    graphs = rng.random() < 0.7
    what = (f"seed {seed}: {doc}; prompts {lengths} + {new}, {seqs} at once, {budget} tokens a step, portions of "
            f"{chunk}, pages of {page}, cache {cache_tokens}, {ahead} steps a plan, graphs {graphs}")
    for dtype in ("float32", "bfloat16"):
        engine = LLMEngine.from_model_dir(folder, EngineConfig(
            dtype=dtype, page_size=page, max_model_len=longest + 1, max_num_seqs=seqs, max_num_batched_tokens=budget,
            max_prefill_chunk=chunk, max_cache_tokens=cache_tokens, use_graphs=graphs, greedy_steps_ahead=ahead))
        results = engine.generate(prompts, SamplingParams(), new, (), True)
        for i, (prompt, result) in enumerate(zip(prompts, results)):
            assert len(result.tokens) == new and result.finish_reason == "length", f"{what}: {dtype}, request {i}"
            logits = plain_gemma.forward(weights, cfg, (list(prompt) + result.tokens)[:-1], torch.float64)
            slack = 2 * tt.TOLERANCE[dtype] * logits.abs().max().item()  # a near-tie may fall either way
            for j, token in enumerate(result.tokens):
                row = logits[len(prompt) - 1 + j]
                assert row[token] >= row.max() - slack, f"{what}: {dtype}, request {i}, token {j} is not the arg-max"
        engine.runner.cache.check()
        del engine


@pytest.mark.parametrize("hidden,inter,vocab", [(100, 150, 333), (36, 50, 101), (66, 130, 99), (7, 6, 11)])
def test_widths_that_are_no_multiple_of_eight(tmp_path, hidden, inter, vocab):
    """Widths that no 16-byte access divides (100, 36, 66, even 7 with a feed-forward of 6 and 11 tokens in the
    vocabulary): whichever kernels take them, both dtypes, whole sequences and mixed steps."""
    import tiny_models
    from rvllm_amd.config.engine_config import EngineConfig
    from rvllm_amd.engine.runner import ModelRunner
    from rvllm_amd.models.registry import architecture_of
    import rvllm_amd.models.gemma3  # noqa: F401
    from rvllm_amd.weights.random_init import write_random_model

    doc = dict(tiny_models.CONFIG_A, hidden_size=hidden, intermediate_size=inter, vocab_size=vocab)
    config = architecture_of(doc).read_config(doc, "a narrow configuration")
    folder = write_random_model(tmp_path / "model", config, 1, torch.bfloat16)
    (folder / "config.json").write_text(json.dumps(doc))
    weights, cfg = plain_gemma.load_weights(folder), plain_gemma.read_config(folder)
    seqs = tt.make_sequences(vocab, [70, 9, 33], seed=1)
    want = {name: plain_gemma.forward(weights, cfg, ids, torch.float64) for name, ids in seqs.items()}
    for dtype in ("float32", "bfloat16"):
        for steps in (tt.trace_whole(seqs), tt.trace_mixed(seqs, seed=1)):
            runner = ModelRunner.from_model_dir(folder, EngineConfig(
                dtype=dtype, max_model_len=128, max_num_seqs=4, max_num_batched_tokens=128, max_prefill_chunk=128,
                max_cache_tokens=256))
            got = tt.collect(steps, tt.run_in_process(runner, steps), vocab)
            assert len(got) == len(seqs)
            for rid, logits in got.items():
                tt.compare(logits, want[rid.split("-", 1)[1]], dtype, f"{hidden} wide, {dtype}, {rid}")
            del runner


@pytest.mark.parametrize("nq,nkv,hd", [(1, 1, 16), (64, 1, 32), (2, 2, 512), (40, 2, 64), (3, 1, 24)])
def test_head_counts_and_sizes_at_the_edges(tmp_path, nq, nkv, hd):
    """One head; 64 and 20 query heads on a key/value head (more than the matrix-core kernels take); the largest
    head size there is a kernel for; a head size that is no multiple of 16: both dtypes, whole and mixed."""
    import tiny_models
    from rvllm_amd.config.engine_config import EngineConfig
    from rvllm_amd.engine.runner import ModelRunner
    from rvllm_amd.models.registry import architecture_of
    import rvllm_amd.models.gemma3  # noqa: F401
    from rvllm_amd.weights.random_init import write_random_model

    doc = dict(tiny_models.CONFIG_A, num_attention_heads=nq, num_key_value_heads=nkv, head_dim=hd,
               query_pre_attn_scalar=hd)
    config = architecture_of(doc).read_config(doc, "heads at the edges")
    folder = write_random_model(tmp_path / "model", config, 1, torch.bfloat16)
    (folder / "config.json").write_text(json.dumps(doc))
    weights, cfg = plain_gemma.load_weights(folder), plain_gemma.read_config(folder)
    seqs = tt.make_sequences(doc["vocab_size"], [70, 9, 33], seed=1)
    want = {name: plain_gemma.forward(weights, cfg, ids, torch.float64) for name, ids in seqs.items()}
    for dtype in ("float32", "bfloat16"):
        for steps in (tt.trace_whole(seqs), tt.trace_mixed(seqs, seed=1)):
            runner = ModelRunner.from_model_dir(folder, EngineConfig(
                dtype=dtype, max_model_len=128, max_num_seqs=4, max_num_batched_tokens=128, max_prefill_chunk=128,
                max_cache_tokens=256))
            got = tt.collect(steps, tt.run_in_process(runner, steps), doc["vocab_size"])
            assert len(got) == len(seqs)
            for rid, logits in got.items():
                tt.compare(logits, want[rid.split("-", 1)[1]], dtype, f"{nq}:{nkv} heads of {hd}, {dtype}, {rid}")
            del runner


def test_a_head_size_beyond_the_kernels_is_refused_by_name(tmp_path):
    import tiny_models
    from rvllm_amd.config.engine_config import EngineConfig
    from rvllm_amd.engine.runner import ModelRunner
    from rvllm_amd.kernels import ops
    from rvllm_amd.models.registry import architecture_of
    import rvllm_amd.models.gemma3  # noqa: F401
    from rvllm_amd.weights.random_init import write_random_model

    doc = dict(tiny_models.CONFIG_A, num_attention_heads=2, num_key_value_heads=1, head_dim=528)
    config = architecture_of(doc).read_config(doc, "a head too large")
    folder = write_random_model(tmp_path / "model", config, 1, torch.bfloat16)
    (folder / "config.json").write_text(json.dumps(doc))
    for dtype in ("float32", "bfloat16"):
        runner = ModelRunner.from_model_dir(folder, EngineConfig(dtype=dtype, max_model_len=64, max_num_seqs=1))
        runner.add_request("x")
        with pytest.raises(ops.KernelError, match="head_dim 528"):
            runner.step([("x", [1, 2, 3], [2])])
