"""Configurations and schedules beside the main replay tests: a head of its own
(not tied to the embedding), flat and beside a nested decoder; bf16 on pages of
32 and 64 slots; steps with more decoding requests than the few-row product
takes (the library's products, no graph); a folder in several shards; and
the bounds of the cache's bookkeeping under long decoding and mixed traces."""

import json

import numpy as np
import pytest
import torch

import plain_gemma
import tiny_models
import trace_tools as tt
from rvllm_amd.cache.manager import window_pages_bound
from rvllm_amd.config.engine_config import EngineConfig
from rvllm_amd.engine.engine import LLMEngine
from rvllm_amd.engine.runner import ModelRunner
from rvllm_amd.kernels import ops

pytestmark = pytest.mark.gpu


def runner_for(folder, dtype, max_tokens, page_size=16, max_num_seqs=4, **more):
    cfg = EngineConfig(dtype=dtype, page_size=page_size, max_model_len=max_tokens, max_num_seqs=max_num_seqs,
                       max_num_batched_tokens=max_tokens, max_prefill_chunk=max_tokens, max_cache_tokens=max_tokens,
                       **more)
    return ModelRunner.from_model_dir(folder, cfg)


# ---- a head that is not tied ---------------------------------------------------------------------------------
def write_untied(folder, nested: bool):
    """Config B with tie_word_embeddings false and a head of its own; ``nested`` keeps the decoder under
    ``language_model.model`` and the head beside it, as multimodal checkpoints do."""
    from safetensors.torch import load_file, save_file

    base = tiny_models.write_model(folder / "base", "B")
    tensors = load_file(str(base / "model.safetensors"))
    g = torch.Generator().manual_seed(21)
    head = (torch.randn(509, 96, generator=g) * 0.05).to(torch.bfloat16)
    out = folder / ("nested" if nested else "flat")
    out.mkdir()
    if nested:
        tensors = {"language_model." + k: v for k, v in tensors.items()}
        tensors["language_model.lm_head.weight"] = head
        tensors["vision_tower.patch.weight"] = torch.zeros(3, dtype=torch.bfloat16)  # left alone
    else:
        tensors["lm_head.weight"] = head
    doc = dict(tiny_models.CONFIG_B, tie_word_embeddings=False)
    (out / "config.json").write_text(json.dumps(doc))
    save_file(tensors, str(out / "model.safetensors"))
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nested", [False, True])
def test_a_head_of_its_own(tmp_path, dtype, nested):
    folder = write_untied(tmp_path, nested)
    weights, cfg = plain_gemma.load_weights(folder), plain_gemma.read_config(folder)
    assert cfg["tied"] is False
    seqs = tt.make_sequences(cfg["vocab"], [3, 40, 77], seed=6)
    refs = {rid: plain_gemma.forward(weights, cfg, ids, torch.float64) for rid, ids in seqs.items()}
    tied = plain_gemma.forward(weights, dict(cfg, tied=True), seqs["r1"], torch.float64)
    assert (tied - refs["r1"]).abs().max() > 0.1 * refs["r1"].abs().max()  # the head's own matrix matters
    for mode in ("whole", "mixed"):
        steps = (tt.trace_whole if mode == "whole" else tt.trace_mixed)(seqs)
        runner = runner_for(folder, dtype, tt.required_tokens(steps))
        assert runner.model.head.weight is not runner.model.embedding.table
        got = tt.collect(steps, tt.run_in_process(runner, steps), cfg["vocab"])
        prefix = steps[0]["entries"][0]["id"].split("-")[0]
        for rid, ref in refs.items():
            tt.compare(got[f"{prefix}-{rid}"], ref, dtype, f"untied {mode} {rid}")
    # generation picks from the head's logits
    engine = LLMEngine.from_model_dir(folder, EngineConfig(dtype="float32", max_model_len=64, max_num_seqs=1))
    res = engine.generate([seqs["r0"]], None, max_new_tokens=5, ignore_eos=True)[0]
    assert res.tokens == plain_gemma.greedy(weights, cfg, seqs["r0"], 5, torch.float64)


def test_a_missing_head_is_named(tmp_path):
    from safetensors.torch import load_file, save_file

    from rvllm_amd.weights.loader import WeightError

    folder = write_untied(tmp_path, nested=False)
    tensors = load_file(str(folder / "model.safetensors"))
    del tensors["lm_head.weight"]
    save_file(tensors, str(folder / "model.safetensors"))
    with pytest.raises(WeightError) as e:
        runner_for(folder, "float32", 64)
    assert e.value.missing == ["lm_head.weight"]


# ---- bf16 on larger pages ------------------------------------------------------------------------------------
@pytest.mark.parametrize("page_size", [32, 64])
@pytest.mark.parametrize("mode", ["whole", "tail", "portions", "mixed"])
@pytest.mark.parametrize("name", ["B", "C"])
def test_cuttings_on_larger_pages_in_bf16(model_dirs, plain_models, name, mode, page_size):
    """The matrix-core attention kernels (decode and prompt) on pages of 32 and 64 slots."""
    weights, cfg = plain_models[name]
    lengths = [1, 2, 23, 64, 65, 131] if name == "B" else [40, 150, 71, 200, 16, 90]
    seqs = tt.make_sequences(cfg["vocab"], lengths, seed=ord(name))
    refs = {rid: plain_gemma.forward(weights, cfg, ids, torch.float64) for rid, ids in seqs.items()}
    make = {"whole": tt.trace_whole, "tail": tt.trace_tail, "portions": tt.trace_portions, "mixed": tt.trace_mixed}[mode]
    steps = make(seqs)
    runner = runner_for(model_dirs[name], "bfloat16", tt.required_tokens(steps, round_to=64), page_size=page_size)
    got = tt.collect(steps, tt.run_in_process(runner, steps), cfg["vocab"])
    prefix = steps[0]["entries"][0]["id"].split("-")[0]
    for rid, ref in refs.items():
        tt.compare(got[f"{prefix}-{rid}"], ref, "bfloat16", f"page {page_size} {name} {mode} {rid}")


# ---- more decoding requests than the few-row product takes -----------------------------------------------
def many_requests_trace(vocab, count, seed, prompt_lengths=(3, 19), decode=6):
    """``count`` requests: their prompts in a few steps of several requests each, then ``decode`` steps in which
    all of them bring one token."""
    rng = np.random.default_rng(seed)
    seqs = {f"q{i}": rng.integers(0, vocab, int(rng.integers(*prompt_lengths)) + decode).tolist() for i in range(count)}
    steps, names = [], list(seqs)
    for at in range(0, count, 24):
        steps.append(tt.step(len(steps), [{"id": n, "tokens": seqs[n][:-decode], "want": [len(seqs[n]) - decode - 1]}
                                         for n in names[at:at + 24]]))
    for d in range(decode, 0, -1):
        steps.append(tt.step(len(steps), [{"id": n, "tokens": [seqs[n][-d]], "want": [0]} for n in names],
                             names if d == 1 else []))
    return seqs, steps


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,count", [("A", 80), ("D", 65)])
def test_more_decoding_requests_than_the_few_row_product_takes(model_dirs, plain_models, tmp_path, name, count, dtype):
    """65 to 80 live requests decode together: beyond 64 rows the bf16 products go to the library; such a step is
    recorded too, and the recording replayed three times against the step run kernel by kernel before it is
    trusted; every request's logits still equal the plain implementation's."""
    assert count > ops.SKINNY_MAX_ROWS
    if name == "D":
        folder = tiny_models.write_model(tmp_path / "D", "D")
        weights, cfg = plain_gemma.load_weights(folder), plain_gemma.read_config(folder)
    else:
        folder, (weights, cfg) = model_dirs[name], plain_models[name]
    seqs, steps = many_requests_trace(cfg["vocab"], count, seed=count)
    runner = runner_for(folder, dtype, 64 * count, max_num_seqs=count)
    got = tt.collect(steps, tt.run_in_process(runner, steps), cfg["vocab"])
    assert (runner.graph_replays >= 4) == (dtype == "bfloat16")  # the six decode steps but the first
    assert runner._library_steps_from_graphs
    for rid in list(seqs)[:: 1 if name == "A" else 8]:  # the wide model's reference on the CPU is slow: every eighth
        ref = plain_gemma.forward(weights, cfg, seqs[rid], torch.float64)
        want = ref[len(seqs[rid]) - 7:]  # the prompt's last place and the six decoded ones
        tt.compare(got[rid], want, dtype, f"{name} {count} requests {rid}")


# ---- the steps a scheduler builds under load: dozens of decoders beside a long portion ------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_dozens_of_decoding_requests_beside_a_long_portion(model_dirs, plain_models, name, dtype):
    """44 requests through the engine with a budget of 100 tokens a step and portions of at most 64: most have
    short prompts and are soon decoding, the others' prompts of 130 to 200 tokens then arrive in portions beside
    thirty and more decoded tokens, so that one step runs both attention kernels (and the library's products,
    where the step has more than 64 rows).  Every token is the plain implementation's."""
    weights, cfg = plain_models[name]
    rng = np.random.default_rng(44)
    lengths = [int(rng.integers(2, 12)) for _ in range(36)] + [130, 200, 177, 64, 150, 199, 131, 166]
    prompts = list(tt.make_sequences(cfg["vocab"], lengths, seed=44).values())
    new = 30
    engine = LLMEngine.from_model_dir(model_dirs[name], EngineConfig(
        dtype=dtype, max_model_len=256, max_num_seqs=44, max_num_batched_tokens=100, max_prefill_chunk=64))
    shapes = []
    run_step = engine.runner.step

    def watched(entries, **kw):
        shapes.append((sum(len(tokens) == 1 for _, tokens, _ in entries), max(len(tokens) for _, tokens, _ in entries)))
        return run_step(entries, **kw)

    engine.runner.step = watched
    results = engine.generate(prompts, None, max_new_tokens=new, ignore_eos=True)
    assert any(singles >= 30 and longest >= 60 for singles, longest in shapes), shapes
    assert sum(singles >= 30 and longest >= 16 for singles, longest in shapes) >= 10
    from test_gpu_generate import assert_greedy

    for prompt, res in zip(prompts, results):
        assert len(res.tokens) == new and res.set_backs == 0
        assert_greedy(weights, cfg, prompt, res.tokens, dtype)
    if dtype == "float32":
        for prompt, res in list(zip(prompts, results))[::4]:
            assert res.tokens == plain_gemma.greedy(weights, cfg, prompt, new, torch.float64)


# ---- heads that only the kernel for any size takes -----------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", ["whole", "mixed"])
def test_a_head_size_above_256_and_17_query_heads_a_group(tmp_path, dtype, mode):
    """Head size 272 with 34 query heads on 2 key/value heads: neither matrix-core attention kernel takes these,
    so bf16 too runs the one for any size; the q/k norm takes its path for odd sizes."""
    folder = tiny_models.write_model(tmp_path / "G", "G")
    weights, cfg = plain_gemma.load_weights(folder), plain_gemma.read_config(folder)
    seqs = tt.make_sequences(cfg["vocab"], [3, 40, 77, 130], seed=7)
    steps = (tt.trace_whole if mode == "whole" else tt.trace_mixed)(seqs)
    runner = runner_for(folder, dtype, tt.required_tokens(steps))
    view = runner.storage.views[0]
    assert not ops.mfma_attention_covers(view.k_pages, view.v_pages, cfg["nq"])
    got = tt.collect(steps, tt.run_in_process(runner, steps), cfg["vocab"])
    prefix = steps[0]["entries"][0]["id"].split("-")[0]
    for rid, ids in seqs.items():
        tt.compare(got[f"{prefix}-{rid}"], plain_gemma.forward(weights, cfg, ids, torch.float64), dtype, f"G {mode} {rid}")


def test_a_recording_that_does_not_reproduce_its_step_is_not_trusted(model_dirs):
    """The check of a recorded step with library products, made to fail from the host: the step's logits come from
    the run kernel by kernel, no graph is kept, and later steps of that kind are not recorded again; steps of few
    requests still come from graphs."""
    seqs, steps = many_requests_trace(256, 70, seed=3)
    runner = runner_for(model_dirs["A"], "bfloat16", 64 * 70, max_num_seqs=70)
    runner.GRAPH_LIBRARY_TOLERANCE = -1.0  # nothing is close enough
    with pytest.warns(UserWarning, match="did not reproduce"):
        tt.collect(steps, tt.run_in_process(runner, steps), 256)
    assert runner.graph_replays == 0 and not runner._library_steps_from_graphs and not runner._graphs
    runner.add_request("few")
    runner.step([("few", [1, 2, 3], [])])
    for token in (4, 5, 6):
        runner.step([("few", [token], [0])])
    assert runner.graph_replays >= 2


# ---- a folder in several shards ------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_folder_in_three_shards(model_dirs, plain_models, tmp_path, dtype):
    from safetensors.torch import load_file, save_file

    tensors = load_file(str(model_dirs["B"] / "model.safetensors"))
    names = sorted(tensors)
    shards = {f"model-{i + 1:05d}-of-00003.safetensors": names[i::3] for i in range(3)}
    for fname, held in shards.items():
        save_file({n: tensors[n] for n in held}, str(tmp_path / fname))
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(
        {"metadata": {}, "weight_map": {n: fname for fname, held in shards.items() for n in held}}))
    (tmp_path / "config.json").write_text((model_dirs["B"] / "config.json").read_text())
    weights, cfg = plain_models["B"]
    ids = tt.make_sequences(cfg["vocab"], [50], seed=2)["r0"]
    runner = runner_for(tmp_path, dtype, 64)
    runner.add_request("x")
    got = runner.step([("x", ids, list(range(len(ids))))]).float().cpu().numpy()
    tt.compare(got, plain_gemma.forward(weights, cfg, ids, torch.float64), dtype, "three shards")
    # an index that names a tensor in the wrong file is refused
    from rvllm_amd.weights.safetensors_io import SafetensorsError

    doc = json.loads((tmp_path / "model.safetensors.index.json").read_text())
    doc["weight_map"][names[0]] = "model-00002-of-00003.safetensors"
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(doc))
    with pytest.raises(SafetensorsError, match="do not hold"):
        runner_for(tmp_path, dtype, 64)


# ---- the cache's bounds -----------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_window_never_holds_more_pages_than_its_bound(model_dirs, dtype):
    """Sliding layers keep pages that return to the pool behind the window, not a ring: what a request holds in
    the window's group stays within window_pages_bound, under decoding one by one and under portions."""
    for chunk, new in ((1, 300), (23, 40)):
        engine = LLMEngine.from_model_dir(model_dirs["A"], EngineConfig(
            dtype=dtype, max_model_len=512, max_num_seqs=1, max_cache_tokens=512, max_num_batched_tokens=max(chunk, 8),
            max_prefill_chunk=chunk))
        pool = engine.runner.cache.groups["window8"].pool
        prompt = list(range(1, 120)) if chunk > 1 else [11, 22, 33]
        res = engine.generate([prompt], None, max_new_tokens=new, ignore_eos=True)[0]
        assert len(res.tokens) == new
        step_tokens = chunk if chunk > 1 else engine.runner.config.greedy_steps_ahead
        assert 0 < pool.most_held_by_one <= window_pages_bound(8, 16, step_tokens)
        full = engine.runner.cache.groups["full"].pool
        assert full.most_held_by_one == -(-(len(prompt) + new - 1) // 16)  # the other group keeps everything
        assert pool.free_count == pool.num_pages


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_pages_change_hands_in_a_mixed_trace(model_dirs, plain_models, dtype):
    """With a pool as small as the trace allows, pages that one request gave back are held by another later; the
    logits are those of the plain implementation all the same."""
    weights, cfg = plain_models["B"]
    seqs = tt.make_sequences(cfg["vocab"], [1, 2, 23, 64, 65, 131], seed=ord("B"))
    steps = tt.trace_mixed(seqs)
    runner = runner_for(model_dirs["B"], dtype, tt.required_tokens(steps))
    for g in runner.cache.groups.values():
        g.pool.keep_history = True
    got = tt.collect(steps, tt.run_in_process(runner, steps), cfg["vocab"])
    for rid, ids in seqs.items():
        tt.compare(got[f"m-{rid}"], plain_gemma.forward(weights, cfg, ids, torch.float64), dtype, rid)
    for name, g in runner.cache.groups.items():
        shared = [owners for owners in g.pool.history.values() if len(set(owners)) > 1]
        assert shared, f"no page of group {name} was held by two requests"


# ---- memory ------------------------------------------------------------------------------------------------
def test_weights_are_counted_and_a_cache_that_does_not_fit_is_refused_with_the_numbers(model_dirs, monkeypatch):
    from rvllm_amd.cache.storage import CacheTooLarge

    tiled = runner_for(model_dirs["B"], "bfloat16", 256)
    rows = runner_for(model_dirs["B"], "bfloat16", 256, tiled_weights=False)
    params = sum(t.numel() for t in plain_gemma.load_weights(model_dirs["B"]).values())
    assert rows.weight_bytes == 2 * params  # bf16, the tied head's table once
    # in tiles every matrix lies there a second time, its rows and columns filled up to whole tiles
    assert 1.9 * rows.weight_bytes < tiled.weight_bytes < 2.6 * rows.weight_bytes
    # a device with 64 MiB free (said by the host: nothing is filled up for this)
    monkeypatch.setattr(torch.cuda, "mem_get_info", lambda device=None: (64 << 20, 288 << 30))
    monkeypatch.setattr(torch.cuda, "memory_reserved", lambda device=None: torch.cuda.memory_allocated(device))
    with pytest.raises(CacheTooLarge, match=r"needs \d+\.\d GiB, 0\.1 GiB of 288\.0 GiB are free; the weights hold"):
        ModelRunner.from_model_dir(model_dirs["B"], EngineConfig(dtype="bfloat16", max_model_len=2048, max_num_seqs=64,
                                                                 max_cache_tokens=600_000))
    runner_for(model_dirs["B"], "bfloat16", 256)  # what fits is built as ever


# ---- logits of replayed steps ----------------------------------------------------------------------------
def test_logits_of_a_replayed_step_live_until_the_next_step_of_its_shape(model_dirs):
    """A decode step replayed from a graph returns the graph's own output buffer: the next step of the same shape
    writes it again, so a caller that keeps logits copies them (as the engine's sampler does at once)."""
    runner = runner_for(model_dirs["B"], "bfloat16", 256)
    runner.add_request("x")
    runner.step([("x", [5, 6, 7], [])])
    kept = []
    for token in (8, 9, 10, 11):
        logits = runner.step([("x", [token], [0])])
        kept.append((logits, logits.clone()))
    assert runner.graph_replays >= 2
    (_, a_then), (b, b_then) = kept[-2], kept[-1]
    assert torch.equal(b, b_then) and not torch.equal(a_then, b_then)
    assert kept[-2][0].data_ptr() == b.data_ptr()  # one buffer: the older result now reads as the newer one
