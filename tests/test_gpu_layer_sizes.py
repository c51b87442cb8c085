"""The engine at the layer sizes of the 4B model (two layers, a small
vocabulary), and with the heads of the 27B model, against the plain implementation: sequences that cross the edge of
the window of 1024, whole, with the last tokens decoded one by one, in large
and small portions, and two requests mixed.  What the tiny configurations
cannot show lies here: portions of more than a thousand tokens (the library's
matrix products, the prompt attention kernel over many blocks of keys), a
window that ends in the middle of a long cache, decoding over split keys."""

import pytest
import torch

import plain_gemma
import tiny_models
import trace_tools as tt
from rvllm_amd.config.engine_config import EngineConfig
from rvllm_amd.engine.runner import ModelRunner

pytestmark = pytest.mark.gpu

LENGTHS = [1300, 700]


@pytest.fixture(scope="module", params=["D", "E"])
def model(request, tmp_path_factory):
    """D: two layers of the 4B model's sizes.  E: three narrow layers with the 27B model's heads."""
    folder = tiny_models.write_model(tmp_path_factory.mktemp("larger") / request.param, request.param)
    weights, cfg = plain_gemma.load_weights(folder), plain_gemma.read_config(folder)
    seqs = tt.make_sequences(cfg["vocab"], LENGTHS, seed=4)
    refs = {rid: plain_gemma.forward(weights, cfg, ids, torch.float64) for rid, ids in seqs.items()}
    return folder, cfg, seqs, refs


def big_portions(seqs):
    return tt.trace_portions(seqs, seed=2, sizes=(300, 257, 64, 33, 17, 2, 129))


def mixed(seqs):
    return tt.trace_mixed(seqs, seed=5, max_live=2, decode_tail=20, sizes=(31, 64, 200, 97))


MODES = {"whole": tt.trace_whole, "tail": tt.trace_tail, "portions": big_portions, "mixed": mixed}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", list(MODES))
def test_cuttings_at_the_4b_layer_sizes(model, dtype, mode):
    folder, cfg, seqs, refs = model
    steps = MODES[mode](seqs)
    most = tt.required_tokens(steps)
    runner = ModelRunner.from_model_dir(folder, EngineConfig(
        dtype=dtype, page_size=16, max_model_len=max(LENGTHS) + 20, max_num_seqs=2, max_num_batched_tokens=most,
        max_prefill_chunk=most, max_cache_tokens=most))
    outputs = tt.run_in_process(runner, steps)
    got = tt.collect(steps, outputs, cfg["vocab"])
    prefix = steps[0]["entries"][0]["id"].split("-")[0]
    for name, ref in refs.items():
        tt.compare(got[f"{prefix}-{name}"], ref, dtype, f"4B layer sizes, {dtype}, {mode}, {name}")
    assert all(free == g.pool.num_pages for free, g in zip(runner.cache.free_pages().values(),
                                                           runner.cache.groups.values()))


@pytest.mark.parametrize("mode", ["portions", "mixed"])
def test_a_cache_that_held_nan_before_at_the_4b_layer_sizes(model, mode):
    """Pages come with what their last holder left, which need not be finite:
    every slot of the cache is NaN before the first step, and no logit may show
    it (the slots beyond a request's newest token are left out, not multiplied
    by zero)."""
    folder, cfg, seqs, refs = model
    steps = MODES[mode](seqs)
    most = tt.required_tokens(steps)
    runner = ModelRunner.from_model_dir(folder, EngineConfig(
        dtype="bfloat16", page_size=16, max_model_len=max(LENGTHS) + 20, max_num_seqs=2, max_num_batched_tokens=most,
        max_prefill_chunk=most, max_cache_tokens=most))
    for view in runner.storage.views:
        view.k_pages.fill_(float("nan"))
        view.v_pages.fill_(float("nan"))
    got = tt.collect(steps, tt.run_in_process(runner, steps), cfg["vocab"])
    prefix = steps[0]["entries"][0]["id"].split("-")[0]
    for name, ref in refs.items():
        tt.compare(got[f"{prefix}-{name}"], ref, "bfloat16", f"4B layer sizes, NaN pages, {mode}, {name}")
