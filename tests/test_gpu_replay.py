"""The engine against the plain implementation under every way of cutting the
work: each request alone and whole; most of it in one step and the last 32
tokens one by one; portions of changing size down to two tokens; up to four
live requests mixed, with so few pages that they are used again.  In 32-bit and
in bfloat16, for every tiny configuration, through the step function and
through bin/trace_run."""

import numpy as np
import pytest
import torch

import plain_gemma
import trace_tools as tt
from rvllm_amd.config.engine_config import EngineConfig
from rvllm_amd.engine.runner import ModelRunner

pytestmark = pytest.mark.gpu

LENGTHS = {"A": [5, 9, 13, 17, 70, 150], "B": [1, 2, 23, 64, 65, 131], "C": [40, 150, 71, 200, 16, 90]}
MODES = {
    "whole": tt.trace_whole,
    "tail": tt.trace_tail,
    "portions": tt.trace_portions,
    "mixed": tt.trace_mixed,
}


@pytest.fixture(scope="module")
def references(plain_models):
    """Logits of the plain implementation in 64-bit for every test sequence."""
    out = {}
    for name, (weights, cfg) in plain_models.items():
        seqs = tt.make_sequences(cfg["vocab"], LENGTHS[name], seed=ord(name))
        out[name] = (seqs, {rid: plain_gemma.forward(weights, cfg, ids, torch.float64) for rid, ids in seqs.items()})
    return out


def make_runner(model_dir, dtype, max_tokens, page_size=16):
    cfg = EngineConfig(dtype=dtype, page_size=page_size, max_model_len=max_tokens, max_num_seqs=4,
                       max_num_batched_tokens=max_tokens, max_prefill_chunk=max_tokens, max_cache_tokens=max_tokens)
    return ModelRunner.from_model_dir(model_dir, cfg)


def check(steps, outputs, refs, vocab, dtype, prefix, what):
    got = tt.collect(steps, outputs, vocab)
    assert len(got) == len(refs)
    worst = 0.0
    for name, ref in refs.items():
        worst = max(worst, tt.compare(got[f"{prefix}-{name}"], ref, dtype, f"{what} {name}"))
    return worst


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("mode", list(MODES))
def test_cuttings_in_process(model_dirs, references, name, dtype, mode):
    seqs, refs = references[name]
    vocab = next(iter(refs.values())).shape[1]
    steps = MODES[mode](seqs)
    # the pool holds exactly what the trace needs at its fullest, so pages are used again
    runner = make_runner(model_dirs[name], dtype, max_tokens=tt.required_tokens(steps))
    outputs = tt.run_in_process(runner, steps)
    check(steps, outputs, refs, vocab, dtype, steps[0]["entries"][0]["id"].split("-")[0], f"{name} {dtype} {mode}")
    assert all(free == g.pool.num_pages for free, g in zip(runner.cache.free_pages().values(),
                                                           runner.cache.groups.values()))


@pytest.mark.parametrize("name", ["A", "B"])
def test_cuttings_agree_bit_for_bit_in_32_bit(model_dirs, references, name):
    """In 32-bit every kernel adds in an order that depends on the token's
    position alone, so all four cuttings give the same bits."""
    seqs, refs = references[name]
    vocab = next(iter(refs.values())).shape[1]
    runner = make_runner(model_dirs[name], "float32", 4 * 256)
    results = {}
    for mode, make in MODES.items():
        steps = make(seqs)
        got = tt.collect(steps, tt.run_in_process(runner, steps), vocab)
        results[mode] = {rid.split("-", 1)[1]: arr for rid, arr in got.items()}
    for mode in ("tail", "portions", "mixed"):
        for rid in seqs:
            assert np.array_equal(results[mode][rid], results["whole"][rid]), f"{name} {mode} {rid}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "C"])
@pytest.mark.parametrize("mode", ["whole", "tail", "portions", "mixed"])
def test_what_a_page_held_before_reaches_no_logit(model_dirs, references, name, dtype, mode):
    """A page comes to a request with whatever its last holder left in it, and
    that need not be finite.  Here every slot of the cache holds NaN before the
    first step: a kernel that multiplies a slot beyond the request's newest
    token by a probability of zero, instead of leaving it out, shows it."""
    seqs, refs = references[name]
    vocab = next(iter(refs.values())).shape[1]
    steps = MODES[mode](seqs)
    runner = make_runner(model_dirs[name], dtype, max_tokens=tt.required_tokens(steps))
    poisoned = 0
    for view in runner.storage.views:
        if view is not None and hasattr(view, "k_pages"):
            view.k_pages.fill_(float("nan"))
            view.v_pages.fill_(float("nan"))
            poisoned += 1
    assert poisoned > 0
    outputs = tt.run_in_process(runner, steps)
    check(steps, outputs, refs, vocab, dtype, steps[0]["entries"][0]["id"].split("-")[0], f"NaN pages {name} {dtype} {mode}")


@pytest.mark.parametrize("page_size", [32, 64])
def test_other_page_sizes(model_dirs, references, page_size):
    seqs, refs = references["B"]
    vocab = next(iter(refs.values())).shape[1]
    steps = tt.trace_mixed(seqs, seed=3)
    runner = make_runner(model_dirs["B"], "float32", tt.required_tokens(steps), page_size=page_size)
    check(steps, tt.run_in_process(runner, steps), refs, vocab, "float32", "m", f"page {page_size}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(model_dirs, references, tmp_path, dtype):
    """All four cuttings through bin/trace_run as a user drives it."""
    seqs, refs = references["B"]
    vocab = next(iter(refs.values())).shape[1]
    steps, n = [], 0
    for mode, make in MODES.items():
        part = make(seqs, first_step=n)
        steps += part
        n += len(part)
    outputs = tt.run_trace_program(model_dirs["B"], dtype, steps, tmp_path / "out",
                                   max_tokens=tt.required_tokens(steps))
    got = tt.collect(steps, outputs, vocab)
    for prefix in ("w", "t", "p", "m"):
        for name, ref in refs.items():
            tt.compare(got[f"{prefix}-{name}"], ref, dtype, f"trace_run {dtype} {prefix}-{name}")


def test_trace_run_skips_files_for_steps_that_want_nothing(model_dirs, tmp_path):
    steps = [
        tt.step(0, [{"id": "a", "tokens": [1, 2, 3], "want": []}]),
        tt.step(1, [{"id": "a", "tokens": [4], "want": [0]}, {"id": "b", "tokens": [9, 8], "want": [1, 0]}], ["a"]),
        tt.step(2, [{"id": "b", "tokens": [7], "want": []}], ["b"]),
    ]
    outputs = tt.run_trace_program(model_dirs["A"], "float32", steps, tmp_path / "out", max_tokens=128)
    assert set(outputs) == {1} and outputs[1].size == 3 * 256
    weights, cfg = plain_gemma.load_weights(model_dirs["A"]), plain_gemma.read_config(model_dirs["A"])
    ref_a = plain_gemma.forward(weights, cfg, [1, 2, 3, 4], torch.float64)
    ref_b = plain_gemma.forward(weights, cfg, [9, 8], torch.float64)
    rows = outputs[1].reshape(3, 256)
    tt.compare(rows[0:1], ref_a[3:4], "float32", "a")
    tt.compare(rows[1:2], ref_b[1:2], "float32", "b place 1")  # the order of `want` is kept
    tt.compare(rows[2:3], ref_b[0:1], "float32", "b place 0")
