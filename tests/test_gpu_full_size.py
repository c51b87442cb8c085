"""The whole model at the sizes of Gemma 3 4B (34 layers, a vocabulary of
262 208) with random weights, written to a folder and loaded from it, against
the plain implementation in 64-bit: a prompt run whole, then tokens decoded
one by one, in 32-bit and in bfloat16.  What two layers of these sizes cannot
show lies here: errors that grow over 34 layers, the head over the whole
vocabulary, a folder of several gigabytes through the loader."""

import shutil

import numpy as np
import pytest
import torch

import plain_gemma
import tiny_models
import trace_tools as tt
from rvllm_amd.config.engine_config import EngineConfig
from rvllm_amd.engine.runner import ModelRunner

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    folder = tiny_models.write_model(tmp_path_factory.mktemp("full") / "4B", "4B")
    cfg = plain_gemma.read_config(folder)
    ids = tt.make_sequences(cfg["vocab"], [32], seed=6)["r0"]
    want = plain_gemma.forward(plain_gemma.load_weights(folder), cfg, ids, torch.float64)
    yield folder, ids, want
    shutil.rmtree(folder)  # eight gigabytes: not left for the temporary folder's own cleaning


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_whole_4b_sized_model(model, dtype):
    folder, ids, want = model
    runner = ModelRunner.from_model_dir(folder, EngineConfig(
        dtype=dtype, max_model_len=64, max_num_seqs=1, max_num_batched_tokens=64, max_prefill_chunk=64,
        max_cache_tokens=64))
    runner.add_request("r")
    got = [runner.step([("r", ids[:24], list(range(24)))]).float().cpu().numpy()]
    for token in ids[24:]:
        got.append(runner.step([("r", [token], [0])]).float().cpu().numpy())
    tt.compare(np.concatenate(got), want, dtype, f"the whole 4B-sized model, {dtype}")
