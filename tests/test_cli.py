"""The command line's options: names and meanings of the reference's flags
(v3/crates/rvllm-serve/src/lib.rs:54-175), without a GPU."""

import json

import pytest

import tiny_models
from rvllm_amd import cli


def test_defaults_are_the_references():
    o = cli.parse(["--model", "m"], {})
    assert (o["max_model_len"], o["max_num_batched_tokens"], o["max_prefill_chunk"]) == (8192, 2048, 128)
    assert o["temperature"] == 0.0 and o["top_p"] == 1.0 and o["max_tokens"] == 200


def test_both_spellings_of_a_value_and_the_environment():
    o = cli.parse(["--model=m", "--max-model-len", "512", "--max-prefill-chunk=64", "--prompt-ids", "1 2,3"],
                  {"RVLLM_SAMPLE_T": "0.7", "RVLLM_SAMPLE_TOPK": "40", "RVLLM_GEN_TOKENS": "9", "RVLLM_EOS": "1,107"})
    assert o["max_model_len"] == 512 and o["max_prefill_chunk"] == 64 and o["prompt_ids"] == [[1, 2, 3]]
    assert o["temperature"] == 0.7 and o["top_k"] == 40 and o["max_tokens"] == 9 and o["eos"] == "1,107"
    assert cli.parse([], {"RVLLM_MODEL_DIR": "/x"})["model"] == "/x"


def test_tuning_of_the_librarys_products_is_asked_for_by_flag_or_environment():
    assert cli.parse(["--model", "m"], {})["tune_products"] is False
    assert cli.parse(["--model", "m", "--tune-products"], {})["tune_products"] is True
    assert cli.parse(["--model", "m"], {"RVLLM_TUNE_PRODUCTS": "1"})["tune_products"] is True
    assert cli.parse(["--model", "m"], {"RVLLM_TUNE_PRODUCTS": "0"})["tune_products"] is False
    cli.parse(["--model", "m"], {"RVLLM_AMD_LIBRARY_PLANS": "/tmp/plans.json"})  # a known variable


@pytest.mark.parametrize("argv,env,needle", [
    (["--model", "m", "--frobnicate"], {}, "unknown argument: --frobnicate"),
    (["--model", "m"], {"RVLLM_NO_SUCH_THING": "1"}, "unknown environment variable: RVLLM_NO_SUCH_THING"),
    (["--model", "m", "--port", "80"], {}, "no HTTP server"),
    (["--model", "m", "--max-prefill-chunk", "4096"], {}, "max_prefill_chunk must not exceed max_num_batched_tokens"),
    (["--model", "m", "--max-model-len", "0"], {}, "must be >= 1"),
    (["--model", "m", "--max-tokens"], {}, "needs a value"),
    (["--model", "m", "--top-k", "many"], {}, "invalid value"),
    ([], {}, "no model"),
])
def test_errors(argv, env, needle):
    with pytest.raises(cli.UsageError, match=needle):
        cli.parse(argv, env)


def test_synthetic_prompt_is_the_references():
    # v3/crates/rvllm-bench/src/main.rs:970-977: token 2, then 100 + lcg % (vocab - 100)
    p = cli._synthetic_prompt(4, 262208)
    s = (0x12345678 * 1103515245 + 12345) & 0xFFFFFFFF
    assert p[0] == 2 and p[1] == 100 + (s >> 16) % (262208 - 100) and len(p) == 4
    assert all(0 <= t < 50 for t in cli._synthetic_prompt(10, 50))


def test_dry_run_checks_everything_and_loads_nothing(tmp_path, capsys):
    (tmp_path / "config.json").write_text(json.dumps(tiny_models.CONFIG_B))
    assert cli.main(["--model", str(tmp_path), "--dry-run", "--prompt-ids", "1 2 3"], {}) == 0
    out = json.loads(capsys.readouterr().out)
    assert out["dry_run"] is True and out["architecture"] == "Gemma3ForCausalLM" and out["prompts"] == 1
    # a token outside the vocabulary, a bad configuration and bad sampling parameters are usage errors
    assert cli.main(["--model", str(tmp_path), "--dry-run", "--prompt-ids", "1 509"], {}) == 2
    assert cli.main(["--model", str(tmp_path), "--dry-run", "--page-size", "24"], {}) == 2
    assert cli.main(["--model", str(tmp_path), "--dry-run", "--temperature", "0.8", "--top-p", "1.5"], {}) == 2
    assert "top_p" in capsys.readouterr().err
