"""Configuration: reading config.json's keys, the registry, the errors."""

import copy
import json

import pytest

import tiny_models
from rvllm_amd.config.engine_config import EngineConfig
from rvllm_amd.config.errors import ConfigError, UnknownArchitectureError
from rvllm_amd.config.gemma3 import GLOBAL, SLIDING, Gemma3Config
from rvllm_amd.models import architecture_names, architecture_of, load_config
from rvllm_amd.models.gemma3 import build_spec


def read(doc):
    return Gemma3Config.from_dict(doc)


def test_config_a_fields():
    c = read(tiny_models.CONFIG_A)
    assert (c.num_hidden_layers, c.hidden_size, c.num_attention_heads, c.num_key_value_heads, c.head_dim) == (2, 64, 4, 2, 16)
    assert c.layer_types == (SLIDING, GLOBAL)
    assert c.rope_local.theta == 10000.0 and c.rope_global.theta == 1e6
    assert c.rope_local.factor == 1.0 and c.rope_global.factor == 1.0
    assert c.query_pre_attn_scalar == 16 and c.rms_norm_eps == 1e-6 and c.sliding_window == 8
    assert c.final_logit_softcapping is None and c.tie_word_embeddings


def test_config_b_pattern_and_scaling():
    c = read(tiny_models.CONFIG_B)
    # layer l is global iff (l + 1) % pattern == 0 (gemma4_arch.rs:566-577)
    assert c.layer_types == (SLIDING, SLIDING, GLOBAL)
    assert c.rope_global.factor == 4.0 and c.rope_local.factor == 1.0
    assert c.rope_global.theta == 500000.0
    assert c.q_size == 192 != c.hidden_size


def test_pattern_six_over_34_layers():
    doc = dict(tiny_models.CONFIG_B, num_hidden_layers=34, sliding_window_pattern=6)
    kinds = read(doc).layer_types
    assert [i for i, k in enumerate(kinds) if k == GLOBAL] == [5, 11, 17, 23, 29]


def test_text_config_nesting_and_outer_fallback():
    inner = {k: v for k, v in tiny_models.CONFIG_A.items() if k not in ("architectures", "tie_word_embeddings")}
    doc = {"architectures": ["Gemma3ForConditionalGeneration"], "text_config": inner, "tie_word_embeddings": True}
    c = read(doc)
    assert c.hidden_size == 64 and c.tie_word_embeddings


def test_reference_rope_spelling():
    doc = {k: v for k, v in tiny_models.CONFIG_A.items() if not k.startswith("rope")}
    doc["rope_parameters"] = {"sliding_attention": {"rope_theta": 1e4},
                              "full_attention": {"rope_theta": 2e6, "rope_type": "linear", "factor": 2.0}}
    c = read(doc)
    assert c.rope_local.theta == 1e4 and c.rope_global.theta == 2e6 and c.rope_global.factor == 2.0
    # flat fallback of the reference: bare rope_theta is the local base
    doc = {k: v for k, v in tiny_models.CONFIG_A.items() if not k.startswith("rope")}
    doc.update(rope_theta=1e4, rope_theta_global=3e6)
    c = read(doc)
    assert c.rope_local.theta == 1e4 and c.rope_global.theta == 3e6
    # only one base: both kinds share it
    doc = {k: v for k, v in tiny_models.CONFIG_A.items() if not k.startswith("rope")}
    doc.update(rope_theta=7e4)
    c = read(doc)
    assert c.rope_local.theta == c.rope_global.theta == 7e4


def test_query_pre_attn_scalar_defaults_to_head_dim():
    doc = {k: v for k, v in tiny_models.CONFIG_B.items() if k != "query_pre_attn_scalar"}
    assert read(doc).query_pre_attn_scalar == 32.0


def test_all_problems_reported_at_once():
    doc = copy.deepcopy(tiny_models.CONFIG_A)
    del doc["hidden_size"]
    doc["num_attention_heads"] = 5  # not a multiple of 2 kv heads
    doc["rms_norm_eps"] = "tiny"
    doc["layer_types"] = ["sliding_attention"]
    with pytest.raises(ConfigError) as e:
        read(doc)
    text = str(e.value)
    assert "hidden_size" in text and "multiple" in text and "rms_norm_eps" in text and "layer_types has len 1" in text
    assert len(e.value.problems) >= 4


@pytest.mark.parametrize("key,value,needle", [
    ("num_kv_shared_layers", 2, "num_kv_shared_layers"),
    ("hidden_size_per_layer_input", 8, "per-layer"),
    ("global_head_dim", 32, "global_head_dim"),
    ("attention_k_eq_v", True, "attention_k_eq_v"),
    ("attn_logit_softcapping", 50.0, "attn_logit_softcapping"),
    ("hidden_activation", "relu", "hidden_activation"),
    ("head_dim", 15, "even"),
    ("sliding_window", 100000, "exceeds"),
    ("rope_scaling", {"rope_type": "yarn", "factor": 2.0}, "rope_type"),
])
def test_unsupported_values_are_named(key, value, needle):
    doc = dict(tiny_models.CONFIG_A)
    doc[key] = value
    with pytest.raises(ConfigError) as e:
        read(doc)
    assert needle in str(e.value)


def test_bool_is_not_an_integer():
    with pytest.raises(ConfigError):
        read(dict(tiny_models.CONFIG_A, num_hidden_layers=True))


def test_unknown_architecture_lists_the_known():
    doc = dict(tiny_models.CONFIG_A, architectures=["LlamaForCausalLM"])
    with pytest.raises(UnknownArchitectureError) as e:
        architecture_of(doc)
    assert "LlamaForCausalLM" in str(e.value) and "Gemma3ForCausalLM" in str(e.value)
    assert "Gemma3ForCausalLM" in architecture_names()


def test_round_trip_through_config_json(tmp_path):
    for doc in (tiny_models.CONFIG_A, tiny_models.CONFIG_B, tiny_models.CONFIG_C):
        c = read(doc)
        (tmp_path / "config.json").write_text(json.dumps(c.to_dict()))
        arch, again = load_config(tmp_path)
        assert again == c and arch.name == "Gemma3ForCausalLM"


def test_config_file_errors(tmp_path):
    with pytest.raises(ConfigError, match="not found"):
        load_config(tmp_path)
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="not valid JSON"):
        load_config(tmp_path)
    (tmp_path / "config.json").write_text("[1]")
    with pytest.raises(ConfigError, match="object"):
        load_config(tmp_path)


def test_spec_takes_every_size_from_the_configuration():
    c = read(tiny_models.CONFIG_B)
    spec = build_spec(c)
    assert len(spec.layers) == 3 and [e.layer for e in spec.schedule] == [0, 1, 2]
    windows = [l.mixer["window"] for l in spec.layers]
    assert windows == [5, 5, None]
    thetas = [l.mixer["position"]["theta"] for l in spec.layers]
    factors = [l.mixer["position"]["factor"] for l in spec.layers]
    assert thetas == [10000.0, 10000.0, 500000.0] and factors == [1.0, 1.0, 4.0]
    assert spec.layers[0].mixer["scale"] == pytest.approx(48 ** -0.5)
    assert spec.embedding["scale"] == pytest.approx(96 ** 0.5)
    assert spec.layers[0].norm["eps"] == 1e-5 and spec.layers[0].norm["unit_offset"] is True
    assert spec.head["tied"] is True and spec.head["softcap"] is None
    assert build_spec(read(tiny_models.CONFIG_C)).head["softcap"] == 30.0


def test_engine_config_reports_every_bad_field():
    with pytest.raises(ConfigError) as e:
        EngineConfig(dtype="fp8", page_size=24, max_num_seqs=0, max_prefill_chunk=4096,
                     max_num_batched_tokens=128).validate()
    assert len(e.value.problems) == 4
    assert EngineConfig().validate().cache_tokens() == 8 * 8192
