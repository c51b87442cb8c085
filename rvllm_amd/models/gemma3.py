"""The Gemma dense text decoder as a ``ModelSpec``.

What the architecture fixes (not read from config.json), each as the reference
has it:
  * embeddings are multiplied by sqrt(hidden_size)
    (v3/crates/rvllm-loader/src/gemma4_load.rs:219-253, metal_host.rs:298);
  * every layer is a sandwich of four RMSNorms around attention and a gated
    feed-forward (v3/crates/rvllm-runtime/src/gemma4_layer_exec.rs:1-28);
  * queries and keys are RMS-normed per head before the rotation
    (v3/kernels/fused_qk_rmsnorm.cu:3-6);
  * sliding layers rotate with the local base, global layers with the global
    base (v3/crates/rvllm-runtime/src/gemma4_bring_up.rs:3893-3902).
Where this decoder departs from the reference's Gemma-4 path it follows the
Gemma-3 checkpoints: norm gains are 1 + weight, the score scale is
query_pre_attn_scalar^-1/2, global layers divide positions by the linear
factor, values are not normed and there is no per-layer scalar.
"""

from __future__ import annotations

import math

from ..config.gemma3 import Gemma3Config
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
from .registry import Architecture, register_architecture


def build_spec(cfg: Gemma3Config, prefix: str = "model") -> ModelSpec:
    norm = PartSpec("rmsnorm", {"eps": cfg.rms_norm_eps, "unit_offset": True})
    qk_norm = {"eps": cfg.rms_norm_eps, "unit_offset": True}
    scale = cfg.query_pre_attn_scalar ** -0.5
    layers = []
    for l in range(cfg.num_hidden_layers):
        sliding = cfg.is_sliding(l)
        rope = cfg.rope_local if sliding else cfg.rope_global
        mixer = PartSpec("attention", {
            "num_heads": cfg.num_attention_heads,
            "num_kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim,
            "scale": scale,
            "window": cfg.sliding_window if sliding else None,
            "qk_norm": qk_norm,
            "position": PartSpec("rope", {"theta": rope.theta, "factor": rope.factor, "rotary_dim": cfg.head_dim}),
        })
        ff = PartSpec("gated_mlp", {
            "intermediate_size": cfg.intermediate_size,
            "activation": cfg.hidden_activation,
        })
        layers.append(LayerSpec(prefix=f"{prefix}.layers.{l}", block=PartSpec("sandwich"), mixer=mixer,
                                feed_forward=ff, norm=norm))
    return ModelSpec(
        architecture=cfg.architecture,
        hidden_size=cfg.hidden_size,
        vocab_size=cfg.vocab_size,
        max_position=cfg.max_position_embeddings,
        embedding=PartSpec("scaled_embedding", {"scale": math.sqrt(cfg.hidden_size)}),
        layers=tuple(layers),
        schedule=tuple(ScheduleEntry(l) for l in range(cfg.num_hidden_layers)),
        final_norm=norm,
        head=PartSpec("lm_head", {"tied": cfg.tie_word_embeddings, "softcap": cfg.final_logit_softcapping}),
        prefix=prefix,
    )


# Names under which config.json may announce this decoder.  The multimodal
# name is accepted for its text part (fields under text_config).
NAMES = ("Gemma3ForCausalLM", "Gemma3ForConditionalGeneration", "Gemma3TextModel")

for _name in NAMES:
    register_architecture(Architecture(
        name=_name,
        read_config=Gemma3Config.from_dict,
        build_spec=build_spec,
        write_config=Gemma3Config.to_dict,
    ))
