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


# Prefixes under which a checkpoint may keep the text decoder
# (v3/crates/rvllm-loader/src/gemma4_arch.rs:624-658), told apart by where the embedding table lies.
TENSOR_PREFIXES = ("model.language_model", "language_model.model", "language_model", "model")
# Tensors of a multimodal checkpoint that the text decoder leaves alone.
IGNORED_TENSOR_PREFIXES = ("vision_tower.", "model.vision_tower.", "multi_modal_projector.",
                           "model.multi_modal_projector.")


def locate_tensors(names) -> dict:
    """Where a checkpoint keeps the decoder: the prefix of its layers, and the
    name of an untied head.  The reference looks the head up as plain
    ``lm_head.weight`` (v3/crates/rvllm-loader/src/gemma4_load.rs:431-436);
    checkpoints that nest the decoder keep the head beside it
    (``language_model.lm_head.weight``), so the name under the prefix's own
    first parts is tried too."""
    names = set(names)
    prefix = next((p for p in TENSOR_PREFIXES if f"{p}.embed_tokens.weight" in names), "model")
    parts = prefix.split(".")
    candidates = ["lm_head.weight"] + [".".join(parts[:n]) + ".lm_head.weight" for n in range(len(parts), 0, -1)]
    head = next((c for c in candidates if c in names), "lm_head.weight")
    return {"prefix": prefix, "head_weight": head}


def build_spec(cfg: Gemma3Config, prefix: str = "model", head_weight: str = "lm_head.weight") -> ModelSpec:
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
        head=PartSpec("lm_head", {"tied": cfg.tie_word_embeddings, "softcap": cfg.final_logit_softcapping,
                                  "weight_name": head_weight}),
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
        locate_tensors=locate_tensors,
        ignored_prefixes=IGNORED_TENSOR_PREFIXES,
    ))
