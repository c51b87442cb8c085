"""Typed configuration of the Gemma dense text decoder, read from config.json.

Which keys are read, which are required and what their limits are follows the
reference's parser (v3/crates/rvllm-loader/src/gemma4_arch.rs:107-429):
text fields live under ``text_config`` when that object exists (:129-136),
sizes are required (:155-190), the layer kinds come from ``layer_types`` or
from ``sliding_window_pattern`` (:543-581), the rotation bases from
``rope_parameters`` or flat keys (:255-265).  Keys that only the Gemma-4
variants use (shared KV layers, per-layer inputs, a second head size, partial
rotation) are accepted at their neutral value and rejected otherwise.

Added to what the reference reads, because the Gemma-3 decoder needs them:
``query_pre_attn_scalar`` (score scale), ``rope_scaling`` (linear scaling of
global layers), ``rope_local_base_freq``.
"""

from __future__ import annotations

import dataclasses
import math
from typing import Any, Optional

from .errors import ConfigError
from .fields import FieldReader

# Upper bounds, as in the reference (gemma4_arch.rs:13-17).
MAX_LAYERS = 1024
MAX_WIDTH = 1 << 20
MAX_VOCAB = 1 << 22
MAX_CONTEXT = 1 << 20

SLIDING = "sliding_attention"
GLOBAL = "full_attention"
_GLOBAL_ALIASES = ("full_attention", "global_attention")

ACTIVATIONS = ("gelu_pytorch_tanh", "gelu_tanh", "silu")


@dataclasses.dataclass(frozen=True)
class RopeParameters:
    """Rotation of one kind of layer: base and the linear position divisor."""

    theta: float
    factor: float = 1.0


@dataclasses.dataclass(frozen=True)
class Gemma3Config:
    architecture: str
    num_hidden_layers: int
    hidden_size: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    rms_norm_eps: float
    max_position_embeddings: int
    sliding_window: int
    layer_types: tuple[str, ...]
    rope_local: RopeParameters
    rope_global: RopeParameters
    query_pre_attn_scalar: float
    hidden_activation: str
    tie_word_embeddings: bool
    final_logit_softcapping: Optional[float] = None

    # ---- derived -----------------------------------------------------
    @property
    def q_size(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_key_value_heads * self.head_dim

    def is_sliding(self, layer: int) -> bool:
        return self.layer_types[layer] == SLIDING

    # ---- reading -----------------------------------------------------
    @classmethod
    def from_dict(cls, doc: dict, source: str = "config.json") -> "Gemma3Config":
        if not isinstance(doc, dict):
            raise ConfigError(source, ["top level must be a JSON object"])
        text = doc.get("text_config", doc)
        if not isinstance(text, dict):
            raise ConfigError(source, ["text_config must be an object"])
        r = FieldReader(text, outer=doc if text is not doc else None)

        archs = doc.get("architectures")
        architecture = archs[0] if isinstance(archs, list) and archs and isinstance(archs[0], str) else ""
        if not architecture:
            r.problem("missing or invalid required field architectures[0]")

        layers = r.integer("num_hidden_layers", lo=1, hi=MAX_LAYERS)
        hidden = r.integer("hidden_size", lo=1, hi=MAX_WIDTH)
        nq = r.integer("num_attention_heads", lo=1, hi=MAX_WIDTH)
        nkv = r.integer("num_key_value_heads", lo=1, hi=MAX_WIDTH)
        head_dim = r.integer("head_dim", lo=2, hi=MAX_WIDTH)
        inter = r.integer("intermediate_size", lo=1, hi=MAX_WIDTH)
        vocab = r.integer("vocab_size", lo=1, hi=MAX_VOCAB)
        eps = r.real("rms_norm_eps", positive=True)
        max_pos = r.integer("max_position_embeddings", lo=1, hi=MAX_CONTEXT)
        window = r.integer("sliding_window", "sliding_window_size", lo=1, hi=MAX_CONTEXT)
        tie = r.boolean("tie_word_embeddings")
        act = r.string("hidden_activation", "hidden_act")
        qpas = r.real("query_pre_attn_scalar", default=None, positive=True)
        softcap = r.real("final_logit_softcapping", "logit_softcapping", default=None, positive=True)

        if act and act not in ACTIVATIONS:
            r.problem(f"unsupported hidden_activation {act!r}; supported: {', '.join(ACTIVATIONS)}")
        if nq and nkv and nq % nkv != 0:
            r.problem(f"num_attention_heads={nq} must be a multiple of num_key_value_heads={nkv}")
        if head_dim % 2 != 0:
            r.problem(f"head_dim={head_dim} must be even")
        if window > max_pos:
            r.problem(f"sliding_window={window} exceeds max_position_embeddings={max_pos}")

        layer_types = _read_layer_types(r, layers)
        rope_local, rope_global = _read_rope(r)
        _reject_other_variants(r, head_dim, nkv)

        if r.raw("attn_logit_softcapping") is not None:
            r.problem("attn_logit_softcapping is not supported by this decoder (must be null)")

        if r.problems:
            raise ConfigError(source, r.problems)
        return cls(
            architecture=architecture,
            num_hidden_layers=layers,
            hidden_size=hidden,
            num_attention_heads=nq,
            num_key_value_heads=nkv,
            head_dim=head_dim,
            intermediate_size=inter,
            vocab_size=vocab,
            rms_norm_eps=eps,
            max_position_embeddings=max_pos,
            sliding_window=window,
            layer_types=layer_types,
            rope_local=rope_local,
            rope_global=rope_global,
            query_pre_attn_scalar=float(head_dim) if qpas is None else qpas,
            hidden_activation=act,
            tie_word_embeddings=tie,
            final_logit_softcapping=softcap,
        )

    # ---- writing -----------------------------------------------------
    def to_dict(self) -> dict[str, Any]:
        """The config.json that reads back as this configuration."""
        doc: dict[str, Any] = {
            "architectures": [self.architecture],
            "model_type": "gemma3_text",
            "num_hidden_layers": self.num_hidden_layers,
            "hidden_size": self.hidden_size,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size,
            "vocab_size": self.vocab_size,
            "rms_norm_eps": self.rms_norm_eps,
            "max_position_embeddings": self.max_position_embeddings,
            "sliding_window": self.sliding_window,
            "layer_types": list(self.layer_types),
            "rope_theta": self.rope_global.theta,
            "rope_local_base_freq": self.rope_local.theta,
            "rope_scaling": (
                {"rope_type": "linear", "factor": self.rope_global.factor}
                if self.rope_global.factor != 1.0
                else None
            ),
            "query_pre_attn_scalar": self.query_pre_attn_scalar,
            "hidden_activation": self.hidden_activation,
            "tie_word_embeddings": self.tie_word_embeddings,
            "final_logit_softcapping": self.final_logit_softcapping,
            "attn_logit_softcapping": None,
        }
        return doc


def _read_layer_types(r: FieldReader, layers: int) -> tuple[str, ...]:
    raw = r.raw("layer_types")
    if raw is not None:
        if not isinstance(raw, list):
            r.problem("layer_types must be a list of strings")
            return ()
        if len(raw) != layers:
            r.problem(f"layer_types has len {len(raw)}, expected {layers}")
            return ()
        out = []
        for i, kind in enumerate(raw):
            if kind == SLIDING:
                out.append(SLIDING)
            elif kind in _GLOBAL_ALIASES:
                out.append(GLOBAL)
            else:
                r.problem(f"unsupported layer_types[{i}]={kind!r}")
        return tuple(out)
    if r.has("sliding_window_pattern"):
        pattern = r.integer("sliding_window_pattern", lo=1, hi=MAX_LAYERS)
        # Layer l is global iff (l + 1) is a multiple of the pattern
        # (gemma4_arch.rs:566-577).
        return tuple(GLOBAL if (l + 1) % pattern == 0 else SLIDING for l in range(layers))
    r.problem("config must provide layer_types or sliding_window_pattern")
    return ()


def _read_rope(r: FieldReader) -> tuple[RopeParameters, RopeParameters]:
    """Rotation bases of the local and global layers and the global divisor.

    Three spellings are understood.  ``rope_parameters.{sliding_attention,
    full_attention}.rope_theta`` is the reference's (gemma4_arch.rs:255-265).
    ``rope_local_base_freq`` beside ``rope_theta`` is the Gemma-3 checkpoint
    spelling: there the bare ``rope_theta`` belongs to the *global* layers.
    ``rope_theta`` beside ``rope_theta_global`` is the reference's flat
    fallback, where the bare key belongs to the *local* layers.
    """
    params = r.raw("rope_parameters")
    local_theta = global_theta = None
    factor = 1.0
    if params is not None:
        if not isinstance(params, dict):
            r.problem("rope_parameters must be an object")
            params = {}
        r.used.add("rope_parameters")
        sl = params.get("sliding_attention") or {}
        fu = params.get("full_attention") or {}
        local_theta = sl.get("rope_theta")
        global_theta = fu.get("rope_theta")
        factor = _linear_factor(r, fu, "rope_parameters.full_attention", factor)
        _linear_factor(r, sl, "rope_parameters.sliding_attention", 1.0, must_be_one=True)
        for name, sub in (("sliding_attention", sl), ("full_attention", fu)):
            prf = sub.get("partial_rotary_factor", 1.0)
            if prf != 1.0:
                r.problem(f"rope_parameters.{name}.partial_rotary_factor={prf} is not supported (must be 1)")
    flat = r.real("rope_theta", default=None, positive=True)
    flat_local = r.real("rope_local_base_freq", default=None, positive=True)
    flat_global = r.real("rope_theta_global", default=None, positive=True)
    if local_theta is None:
        local_theta = flat_local if flat_local is not None else flat
    if global_theta is None:
        if flat_global is not None:
            global_theta = flat_global
        elif flat_local is not None:
            global_theta = flat  # Gemma-3 spelling: the bare key is the global base
        else:
            global_theta = local_theta  # the reference falls back to the local base
    scaling = r.raw("rope_scaling")
    if scaling is not None:
        if not isinstance(scaling, dict):
            r.problem("rope_scaling must be an object or null")
        else:
            factor = _linear_factor(r, scaling, "rope_scaling", factor)
    for name, value in (("local", local_theta), ("global", global_theta)):
        if not isinstance(value, (int, float)) or isinstance(value, bool) or not math.isfinite(value) or value <= 0:
            r.problem(f"missing or invalid rope_theta for the {name} layers")
            return RopeParameters(1.0), RopeParameters(1.0)
    return RopeParameters(float(local_theta), 1.0), RopeParameters(float(global_theta), float(factor))


def _linear_factor(r: FieldReader, obj: dict, where: str, current: float, must_be_one: bool = False) -> float:
    kind = obj.get("rope_type", obj.get("type"))
    if kind in (None, "default"):
        return current
    if kind != "linear":
        r.problem(f"{where}: unsupported rope_type {kind!r} (supported: default, linear)")
        return current
    factor = obj.get("factor")
    if isinstance(factor, bool) or not isinstance(factor, (int, float)) or not math.isfinite(factor) or factor <= 0:
        r.problem(f"{where}.factor must be a finite number > 0")
        return current
    if must_be_one and factor != 1.0:
        r.problem(f"{where}: scaling of the local layers is not supported")
    return float(factor)


def _reject_other_variants(r: FieldReader, head_dim: int, nkv: int) -> None:
    """Fields of the Gemma-4 variants must be absent or neutral
    (their meaning: gemma4_arch.rs:156-182,245-289)."""
    if r.integer("num_kv_shared_layers", default=0) != 0:
        r.problem("num_kv_shared_layers > 0 is not supported")
    if r.integer("hidden_size_per_layer_input", default=0) != 0:
        r.problem("hidden_size_per_layer_input > 0 (per-layer embeddings) is not supported")
    if r.integer("global_head_dim", default=head_dim) != head_dim:
        r.problem("global_head_dim different from head_dim is not supported")
    for key in ("num_global_key_value_heads", "num_key_value_heads_global", "global_num_key_value_heads"):
        if r.integer(key, default=nkv) != nkv:
            r.problem(f"{key} different from num_key_value_heads is not supported")
    if r.boolean("attention_k_eq_v", default=False):
        r.problem("attention_k_eq_v=true is not supported")
    if r.real("partial_rotary_factor", default=1.0) != 1.0:
        r.problem("partial_rotary_factor != 1 is not supported")
