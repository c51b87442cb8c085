"""A plain, slow implementation of the Gemma dense text decoder: whole
sequences, no cache, one function per part, plain PyTorch operations (on the CPU
unless a test of many thousand tokens names another device).  It shares no
code with the engine; the tests compare the engine against it.

Every function is written from the reference's formulas and cites them
(paths relative to the reference's root).  Where the Gemma-3 decoder departs
from the reference's Gemma-4 path the docstring says so.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch


# --------------------------------------------------------------------------
# configuration: read straight from config.json's keys
# --------------------------------------------------------------------------
def read_config(model_dir) -> dict:
    """The fields the formulas need, from config.json (text_config if nested:
    v3/crates/rvllm-loader/src/gemma4_arch.rs:129-136)."""
    doc = json.loads((Path(model_dir) / "config.json").read_text())
    tc = doc.get("text_config", doc)
    n = tc["num_hidden_layers"]
    if tc.get("layer_types") is not None:
        kinds = ["sliding" if k == "sliding_attention" else "global" for k in tc["layer_types"]]
    else:
        # layer l is global iff (l + 1) % pattern == 0 (gemma4_arch.rs:566-577)
        pat = tc["sliding_window_pattern"]
        kinds = ["global" if (l + 1) % pat == 0 else "sliding" for l in range(n)]
    scaling = tc.get("rope_scaling") or {}
    return dict(
        layers=n,
        hidden=tc["hidden_size"],
        nq=tc["num_attention_heads"],
        nkv=tc["num_key_value_heads"],
        hd=tc["head_dim"],
        inter=tc["intermediate_size"],
        vocab=tc["vocab_size"],
        eps=tc["rms_norm_eps"],
        window=tc["sliding_window"],
        kinds=kinds,
        theta_local=tc.get("rope_local_base_freq", tc["rope_theta"]),
        theta_global=tc["rope_theta"],
        factor=float(scaling.get("factor", 1.0)),
        qpas=tc.get("query_pre_attn_scalar", tc["head_dim"]),
        softcap=tc.get("final_logit_softcapping"),
        tied=tc.get("tie_word_embeddings", True),
    )


# --------------------------------------------------------------------------
# parts
# --------------------------------------------------------------------------
def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """y = x * rsqrt(mean(x^2) + eps) * gain, eps inside the root
    (v3/kernels/rmsnorm_inplace_f16.cu:44-59, v3/crates/rvllm-fused/src/reference.rs:58-76).
    The reference multiplies by the stored weight; the Gemma-3 checkpoints
    store the gain minus one, so gain = 1 + w here."""
    ms = (x * x).mean(dim=-1, keepdim=True)
    return x * torch.rsqrt(ms + eps) * (1.0 + w)


def rope_inv_freq(hd: int, theta: float, factor: float, dtype=torch.float32) -> torch.Tensor:
    """inv_freq[i] = theta^(-2i/hd), i < hd/2 (v3/crates/rvllm-loader/src/gemma4_load.rs:1168-1179,
    v3/crates/rvllm-loader/src/metal_host.rs:281-289).  Linear scaling divides
    it by ``factor`` (not in the reference: the Gemma-3 global layers)."""
    i = torch.arange(hd // 2, dtype=torch.float64)
    return (theta ** (-2.0 * i / hd) / factor).to(dtype)


def rope(x: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """Split-half rotation of x[T, heads, hd]: pairs (i, i + hd/2),
    x'[i] = x[i] cos - x[i+hd/2] sin, x'[i+hd/2] = x[i] sin + x[i+hd/2] cos,
    angle = pos * inv_freq[i] (v3/kernels/fused_rope_partial_f16kv.cu:50-65,
    v3/crates/rvllm-fused/src/gemma4_reference.rs:155-165,
    v3/crates/rvllm-loader/src/metal_host.rs:1160-1166,1779-1790)."""
    half = x.shape[-1] // 2
    angle = positions.to(inv_freq.dtype)[:, None] * inv_freq[None, :]  # [T, hd/2]
    cos = torch.cos(angle)[:, None, :].to(x.dtype)
    sin = torch.sin(angle)[:, None, :].to(x.dtype)
    a, b = x[..., :half], x[..., half:]
    return torch.cat([a * cos - b * sin, a * sin + b * cos], dim=-1)


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, window) -> torch.Tensor:
    """Causal grouped-query attention of a whole sequence.
    q[T, nq, hd], k and v [T, nkv, hd]; query head h reads kv head h // (nq / nkv)
    (v3/kernels/paged_attention_sm89.cu:71).  Key j is visible to the query at
    p iff j <= p and, with a window, j >= p - window + 1
    (v3/crates/rvllm-runtime/src/gemma4_layer_exec.rs:801-804,
    v3/kernels/paged_attention_sm89.cu:96-105).  s = scale * q.k; softmax with
    the maximum subtracted; weighted sum of v
    (v3/crates/rvllm-loader/src/metal_host.rs:1358-1373)."""
    T, nq, hd = q.shape
    nkv = k.shape[1]
    group = nq // nkv
    out = torch.empty_like(q)
    pos = torch.arange(T, device=q.device)
    # Rows are taken ROWS_AT_A_TIME at a time, so that a long sequence needs no T x T table; a row's result does
    # not depend on the cut (every visible key of a row is in its piece, the others weigh exp(-inf) = 0).
    for r0 in range(0, T, ROWS_AT_A_TIME):
        r1 = min(T, r0 + ROWS_AT_A_TIME)
        c0 = 0 if window is None else max(0, r0 - window + 1)
        visible = pos[None, c0:r1] <= pos[r0:r1, None]
        if window is not None:
            visible &= pos[None, c0:r1] >= pos[r0:r1, None] - window + 1
        for h in range(nq):
            kh = h // group
            s = scale * (q[r0:r1, h, :] @ k[c0:r1, kh, :].T)  # [rows, keys]
            s = s.masked_fill(~visible, float("-inf"))
            s = s - s.max(dim=-1, keepdim=True).values
            p = torch.exp(s)
            p = p / p.sum(dim=-1, keepdim=True)
            out[r0:r1, h, :] = p @ v[c0:r1, kh, :]
    return out


ROWS_AT_A_TIME = 2048


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    """0.5 z (1 + tanh(0.7978845608 (z + 0.044715 z^3)))
    (v3/kernels/fused_gelu_mul_f16.cu:20-27, v3/crates/rvllm-fused/src/gemma4_reference.rs:27-30)."""
    return 0.5 * z * (1.0 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z * z * z)))


def feed_forward(x: torch.Tensor, w_gate, w_up, w_down) -> torch.Tensor:
    """down(gelu_tanh(gate(x)) * up(x)) (v3/crates/rvllm-runtime/src/gemma4_layer_exec.rs:1345-1726,
    steps 10 to 12)."""
    return (gelu_tanh(x @ w_gate.T) * (x @ w_up.T)) @ w_down.T


def softcap(logits: torch.Tensor, cap: float) -> torch.Tensor:
    """cap * tanh(logits / cap) (v3/kernels/logit_softcap.cu:28,
    v3/crates/rvllm-fused/src/gemma4_reference.rs:329-338)."""
    return cap * torch.tanh(logits / cap)


# --------------------------------------------------------------------------
# the whole model
# --------------------------------------------------------------------------
def find_prefix(weights: dict) -> str:
    for p in ("model.language_model", "language_model.model", "language_model", "model"):
        if f"{p}.embed_tokens.weight" in weights:
            return p
    raise KeyError("no embed_tokens.weight found")


def find_head(weights: dict) -> str:
    """An untied head: ``lm_head.weight`` under no prefix, as the reference
    looks it up (v3/crates/rvllm-loader/src/gemma4_load.rs:431-436), or beside
    a nested decoder."""
    for name in ("lm_head.weight", "language_model.lm_head.weight", "model.lm_head.weight"):
        if name in weights:
            return name
    raise KeyError("no lm_head.weight found")


def layer(x, positions, w: dict, p: str, cfg: dict, kind: str) -> torch.Tensor:
    """One decoder layer on a whole sequence x[T, H], in the order of
    v3/crates/rvllm-loader/src/metal_host.rs:492-628: input norm, q/k/v,
    per-head q and k norm (metal_host.rs:562-569), rotation, attention, output
    projection, post-attention norm added to the residual (:606-612),
    pre-feed-forward norm, feed-forward, post-feed-forward norm added (:614-628).
    Departures (Gemma 3): score scale query_pre_attn_scalar^-1/2 instead of
    the reference's 1 or 1/sqrt(hd) (gemma4_bring_up.rs:3840, metal_host.rs:570-573);
    no norm of v (fused_qkv_rmsnorm.cu:85-93 is Gemma-4 only); no layer scalar."""
    T = x.shape[0]
    nq, nkv, hd, eps = cfg["nq"], cfg["nkv"], cfg["hd"], cfg["eps"]
    h = rmsnorm(x, w[f"{p}.input_layernorm.weight"], eps)
    q = (h @ w[f"{p}.self_attn.q_proj.weight"].T).view(T, nq, hd)
    k = (h @ w[f"{p}.self_attn.k_proj.weight"].T).view(T, nkv, hd)
    v = (h @ w[f"{p}.self_attn.v_proj.weight"].T).view(T, nkv, hd)
    q = rmsnorm(q, w[f"{p}.self_attn.q_norm.weight"], eps)
    k = rmsnorm(k, w[f"{p}.self_attn.k_norm.weight"], eps)
    if kind == "sliding":
        inv_freq = rope_inv_freq(hd, cfg["theta_local"], 1.0)
        window = cfg["window"]
    else:
        inv_freq = rope_inv_freq(hd, cfg["theta_global"], cfg["factor"])
        window = None
    inv_freq = inv_freq.to(device=x.device, dtype=torch.float64 if x.dtype == torch.float64 else torch.float32)
    q = rope(q, positions, inv_freq)
    k = rope(k, positions, inv_freq)
    a = attention(q, k, v, float(cfg["qpas"]) ** -0.5, window).reshape(T, nq * hd)
    o = a @ w[f"{p}.self_attn.o_proj.weight"].T
    x = x + rmsnorm(o, w[f"{p}.post_attention_layernorm.weight"], eps)
    h = rmsnorm(x, w[f"{p}.pre_feedforward_layernorm.weight"], eps)
    f = feed_forward(h, w[f"{p}.mlp.gate_proj.weight"], w[f"{p}.mlp.up_proj.weight"], w[f"{p}.mlp.down_proj.weight"])
    return x + rmsnorm(f, w[f"{p}.post_feedforward_layernorm.weight"], eps)


def forward(weights: dict, cfg: dict, token_ids, dtype=torch.float32, device="cpu") -> torch.Tensor:
    """Logits [T, vocab] of a whole sequence.  Embedding times sqrt(hidden)
    (v3/crates/rvllm-loader/src/gemma4_load.rs:233-246, metal_host.rs:298); the
    layers; final norm; head against the *unscaled* embedding table when tied
    (gemma4_load.rs:431-457); optional soft-cap.  ``device``: where these plain
    tensor operations run (sequences of many thousand tokens take the CPU minutes); the
    result comes back to the CPU."""
    w = {k: v.to(device=device, dtype=dtype) for k, v in weights.items()}
    pre = find_prefix(w)
    ids = torch.as_tensor(list(token_ids), dtype=torch.long, device=device)
    positions = torch.arange(len(ids), device=device)
    emb = w[f"{pre}.embed_tokens.weight"]
    x = emb[ids] * torch.tensor(math.sqrt(cfg["hidden"]), dtype=torch.float32).to(dtype)
    for l in range(cfg["layers"]):
        x = layer(x, positions, w, f"{pre}.layers.{l}", cfg, cfg["kinds"][l])
    x = rmsnorm(x, w[f"{pre}.norm.weight"], cfg["eps"])
    head = emb if cfg["tied"] else w[find_head(w)]
    logits = x @ head.T
    if cfg["softcap"] is not None:
        logits = softcap(logits, cfg["softcap"])
    return logits.cpu()


def load_weights(model_dir) -> dict:
    """All tensors of model.safetensors, by name, through the safetensors
    package (not the engine's reader)."""
    from safetensors.torch import load_file

    return load_file(str(Path(model_dir) / "model.safetensors"))


def pick_greedy(row: torch.Tensor) -> int:
    """The id of the largest logit of a row; equal maxima give the lowest id:
    the reference scans from the left with a strict ``>``
    (kernels/argmax.cu:16-25, v3/crates/rvllm-fused/src/reference.rs:200-225)."""
    best, best_value = 0, None
    for i, value in enumerate(row.tolist()):
        if best_value is None or value > best_value:
            best, best_value = i, value
    return best


def greedy(weights: dict, cfg: dict, prompt, steps: int, dtype=torch.float32) -> list[int]:
    """Greedy continuation by re-running the whole sequence every step."""
    ids = list(prompt)
    out = []
    for _ in range(steps):
        best = pick_greedy(forward(weights, cfg, ids, dtype)[-1])
        out.append(best)
        ids.append(best)
    return out
