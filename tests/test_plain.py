"""What fixes the plain implementation beside the reference's text: vectors
that the reference's own tests hold, special cases that reduce to a library
routine, and invariants.  Each is chosen so that a plausible mistake (a wrong
sign or pairing in the rotation, a norm in the wrong place, a window off by
one, the scale on the wrong side of the embedding) fails it."""

import math

import pytest
import torch
import torch.nn.functional as F

import plain_gemma as P

torch.manual_seed(0)


# ---- RMSNorm ---------------------------------------------------------------
def test_rmsnorm_hand_calculation():
    # the reference's own vector: x / rms with unit gain
    # (v3/crates/rvllm-fused/src/reference.rs:341-350); unit gain is w = 0 here
    x = torch.tensor([[1.0, 2.0, 3.0, 4.0]])
    rms = math.sqrt((1 + 4 + 9 + 16) / 4 + 1e-6)
    got = P.rmsnorm(x, torch.zeros(4), 1e-6)
    assert torch.allclose(got, x / rms, atol=1e-7)


def test_rmsnorm_reduces_to_the_library_with_gain_one_plus_w():
    x, w = torch.randn(5, 24), torch.randn(24) * 0.1
    assert torch.allclose(P.rmsnorm(x, w, 1e-5), F.rms_norm(x, (24,), 1.0 + w, 1e-5), atol=1e-6)


def test_rmsnorm_eps_is_inside_the_root_and_scale_invariant_without_it():
    x = torch.full((1, 4), 1e-3)
    # mean(x^2) = 1e-6 = eps: the result is x / sqrt(2e-6), not x / (1e-3 + eps)
    assert torch.allclose(P.rmsnorm(x, torch.zeros(4), 1e-6), x / math.sqrt(2e-6), rtol=1e-5)
    y = torch.randn(3, 16)
    assert torch.allclose(P.rmsnorm(7.0 * y, torch.zeros(16), 0.0), P.rmsnorm(y, torch.zeros(16), 0.0), atol=1e-6)


# ---- rotation ----------------------------------------------------------------
def test_rope_golden_vector_of_the_reference():
    """v3/crates/rvllm-fused/src/gemma4_reference.rs:353-382: inputs (1, 2) and
    (3, 4) in the pairs (0, hd/2) and (1, hd/2 + 1), cos/sin (0.5, 0.8660254)
    and (-0.25, 0.96824586) give [-1.2320508, 1.8660254, -4.6229835, 1.9047375].
    The angles are fed through positions * inv_freq = angle."""
    hd = 8
    x = torch.zeros(1, 1, hd)
    x[0, 0, 0], x[0, 0, hd // 2] = 1.0, 2.0
    x[0, 0, 1], x[0, 0, hd // 2 + 1] = 3.0, 4.0
    x[0, 0, 2] = 7.0
    angles = torch.tensor([math.acos(0.5), math.atan2(0.96824586, -0.25), 0.0, 0.0], dtype=torch.float64)
    out = P.rope(x.double(), torch.tensor([1]), angles)
    want = [-1.2320508, 1.8660254, -4.6229835, 1.9047375]
    got = [out[0, 0, 0], out[0, 0, hd // 2], out[0, 0, 1], out[0, 0, hd // 2 + 1]]
    for g, w in zip(got, want):
        assert abs(g.item() - w) < 1e-5
    assert out[0, 0, 2].item() == 7.0  # angle 0 leaves the pair alone


def test_rope_identity_at_position_zero_and_norm_preserving():
    # v3/crates/rvllm-fused/src/reference.rs:416-418
    x = torch.randn(4, 3, 16)
    inv = P.rope_inv_freq(16, 10000.0, 1.0)
    assert torch.equal(P.rope(x, torch.zeros(4, dtype=torch.long), inv), x)
    y = P.rope(x, torch.tensor([3, 50, 700, 8000]), inv)
    pair = lambda t: t[..., :8] ** 2 + t[..., 8:] ** 2
    assert torch.allclose(pair(y), pair(x), atol=1e-4)


def test_rope_scores_depend_on_distance_only():
    q, k = torch.randn(1, 1, 32).double(), torch.randn(1, 1, 32).double()
    inv = P.rope_inv_freq(32, 10000.0, 1.0, torch.float64)
    dot = lambda pq, pk: (P.rope(q, torch.tensor([pq]), inv) * P.rope(k, torch.tensor([pk]), inv)).sum().item()
    assert abs(dot(5, 2) - dot(105, 102)) < 1e-9
    assert abs(dot(5, 2) - dot(2, 5)) > 1e-6  # the sign of the distance matters


def test_rope_inv_freq_uses_head_dim_and_linear_scaling_divides_positions():
    inv = P.rope_inv_freq(16, 10000.0, 1.0, torch.float64)
    assert inv[0] == 1.0 and abs(inv[1].item() - 10000.0 ** (-2 / 16)) < 1e-12 and len(inv) == 8
    x = torch.randn(2, 2, 16).double()
    scaled = P.rope(x, torch.tensor([8, 40]), P.rope_inv_freq(16, 1e6, 4.0, torch.float64))
    plain = P.rope(x, torch.tensor([2, 10]), P.rope_inv_freq(16, 1e6, 1.0, torch.float64))
    assert torch.allclose(scaled, plain, atol=1e-12)


# ---- attention ---------------------------------------------------------------
def sdpa(q, k, v, scale, mask):
    out = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1)[None], v.transpose(0, 1)[None],
                                         attn_mask=mask, scale=scale, enable_gqa=True)
    return out[0].transpose(0, 1)


def test_attention_reduces_to_the_library_causal_gqa():
    T, nq, nkv, hd = 11, 6, 3, 8
    q, k, v = torch.randn(T, nq, hd), torch.randn(T, nkv, hd), torch.randn(T, nkv, hd)
    causal = torch.tril(torch.ones(T, T, dtype=torch.bool))
    assert torch.allclose(P.attention(q, k, v, 0.3, None), sdpa(q, k, v, 0.3, causal), atol=1e-5)


def test_attention_window_is_a_band_including_self():
    T, nq, nkv, hd, w = 13, 4, 2, 8, 5
    q, k, v = torch.randn(T, nq, hd), torch.randn(T, nkv, hd), torch.randn(T, nkv, hd)
    i = torch.arange(T)
    band = (i[None, :] <= i[:, None]) & (i[:, None] - i[None, :] < w)  # 0 <= p - j < window
    assert torch.allclose(P.attention(q, k, v, 0.25, w), sdpa(q, k, v, 0.25, band), atol=1e-5)
    # a window at least as long as the sequence is no window
    assert torch.equal(P.attention(q, k, v, 0.25, T), P.attention(q, k, v, 0.25, None))
    # window 1: each token sees only itself and returns its own value (metal_host.rs:1297-1311)
    assert torch.allclose(P.attention(q, k, v, 0.25, 1), v.repeat_interleave(nq // nkv, dim=1), atol=1e-6)


def test_attention_far_key_is_found():
    """One key far back is made to stand out: a window or mask that drops it
    changes the result visibly."""
    T, hd = 300, 8
    q, k, v = torch.randn(T, 1, hd) * 0.1, torch.randn(T, 1, hd) * 0.1, torch.randn(T, 1, hd)
    k[3, 0] = 0
    k[3, 0, 0] = 50.0
    q[-1, 0] = 0
    q[-1, 0, 0] = 50.0
    out = P.attention(q, k, v, 1.0, None)
    assert torch.allclose(out[-1, 0], v[3, 0], atol=1e-4)
    assert not torch.allclose(P.attention(q, k, v, 1.0, 64)[-1, 0], v[3, 0], atol=1e-2)


def test_grouping_maps_query_head_to_kv_head_by_division():
    T, hd = 4, 4
    q = torch.randn(T, 4, hd)
    k, v = torch.randn(T, 2, hd), torch.randn(T, 2, hd)
    out = P.attention(q, k, v, 1.0, None)
    # heads 0, 1 read kv head 0; heads 2, 3 read kv head 1 (paged_attention_sm89.cu:71)
    solo = P.attention(q[:, 2:3], k[:, 1:2], v[:, 1:2], 1.0, None)
    assert torch.allclose(out[:, 2:3], solo, atol=1e-6)


# ---- feed-forward ------------------------------------------------------------
def test_gelu_tanh_is_the_library_form_and_its_symmetry():
    z = torch.linspace(-6, 6, 101)
    assert torch.allclose(P.gelu_tanh(z), F.gelu(z, approximate="tanh"), atol=1e-6)
    assert P.gelu_tanh(torch.zeros(1)).item() == 0.0
    assert torch.allclose(P.gelu_tanh(z) - P.gelu_tanh(-z), z, atol=1e-5)


def test_feed_forward_gate_is_activated_not_up():
    x = torch.randn(3, 8)
    wg, wu, wd = torch.randn(12, 8), torch.randn(12, 8), torch.randn(8, 12)
    want = (F.gelu(x @ wg.T, approximate="tanh") * (x @ wu.T)) @ wd.T
    assert torch.allclose(P.feed_forward(x, wg, wu, wd), want, atol=1e-5)
    assert not torch.allclose(P.feed_forward(x, wu, wg, wd), want, atol=1e-3)


def test_softcap_vector_of_the_reference():
    # v3/crates/rvllm-fused/src/gemma4_reference.rs:418-423: +-1000 -> +-30
    out = P.softcap(torch.tensor([1000.0, -1000.0, 0.3]), 30.0)
    assert abs(out[0].item() - 30.0) < 0.01 and abs(out[1].item() + 30.0) < 0.01
    assert abs(out[2].item() - 30.0 * math.tanh(0.01)) < 1e-6


# ---- the whole model -----------------------------------------------------------
def test_embedding_is_scaled_and_the_tied_head_is_not(plain_models):
    """With every layer's branch silenced (post-norm gains of zero, i.e.
    weight -1) the residual stream is the scaled embedding and the logits are
    norm(E[id] * sqrt(H)) . E^T with the unscaled table."""
    w, cfg = plain_models["A"]
    w = {k: v.float().clone() for k, v in w.items()}
    for l in range(cfg["layers"]):
        w[f"model.layers.{l}.post_attention_layernorm.weight"].fill_(-1.0)
        w[f"model.layers.{l}.post_feedforward_layernorm.weight"].fill_(-1.0)
    ids = [3, 200, 77]
    emb = w["model.embed_tokens.weight"]
    x = emb[ids] * math.sqrt(cfg["hidden"])
    want = P.rmsnorm(x, w["model.norm.weight"], cfg["eps"]) @ emb.T
    assert torch.allclose(P.forward(w, cfg, ids), want, atol=1e-5)
    # and the scale matters: eps makes the norm see it
    unscaled = P.rmsnorm(emb[ids], w["model.norm.weight"], cfg["eps"]) @ emb.T
    assert not torch.allclose(want, unscaled, atol=1e-4)


def test_a_shift_of_all_positions_changes_nothing_without_a_window_edge(plain_models):
    """Only distances count: the same tokens at shifted positions give the
    same layer output (full rotation, no absolute term)."""
    w, cfg = plain_models["B"]
    w = {k: v.double() for k, v in w.items()}
    x = torch.randn(6, cfg["hidden"], dtype=torch.float64)
    for kind in ("sliding", "global"):
        a = P.layer(x, torch.arange(6), w, "model.layers.0", cfg, kind)
        b = P.layer(x, torch.arange(6) + 1000, w, "model.layers.0", cfg, kind)
        assert torch.allclose(a, b, atol=1e-9)


def test_later_tokens_do_not_change_earlier_logits(plain_models):
    w, cfg = plain_models["B"]
    ids = list(range(40, 70))
    full = P.forward(w, cfg, ids)
    assert torch.allclose(P.forward(w, cfg, ids[:17]), full[:17], atol=1e-5)


def test_kinds_follow_the_pattern(plain_models):
    assert plain_models["A"][1]["kinds"] == ["sliding", "global"]
    assert plain_models["B"][1]["kinds"] == ["sliding", "sliding", "global"]
    assert plain_models["B"][1]["factor"] == 4.0 and plain_models["A"][1]["factor"] == 1.0


def test_greedy_takes_the_lowest_id_among_equal_maxima():
    # kernels/argmax.cu:16-25, pinned by rvllm-invariants/tests/identity.rs:91-128
    row = torch.tensor([2.0, 9.0, 4.0, 9.0, 1.0])
    assert int(torch.nonzero(row == row.max())[0]) == 1
    assert int(torch.nonzero(torch.full((4,), 1.5) == 1.5)[0]) == 0
