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
    # the reference's golden rows: v3/crates/rvllm-invariants/tests/identity.rs:91-128
    assert P.pick_greedy(torch.tensor([2.0, 9.0, 4.0, 9.0, 1.0])) == 1
    assert P.pick_greedy(torch.full((4,), 1.5)) == 0
    assert P.pick_greedy(torch.tensor([0.1, 0.2, 9.9, 0.3])) == 2
    assert P.pick_greedy(torch.tensor([7.0, 0.0, 1.0, 2.0])) == 0


def test_greedy_generation_feeds_its_choice_back(plain_models):
    """Each chosen token is the pick of the row the whole sequence so far ends in."""
    w, cfg = plain_models["A"]
    prompt = [5, 17, 3]
    out = P.greedy(w, cfg, prompt, 3)
    ids = list(prompt)
    for token in out:
        assert token == P.pick_greedy(P.forward(w, cfg, ids)[-1])
        ids.append(token)


# ---- what the Gemma-3 decoder has beyond the reference's text, pinned by a second composition -------------
def library_layer(x, positions, w, p, cfg, kind):
    """One layer put together from library routines and the other common
    spelling of the rotation (x cos + rotate_half(x) sin): ``F.rms_norm`` with
    the gain 1 + w, ``F.scaled_dot_product_attention`` with an explicit band or
    causal mask, ``F.gelu(approximate="tanh")``.  It shares no line with
    ``plain_gemma.layer``."""
    T = x.shape[0]
    nq, nkv, hd, eps = cfg["nq"], cfg["nkv"], cfg["hd"], cfg["eps"]
    norm = lambda t, name: F.rms_norm(t, (t.shape[-1],), 1.0 + w[f"{p}.{name}.weight"], eps)
    h = norm(x, "input_layernorm")
    q = F.linear(h, w[f"{p}.self_attn.q_proj.weight"]).view(T, nq, hd)
    k = F.linear(h, w[f"{p}.self_attn.k_proj.weight"]).view(T, nkv, hd)
    v = F.linear(h, w[f"{p}.self_attn.v_proj.weight"]).view(T, nkv, hd)
    q, k = norm(q, "self_attn.q_norm"), norm(k, "self_attn.k_norm")
    theta, factor = (cfg["theta_local"], 1.0) if kind == "sliding" else (cfg["theta_global"], cfg["factor"])
    # the inverse frequencies are a 32-bit table (rounded once, after the division by the factor)
    freqs = (1.0 / (theta ** (torch.arange(0, hd, 2, dtype=torch.float64) / hd)) / factor).float().double()
    angle = torch.outer(positions.double(), freqs)
    cos, sin = torch.cat([angle.cos()] * 2, -1)[:, None, :], torch.cat([angle.sin()] * 2, -1)[:, None, :]
    rotate_half = lambda t: torch.cat([-t[..., hd // 2:], t[..., : hd // 2]], -1)
    q, k = q * cos + rotate_half(q) * sin, k * cos + rotate_half(k) * sin
    i = torch.arange(T)
    mask = i[None, :] <= i[:, None]
    if kind == "sliding":
        mask &= i[:, None] - i[None, :] < cfg["window"]
    a = sdpa(q, k, v, cfg["qpas"] ** -0.5, mask).reshape(T, nq * hd)
    x = x + norm(F.linear(a, w[f"{p}.self_attn.o_proj.weight"]), "post_attention_layernorm")
    h = norm(x, "pre_feedforward_layernorm")
    f = F.linear(F.gelu(F.linear(h, w[f"{p}.mlp.gate_proj.weight"]), approximate="tanh")
                 * F.linear(h, w[f"{p}.mlp.up_proj.weight"]), w[f"{p}.mlp.down_proj.weight"])
    return x + norm(f, "post_feedforward_layernorm")


@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("kind", ["sliding", "global"])
def test_layer_equals_a_composition_of_library_routines(plain_models, name, kind):
    w, cfg = plain_models[name]
    w = {k: v.double() for k, v in w.items()}
    T = 3 * cfg["window"] + 5 if cfg["window"] < 40 else cfg["window"] + 30  # past every window's edge
    x = torch.randn(T, cfg["hidden"], dtype=torch.float64)
    positions = torch.arange(T)
    got = P.layer(x, positions, w, "model.layers.0", cfg, kind)
    want = library_layer(x, positions, w, "model.layers.0", cfg, kind)
    assert torch.allclose(got, want, atol=1e-9)


def test_score_scale_is_the_scalar_to_the_power_minus_one_half(plain_models):
    """Scores are q.k * query_pre_attn_scalar^-1/2 with q normed by the gain
    1 + w: a scalar four times as large and a query gain twice as large cancel.
    A scale of 1/scalar, a scale taken from the head size, or a gain of w
    instead of 1 + w each break the equality."""
    w, cfg = plain_models["B"]
    w = {k: v.double() for k, v in w.items()}
    assert cfg["qpas"] != cfg["hd"]
    x = torch.randn(12, cfg["hidden"], dtype=torch.float64)
    pos = torch.arange(12)
    base = P.layer(x, pos, w, "model.layers.2", cfg, "global")
    w2 = dict(w)
    gain = 1.0 + w["model.layers.2.self_attn.q_norm.weight"]
    w2["model.layers.2.self_attn.q_norm.weight"] = 2.0 * gain - 1.0
    other = P.layer(x, pos, w2, "model.layers.2", dict(cfg, qpas=4 * cfg["qpas"]), "global")
    assert torch.allclose(base, other, atol=1e-10)
    assert not torch.allclose(base, P.layer(x, pos, w, "model.layers.2", dict(cfg, qpas=4 * cfg["qpas"]), "global"),
                              atol=1e-6)


def test_each_layer_kind_reads_its_own_base_and_only_global_layers_scale(plain_models):
    w, cfg = plain_models["B"]
    w = {k: v.double() for k, v in w.items()}
    x = torch.randn(9, cfg["hidden"], dtype=torch.float64)
    pos = torch.arange(9) + 40
    run = lambda c, kind: P.layer(x, pos, w, "model.layers.0", c, kind)
    # a sliding layer knows nothing of the global base or the factor; a global one nothing of the local base
    assert torch.equal(run(cfg, "sliding"), run(dict(cfg, theta_global=123.0, factor=9.0), "sliding"))
    assert torch.equal(run(cfg, "global"), run(dict(cfg, theta_local=123.0, window=2), "global"))
    assert not torch.allclose(run(cfg, "global"), run(dict(cfg, theta_global=123.0), "global"), atol=1e-6)
    assert not torch.allclose(run(cfg, "sliding"), run(dict(cfg, theta_local=123.0), "sliding"), atol=1e-6)
    # the factor divides the positions of a global layer: factor 4 at positions 4p is factor 1 at positions p
    a = P.layer(x, 4 * torch.arange(9), w, "model.layers.0", cfg, "global")
    b = P.layer(x, torch.arange(9), w, "model.layers.0", dict(cfg, factor=1.0), "global")
    assert cfg["factor"] == 4.0 and torch.allclose(a, b, atol=1e-10)


def test_query_and_key_norm_come_before_the_rotation(plain_models):
    """With gains that differ inside a rotated pair, norming after the rotation
    would make scores depend on the positions themselves; normed first, only
    distances count, under any gains."""
    w, cfg = plain_models["B"]
    w = {k: v.double() for k, v in w.items()}
    g = torch.Generator().manual_seed(4)
    for n in ("q_norm", "k_norm"):
        w[f"model.layers.2.self_attn.{n}.weight"] = torch.randn(cfg["hd"], generator=g, dtype=torch.float64)
    x = torch.randn(7, cfg["hidden"], dtype=torch.float64, generator=g)
    a = P.layer(x, torch.arange(7), w, "model.layers.2", cfg, "global")
    b = P.layer(x, torch.arange(7) + 333, w, "model.layers.2", cfg, "global")
    assert torch.allclose(a, b, atol=1e-9)


def test_the_untied_head_is_its_own_matrix(plain_models):
    w, cfg = plain_models["A"]
    w = {k: v.float().clone() for k, v in w.items()}
    ids = [9, 8, 7, 6]
    tied = P.forward(w, cfg, ids)
    head = torch.randn(cfg["vocab"], cfg["hidden"], generator=torch.Generator().manual_seed(8)) * 0.02
    for name in ("lm_head.weight", "language_model.lm_head.weight"):
        untied = P.forward(dict(w, **{name: head}), dict(cfg, tied=False), ids)
        # the same final hidden state against another matrix: the input side still reads the embedding table
        x = torch.linalg.lstsq(w["model.embed_tokens.weight"].double(), tied.double().T).solution.T  # hidden rows
        assert torch.allclose(untied.double(), x @ head.double().T, atol=1e-4)
    assert not torch.allclose(untied, tied, atol=1e-3)
