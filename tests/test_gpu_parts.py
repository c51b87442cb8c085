"""Each part of a layer alone against the plain implementation, and a toy
mixer with a state of its own — defined here, not in the framework — that is
registered, built from a model folder and stepped through the same engine."""

import dataclasses
import json
import math

import pytest
import torch

import plain_gemma as P
from rvllm_amd.cache.manager import CacheManager
from rvllm_amd.cache.storage import CacheStorage
from rvllm_amd.config.engine_config import EngineConfig
from rvllm_amd.engine.batch import BatchBuilder, Portion
from rvllm_amd.engine.runner import ModelRunner
from rvllm_amd.kernels import ops
from rvllm_amd.models import Architecture, register_architecture, unregister_architecture
from rvllm_amd.parts import (BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITION_ENCODINGS, Embedding,
                             FeedForward, Head, LayerSpec, Mixer, ModelSpec, ParamSpec, PartSpec, PositionEncoding,
                             ScheduleEntry, StateNeed)
from rvllm_amd.parts.linear import linear
from rvllm_amd.weights.random_init import random_tensors, write_random_model

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def bound(part, prefix, dtype, seed=0):
    tensors = random_tensors(part.param_specs(prefix), seed, "cpu", dtype)
    part.bind(tensors, prefix, DEV, dtype)
    return {k: v.double() for k, v in tensors.items()}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_part(dtype):
    norm = NORMS.build(PartSpec("rmsnorm", {"eps": 1e-5, "unit_offset": True}), width=72, name="some_norm")
    assert [s.name for s in norm.param_specs("model.layers.3")] == ["model.layers.3.some_norm.weight"]
    w = bound(norm, "model.layers.3", dtype)["model.layers.3.some_norm.weight"]
    x = torch.randn(5, 72).to(dtype)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert torch.allclose(norm.forward(x.to(DEV)).cpu().double(), P.rmsnorm(x.double(), w, 1e-5), atol=tol, rtol=tol)
    plain = NORMS.build(PartSpec("rmsnorm", {"eps": 1e-5}), width=72, name="n")
    plain.bind({"p.n.weight": w.to(dtype)}, "p", DEV, dtype)
    want = P.rmsnorm(x.double(), torch.zeros(72).double(), 1e-5) * w.to(dtype).double()
    assert torch.allclose(plain.forward(x.to(DEV)).cpu().double(), want, atol=tol, rtol=tol)


def test_rope_part_tables():
    rope = POSITION_ENCODINGS.build(PartSpec("rope", {"theta": 5e5, "factor": 4.0}), head_dim=32)
    assert rope.rotary_dim == 32
    assert torch.equal(rope.inv_freq(DEV).cpu(), P.rope_inv_freq(32, 5e5, 4.0))
    # the step's tables: made once and shared by parts with the same parameters, not by others
    import types
    step = types.SimpleNamespace(positions=torch.tensor([3, 4, 900], dtype=torch.int32, device=DEV), num_tokens=3,
                                 shared={})
    cos, sin = rope.tables(step)
    angle = torch.tensor([3.0, 4.0, 900.0])[:, None] * P.rope_inv_freq(32, 5e5, 4.0)[None, :]
    assert torch.allclose(cos.cpu(), angle.cos(), atol=1e-6) and torch.allclose(sin.cpu(), angle.sin(), atol=1e-6)
    twin = POSITION_ENCODINGS.build(PartSpec("rope", {"theta": 5e5, "factor": 4.0}), head_dim=32)
    other = POSITION_ENCODINGS.build(PartSpec("rope", {"theta": 5e5, "factor": 1.0}), head_dim=32)
    assert twin.tables(step)[0] is cos and other.tables(step)[0] is not cos and len(step.shared) == 2
    none = POSITION_ENCODINGS.build(PartSpec("none"), head_dim=32)
    assert none.rotary_dim == 0 and none.inv_freq(DEV) is None and none.tables(step) is None
    with pytest.raises(ValueError):
        POSITION_ENCODINGS.build(PartSpec("rope", {"theta": 1e4, "rotary_dim": 7}), head_dim=32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_feed_forward_part(dtype):
    ff = FEED_FORWARDS.build(PartSpec("gated_mlp", {"intermediate_size": 88, "activation": "gelu_pytorch_tanh"}),
                             hidden_size=40)
    w = bound(ff, "L", dtype)
    x = torch.randn(6, 40).to(dtype)
    want = P.feed_forward(x.double(), w["L.mlp.gate_proj.weight"], w["L.mlp.up_proj.weight"],
                          w["L.mlp.down_proj.weight"])
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    got = ops.as_tensor(ff.forward(x.to(DEV), None)).cpu().double()
    assert (got - want).abs().max() <= tol * max(1.0, want.abs().max().item())


def attention_harness(mixer, page_size=16, num_pages=32, max_tokens=256):
    cache = CacheManager([mixer.cache_need()], page_size, num_pages, 2)
    storage = CacheStorage(cache, DEV, mixer.w_o.dtype)
    builder = BatchBuilder(DEV, max_tokens, 2, {name: num_pages for name in cache.groups})
    return cache, storage, builder


def run_portions(mixer, x, cuts):
    """Feed x[T, H] of one request through the mixer in portions."""
    cache, storage, builder = attention_harness(mixer)
    cache.add_request("r")
    outs, start = [], 0
    group = next(iter(cache.groups))
    for n in cuts:
        cache.extend("r", start + n)
        batch = builder.build([Portion("r", [0] * n, start)], {group: [cache.table("r", group)]}, [cache.slot("r")])
        # a part may hand back the unreduced K slices of its last product; as_tensor adds them up
        outs.append(ops.as_tensor(mixer.forward(x[start:start + n].to(DEV), batch, storage.views[0])).cpu())
        cache.commit("r", start + n)
        start += n
    return torch.cat(outs)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window,rope", [(None, True), (6, True), (None, False), (20, False)])
def test_attention_part(dtype, window, rope):
    H, nq, nkv, hd, T = 56, 6, 2, 16, 45
    spec = PartSpec("attention", {
        "num_heads": nq, "num_kv_heads": nkv, "head_dim": hd, "scale": 0.2, "window": window,
        "qk_norm": {"eps": 1e-6, "unit_offset": True},
        "position": PartSpec("rope", {"theta": 1e4, "factor": 2.0}) if rope else PartSpec("none"),
    })
    mixer = MIXERS.build(spec, hidden_size=H)
    w = bound(mixer, "L", dtype, seed=3)
    x = torch.randn(T, H).to(dtype)
    # the plain layer's attention branch
    xd = x.double()
    q = P.rmsnorm((xd @ w["L.self_attn.q_proj.weight"].T).view(T, nq, hd), w["L.self_attn.q_norm.weight"], 1e-6)
    k = P.rmsnorm((xd @ w["L.self_attn.k_proj.weight"].T).view(T, nkv, hd), w["L.self_attn.k_norm.weight"], 1e-6)
    v = (xd @ w["L.self_attn.v_proj.weight"].T).view(T, nkv, hd)
    if rope:
        inv = P.rope_inv_freq(hd, 1e4, 2.0, torch.float64)
        q, k = P.rope(q, torch.arange(T), inv), P.rope(k, torch.arange(T), inv)
    want = P.attention(q, k, v, 0.2, window).reshape(T, nq * hd) @ w["L.self_attn.o_proj.weight"].T
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    for cuts in ([T], [17, 1, 1, 2, 16, 8]):
        got = run_portions(mixer, x, cuts).double()
        assert (got - want).abs().max() <= tol * max(1.0, want.abs().max().item()), cuts


def test_attention_without_rotation_or_norm_is_plain_softmax_attention():
    """The special case that reduces to the library routine."""
    H, nq, hd, T = 32, 2, 16, 12
    spec = PartSpec("attention", {"num_heads": nq, "num_kv_heads": nq, "head_dim": hd, "scale": hd ** -0.5,
                                  "window": None, "qk_norm": None, "position": None})
    mixer = MIXERS.build(spec, hidden_size=H)
    assert len(mixer.param_specs("L")) == 4  # no norm weights asked for
    w = bound(mixer, "L", torch.float32, seed=4)
    x = torch.randn(T, H)
    q, k, v = ((x.double() @ w[f"L.self_attn.{n}_proj.weight"].T).view(T, nq, hd).transpose(0, 1) for n in "qkv")
    lib = torch.nn.functional.scaled_dot_product_attention(q[None], k[None], v[None], is_causal=True)[0]
    want = lib.transpose(0, 1).reshape(T, nq * hd) @ w["L.self_attn.o_proj.weight"].T
    assert torch.allclose(run_portions(mixer, x, [5, 7]).double(), want, atol=1e-5)


def test_block_part_is_the_plain_layer(plain_models):
    from rvllm_amd.models.gemma3 import build_spec
    from rvllm_amd.config.gemma3 import Gemma3Config
    import tiny_models

    weights, cfg = plain_models["B"]
    spec = build_spec(Gemma3Config.from_dict(tiny_models.CONFIG_B))
    for layer_index in (0, 2):  # a sliding and a global layer
        layer = spec.layers[layer_index]
        block = BLOCKS.build(layer.block, layer=layer, hidden_size=spec.hidden_size)
        block.bind({k: v.float() for k, v in weights.items()}, layer.prefix, DEV, torch.float32)
        T = 19
        x = torch.randn(T, spec.hidden_size)
        want = P.layer(x.double(), torch.arange(T), {k: v.double() for k, v in weights.items()}, layer.prefix, cfg,
                       cfg["kinds"][layer_index])
        cache, storage, builder = attention_harness(block.mixer)
        cache.add_request("r")
        cache.extend("r", T)
        group = next(iter(cache.groups))
        batch = builder.build([Portion("r", [0] * T, 0)], {group: [cache.table("r", group)]}, [0])
        xs = x.to(DEV)
        assert block.forward(xs, batch, storage.views[0]) is None  # no next norm was asked for
        assert torch.allclose(xs.cpu().double(), want, atol=2e-5)


# --------------------------------------------------------------------------
# A toy mixer with a state of its own, and a toy architecture around it.
# --------------------------------------------------------------------------
class RunningMeanMixer(Mixer):
    """y[t] = W @ mean(x[0..t]): keeps the running sum and the count of a
    request in a slot of fixed size, portions must continue where the slot
    left off.  It reads the step's slots on the host and launches by what it finds there, so its work
    cannot be recorded into a graph: it says so, and the runner then never takes a step from one."""

    capturable = False

    def __init__(self, spec, *, hidden_size):
        self.hidden = hidden_size
        self.w = None

    def param_specs(self, prefix):
        return [ParamSpec(f"{prefix}.mean_mixer.weight", (self.hidden, self.hidden), init=("normal", 0.3))]

    def bind(self, tensors, prefix, device, dtype):
        self.w = tensors[f"{prefix}.mean_mixer.weight"].to(device=device, dtype=dtype)

    def cache_need(self):
        return StateNeed((self.hidden + 1,), torch.float32)

    def forward(self, x, step, cache):
        out = torch.empty_like(x)
        starts = step.host_q_start
        slots = step.state_slot.cpu().tolist()
        for b in range(step.num_requests):
            lo, hi = int(starts[b]), int(starts[b + 1])
            state = cache.slots[slots[b]]
            sums = state[: self.hidden] + torch.cumsum(x[lo:hi].float(), dim=0)
            counts = state[self.hidden] + torch.arange(1, hi - lo + 1, device=x.device, dtype=torch.float32)
            out[lo:hi] = ((sums / counts[:, None]).to(x.dtype) @ self.w.T)
            if cache.writes:
                state[: self.hidden] = sums[-1]
                state[self.hidden] = counts[-1]
        return out


@dataclasses.dataclass(frozen=True)
class ToyConfig:
    architecture: str
    hidden: int
    vocab: int
    layers: int

    @classmethod
    def from_dict(cls, doc, source="config.json"):
        return cls(doc["architectures"][0], doc["toy_hidden"], doc["toy_vocab"], doc["toy_layers"])

    def to_dict(self):
        return {"architectures": [self.architecture], "toy_hidden": self.hidden, "toy_vocab": self.vocab,
                "toy_layers": self.layers}


def toy_spec(cfg: ToyConfig, prefix="model") -> ModelSpec:
    norm = PartSpec("rmsnorm", {"eps": 1e-6, "unit_offset": False})
    attn = PartSpec("attention", {"num_heads": 2, "num_kv_heads": 1, "head_dim": 16, "scale": 0.25, "window": None,
                                  "qk_norm": None, "position": PartSpec("rope", {"theta": 100.0})})
    ff = PartSpec("gated_mlp", {"intermediate_size": 2 * cfg.hidden, "activation": "silu"})
    layers = []
    for l in range(cfg.layers):
        mixer = PartSpec("running_mean") if l % 2 == 0 else attn  # different mixers in different layers
        layers.append(LayerSpec(f"{prefix}.layers.{l}", PartSpec("sandwich"), mixer, ff, norm))
    # the order of layers is data: layer 1 runs twice, the second time reading its own cache only
    schedule = [ScheduleEntry(l) for l in range(cfg.layers)] + [ScheduleEntry(1, cache_from=1)]
    return ModelSpec(cfg.architecture, cfg.hidden, cfg.vocab, 512, PartSpec("scaled_embedding", {"scale": 1.0}),
                     tuple(layers), tuple(schedule), norm, PartSpec("lm_head", {"tied": True}), prefix)


@pytest.fixture
def toy_architecture():
    MIXERS.register("running_mean", RunningMeanMixer, replace=True)
    arch = register_architecture(Architecture("ToyForCausalLM", ToyConfig.from_dict, toy_spec, ToyConfig.to_dict),
                                 replace=True)
    yield arch
    unregister_architecture("ToyForCausalLM")
    MIXERS.unregister("running_mean")


def toy_plain(weights, cfg: ToyConfig, ids):
    """The toy model on a whole sequence, written out plainly."""
    w = {k: v.double() for k, v in weights.items()}
    norm = lambda x, name: x * torch.rsqrt((x * x).mean(-1, keepdim=True) + 1e-6) * w[name]
    x = w["model.embed_tokens.weight"][ids]
    T = len(ids)
    kept = {}  # keys and values of a layer's first run; a run that reads another run's cache uses these
    for run, l in enumerate(list(range(cfg.layers)) + [1]):
        p = f"model.layers.{l}"
        h = norm(x, f"{p}.input_layernorm.weight")
        if l % 2 == 0:
            mean = torch.cumsum(h, 0) / torch.arange(1, T + 1, dtype=torch.float64)[:, None]
            a = mean @ w[f"{p}.mean_mixer.weight"].T
        else:
            inv = P.rope_inv_freq(16, 100.0, 1.0, torch.float64)
            q = P.rope((h @ w[f"{p}.self_attn.q_proj.weight"].T).view(T, 2, 16), torch.arange(T), inv)
            if run < cfg.layers:
                k = P.rope((h @ w[f"{p}.self_attn.k_proj.weight"].T).view(T, 1, 16), torch.arange(T), inv)
                kept[l] = (k, (h @ w[f"{p}.self_attn.v_proj.weight"].T).view(T, 1, 16))
            k, v = kept[l]
            a = P.attention(q, k, v, 0.25, None).reshape(T, 32) @ w[f"{p}.self_attn.o_proj.weight"].T
        x = x + norm(a, f"{p}.post_attention_layernorm.weight")
        h = norm(x, f"{p}.pre_feedforward_layernorm.weight")
        f = (torch.nn.functional.silu(h @ w[f"{p}.mlp.gate_proj.weight"].T) * (h @ w[f"{p}.mlp.up_proj.weight"].T)) \
            @ w[f"{p}.mlp.down_proj.weight"].T
        x = x + norm(f, f"{p}.post_feedforward_layernorm.weight")
    return norm(x, "model.norm.weight") @ w["model.embed_tokens.weight"].T


def test_toy_mixer_with_state_is_registered_built_and_stepped(tmp_path, toy_architecture):
    cfg = ToyConfig("ToyForCausalLM", hidden=24, vocab=50, layers=3)
    folder = write_random_model(tmp_path / "toy", cfg, seed=7, dtype=torch.float32)
    assert json.loads((folder / "config.json").read_text())["toy_hidden"] == 24
    engine_cfg = EngineConfig(dtype="float32", max_model_len=128, max_num_seqs=3, max_num_batched_tokens=128,
                              max_prefill_chunk=128, max_cache_tokens=256)
    runner = ModelRunner.from_model_dir(folder, engine_cfg)
    # layer 0 and 2 keep a state slot, layer 1 keeps pages
    assert runner.cache.state_layers == [0, 2] and runner.cache.layer_group == [None, "full", None]
    weights = P.load_weights(folder)
    seqs = {"a": [3, 14, 15, 9, 26, 5, 35, 8, 9, 7, 9, 3], "b": [2, 7, 18, 28, 18, 28, 4, 5]}
    want = {k: toy_plain(weights, cfg, v) for k, v in seqs.items()}
    # whole
    for name, ids in seqs.items():
        runner.add_request(name)
        got = runner.step([(name, ids, list(range(len(ids))))]).cpu().double()
        assert torch.allclose(got, want[name], atol=1e-4), name
        runner.release(name)
    # cut and mixed: the slot carries the state from portion to portion, and a
    # slot that is handed out again starts from zero
    runner.add_request("a2")
    runner.add_request("b2")
    g1 = runner.step([("a2", seqs["a"][:5], list(range(5))), ("b2", seqs["b"][:2], [0, 1])]).cpu().double()
    g2 = runner.step([("b2", seqs["b"][2:3], [0]), ("a2", seqs["a"][5:], list(range(7)))]).cpu().double()
    g3 = runner.step([("b2", seqs["b"][3:], list(range(5)))]).cpu().double()
    got_a = torch.cat([g1[:5], g2[1:]])
    got_b = torch.cat([g1[5:], g2[:1], g3])
    assert torch.allclose(got_a, want["a"], atol=1e-4) and torch.allclose(got_b, want["b"], atol=1e-4)
    runner.release("a2")
    runner.release("b2")
    runner.cache.check()


# --------------------------------------------------------------------------
# A toy feed-forward with routing and a toy position encoding, defined here and
# plugged in through the registries: no file of the framework changes.
# --------------------------------------------------------------------------
class TopOneExperts(FeedForward):
    """A router picks one of E small gated MLPs per token (router logits in 32-bit)."""

    def __init__(self, spec, *, hidden_size):
        self.hidden, self.experts, self.inter = hidden_size, int(spec["experts"]), int(spec["intermediate_size"])

    def param_specs(self, prefix):
        p = f"{prefix}.moe"
        specs = [ParamSpec(f"{p}.router.weight", (self.experts, self.hidden), init=("normal", 0.5))]
        for e in range(self.experts):
            specs += [ParamSpec(f"{p}.experts.{e}.gate_up.weight", (2 * self.inter, self.hidden), init=("normal", 0.2)),
                      ParamSpec(f"{p}.experts.{e}.down.weight", (self.hidden, self.inter), init=("normal", 0.2))]
        return specs

    def bind(self, tensors, prefix, device, dtype):
        p = f"{prefix}.moe"
        self.router = tensors[f"{p}.router.weight"].to(device=device, dtype=torch.float32)
        self.gate_up = [tensors[f"{p}.experts.{e}.gate_up.weight"].to(device=device, dtype=dtype) for e in range(self.experts)]
        self.down = [tensors[f"{p}.experts.{e}.down.weight"].to(device=device, dtype=dtype) for e in range(self.experts)]

    def forward(self, x, step):
        choice = (x.float() @ self.router.T).argmax(dim=-1)
        out = torch.zeros_like(x)
        for e in range(self.experts):
            rows = (choice == e).nonzero().flatten()
            if rows.numel():
                act = ops.gated_act(linear(x[rows].contiguous(), self.gate_up[e]), "silu")  # the framework's kernels
                out[rows] = linear(act, self.down[e])
        return out


class RootPositions(PositionEncoding):
    """Rotation by the angle sqrt(position) * inv_freq[i]: another rule for the angles, the same kernel."""

    def __init__(self, spec, *, head_dim):
        self.rotary_dim = head_dim
        self.inv = 50.0 ** (-2.0 * torch.arange(head_dim // 2, dtype=torch.float64) / head_dim)

    def tables(self, step):
        key = ("root", self.rotary_dim)
        if key not in step.shared:
            angle = step.positions[: step.num_tokens].double().sqrt()[:, None] * self.inv.to(step.positions.device)[None, :]
            step.shared[key] = (angle.cos().float().contiguous(), angle.sin().float().contiguous())
        return step.shared[key]


def toy2_spec(cfg: ToyConfig, prefix="model") -> ModelSpec:
    norm = PartSpec("rmsnorm", {"eps": 1e-6, "unit_offset": True})
    attn = PartSpec("attention", {"num_heads": 2, "num_kv_heads": 2, "head_dim": 16, "scale": 0.25, "window": 6,
                                  "qk_norm": None, "position": PartSpec("root_positions")})
    dense = PartSpec("gated_mlp", {"intermediate_size": 2 * cfg.hidden, "activation": "silu"})
    routed = PartSpec("top_one_experts", {"experts": 3, "intermediate_size": cfg.hidden})
    layers = tuple(LayerSpec(f"{prefix}.layers.{l}", PartSpec("sandwich"), attn, routed if l % 2 else dense, norm)
                   for l in range(cfg.layers))  # different feed-forwards in different layers
    return ModelSpec(cfg.architecture, cfg.hidden, cfg.vocab, 512, PartSpec("scaled_embedding", {"scale": 1.0}),
                     layers, tuple(ScheduleEntry(l) for l in range(cfg.layers)), norm, PartSpec("lm_head", {"tied": True}),
                     prefix)


def toy2_plain(weights, cfg: ToyConfig, ids):
    w = {k: v.double() for k, v in weights.items()}
    norm = lambda x, name: x * torch.rsqrt((x * x).mean(-1, keepdim=True) + 1e-6) * (1.0 + w[name])
    x = w["model.embed_tokens.weight"][ids]
    T = len(ids)
    inv = 50.0 ** (-2.0 * torch.arange(8, dtype=torch.float64) / 16)
    angle = torch.arange(T, dtype=torch.float64).sqrt()[:, None] * inv[None, :]
    cos, sin = angle.cos().float().double()[:, None, :], angle.sin().float().double()[:, None, :]  # tables are 32-bit

    def rotate(v):
        a, b = v[..., :8], v[..., 8:]
        return torch.cat([a * cos - b * sin, a * sin + b * cos], dim=-1)

    for l in range(cfg.layers):
        p = f"model.layers.{l}"
        h = norm(x, f"{p}.input_layernorm.weight")
        q = rotate((h @ w[f"{p}.self_attn.q_proj.weight"].T).view(T, 2, 16))
        k = rotate((h @ w[f"{p}.self_attn.k_proj.weight"].T).view(T, 2, 16))
        v = (h @ w[f"{p}.self_attn.v_proj.weight"].T).view(T, 2, 16)
        a = P.attention(q, k, v, 0.25, 6).reshape(T, 32) @ w[f"{p}.self_attn.o_proj.weight"].T
        x = x + norm(a, f"{p}.post_attention_layernorm.weight")
        h = norm(x, f"{p}.pre_feedforward_layernorm.weight")
        if l % 2:
            choice = (h.float() @ weights[f"{p}.moe.router.weight"].float().T).argmax(-1)
            f = torch.zeros_like(h)
            for t in range(T):
                e = int(choice[t])
                gu = h[t] @ w[f"{p}.moe.experts.{e}.gate_up.weight"].T
                f[t] = (torch.nn.functional.silu(gu[: cfg.hidden]) * gu[cfg.hidden:]) @ w[f"{p}.moe.experts.{e}.down.weight"].T
        else:
            f = (torch.nn.functional.silu(h @ w[f"{p}.mlp.gate_proj.weight"].T) * (h @ w[f"{p}.mlp.up_proj.weight"].T)) \
                @ w[f"{p}.mlp.down_proj.weight"].T
        x = x + norm(f, f"{p}.post_feedforward_layernorm.weight")
    return norm(x, "model.norm.weight") @ w["model.embed_tokens.weight"].T


def test_toy_routed_feed_forward_and_position_encoding_plug_in(tmp_path):
    FEED_FORWARDS.register("top_one_experts", TopOneExperts, replace=True)
    POSITION_ENCODINGS.register("root_positions", RootPositions, replace=True)
    register_architecture(Architecture("Toy2ForCausalLM", ToyConfig.from_dict, toy2_spec, ToyConfig.to_dict), replace=True)
    try:
        cfg = ToyConfig("Toy2ForCausalLM", hidden=24, vocab=40, layers=4)
        folder = write_random_model(tmp_path / "toy2", cfg, seed=11, dtype=torch.float32)
        runner = ModelRunner.from_model_dir(folder, EngineConfig(dtype="float32", max_model_len=64, max_num_seqs=2,
                                                                max_num_batched_tokens=64, max_prefill_chunk=64,
                                                                max_cache_tokens=128))
        weights = P.load_weights(folder)
        assert any(".moe.experts.2.down.weight" in k for k in weights)  # the experts' tensors were written and read by name
        ids = [5, 1, 33, 7, 7, 20, 39, 0, 12, 3, 18, 25, 6, 31]
        want = toy2_plain(weights, cfg, ids)
        runner.add_request("whole")
        got = runner.step([("whole", ids, list(range(len(ids))))]).cpu().double()
        assert torch.allclose(got, want, atol=1e-4)
        # cut into portions and single tokens beside another request: the same logits
        runner.add_request("cut")
        parts, at = [], 0
        for n in (3, 1, 6, 1, 3):
            parts.append(runner.step([("cut", ids[at:at + n], list(range(n)))]).cpu().double())
            at += n
        assert torch.allclose(torch.cat(parts), want, atol=1e-4)
    finally:
        unregister_architecture("Toy2ForCausalLM")
        FEED_FORWARDS.unregister("top_one_experts")
        POSITION_ENCODINGS.unregister("root_positions")


def test_a_part_that_cannot_be_recorded_keeps_its_model_out_of_graphs(tmp_path, toy_architecture):
    """The toy mixer waits for the device inside its forward.  In bf16 with graphs switched on (the default)
    decode steps of its model run kernel by kernel; the same engine replays graphs for a model whose parts all
    can be recorded."""
    cfg = ToyConfig("ToyForCausalLM", hidden=24, vocab=50, layers=3)
    folder = write_random_model(tmp_path / "toy", cfg, seed=7, dtype=torch.bfloat16)
    engine_cfg = EngineConfig(dtype="bfloat16", max_model_len=128, max_num_seqs=3, max_num_batched_tokens=128,
                              max_prefill_chunk=128, max_cache_tokens=256, use_graphs=True)
    runner = ModelRunner.from_model_dir(folder, engine_cfg)
    assert not runner.model.capturable
    weights = P.load_weights(folder)
    ids = [3, 14, 15, 9, 26, 5, 35, 8, 9, 7, 9, 3]
    want = toy_plain(weights, cfg, ids)
    runner.add_request("a")
    got = [runner.step([("a", ids[:4], list(range(4)))]).float().cpu()]
    for t in ids[4:]:  # decoded one by one: steps that a model of recordable parts would take from a graph
        got.append(runner.step([("a", [t], [0])]).float().cpu())
    assert runner.graph_replays == 0
    got = torch.cat(got).double()
    assert (got - want).abs().max() <= 3e-2 * want.abs().max()


# --------------------------------------------------------------------------
# A toy embedding (token table plus a learned table of absolute positions) and a toy head (with a bias),
# registered from here: the model builds both through the registries.
# --------------------------------------------------------------------------
class TokenAndPositionEmbedding(Embedding):
    def __init__(self, spec, *, hidden_size, vocab_size):
        self.hidden, self.vocab, self.positions = hidden_size, vocab_size, int(spec["positions"])

    def param_specs(self, prefix):
        return [ParamSpec(f"{prefix}.wte.weight", (self.vocab, self.hidden), init=("normal", 0.5)),
                ParamSpec(f"{prefix}.wpe.weight", (self.positions, self.hidden), init=("normal", 0.5))]

    def bind(self, tensors, prefix, device, dtype):
        self.table = tensors[f"{prefix}.wte.weight"].to(device=device, dtype=dtype).contiguous()
        self.places = tensors[f"{prefix}.wpe.weight"].to(device=device, dtype=dtype).contiguous()

    def forward(self, step, out):
        ops.embed_gather(self.table, step.token_ids, 1.0, out)  # the framework's kernel, twice
        places = torch.empty_like(out)
        ops.embed_gather(self.places, step.positions, 1.0, places)
        return out.add_(places)


class BiasedHead(Head):
    def __init__(self, spec, *, hidden_size, vocab_size, embedding):
        self.hidden, self.vocab, self.embedding = hidden_size, vocab_size, embedding

    def param_specs(self, prefix):
        return [ParamSpec("out_bias", (self.vocab,), init=("normal", 1.0))]

    def bind(self, tensors, prefix, device, dtype):
        self.bias = tensors["out_bias"].to(device=device, dtype=torch.float32)

    def forward(self, x):
        return linear(x, self.embedding.table, out_dtype=torch.float32).add_(self.bias)


def toy3_spec(cfg: ToyConfig, prefix="model") -> ModelSpec:
    norm = PartSpec("rmsnorm", {"eps": 1e-6, "unit_offset": False})
    attn = PartSpec("attention", {"num_heads": 2, "num_kv_heads": 1, "head_dim": 16, "scale": 0.25, "window": None,
                                  "qk_norm": None, "position": None})  # positions come from the embedding alone
    ff = PartSpec("gated_mlp", {"intermediate_size": 2 * cfg.hidden, "activation": "silu"})
    layers = tuple(LayerSpec(f"{prefix}.h.{l}", PartSpec("sandwich"), attn, ff, norm) for l in range(cfg.layers))
    return ModelSpec(cfg.architecture, cfg.hidden, cfg.vocab, 64, PartSpec("token_and_position", {"positions": 64}),
                     layers, tuple(ScheduleEntry(l) for l in range(cfg.layers)), norm, PartSpec("biased_head"), prefix,
                     final_norm_name="ln_f")


def toy3_plain(weights, cfg: ToyConfig, ids):
    w = {k: v.double() for k, v in weights.items()}
    norm = lambda x, name: x * torch.rsqrt((x * x).mean(-1, keepdim=True) + 1e-6) * w[name]
    T = len(ids)
    x = w["model.wte.weight"][ids] + w["model.wpe.weight"][:T]
    for l in range(cfg.layers):
        p = f"model.h.{l}"
        h = norm(x, f"{p}.input_layernorm.weight")
        q, k, v = ((h @ w[f"{p}.self_attn.{n}_proj.weight"].T).view(T, -1, 16) for n in "qkv")
        a = P.attention(q, k, v, 0.25, None).reshape(T, 32) @ w[f"{p}.self_attn.o_proj.weight"].T
        x = x + norm(a, f"{p}.post_attention_layernorm.weight")
        h = norm(x, f"{p}.pre_feedforward_layernorm.weight")
        f = (torch.nn.functional.silu(h @ w[f"{p}.mlp.gate_proj.weight"].T) * (h @ w[f"{p}.mlp.up_proj.weight"].T)) \
            @ w[f"{p}.mlp.down_proj.weight"].T
        x = x + norm(f, f"{p}.post_feedforward_layernorm.weight")
    return norm(x, "model.ln_f.weight") @ w["model.wte.weight"].T + w["out_bias"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_embedding_and_head_plug_in_and_replay_from_graphs(tmp_path, dtype):
    EMBEDDINGS.register("token_and_position", TokenAndPositionEmbedding, replace=True)
    HEADS.register("biased_head", BiasedHead, replace=True)
    register_architecture(Architecture("Toy3ForCausalLM", ToyConfig.from_dict, toy3_spec, ToyConfig.to_dict), replace=True)
    try:
        cfg = ToyConfig("Toy3ForCausalLM", hidden=24, vocab=40, layers=2)
        store = torch.float32 if dtype == "float32" else torch.bfloat16
        folder = write_random_model(tmp_path / "toy3", cfg, seed=13, dtype=store)
        weights = P.load_weights(folder)
        assert {"model.wte.weight", "model.wpe.weight", "out_bias", "model.ln_f.weight"} <= set(weights)
        assert not any("embed_tokens" in k or k.startswith("model.norm.") for k in weights)  # its own names only
        runner = ModelRunner.from_model_dir(folder, EngineConfig(dtype=dtype, max_model_len=64, max_num_seqs=2,
                                                                max_num_batched_tokens=64, max_prefill_chunk=64,
                                                                max_cache_tokens=128, use_graphs=True))
        assert runner.model.capturable
        ids = [5, 1, 33, 7, 7, 20, 39, 0, 12, 3, 18, 25, 6, 31]
        want = toy3_plain(weights, cfg, ids)
        tol = 1e-4 if dtype == "float32" else 3e-2 * want.abs().max().item()
        runner.add_request("whole")
        got = runner.step([("whole", ids, list(range(len(ids))))]).float().cpu().double()
        assert (got - want).abs().max() <= tol
        runner.add_request("cut")
        parts = [runner.step([("cut", ids[:6], list(range(6)))]).float().cpu()]
        for t in ids[6:]:
            parts.append(runner.step([("cut", [t], [0])]).float().cpu())
        assert (torch.cat(parts).double() - want).abs().max() <= tol
        assert (runner.graph_replays > 0) == (dtype == "bfloat16")  # positions reach the embedding from the step's arrays
    finally:
        unregister_architecture("Toy3ForCausalLM")
        EMBEDDINGS.unregister("token_and_position")
        HEADS.unregister("biased_head")


# --------------------------------------------------------------------------
# The framework's own mixer and feed-forward under another architecture's tensor names, with biases and with
# projections that the checkpoint stores fused: parameters of their specs, no copy of the parts.
# --------------------------------------------------------------------------
def toy4_spec(cfg: ToyConfig, prefix="transformer") -> ModelSpec:
    norm = PartSpec("rmsnorm", {"eps": 1e-6, "unit_offset": False})
    heads = {"num_heads": 4, "num_kv_heads": 2, "head_dim": 16, "scale": 0.25, "window": None, "qk_norm": None,
             "position": PartSpec("rope", {"theta": 100.0})}
    layers = []
    for l in range(cfg.layers):
        if l % 2 == 0:  # q, k and v stored as one matrix with a bias; so are gate and up; every projection has a bias
            attn = PartSpec("attention", dict(heads, names={"qkv": "attn.c_attn", "o": "attn.c_proj"}, bias=True))
            ff = PartSpec("gated_mlp", {"intermediate_size": 2 * cfg.hidden, "activation": "silu", "bias": True,
                                        "names": {"gate_up": "ffn.w13", "down": "ffn.w2"}})
        else:  # stored apart under other names; a bias on the queries and on the down projection only
            attn = PartSpec("attention", dict(heads, names={"q": "attn.wq", "k": "attn.wk", "v": "attn.wv",
                                                            "o": "attn.wo"}, bias=["q"]))
            ff = PartSpec("gated_mlp", {"intermediate_size": 2 * cfg.hidden, "activation": "silu", "bias": ["down"],
                                        "names": {"gate": "ffn.w1", "up": "ffn.w3", "down": "ffn.w2"}})
        layers.append(LayerSpec(f"{prefix}.h.{l}", PartSpec("sandwich"), attn, ff, norm))
    return ModelSpec(cfg.architecture, cfg.hidden, cfg.vocab, 256, PartSpec("scaled_embedding", {"scale": 1.0}),
                     tuple(layers), tuple(ScheduleEntry(l) for l in range(cfg.layers)), norm,
                     PartSpec("lm_head", {"tied": True}), prefix)


def toy4_plain(weights, cfg: ToyConfig, ids):
    w = {k: v.double() for k, v in weights.items()}
    norm = lambda x, name: x * torch.rsqrt((x * x).mean(-1, keepdim=True) + 1e-6) * w[name]
    T, H = len(ids), cfg.hidden
    x = w["transformer.embed_tokens.weight"][ids]
    inv = P.rope_inv_freq(16, 100.0, 1.0, torch.float64)
    pos = torch.arange(T)
    for l in range(cfg.layers):
        p = f"transformer.h.{l}"
        h = norm(x, f"{p}.input_layernorm.weight")
        if l % 2 == 0:
            qkv = h @ w[f"{p}.attn.c_attn.weight"].T + w[f"{p}.attn.c_attn.bias"]
            q, k, v = qkv[:, :64], qkv[:, 64:96], qkv[:, 96:]
        else:
            q = h @ w[f"{p}.attn.wq.weight"].T + w[f"{p}.attn.wq.bias"]
            k, v = h @ w[f"{p}.attn.wk.weight"].T, h @ w[f"{p}.attn.wv.weight"].T
        q, k, v = P.rope(q.reshape(T, 4, 16), pos, inv), P.rope(k.reshape(T, 2, 16), pos, inv), v.reshape(T, 2, 16)
        a = P.attention(q, k, v, 0.25, None).reshape(T, 64)
        a = a @ w[f"{p}.attn.c_proj.weight"].T + w[f"{p}.attn.c_proj.bias"] if l % 2 == 0 else a @ w[f"{p}.attn.wo.weight"].T
        x = x + norm(a, f"{p}.post_attention_layernorm.weight")
        h = norm(x, f"{p}.pre_feedforward_layernorm.weight")
        if l % 2 == 0:
            gu = h @ w[f"{p}.ffn.w13.weight"].T + w[f"{p}.ffn.w13.bias"]
            f = (torch.nn.functional.silu(gu[:, :2 * H]) * gu[:, 2 * H:]) @ w[f"{p}.ffn.w2.weight"].T + w[f"{p}.ffn.w2.bias"]
        else:
            f = (torch.nn.functional.silu(h @ w[f"{p}.ffn.w1.weight"].T) * (h @ w[f"{p}.ffn.w3.weight"].T)) \
                @ w[f"{p}.ffn.w2.weight"].T + w[f"{p}.ffn.w2.bias"]
        x = x + norm(f, f"{p}.post_feedforward_layernorm.weight")
    return norm(x, "transformer.norm.weight") @ w["transformer.embed_tokens.weight"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_same_mixer_and_feed_forward_under_other_names_with_biases(tmp_path, dtype):
    register_architecture(Architecture("Toy4ForCausalLM", ToyConfig.from_dict, toy4_spec, ToyConfig.to_dict), replace=True)
    try:
        cfg = ToyConfig("Toy4ForCausalLM", hidden=40, vocab=60, layers=4)
        store = torch.float32 if dtype == "float32" else torch.bfloat16
        folder = write_random_model(tmp_path / "toy4", cfg, seed=17, dtype=store)
        weights = P.load_weights(folder)
        assert {"transformer.h.0.attn.c_attn.bias", "transformer.h.1.attn.wq.bias", "transformer.h.0.ffn.w13.weight",
                "transformer.h.1.ffn.w2.bias", "transformer.h.0.attn.c_proj.bias"} <= set(weights)
        assert not any("self_attn" in k or ".mlp." in k or k.endswith("wk.bias") for k in weights)
        assert weights["transformer.h.0.attn.c_attn.weight"].shape == (128, 40)
        for name in [k for k in weights if k.endswith(".bias")]:  # biases large enough to matter
            weights[name] = (weights[name].float() * 20).to(store)
        from safetensors.torch import save_file
        save_file(weights, str(folder / "model.safetensors"))
        runner = ModelRunner.from_model_dir(folder, EngineConfig(dtype=dtype, max_model_len=64, max_num_seqs=2,
                                                                max_num_batched_tokens=64, max_prefill_chunk=64,
                                                                max_cache_tokens=128, use_graphs=True))
        ids = [5, 1, 33, 7, 7, 20, 39, 0, 12, 3, 18, 25, 6, 31, 59, 2, 44, 8, 9, 50]
        want = toy4_plain(weights, cfg, ids)
        no_bias = toy4_plain({k: (v * 0 if k.endswith(".bias") else v) for k, v in weights.items()}, cfg, ids)
        assert (no_bias - want).abs().max() > 0.1 * want.abs().max()  # the biases move the logits
        tol = (2e-5 if dtype == "float32" else 3e-2) * want.abs().max().item()
        runner.add_request("whole")
        got = runner.step([("whole", ids, list(range(len(ids))))]).float().cpu().double()
        assert (got - want).abs().max() <= tol
        runner.add_request("cut")
        parts = [runner.step([("cut", ids[:6], list(range(6)))]).float().cpu()]
        for t in ids[6:]:  # in bf16 from graphs: the few-row products leave K slices, to which the bias is added
            parts.append(runner.step([("cut", [t], [0])]).float().cpu())
        assert (torch.cat(parts).double() - want).abs().max() <= tol
        assert (runner.graph_replays > 0) == (dtype == "bfloat16")
    finally:
        unregister_architecture("Toy4ForCausalLM")


def test_two_engines_in_one_process_keep_their_own_weight_layouts(model_dirs):
    """Whether a model's matrices lie in tiles is its engine's setting and travels with the model: an engine built
    later with the other setting changes nothing for the first."""
    common = dict(dtype="bfloat16", max_model_len=64, max_num_seqs=2)
    tiled = ModelRunner.from_model_dir(model_dirs["B"], EngineConfig(tiled_weights=True, **common))
    rows = ModelRunner.from_model_dir(model_dirs["B"], EngineConfig(tiled_weights=False, **common))
    again = ModelRunner.from_model_dir(model_dirs["B"], EngineConfig(tiled_weights=True, **common))
    for runner, want in ((tiled, ops.TiledWeight), (rows, torch.Tensor), (again, ops.TiledWeight)):
        mixer = runner.model.blocks[0].mixer
        assert isinstance(mixer.w_qkv, want) and isinstance(mixer.w_o, want)
        assert isinstance(runner.model.blocks[1].feed_forward.w_down, want)
        assert isinstance(runner.model.head.weight, want)
    ids = [3, 1, 4, 1, 5, 9, 2, 6]
    outs = []
    for runner in (tiled, rows):
        runner.add_request("x")
        outs.append(runner.step([("x", ids, list(range(len(ids))))]).clone())
    assert torch.equal(outs[0], outs[1])  # the same sums in the same order from either layout
