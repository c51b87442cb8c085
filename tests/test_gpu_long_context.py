"""Decoding at the contexts that serving and the measurements run at: 8 192, 32 768 and 131 072 keys.

At the kernel's level: the matrix-core decode kernel under the plan that the dispatcher itself makes (the
number of key splits, the merge, block tables of up to 8 192 pages), one decoded token a request, against
64-bit attention over the same keys.  Random keys at the usual score scale make a softmax over a hundred
thousand keys nearly flat, so that a lost split would change the output by less than the tolerance; here the
scores are three times wider (a few dozen keys, anywhere in the context, carry most of the weight), the error
is measured against the size of the outputs, and one planted key far back carries all of it in a test of its
own.

At the engine's level: requests decoding through ``LLMEngine`` from recorded graphs, several steps from one
plan, across the edges of the graphs' context buckets (8 192 -> 9 216, and 16 384 -> 18 432 where the buckets
start to double), every token and a handful of logits against the plain implementation."""

import types

import pytest
import torch
from safetensors.torch import load_file, save_file

import plain_gemma
import tiny_models
import trace_tools as tt
from rvllm_amd.config.engine_config import EngineConfig
from rvllm_amd.engine.engine import LLMEngine
from rvllm_amd.engine.runner import ModelRunner
from rvllm_amd.kernels import ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


class LongDecode:
    """Requests of one decoded token each at the given contexts (the token is the context's last position), their
    keys and values made on the device and scattered over pages in a shuffled order.  With a window, the pages
    that it has passed are gone: their table entries are -1, and so is everything that lies around in the pool
    NaN, so a kernel that touches a page it should not shows it."""

    def __init__(self, contexts, nq, nkv, hd, page_size, window, seed, plan_for=None):
        g = torch.Generator(device=DEV).manual_seed(seed)
        cpu = torch.Generator().manual_seed(seed)
        self.nq, self.nkv, self.hd, self.page_size, self.window = nq, nkv, hd, page_size, window
        self.contexts = list(contexts)
        B = len(self.contexts)
        first_page = [0 if window is None else max(0, L - window) // page_size for L in self.contexts]
        held = [-(-L // page_size) - f for L, f in zip(self.contexts, first_page)]
        num_pages = sum(held) + 7
        order = torch.randperm(num_pages, generator=cpu)
        self.k_pages = torch.full((num_pages, nkv, page_size, hd), float("nan"), dtype=torch.bfloat16, device=DEV)
        self.v_pages = torch.full((num_pages, nkv, page_size // 16, hd, 16), float("nan"), dtype=torch.bfloat16,
                                  device=DEV)  # transposed inside groups of 16 slots
        width = max(-(-L // page_size) for L in self.contexts) + 3
        table = torch.full((B, width), -1, dtype=torch.int32)
        self.keys, self.values, self.first_key = [], [], []
        taken = 0
        for b, L in enumerate(self.contexts):
            first = first_page[b] * page_size
            n = held[b] * page_size  # whole pages; what lies beyond the context is random too, and never visible
            k = torch.randn(n, nkv, hd, device=DEV, generator=g).bfloat16()
            v = torch.randn(n, nkv, hd, device=DEV, generator=g).bfloat16()
            pages = order[taken:taken + held[b]]
            taken += held[b]
            table[b, first_page[b]:first_page[b] + held[b]] = pages.int()
            self.keys.append(k)
            self.values.append(v)
            self.first_key.append(first)
            self._store(b, pages)
        self.table = table.to(DEV)
        self.q = torch.randn(B, nq, hd, device=DEV, generator=g).bfloat16()
        starts = list(range(B + 1))
        self.step = types.SimpleNamespace(
            num_tokens=B, num_requests=B,
            positions=torch.tensor([L - 1 for L in self.contexts], dtype=torch.int32, device=DEV),
            token_req=torch.arange(B, dtype=torch.int32, device=DEV),
            q_start=torch.tensor(starts, dtype=torch.int32, device=DEV),
            chunk_start=torch.tensor([L - 1 for L in self.contexts], dtype=torch.int32, device=DEV),
            max_portion=1, max_context=plan_for or max(self.contexts), host_q_start=starts)

    def _store(self, b, pages=None):
        if pages is None:
            first_page = self.first_key[b] // self.page_size
            pages = self.table[b, first_page:first_page + self.keys[b].shape[0] // self.page_size].long()
        pages = pages.to(DEV)
        k = self.keys[b].view(-1, self.page_size, self.nkv, self.hd)
        v = self.values[b].view(-1, self.page_size, self.nkv, self.hd)
        self.k_pages[pages] = k.permute(0, 2, 1, 3)
        self.v_pages[pages] = v.view(-1, self.page_size // 16, 16, self.nkv, self.hd).permute(0, 3, 1, 4, 2)

    def plant(self, b, key, head, dim, value):
        """Key ``key`` of request b becomes ``value`` at one dimension and nothing else."""
        row = key - self.first_key[b]
        self.keys[b][row, head] = 0
        self.keys[b][row, head, dim] = value
        self._store(b)

    def reference(self, scale):
        """64-bit attention of each request's token over the keys it sees."""
        out = torch.empty(len(self.contexts), self.nq, self.hd, dtype=torch.float64, device=DEV)
        group = self.nq // self.nkv
        for b, L in enumerate(self.contexts):
            lo = 0 if self.window is None else max(0, L - self.window)
            rows = slice(lo - self.first_key[b], L - self.first_key[b])
            for h in range(self.nkv):
                k = self.keys[b][rows, h].double()
                v = self.values[b][rows, h].double()
                s = scale * (self.q[b, h * group:(h + 1) * group].double() @ k.T)
                out[b, h * group:(h + 1) * group] = torch.softmax(s, dim=-1) @ v
        return out.cpu()

    def run(self, scale, **kw):
        B = len(self.contexts)
        out = torch.full((B, self.nq * self.hd), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops.paged_attention_mfma(self.q.view(B, -1).contiguous(), self.k_pages, self.v_pages, self.table, self.step,
                                 out, self.nq, scale, self.window, **kw)
        return out.cpu().view(B, self.nq, self.hd).double()


def close(got, want):
    """Within bf16's rounding of the outputs' own size: a split of the keys that were lost would be missed by
    an absolute tolerance when the outputs are small, as sums over many thousand keys are."""
    assert torch.isfinite(got).all()
    size = want.abs().max().item()
    err = (got - want).abs().max().item()
    return err <= 2e-2 * size, f"largest difference {err:.3e} against outputs of size {size:.3e}"


HEADS = [(8, 4, 256), (32, 16, 128)]  # the 4B model's heads, the 27B model's


@pytest.mark.parametrize("nq,nkv,hd", HEADS)
@pytest.mark.parametrize("context", [8192, 32768, 131072])
@pytest.mark.parametrize("batch", [1, 8])
@pytest.mark.parametrize("window", [None, 1024])
@pytest.mark.parametrize("page_size", [16, 64])
def test_decode_attention_under_its_own_plan_at_long_contexts(nq, nkv, hd, context, batch, window, page_size):
    """One decoded token a request under the dispatcher's own plan (no override of the splits), contexts that
    differ from request to request and end inside a page; once planned for the contexts themselves, once for
    the upper end of the graph's bucket, as a replayed graph runs it (the splits beyond a request's keys are
    empty)."""
    contexts = [context - 37 * i for i in range(batch)]
    scale = 3.0 * hd ** -0.5
    case = LongDecode(contexts, nq, nkv, hd, page_size, window, seed=context // 64 + batch)
    want = case.reference(scale)
    ok, why = close(case.run(scale), want)
    assert ok, why
    tiles, splits, split_len = ops.plan_attention_splits(batch, 1, context, nkv, nq // nkv, window, hd,
                                                           ops.attention_wave_slots(hd))
    if window is None:
        assert splits * split_len >= context and splits > 1  # the keys are split over many waves, then merged
    bucket = ModelRunner.context_bucket(context + 1)
    case.step.max_context = bucket
    ok, why = close(case.run(scale), want)
    assert ok, f"planned for {bucket} keys: {why}"


@pytest.mark.parametrize("nq,nkv,hd", HEADS)
@pytest.mark.parametrize("batch", [1, 8])
def test_decode_attention_finds_one_key_131_thousand_back(nq, nkv, hd, batch):
    """All the weight on key 17 of a context of 131 072: the output is that key's value, so a split that is lost,
    merged with the wrong weight or read from another request's pages shows.  Then the same key at the edge of a
    window that reaches exactly that far (seen), and of one that ends a key short (not seen)."""
    context, far = 131072, 17
    contexts = [context - 37 * i for i in range(batch)]
    for window_of, found in ((lambda L: None, True), (lambda L: L - far, True), (lambda L: L - far - 1, False)):
        for b in {0, batch - 1}:
            window = window_of(contexts[b])
            case = LongDecode(contexts, nq, nkv, hd, 16, window, seed=5)
            for i in range(batch):
                case.keys[i].mul_(0.01)
                case._store(i)
            head = nkv - 1
            case.plant(b, far, head, 3, 40.0)
            case.q.zero_()
            case.q[:, :, 3] = 40.0
            got = case.run(1.0)
            group = nq // nkv
            value = case.values[b][far - case.first_key[b], head].double().cpu()
            hit = torch.allclose(got[b, head * group:(head + 1) * group], value.expand(group, hd), atol=2e-2)
            assert hit == found, (window, b)
            if found:  # and nobody else's output is that value
                ok, why = close(got, case.reference(1.0))
                assert ok, why


@pytest.mark.parametrize("nq,nkv,hd", HEADS)
@pytest.mark.parametrize("back", [1023, 1024, 1025])
def test_decode_attention_at_the_edge_of_the_window_deep_in_a_context(nq, nkv, hd, back):
    """A window of 1024 at contexts of 32 768 and 131 072: the key 1023 back is the last one seen, the keys 1024
    and 1025 back are not (the reference pins its window metadata at the same three distances:
    v3/crates/rvllm-runtime/src/gemma4_bring_up.rs:6357-6381)."""
    for context in (32768 - 5, 131072):
        case = LongDecode([context, context - 333], nq, nkv, hd, 16, 1024, seed=back)
        for i in range(2):
            case.keys[i].mul_(0.01)
            case._store(i)
        key = context - 1 - back
        if key >= case.first_key[0]:
            case.plant(0, key, 0, 3, 40.0)
        case.q.zero_()
        case.q[:, :, 3] = 40.0
        got = case.run(1.0)
        group = nq // nkv
        ok, why = close(got, case.reference(1.0))
        assert ok, why
        if key >= case.first_key[0]:
            value = case.values[0][key - case.first_key[0], 0].double().cpu()
            hit = torch.allclose(got[0, :group], value.expand(group, hd), atol=2e-2)
            assert hit == (back <= 1023), (context, back)


# ---------------------------------------------------------------------------------------------------------------
# through the engine
# ---------------------------------------------------------------------------------------------------------------
@pytest.fixture(scope="module")
def long_model(tmp_path_factory):
    """Three narrow layers with the 27B model's heads (sliding, global, sliding; window 1024).  The query gains
    are raised (by 1.5, scores two and a half times wider) so that scores over many thousand keys are not flat: a
    few hundred keys anywhere in the context carry the weight, and a lost part of the context moves the logits.
    (Wider still, and bf16's rounding of queries and keys alone moves the logits by the tolerance: at + 3 the
    whole prompt in one step and decoding both differ from the 64-bit logits by 3 % of their size.)"""
    folder = tiny_models.write_model(tmp_path_factory.mktemp("long") / "LONG", "LONG")
    path = folder / "model.safetensors"
    tensors = load_file(str(path))
    for name in tensors:
        if name.endswith("q_norm.weight"):
            tensors[name] = tensors[name] + 1.5
    save_file(tensors, str(path))
    return folder, plain_gemma.load_weights(folder), plain_gemma.read_config(folder)


@pytest.mark.parametrize("prompt_len,edge", [(8150, 8192), (16300, 16384)])
def test_decoding_across_the_edge_of_a_graphs_bucket(long_model, prompt_len, edge):
    """Three requests decode 100 tokens through the engine, from graphs, four steps from a plan, the longest
    from ``prompt_len`` tokens across ``edge`` (where the next graph, planned for a longer context, takes over),
    one a few hundred tokens behind it and a short one.  Every token is the plain implementation's arg-max; then
    the longest sequence is replayed through the step function, its last 70 tokens one by one from the graphs
    on both sides of the edge, and the logits compared."""
    folder, weights, cfg = long_model
    new = 100
    lengths = [prompt_len, prompt_len - 300, 700]
    prompts = list(tt.make_sequences(cfg["vocab"], lengths, seed=prompt_len).values())
    engine = LLMEngine.from_model_dir(folder, EngineConfig(
        dtype="bfloat16", max_model_len=prompt_len + 200, max_num_seqs=4, max_num_batched_tokens=2048,
        max_prefill_chunk=2048, greedy_steps_ahead=4, use_graphs=True))
    runner = engine.runner
    results = engine.generate(prompts, None, max_new_tokens=new, ignore_eos=True)
    assert runner.graph_replays > new // 2 and engine.plans < engine.steps
    buckets = {key[1] for key in runner._graphs}
    assert edge in buckets and ModelRunner.context_bucket(edge + 1) in buckets
    refs = []
    for prompt, res in zip(prompts, results):
        assert len(res.tokens) == new
        ids = prompt + res.tokens
        logits = plain_gemma.forward(weights, cfg, ids[:-1], torch.float64, device=DEV)
        refs.append(logits)
        slack = 2 * tt.TOLERANCE["bfloat16"] * logits.abs().max().item()
        for i, token in enumerate(res.tokens):
            row = logits[len(prompt) - 1 + i]
            assert row[token] >= row.max() - slack, f"request of {len(prompt)}: token {i} is not the arg-max"
    # the longest again, through the step function: the prompt in portions, then token by token from the graphs
    ids = (prompts[0] + results[0].tokens)[:-1]
    runner.add_request("again")
    head = len(ids) - 70
    for at in range(0, head, 2048):
        runner.step([("again", ids[at:min(head, at + 2048)], [])])
    replays = runner.graph_replays
    rows = []
    for t in range(head, len(ids)):
        rows.append(runner.step([("again", [ids[t]], [0])]).float().cpu().clone())
    runner.release("again")
    assert runner.graph_replays - replays >= 60  # from graphs, but for the first step of each bucket
    assert head < edge < len(ids)
    tt.compare(torch.cat(rows).numpy(), refs[0][head:], "bfloat16", f"decoding across {edge}")
