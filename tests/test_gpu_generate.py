"""Generation through the entry points: greedy and sampled, long decoding,
the first tokens of a sequence, requests set back when pages run out, the
command line."""

import json
import subprocess
import sys

import pytest
import torch

import plain_gemma
import rvllm_amd
import trace_tools as tt
from rvllm_amd.config.engine_config import EngineConfig
from rvllm_amd.engine.engine import LLMEngine
from rvllm_amd.sampling.params import SamplingParams
from rvllm_amd.sampling.sampler import SplitMix64, sample_from_candidates

pytestmark = pytest.mark.gpu


def assert_greedy(weights, cfg, prompt, output, dtype):
    """Every generated token is the arg-max of the plain implementation's
    logits for the tokens before it — up to the engine's tolerance, so that a
    near-tie cannot fail the test, and nothing else can pass it."""
    ids = list(prompt) + list(output)
    logits = plain_gemma.forward(weights, cfg, ids[:-1], torch.float64)
    slack = 2 * tt.TOLERANCE[dtype] * logits.abs().max().item()
    for i, token in enumerate(output):
        row = logits[len(prompt) - 1 + i]
        assert row[token] >= row.max() - slack, f"token {i} ({token}) is not the arg-max: {row[token]} < {row.max()}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_python_entry(model_dirs, plain_models, dtype):
    """Workload of the first tiny configuration: prompts of 5, 9, 13 and 17
    tokens, 12 greedy tokens each."""
    weights, cfg = plain_models["A"]
    prompts = list(tt.make_sequences(cfg["vocab"], [5, 9, 13, 17], seed=0).values())
    outputs = rvllm_amd.generate(str(model_dirs["A"]), prompts, max_tokens=12, dtype=dtype, max_model_len=64,
                                 max_num_seqs=4, max_num_batched_tokens=64, max_prefill_chunk=64)
    assert [len(o) for o in outputs] == [12] * 4
    for prompt, out in zip(prompts, outputs):
        assert_greedy(weights, cfg, prompt, out, dtype)
    if dtype == "float32":
        assert outputs == [plain_gemma.greedy(weights, cfg, p, 12, torch.float64) for p in prompts]


def test_generation_with_the_librarys_products_tuned_at_start_up(model_dirs, plain_models, tmp_path, monkeypatch):
    """``tune_products``: the engine times the library's algorithms for a ladder of row counts before the first
    request and writes its choices to the file the environment names; a second engine takes them from the file.
    Prompts of 150 tokens in portions of 100 go through those products; every token is the plain model's."""
    import json

    from rvllm_amd.kernels import ops

    weights, cfg = plain_models["B"]
    plans = tmp_path / "plans.json"
    monkeypatch.setenv(ops.LIBRARY_PLANS_ENV, str(plans))
    prompts = list(tt.make_sequences(cfg["vocab"], [150, 97], seed=4).values())
    options = dict(max_tokens=6, dtype="bfloat16", max_model_len=256, max_num_seqs=2, max_num_batched_tokens=160,
                   max_prefill_chunk=100, tune_products=True)
    first = rvllm_amd.generate(str(model_dirs["B"]), prompts, **options)
    for prompt, out in zip(prompts, first):
        assert_greedy(weights, cfg, prompt, out, "bfloat16")
    doc = json.loads(plans.read_text())
    rows = sorted({p[0] for p in doc["plans"]})
    # the ladder of this engine: 96, 144, the portion, the budget (the file also holds what else this process tuned)
    assert {96, 100, 144, 160} <= set(rows)
    again = rvllm_amd.generate(str(model_dirs["B"]), prompts, **options)
    for prompt, out in zip(prompts, again):
        assert_greedy(weights, cfg, prompt, out, "bfloat16")
    assert json.loads(plans.read_text())["plans"] == doc["plans"]  # nothing was tuned again
    # a file that cannot be written is a warning, not an error
    monkeypatch.setenv(ops.LIBRARY_PLANS_ENV, str(tmp_path / "no" / "such" / "folder" / "plans.json"))
    with pytest.warns(UserWarning, match="were not written"):
        rvllm_amd.generate(str(model_dirs["B"]), prompts[:1], **options)


def test_sampled_generation_with_chunked_prompts_is_the_plain_models_stream(model_dirs, plain_models):
    """Workload of the second tiny configuration: six requests with prompts of
    1 to 23 tokens, prompts cut into portions of 7 beside decoding requests,
    10 tokens each at temperature 0.8 from fixed seeds.  The same draws on the
    plain implementation's logits give the same tokens."""
    weights, cfg = plain_models["B"]
    prompts = list(tt.make_sequences(cfg["vocab"], [1, 5, 9, 14, 19, 23], seed=1).values())
    engine = LLMEngine.from_model_dir(model_dirs["B"], EngineConfig(
        dtype="float32", max_model_len=64, max_num_seqs=4, max_num_batched_tokens=16, max_prefill_chunk=7))
    params = [SamplingParams(0.8, 0, 1.0, seed=100 + i) for i in range(len(prompts))]
    results = engine.generate(prompts, params, max_new_tokens=10)
    assert engine.steps > 10  # portions and decodes shared steps
    for i, (prompt, res) in enumerate(zip(prompts, results)):
        rng = SplitMix64(100 + i)
        ids = list(prompt)
        for token in res.tokens:
            row = plain_gemma.forward(weights, cfg, ids, torch.float64)[-1].float()
            cands = [(v / 0.8, j) for j, v in enumerate(row.tolist())]
            want = sample_from_candidates(cands, 0, 1.0, rng, cfg["vocab"])
            assert token == want, f"request {i}, token {len(ids) - len(prompt)}"
            ids.append(token)
    # the same seeds give the same streams again, other seeds give others
    again = engine.generate(prompts, params, max_new_tokens=10)
    assert [r.tokens for r in again] == [r.tokens for r in results]
    other = engine.generate(prompts, [SamplingParams(0.8, 0, 1.0, seed=7 + i) for i in range(6)], max_new_tokens=10)
    assert [r.tokens for r in other] != [r.tokens for r in results]


def test_top_k_one_and_top_p_zero_are_greedy(model_dirs):
    engine = LLMEngine.from_model_dir(model_dirs["A"], EngineConfig(dtype="float32", max_model_len=64, max_num_seqs=4))
    prompt = [[7, 8, 9, 10]]
    greedy = engine.generate(prompt, SamplingParams(), max_new_tokens=8)[0].tokens
    assert engine.generate(prompt, SamplingParams(0.9, 1, 1.0, 5), max_new_tokens=8)[0].tokens == greedy
    assert engine.generate(prompt, SamplingParams(0.9, 0, 0.0, 5), max_new_tokens=8)[0].tokens == greedy


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(model_dirs, plain_models, dtype):
    """300 tokens decoded one by one: the window passes many pages, pages of
    the window group are given back and used again by the same request."""
    weights, cfg = plain_models["A"]
    engine = LLMEngine.from_model_dir(model_dirs["A"], EngineConfig(
        dtype=dtype, max_model_len=512, max_num_seqs=1, max_cache_tokens=512))
    prompt = [11, 22, 33]
    res = engine.generate([prompt], None, max_new_tokens=300, ignore_eos=True)[0]
    assert len(res.tokens) == 300 and res.finish_reason == "length"
    assert_greedy(weights, cfg, prompt, res.tokens, dtype)
    assert engine.runner.cache.free_pages()["window8"] == engine.runner.cache.groups["window8"].pool.num_pages


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_first_tokens_of_a_sequence(model_dirs, plain_models, name):
    weights, cfg = plain_models[name]
    engine = LLMEngine.from_model_dir(model_dirs[name], EngineConfig(dtype="float32", max_model_len=64, max_num_seqs=2))
    runner = engine.runner
    ids = [cfg["vocab"] - 1, 0, 3]
    want = plain_gemma.forward(weights, cfg, ids, torch.float64)
    runner.add_request("x")
    for i, t in enumerate(ids):
        got = runner.step([("x", [t], [0])]).cpu().numpy()
        tt.compare(got, want[i:i + 1], "float32", f"{name} position {i}")
    runner.release("x")


def test_requests_set_back_when_pages_run_out_give_the_same_tokens(model_dirs):
    prompts = list(tt.make_sequences(256, [20, 28, 24, 18], seed=5).values())
    common = dict(dtype="float32", max_model_len=128, max_num_seqs=4, max_num_batched_tokens=64, max_prefill_chunk=16)
    roomy = LLMEngine.from_model_dir(model_dirs["A"], EngineConfig(max_cache_tokens=1024, **common))
    tight = LLMEngine.from_model_dir(model_dirs["A"], EngineConfig(max_cache_tokens=160, **common))
    want = roomy.generate(prompts, None, max_new_tokens=40, ignore_eos=True)
    got = tight.generate(prompts, None, max_new_tokens=40, ignore_eos=True)
    assert sum(r.set_backs for r in want) == 0 and sum(r.set_backs for r in got) >= 1
    assert [r.tokens for r in got] == [r.tokens for r in want]
    tight.runner.cache.check()
    assert all(free == g.pool.num_pages for free, g in zip(tight.runner.cache.free_pages().values(),
                                                           tight.runner.cache.groups.values()))


@pytest.mark.parametrize("name", ["A", "C"])
def test_decode_steps_replayed_from_a_graph_match_eager_steps(model_dirs, plain_models, name):
    """Every replay is checked, with eager work (prompts of new requests, a
    request leaving) and synchronisations between the replays."""
    weights, cfg = plain_models[name]
    common = dict(dtype="bfloat16", max_model_len=256, max_num_seqs=4, max_num_batched_tokens=64,
                  max_prefill_chunk=64, max_cache_tokens=1024)
    eager = LLMEngine.from_model_dir(model_dirs[name], EngineConfig(use_graphs=False, **common)).runner
    graph = LLMEngine.from_model_dir(model_dirs[name], EngineConfig(use_graphs=True, **common)).runner
    seqs = tt.make_sequences(cfg["vocab"], [40, 75, 23], seed=8)
    refs = {rid: plain_gemma.forward(weights, cfg, ids, torch.float64) for rid, ids in seqs.items()}
    done = {rid: 0 for rid in seqs}
    for runner in (eager, graph):
        for rid, ids in seqs.items():
            runner.add_request(rid)
            runner.step([(rid, ids[:10], [])])  # prompts run eagerly
    for rid in seqs:
        done[rid] = 10
    live = list(seqs)
    for it in range(30):
        if it == 12:  # one request leaves: another shape, another graph
            for runner in (eager, graph):
                runner.release("r2")
            live.remove("r2")
        entries = [(rid, [seqs[rid][done[rid]]], [0]) for rid in live if done[rid] < len(seqs[rid])]
        if not entries:
            break
        a = eager.step(entries).float().cpu()
        b = graph.step(entries).float().cpu()  # .cpu() synchronises between the replays
        for row, (rid, _, _) in enumerate(entries):
            tt.compare(b[row:row + 1].numpy(), refs[rid][done[rid]:done[rid] + 1], "bfloat16", f"replay {it} {rid}")
            tt.compare(a[row:row + 1].numpy(), refs[rid][done[rid]:done[rid] + 1], "bfloat16", f"eager {it} {rid}")
            done[rid] += 1
        assert (a - b).abs().max() <= 1e-2 * a.abs().max(), f"replay {it} differs from the eager step"
    assert graph.graph_replays >= 20 and eager.graph_replays == 0
    assert len(graph._graphs) >= 2


def test_a_graph_dropped_for_room_is_recorded_again(model_dirs, plain_models):
    """Only so many shapes keep their graphs.  With room for one, a shape that comes back after another was met
    runs eagerly once more, is recorded again and replayed, with right logits all the way."""
    weights, cfg = plain_models["A"]
    runner = LLMEngine.from_model_dir(model_dirs["A"], EngineConfig(
        dtype="bfloat16", max_model_len=256, max_num_seqs=4, max_num_batched_tokens=64, max_prefill_chunk=64,
        max_cache_tokens=1024, use_graphs=True)).runner
    runner.GRAPH_MAX_KEPT = 1
    seqs = tt.make_sequences(cfg["vocab"], [60, 60, 60], seed=9)
    refs = {rid: plain_gemma.forward(weights, cfg, ids, torch.float64) for rid, ids in seqs.items()}
    for rid, ids in seqs.items():
        runner.add_request(rid)
        runner.step([(rid, ids[:10], [])])
    done = {rid: 10 for rid in seqs}
    replays = []
    for it in range(15):
        live = list(seqs) if (it // 5) % 2 == 0 else list(seqs)[:2]  # three requests, two, three again
        before = runner.graph_replays
        got = runner.step([(rid, [seqs[rid][done[rid]]], [0]) for rid in live]).float().cpu()
        replays.append(runner.graph_replays - before)
        for row, rid in enumerate(live):
            tt.compare(got[row:row + 1].numpy(), refs[rid][done[rid]:done[rid] + 1], "bfloat16", f"step {it} {rid}")
            done[rid] += 1
        assert len(runner._graphs) == 1
    assert replays == [0, 1, 1, 1, 1] * 3  # the first step of each run of a shape is eager


def test_the_garbage_collector_rests_while_a_step_is_recorded(model_dirs):
    """An engine that was dropped may lie in a cycle with its graphs; were it collected while another step is being
    recorded, its memory would be freed during the recording, which the runtime does not allow.  So what is garbage
    goes before the recording and the collector is off during it, and as it was afterwards."""
    import gc

    cfg = EngineConfig(dtype="bfloat16", max_model_len=256, max_num_seqs=2, max_num_batched_tokens=256,
                       max_prefill_chunk=256, max_cache_tokens=512, use_graphs=True)
    runner = LLMEngine.from_model_dir(model_dirs["A"], cfg).runner
    seen = []
    forward = runner.model.forward

    def watched(batch, views):
        seen.append((torch.cuda.is_current_stream_capturing(), gc.isenabled()))
        return forward(batch, views)

    runner.model.forward = watched
    runner.add_request("a")
    runner.step([("a", [1, 2, 3], [2])])
    assert gc.isenabled()
    for token in (4, 5, 6):
        runner.step([("a", [token], [0])])
    # the prompt, the first decoded token run as it comes and then recorded; the rest are replays
    assert seen == [(False, True), (False, True), (True, False)] and gc.isenabled() and runner.graph_replays == 2


@pytest.mark.parametrize("name", ["A", "C"])
def test_several_greedy_steps_in_a_row_choose_what_single_steps_choose(model_dirs, name):
    """``decode_greedy`` hands each request's arg-max token to its next step on the device.  Against a twin runner
    that takes one step at a time: the same tokens, over page edges, with requests of different lengths; one step
    only while the shape has no graph yet, and no step past the end of the graph's bucket of contexts.  (The engine
    against the engine: what a single step computes is held to the plain model by the replay tests.)"""
    common = dict(dtype="bfloat16", max_model_len=1100, max_num_seqs=4, max_num_batched_tokens=1100,
                  max_prefill_chunk=1100, max_cache_tokens=3400, use_graphs=True)
    one = LLMEngine.from_model_dir(model_dirs[name], EngineConfig(**common)).runner
    many = LLMEngine.from_model_dir(model_dirs[name], EngineConfig(**common)).runner
    vocab = one.model.spec.vocab_size
    prompts = {"a": [(7 * i + 1) % vocab for i in range(10)], "b": [(3 * i + 2) % vocab for i in range(27)],
               "c": [(5 * i + 3) % vocab for i in range(1000)]}  # c is 19 tokens from the end of the first bucket
    last = {}
    for runner in (one, many):
        for rid, ids in prompts.items():
            runner.add_request(rid)
            last[rid] = int(runner.step([(rid, ids, [len(ids) - 1])]).argmax())
    nxt_one, nxt_many = dict(last), dict(last)
    taken = []
    total = 0
    while total < 40:
        rows = many.decode_greedy([(rid, nxt_many[rid]) for rid in prompts], 6)
        taken.append(len(rows))
        for row in rows:
            got = one.step([(rid, [nxt_one[rid]], [0]) for rid in prompts]).argmax(dim=1).tolist()
            assert row == got, f"step {total}"
            nxt_one = dict(zip(prompts, got))
            total += 1
        nxt_many = dict(zip(prompts, rows[-1]))
        assert {rid: many.length(rid) for rid in prompts} == {rid: one.length(rid) for rid in prompts}
    # the first call meets a shape without a graph; the contexts reach 1024 after 24 steps: the call before
    # runs only as far as the bucket goes, the one after starts a new shape
    assert taken[0] == 1 and max(taken) == 6 and sum(taken[: taken.index(1, 1)]) == 24, taken
    assert many.graph_replays > one.graph_replays // 2


@pytest.mark.parametrize("name", ["A", "C"])
def test_greedy_steps_ahead_change_no_token(model_dirs, name):
    """Several greedy decode steps from one plan against one plan a step: the same tokens and reasons for requests
    that end at different lengths, one of them at an end id met on the way, and with so few pages that requests are
    set back.  With requests that sample among them the steps still follow one another: the device then draws for
    them as the host does, from each request's own stream of numbers, so the tokens are those of single steps with
    the host's draw (temperatures, nucleus, seeds and numbers of candidates that differ).  (The engine against the
    engine: what a single step computes is held to the plain model by the replay tests.)"""
    def run(ahead, tight, places=4):
        engine = LLMEngine.from_model_dir(model_dirs[name], EngineConfig(
            dtype="bfloat16", max_model_len=200, max_num_seqs=places, max_num_batched_tokens=64, max_prefill_chunk=64,
            max_cache_tokens=112 if tight else 800, greedy_steps_ahead=ahead))
        vocab = engine.runner.model.spec.vocab_size
        params_of = {}
        engine.draws = []  # every step whose tokens the device drew: (request ids, logits, streams before, tokens)
        decode_ahead = engine.runner.decode_ahead

        def watched(entries, steps, choose=None):
            if choose is None:
                return decode_ahead(entries, steps, None)

            def recording(logits, out):
                before = choose.state.clone()
                choose(logits, out)
                engine.draws.append(([rid for rid, _ in entries], logits.clone(), before.cpu().tolist(), out.clone()))
                return out

            return decode_ahead(entries, steps, recording)

        engine.runner.decode_ahead = watched
        engine.params_of = params_of
        engine.set_backs = 0
        prompts = [[(11 * i + j) % vocab for i in range(n)] for j, n in enumerate((5, 18, 33, 9))]
        out = {}
        sampling = {"all greedy": {}, "one samples": {2: SamplingParams(0.9, 20, 1.0, seed=3)},
                    "three sample": {0: SamplingParams(0.7, 20, 0.9, seed=5), 2: SamplingParams(1.3, 20, 1.0, seed=3),
                                     3: SamplingParams(1.0, 20, 0.5, seed=(1 << 64) - 3)},
                    "other candidates": {0: SamplingParams(0.7, 10, 1.0, seed=5), 2: SamplingParams(0.9, 20, 1.0, seed=3)}}
        for phase, sampled in sampling.items():
            before = engine.plans, engine.steps
            for j, prompt in enumerate(prompts):
                params = sampled.get(j, SamplingParams())
                params_of[(phase, j)] = params
                engine.add_request((phase, j), prompt, params, max_new_tokens=(37, 50, 23, 44)[j],
                                   eos_ids=run.eos if j == 1 else (), ignore_eos=False)
            while engine.has_work():
                for res in engine.step():
                    out[res.request_id] = (res.tokens, res.finish_reason)
                    engine.set_backs += res.set_backs
            run.planned[(ahead, tight, places, phase)] = (engine.plans - before[0], engine.steps - before[1])
        return out, engine

    run.eos = ()
    run.planned = {}
    free, _ = run(1, False)
    run.eos = (free[("all greedy", 1)][0][29],)  # request 1 will stop at this token, or at its first appearance
    single, e1 = run(1, False)
    ahead, e4 = run(4, False)
    assert single == ahead
    assert single[("all greedy", 1)][1] == "stop" and len(single[("all greedy", 1)][0]) <= 30
    assert [single[("all greedy", j)][1] for j in (0, 2, 3)] == ["length"] * 3
    assert e4.steps == e1.steps  # a step is a step, however many were planned at once
    assert e1.plans == e1.steps and e4.plans < 0.7 * e4.steps
    for phase in ("one samples", "three sample", "other candidates"):  # steps follow one another with draws on the device
        plans, steps = run.planned[(4, False, 4, phase)]
        assert plans < 0.7 * steps, phase
        assert single[(phase, 2)][0] != single[("all greedy", 2)][0]  # and the draws are draws
    # Where requests are set back or wait for a place, steps that follow one another notice an end a few steps
    # late, so the requests share their steps differently; the logits then differ in their last bits (the
    # attention's split of the keys and the products' kernels go by what a step holds), which the arg-max does
    # not feel and a draw now and then does: these runs are compared by their greedy requests.
    greedy_only = lambda out: {key: value for key, value in out.items() if key[0] == "all greedy"}
    tight_single, t1 = run(1, True)
    tight_ahead, t4 = run(4, True)
    assert greedy_only(tight_single) == greedy_only(tight_ahead) == greedy_only(single)
    # two places for four requests: the waiting ones get theirs when a running one ends, and steps follow one
    # another meanwhile
    few_single, f1 = run(1, False, places=2)
    few_ahead, f4 = run(4, False, places=2)
    assert greedy_only(few_single) == greedy_only(few_ahead) == greedy_only(single) and f4.plans < 0.8 * f4.steps
    for out in (tight_single, tight_ahead, few_single, few_ahead):  # and the others ran to their ends
        assert {key: (len(tokens), reason) for key, (tokens, reason) in out.items()} == \
               {key: (len(tokens), reason) for key, (tokens, reason) in single.items()}
    # The requests that sample, in exactly these runs: every token that the device drew, with requests set back
    # or waiting around it, is the token that the host's sampler draws from the same logits with the request's
    # stream as it stood before the draw; and a greedy request's among them is the arg-max's.
    from rvllm_amd.sampling.sampler import Sampler, SplitMix64

    for engine in (e4, t4, f4):
        assert len(engine.draws) > 30
        sampler = Sampler(engine.runner.model.spec.vocab_size)
        for rids, logits, states, tokens in engine.draws:
            params = [engine.params_of[rid] for rid in rids]
            rngs = [SplitMix64(state) for state in states]
            assert sampler.sample(logits, params, rngs) == tokens.cpu().tolist()
    assert t4.set_backs >= 1 and t1.set_backs >= 1 and e4.set_backs == 0  # the tight runs did set requests back


def test_eos_and_capacity_reasons(model_dirs):
    engine = LLMEngine.from_model_dir(model_dirs["A"], EngineConfig(dtype="float32", max_model_len=128,
                                                                    max_num_seqs=2, max_cache_tokens=32))
    prompt = [5, 6, 7, 8]
    free_run = engine.generate([prompt], None, max_new_tokens=6)[0].tokens
    stopped = engine.generate([prompt], None, max_new_tokens=6, eos_ids=[free_run[2]])[0]
    first = free_run.index(free_run[2])
    assert stopped.tokens == free_run[:first + 1] and stopped.finish_reason == "stop"
    # 32 tokens of cache: a request that wants more ends with "capacity" and keeps what it produced
    res = engine.generate([prompt], None, max_new_tokens=100, ignore_eos=True)[0]
    assert res.finish_reason == "capacity" and 0 < len(res.tokens) < 100


@pytest.mark.parametrize("how", ["module", "script"])
def test_command_line(model_dirs, tmp_path, how):
    """As ``python -m rvllm_amd.cli`` and as the script ``bin/rvllm-amd``, from another working folder."""
    prompts = tmp_path / "prompts.txt"
    prompts.write_text("1 2 3 4\n9 8 7\n")
    dump = tmp_path / "out.txt"
    start = [sys.executable, "-m", "rvllm_amd.cli"] if how == "module" else [str(tt.ROOT / "bin" / "rvllm-amd")]
    cmd = [*start, "--model", str(model_dirs["A"]), "--dtype=float32",
           "--max-model-len", "64", "--max-num-seqs", "2", "--prompt-file", str(prompts), "--max-tokens", "5",
           "--dump", str(dump)]
    proc = subprocess.run(cmd, capture_output=True, text=True, cwd=str(tt.ROOT if how == "module" else tmp_path),
                          timeout=300)
    assert proc.returncode == 0, proc.stderr
    lines = [json.loads(l) for l in proc.stdout.strip().splitlines()]
    assert [l["completion_tokens"] for l in lines] == [5, 5] and lines[0]["finish_reason"] == "length"
    assert dump.read_text().splitlines() == [" ".join(map(str, l["token_ids"])) for l in lines]
    direct = rvllm_amd.generate(str(model_dirs["A"]), [[1, 2, 3, 4], [9, 8, 7]], max_tokens=5, dtype="float32",
                                max_model_len=64, max_num_seqs=2)
    assert direct == [l["token_ids"] for l in lines]
