"""Generation through the Python entry point and the command line, against the plain
implementation; the same tokens alone, batched, cut into portions, after a warm prefix cache
and after forced preemption (reference: tests/test_runner.py:84-155)."""

from __future__ import annotations

import json
import subprocess
import sys

import pytest
import torch

from tests import helpers
from tests.plain import qwen2_plain as plain

pytestmark = pytest.mark.gpu

PROMPT = [(i * 13 + 7) % 500 for i in range(80)]
OTHER = [(i * 29 + 3) % 500 for i in range(56)]


def engine(name="A", dtype="float32", **kw):
    from mercury_amd import Engine, EngineConfig

    kw.setdefault("num_blocks", 64)
    kw.setdefault("max_model_len", 512)
    return Engine(EngineConfig(model=str(helpers.model_folder(name)), dtype=dtype, **kw))


def generate(eng, prompts, max_tokens=12, **params):
    from mercury_amd import SamplingParams

    out = eng.generate(prompts, SamplingParams(ignore_eos=True, **params), max_tokens)
    assert eng.leaked_blocks() == 0
    return out


def plausible(folder, prompt, tokens, exact_share=0.75):
    """Every generated token is the plain model's argmax at its place, or so close to it that
    the bfloat16 error allowed on each of the two logits (the bound the replay tests derive
    from the plain implementation's own bfloat16 run) can have swapped them; and most of them
    (`exact_share`) are the argmax itself: near-ties are the exception among random-weight
    logits, so an engine that picked a runner-up at most places is wrong however close the
    runner-up was."""
    from tests.test_gpu_replay import BF16_SLACK, bf16_cost

    w, cfg = helpers.plain_model(folder)
    whole = plain.forward_logits(w, cfg, prompt + tokens)
    allowed = 2 * BF16_SLACK * bf16_cost(folder, cfg, prompt + tokens, whole)
    logits = whole[len(prompt) - 1:-1]
    chosen = logits[torch.arange(len(tokens)), torch.tensor(tokens)]
    exact = int((logits.argmax(-1) == torch.tensor(tokens)).sum())
    return bool((logits.max(-1).values - chosen <= allowed).all()) and \
        exact >= int(exact_share * len(tokens))     # (of two tokens, one may be a near-tie)


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_greedy_generation_equals_the_plain_implementation(name):
    folder = helpers.model_folder(name)
    w, cfg = helpers.plain_model(folder)
    vocab = cfg["vocab_size"]
    prompts = [helpers.random_tokens(vocab, n, seed=n) for n in (5, 17, 33, 1)]
    want = [plain.greedy_generate(w, cfg, p, 8) for p in prompts]
    assert generate(engine(name), prompts, 8) == want
    got = generate(engine(name, "bfloat16"), prompts, 8)
    assert all(plausible(folder, p, g) for p, g in zip(prompts, got))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_same_tokens_however_the_work_is_cut(dtype):
    alone = {k: generate(engine(dtype=dtype), [p])[0] for k, p in (("a", PROMPT), ("b", OTHER))}
    together = generate(engine(dtype=dtype), [PROMPT, OTHER])
    assert together == [alone["a"], alone["b"]]
    portions = generate(engine(dtype=dtype, prefill_budget=24), [PROMPT, OTHER])
    assert portions == together
    crowd = [[(i * 31 + j) % 500 for j in range(48)] for i in range(6)] + [PROMPT]
    assert generate(engine(dtype=dtype, max_running=8), crowd)[-1] == alone["a"]
    small_pages = generate(engine(dtype=dtype, block_size=8, num_blocks=128), [PROMPT, OTHER])
    assert small_pages == together


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_warm_prefix_cache_and_rope_positions_after_it(dtype):
    eng = engine(dtype=dtype)
    cold = generate(eng, [PROMPT])[0]
    assert eng.manager.main_pool.stats["hit_tokens"] == 0
    assert generate(eng, [PROMPT])[0] == cold
    assert eng.manager.main_pool.stats["hit_tokens"] == 64
    longer = PROMPT + OTHER
    assert generate(eng, [longer])[0] == generate(engine(dtype=dtype), [longer])[0]
    assert eng.manager.main_pool.stats["hit_tokens"] > 64


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_forced_preemption_does_not_change_the_output(dtype):
    expected = generate(engine(dtype=dtype), [PROMPT], 24)[0]
    tight = engine(dtype=dtype, num_blocks=11, max_running=4, max_model_len=176,
                   debug_invariants=True)
    crowd = [PROMPT] + [[(i * 37 + j) % 500 for j in range(80)] for i in range(3)]
    got = generate(tight, crowd, 24)
    assert tight.sched.stats["preemptions"] > 0
    assert got[0] == expected


def test_every_policy_produces_the_same_tokens():
    prompts = [PROMPT, OTHER, PROMPT + [5] * 16]
    base = generate(engine(policy="fcfs"), prompts)
    for policy in ("lpm", "lpm_aging"):
        assert generate(engine(policy=policy), prompts) == base


def test_temperature_sampling_is_per_request_reproducible():
    """Tiny configuration B with its own workload: pages of 8 tokens, prompts of 1, 9, 40 and
    64 tokens of which two share their first 24, portions of 16 beside decoded tokens,
    temperature 0.8 under a seeded generator.  A request draws
    the same tokens alone, in a batch and cut into portions of 16."""
    folder = helpers.model_folder("B")
    vocab = 1000
    shared = helpers.random_tokens(vocab, 24, seed=99)
    prompts = [helpers.random_tokens(vocab, 1, seed=1), helpers.random_tokens(vocab, 9, seed=2),
               shared + helpers.random_tokens(vocab, 16, seed=3),
               shared + helpers.random_tokens(vocab, 40, seed=4)]

    def run(which, **kw):
        from mercury_amd import SamplingParams

        kw.setdefault("seed", 5)
        eng = engine("B", block_size=8, num_blocks=64, **kw)
        outs = {}
        for i in which:
            eng.submit(f"req{i}", prompts[i], 6, lambda e, i=i: outs.setdefault(i, []).append(e),
                       params=SamplingParams(temperature=0.8, ignore_eos=True))
        eng._take_commands()
        while eng.sched.has_work():
            eng.step()
        return {i: [e.token for e in ev if e.kind == "token"] for i, ev in outs.items()}

    batched = run(range(4), prefill_budget=16)
    for i in range(4):
        assert run([i])[i] == batched[i]
    assert len({tuple(v) for v in batched.values()}) == 4
    # another seed draws other tokens: over four requests of six tokens from a flat
    # distribution (the largest probability is a few per cent) at least one draw differs
    other = run(range(4), prefill_budget=16, seed=6)
    assert any(other[i] != batched[i] for i in range(4))


@pytest.mark.parametrize("lookahead", [False, True])
def test_sampled_tokens_are_the_plain_rule_on_the_plain_logits(lookahead):
    """Configuration B in float32: every sampled token is
    inverse_cdf_draw(sampling_distribution(plain logits), uniform_for(seed, request id, output
    index)) (reference: mercury/sampling.py:17-35 for the distribution).  An output index off
    by one, or the draw of another request, would give other tokens at once.  Where the
    uniform number falls within 1e-5 of the boundary between two tokens' shares, float32 and
    float64 sums may put it on either side, and either token is taken."""
    from mercury_amd import SamplingParams
    from mercury_amd.sampling.sampler import uniform_for

    folder = helpers.model_folder("B")
    w, cfg = helpers.plain_model(folder)
    prompts = {"plain": helpers.random_tokens(1000, 9, seed=2),
               "nucleus": helpers.random_tokens(1000, 40, seed=3),
               "own-seed": helpers.random_tokens(1000, 17, seed=4)}
    params = {"plain": dict(temperature=0.8), "nucleus": dict(temperature=1.3, top_p=0.6),
              "own-seed": dict(temperature=0.7, seed=1234)}
    eng = engine("B", block_size=8, num_blocks=64, seed=5, lookahead=lookahead, prefill_budget=16)
    outs = {rid: [] for rid in prompts}
    for rid, prompt in prompts.items():
        eng.submit(rid, prompt, 12, outs[rid].append,
                   params=SamplingParams(ignore_eos=True, **params[rid]))
    eng.run_until_idle()
    if lookahead:
        assert eng.runner.stats["ahead_used"] > 0
    for rid, prompt in prompts.items():
        got = [e.token for e in outs[rid] if e.kind == "token"]
        assert len(got) == 12
        seed = params[rid].get("seed", 5)
        tokens = list(prompt)
        for index, token in enumerate(got):
            logits = plain.forward_logits(w, cfg, tokens)[-1]
            probs = plain.sampling_distribution(logits, params[rid]["temperature"],
                                                params[rid].get("top_p", 1.0))
            u = uniform_for(seed, rid, index)
            want = plain.inverse_cdf_draw(probs, u)
            if token != want:
                cumulative = probs.double().cumsum(-1)
                lo, hi = sorted((token, want))
                between = cumulative[lo:hi]          # the boundaries that separate the two
                assert len(between) and float((between - u).abs().max()) < 1e-5, \
                    f"{rid} output {index}: drew {token}, the plain rule draws {want} (u = {u})"
            tokens.append(token)
    assert eng.leaked_blocks() == 0


def test_command_line_generates_and_writes_random_weights(tmp_path):
    config = tmp_path / "config.json"
    config.write_text(json.dumps(helpers.TINY_A))
    out = subprocess.run([sys.executable, "-m", "mercury_amd", "random-weights", "--config",
                          str(config), "--out", str(tmp_path / "m"), "--seed", "3", "--std", "0.05"],
                         capture_output=True, text=True, cwd=helpers.ROOT)
    assert out.returncode == 0, out.stderr
    prompt = [(i * 7) % 500 for i in range(20)]
    run = subprocess.run([sys.executable, "-m", "mercury_amd", "generate", "--model",
                          str(tmp_path / "m"), "--prompt-ids", ",".join(map(str, prompt)),
                          "--prompt-ids", "1 2 3", "--max-tokens", "5", "--dtype", "float32",
                          "--num-blocks", "32", "--max-model-len", "256", "--ignore-eos"],
                         capture_output=True, text=True, cwd=helpers.ROOT)
    assert run.returncode == 0, run.stderr
    lines = [json.loads(line) for line in run.stdout.strip().splitlines()]
    w, cfg = helpers.plain_model(tmp_path / "m")
    assert lines[0] == {"prompt_index": 0, "tokens": plain.greedy_generate(w, cfg, prompt, 5)}
    assert lines[1]["tokens"] == plain.greedy_generate(w, cfg, [1, 2, 3], 5)


def test_smoke_entry_point():
    import __graft_entry__

    __graft_entry__.smoke()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_captured_decode_graphs_replay_like_eager_steps(dtype):
    """Decode steps run through captured HIP graphs.  Replays of one graph, with other work
    (prompts, other batch sizes, synchronisations) between them, give the tokens of an engine
    that never captures."""
    prompts = [PROMPT, OTHER, PROMPT[:33], OTHER[:7]]
    eager = generate(engine(dtype=dtype, use_graphs=False), prompts, 40)
    graphed_engine = engine(dtype=dtype, use_graphs=True)
    assert generate(graphed_engine, prompts, 40) == eager
    assert len(graphed_engine.runner.runner.graphs) >= 1
    # the same graphs again, after unrelated work in between
    assert generate(graphed_engine, prompts[:2], 20) == [e[:20] for e in eager[:2]]
    assert generate(graphed_engine, prompts, 40) == eager


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_graph_row_changes_its_owner(dtype):
    """With two requests running at a time and five waiting in turn, the rows of the
    two-sequence graph pass from request to request, and with few pages a preempted request
    comes back under its own key with other pages: the graph's host copy of the block tables
    has to follow.  The tokens are those of an engine that never captures."""
    from mercury_amd import SamplingParams

    prompts = [PROMPT[:40], OTHER[:30], PROMPT[:9], OTHER[:50], PROMPT[:25]]
    lengths = [30, 12, 44, 7, 21]

    def run(**kw):
        eng = engine(dtype=dtype, max_running=2, **kw)
        outs = {i: [] for i in range(len(prompts))}
        for i, (p, n) in enumerate(zip(prompts, lengths)):
            eng.submit(f"r{i}", list(p), n, outs[i].append, params=SamplingParams(ignore_eos=True))
        eng._take_commands()
        while eng.sched.has_work():
            eng.step()
        assert eng.leaked_blocks() == 0
        return {i: [e.token for e in ev if e.kind == "token"] for i, ev in outs.items()}, eng

    eager, _ = run(use_graphs=False)
    graphed, eng = run(use_graphs=True)
    assert graphed == eager
    assert any(key[0] == 2 for key in eng.runner.runner.graphs)
    # 6 pages of 16 tokens hold two requests only until they have grown: the newer one is
    # preempted and starts over
    tight, eng = run(use_graphs=True, num_blocks=6, max_model_len=96)
    assert tight == eager
    assert eng.sched.stats["preemptions"] > 0


def run_requests(eng, submissions, max_tokens, aborts=(), **params):
    """Drive the engine by hand: `submissions` maps a step number to the prompts submitted
    before it, `aborts` a step number to the request ids aborted before it."""
    from mercury_amd import SamplingParams

    outs, step, count = {}, 0, 0
    while True:
        for prompt in submissions.get(step, []):
            rid = f"r{count}"
            outs[rid] = []
            eng.submit(rid, list(prompt), max_tokens, outs[rid].append,
                       params=SamplingParams(**params))
            count += 1
        for rid in dict(aborts).get(step, []):
            eng.abort(rid)
        eng._take_commands()
        if not eng.sched.has_work() and step > max(submissions):
            break
        eng.step()
        step += 1
    assert eng.leaked_blocks() == 0
    return {rid: [e.token for e in ev if e.kind == "token"] for rid, ev in outs.items()}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_steps_started_ahead_give_the_same_tokens(dtype):
    """A decode step launched before the previous one's tokens were read (the scheduler
    expected the same requests to go on) yields what the step launched afterwards yields:
    greedy and sampled, with requests that arrive, stop at a stop token, reach their length
    or are aborted while a step runs ahead."""
    prompts = [PROMPT, OTHER, PROMPT[:33], OTHER[:7]]
    plain_run = run_requests(engine(dtype=dtype, lookahead=False), {0: prompts}, 40, ignore_eos=True)
    eng = engine(dtype=dtype, lookahead=True)
    assert run_requests(eng, {0: prompts}, 40, ignore_eos=True) == plain_run
    stats = eng.runner.stats
    assert stats["ahead_used"] >= 30 and stats["ahead_started"] - stats["ahead_used"] <= 2

    sampling = dict(temperature=0.8, top_p=0.9)
    sampled = run_requests(engine(dtype=dtype, lookahead=False), {0: prompts}, 24, ignore_eos=True,
                           **sampling)
    assert run_requests(engine(dtype=dtype, lookahead=True), {0: prompts}, 24, ignore_eos=True,
                        **sampling) == sampled

    # a token some request first draws a few steps into decoding becomes the stop token: the
    # request ends there, the others go on, and the step that ran ahead with it is dropped
    stop = next(tok for toks in sampled.values() for i, tok in enumerate(toks)
                if i >= 3 and tok not in toks[:i])
    cut = {rid: (toks[:toks.index(stop) + 1] if stop in toks else toks) for rid, toks in sampled.items()}
    from mercury_amd import Engine, EngineConfig
    for look in (False, True):
        eng = Engine(EngineConfig(model=str(helpers.model_folder("A")), dtype=dtype, num_blocks=64,
                                  max_model_len=512, lookahead=look), eos_token_ids=[stop])
        assert run_requests(eng, {0: prompts}, 24, **sampling) == cut
    assert eng.runner.stats["ahead_started"] > eng.runner.stats["ahead_used"] > 0

    # arrivals and an abort in the middle of decoding
    late = {0: prompts[:2], 9: prompts[2:3], 15: prompts[3:]}
    aborts = {12: ["r0"]}
    want = run_requests(engine(dtype=dtype, lookahead=False), late, 30, aborts, ignore_eos=True)
    eng = engine(dtype=dtype, lookahead=True)
    assert run_requests(eng, late, 30, aborts, ignore_eos=True) == want
    assert len(want["r0"]) < 30 and want["r1"] == plain_run["r1"][:30]
    assert eng.runner.stats["ahead_used"] > 0
