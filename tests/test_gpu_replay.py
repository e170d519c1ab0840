"""Replay of the same requests in different cuts, in float32 and in bfloat16, against the
plain implementation: whole; most in one step and the last 32 tokens one by one; in portions
of changing size down to two tokens; mixed with other requests in a pool so small that pages
are used again; long decoding from the first token on."""

from __future__ import annotations

import pytest
import torch

from tests import helpers
from tests.plain import qwen2_plain as plain

pytestmark = pytest.mark.gpu

# float32: the reference's own bound for this comparison (tests/test_runner.py:182).
# bfloat16: the bound is derived, not fitted.  The plain implementation is run a second time
# with its tensors in bfloat16, which rounds wherever the reference rounds to its model dtype
# (mercury/model/qwen2.py:27-31, mercury/model/rope.py:46-47, every projection's output); the
# largest distance of that run's logits from the float32 run's is what bfloat16 costs the
# reference itself on this request.  The engine (float32 residual stream, float32 logits)
# may be off by at most BF16_SLACK times that, at every place.
TOL = {"float32": dict(atol=1e-5, rtol=1e-5)}
BF16_SLACK = 1.5
LENGTHS = {"a": 200, "b": 97, "c": 150, "d": 40, "e": 64, "f": 33}
PORTIONS = [16, 7, 2, 5, 3, 2, 33, 2, 64, 9, 2, 17]

# Beside the tiny configurations (B with the 8-token pages its workload names), two layers of
# the sizes whose kernels serving runs: heads of 64 in groups of 7 (the matrix-core attention,
# the fused q/k/v projection and the K-split projections whose partial sums the norms add
# up), and heads of 128 in groups of 4.
SIZED = {
    "S64": {"hidden_size": 896, "intermediate_size": 4864, "num_attention_heads": 14,
            "num_key_value_heads": 2, "head_dim": 64, "vocab_size": 5003,
            "tie_word_embeddings": True, "rms_norm_eps": 1e-6},
    "S128": {"hidden_size": 1024, "intermediate_size": 2816, "num_attention_heads": 8,
             "num_key_value_heads": 2, "head_dim": 128, "vocab_size": 3001,
             "tie_word_embeddings": False, "rms_norm_eps": 1e-5},
}
CASES = [("A", 16), ("B", 8), ("C", 16), ("S64", 16), ("S128", 32)]


def sized_folder(name):
    import tempfile
    from pathlib import Path

    from mercury_amd.weights import write_random_model

    if name not in helpers._FOLDERS:
        cfg = {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
               "num_hidden_layers": 2, "rope_theta": 1000000.0,
               "max_position_embeddings": 4096, **SIZED[name]}
        folder = Path(tempfile.mkdtemp(prefix=f"mercury_sized_{name}_"))
        write_random_model(folder, cfg, seed=3, std=0.02, dtype=torch.bfloat16)
        helpers._FOLDERS[name] = folder
    return helpers._FOLDERS[name]


def bf16_cost(folder, cfg, tokens, want):
    """The largest distance of the bfloat16 plain run's logits from the float32 run's."""
    rounded = plain.forward_logits(plain.read_weights(folder, torch.bfloat16), cfg, tokens)
    return float((rounded.float() - want).abs().max())


class Case:
    def __init__(self, name, page):
        self.name, self.page = name, page
        self.folder = sized_folder(name) if name in SIZED else helpers.model_folder(name)
        weights, cfg = helpers.plain_model(self.folder)
        self.reqs = {k: helpers.random_tokens(cfg["vocab_size"], n, seed=ord(k))
                     for k, n in LENGTHS.items()}
        self.want = {k: plain.forward_logits(weights, cfg, v) for k, v in self.reqs.items()}
        self.cost = {k: bf16_cost(self.folder, cfg, v, self.want[k]) for k, v in self.reqs.items()}

    def session(self, dtype, max_tokens):
        from mercury_amd.engine.replay import ReplaySession

        return ReplaySession(self.folder, dtype, max_tokens, page_size=self.page)

    def check(self, got, key, dtype, what, rows=None):
        want = self.want[key] if rows is None else self.want[key][rows]
        check(got, want, dtype, f"{self.name} {what} {key}", self.cost[key])


@pytest.fixture(scope="module", params=CASES, ids=[f"{n}-page{p}" for n, p in CASES])
def model(request):
    return Case(*request.param)


def entry(key, tokens):
    return {"id": key, "tokens": tokens, "want": list(range(len(tokens)))}


def check(got, want, dtype, what, bf16_cost=None, f32_cost=0.0):
    """`f32_cost`: where `want` was computed in float64, the plain implementation's own
    float32 distance from it; the engine's float32 result may add that (times the slack) to
    the reference's bound.  Zero wherever `want` is the plain float32 result itself."""
    assert got.shape == want.shape, f"{what}: {tuple(got.shape)} vs {tuple(want.shape)}"
    assert torch.isfinite(got).all(), f"{what}: non-finite logits"
    diff = (got - want).abs()
    if dtype == "bfloat16":
        assert bf16_cost is not None and bf16_cost > 0
        bound = torch.full_like(want, BF16_SLACK * bf16_cost)
    else:
        bound = TOL[dtype]["atol"] + TOL[dtype]["rtol"] * want.abs() + BF16_SLACK * f32_cost
    bad = (diff > bound).any(-1)
    if bad.any():
        first = int(bad.nonzero()[0])
        raise AssertionError(
            f"{what}: worst difference {diff.max().item():.3e} (bound {bound.max().item():.3e}), "
            f"first wrong token {first} of {got.shape[0]}, {int(bad.sum())} wrong")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_each_request_alone_and_whole(model, dtype):
    s = model.session(dtype, 256)
    for key, tokens in model.reqs.items():
        got = s.step([entry(key, tokens)], [key])
        model.check(got, key, dtype, "whole")
    assert s.manager.leaked_pages() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_most_in_one_step_then_the_last_32_one_by_one(model, dtype):
    s = model.session(dtype, 256)
    for key in ("a", "d", "f"):
        tokens = model.reqs[key]
        head = len(tokens) - 32
        rows = [s.step([entry(key, tokens[:head])], [])]
        for i in range(head, len(tokens)):
            rows.append(s.step([entry(key, tokens[i:i + 1])], [key] if i == len(tokens) - 1 else []))
        model.check(torch.cat(rows), key, dtype, "tail-decode")
    assert s.manager.leaked_pages() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_portions_of_changing_size(model, dtype):
    s = model.session(dtype, 256)
    for shift, key in enumerate(("a", "b", "c")):
        tokens, done, rows, n = model.reqs[key], 0, [], shift
        while done < len(tokens):
            size = PORTIONS[n % len(PORTIONS)]
            part = tokens[done:done + size]
            done += len(part)
            rows.append(s.step([entry(key, part)], [key] if done == len(tokens) else []))
            n += 1
        model.check(torch.cat(rows), key, dtype, "portions")
    assert s.manager.leaked_pages() == 0


def held(count):
    """What a request counts against the pool: its length rounded up to a multiple of 64."""
    return -(-count // 64) * 64


def mixed_run(step_fn, reqs, max_tokens, live_limit=4):
    """Up to four live requests; each runs its first 60% in portions of changing size and the
    rest token by token, so portions of some stand beside decoded tokens of others.  Finished
    requests give their pages back and the waiting ones take them."""
    order = ["a", "b", "d", "c", "e", "f", "a2", "c2"]
    pending = list(order)
    live, done, got = [], {}, {}
    n = 0
    while pending or live:
        while pending and len(live) < live_limit and \
                sum(held(len(reqs[k])) for k in live + pending[:1]) <= max_tokens:
            key = pending.pop(0)
            live.append(key)
            done[key], got[key] = 0, []
        entries, ends = [], []
        for i, key in enumerate(live):
            tokens = reqs[key]
            if done[key] < int(0.6 * len(tokens)):
                size = PORTIONS[(n + 3 * i) % len(PORTIONS)]
            else:
                size = 1
            part = tokens[done[key]:done[key] + size]
            entries.append(entry(key, part))
            if done[key] + len(part) == len(tokens):
                ends.append(key)
        out = step_fn(entries, ends)
        at = 0
        for e in entries:
            count = len(e["tokens"])
            got[e["id"]].append(out[at:at + count])
            at += count
            done[e["id"]] += count
        for key in ends:
            live.remove(key)
        n += 1
    return {k: torch.cat(v) for k, v in got.items()}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_requests_in_a_pool_whose_pages_are_used_again(model, dtype):
    reqs = dict(model.reqs, a2=model.reqs["a"], c2=model.reqs["c"])
    # a + b + d + c live together count 256+128+64+192 = 640 tokens; the eight requests
    # together count 1216, so pages are taken again by later requests.
    s = model.session(dtype, 640)
    used = set()

    def step_fn(entries, ends):
        out = s.step(entries, ends)
        for g in s.manager.groups:
            used.update(p for p in range(g.pool.num_pages) if g.pool.holders[p])
        s.manager.check_invariants()
        return out

    got = mixed_run(step_fn, reqs, 640)
    for key in got:
        model.check(got[key], key[0], dtype, f"mixed ({key})")
    assert s.manager.leaked_pages() == 0
    assert len(used) <= 640 // model.page


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_from_the_first_token(model, dtype):
    s = model.session(dtype, 256)
    tokens = model.reqs["a"]
    rows = [s.step([entry("x", tokens[i:i + 1])], []) for i in range(len(tokens))]
    model.check(torch.cat(rows), "a", dtype, "token by token")
    # the first tokens of a sequence, each alone in its step, are right on their own
    model.check(torch.cat(rows[:3]), "a", dtype, "first tokens", rows=slice(0, 3))


def test_position_shift_invariance_of_the_plain_model():
    """Only distances enter the rotary scores, so shifting every position leaves the logits
    unchanged; a plain implementation with a wrong pairing or sign fails this."""
    folder = helpers.model_folder("A")
    weights, cfg = helpers.plain_model(folder)
    tokens = helpers.random_tokens(cfg["vocab_size"], 24, seed=5)
    base = plain.forward_logits(weights, cfg, tokens)
    moved = plain.forward_logits(weights, cfg, tokens, first_position=37)
    torch.testing.assert_close(base, moved, atol=2e-5, rtol=1e-4)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,page", [("A", None), ("B", 8)])
def test_the_replay_program_itself(name, page, dtype):
    """Through bin/trace_run as a child process: whole, then chunked beside another request,
    in a pool that forces page reuse; files and `done` lines as documented; with the default
    page size and with --block-size 8; a place wanted twice comes back twice."""
    case = Case(name, page or 16)
    reqs = case.reqs
    run = helpers.TraceRun(case.folder, dtype, 320, block_size=page, max_live=4)
    got = run.step([entry("a", reqs["a"])], ["a"])
    case.check(got, "a", dtype, "program whole")
    assert run.step([{"id": "b", "tokens": reqs["b"][:50], "want": []}]) is None
    out = run.step([{"id": "b", "tokens": reqs["b"][50:], "want": [46]},
                    {"id": "c", "tokens": reqs["c"], "want": [149, 0, 149]}], ["b", "c"])
    case.check(out[0:1], "b", dtype, "program last", rows=slice(96, 97))
    case.check(out[1:4], "c", dtype, "program repeated", rows=[149, 0, 149])
    assert torch.equal(out[1], out[3])
    got = run.step([entry("d", reqs["d"]), entry("a", reqs["a"])], ["d", "a"])
    case.check(got[:40], "d", dtype, "program")
    case.check(got[40:], "a", dtype, "program again")
    assert run.close() == 0
