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
# bfloat16: the reference bounds its float16 run by 1e-2 on logits that reach about 10
# (tests/test_parity.py:126), a thousandth of their range with 11 bits of mantissa; bfloat16
# keeps 8 bits, 8 times coarser, and between kernels every activation is rounded to it, so
# the bound here is 2% of the largest logit of the request (the tiny models' logits reach 2
# to 4), with weights that are exactly representable in bfloat16 on both sides.
TOL = {"float32": dict(atol=1e-5, rtol=1e-5), "bfloat16": dict(atol=0.0, rtol=0.0)}
BF16_FRACTION = 0.02
LENGTHS = {"a": 200, "b": 97, "c": 150, "d": 40, "e": 64, "f": 33}
PORTIONS = [16, 7, 2, 5, 3, 2, 33, 2, 64, 9, 2, 17]


@pytest.fixture(scope="module", params=["A", "B", "C"])
def model(request):
    folder = helpers.model_folder(request.param)
    weights, cfg = helpers.plain_model(folder)
    reqs = {k: helpers.random_tokens(cfg["vocab_size"], n, seed=ord(k)) for k, n in LENGTHS.items()}
    want = {k: plain.forward_logits(weights, cfg, v) for k, v in reqs.items()}
    return folder, reqs, want


def session(folder, dtype, max_tokens):
    from mercury_amd.engine.replay import ReplaySession

    return ReplaySession(folder, dtype, max_tokens)


def entry(key, tokens):
    return {"id": key, "tokens": tokens, "want": list(range(len(tokens)))}


def check(got, want, dtype, what):
    assert got.shape == want.shape, f"{what}: {tuple(got.shape)} vs {tuple(want.shape)}"
    assert torch.isfinite(got).all(), f"{what}: non-finite logits"
    diff = (got - want).abs()
    if dtype == "bfloat16":
        bound = torch.full_like(want, BF16_FRACTION * float(want.abs().max()))
    else:
        bound = TOL[dtype]["atol"] + TOL[dtype]["rtol"] * want.abs()
    bad = (diff > bound).any(-1)
    if bad.any():
        first = int(bad.nonzero()[0])
        raise AssertionError(
            f"{what}: worst difference {diff.max().item():.3e} (bound {bound.max().item():.3e}), "
            f"first wrong token {first} of {got.shape[0]}, {int(bad.sum())} wrong")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_each_request_alone_and_whole(model, dtype):
    folder, reqs, want = model
    s = session(folder, dtype, 256)
    for key, tokens in reqs.items():
        got = s.step([entry(key, tokens)], [key])
        check(got, want[key], dtype, f"whole {key}")
    assert s.manager.leaked_pages() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_most_in_one_step_then_the_last_32_one_by_one(model, dtype):
    folder, reqs, want = model
    s = session(folder, dtype, 256)
    for key in ("a", "d", "f"):
        tokens = reqs[key]
        head = len(tokens) - 32
        rows = [s.step([entry(key, tokens[:head])], [])]
        for i in range(head, len(tokens)):
            rows.append(s.step([entry(key, tokens[i:i + 1])], [key] if i == len(tokens) - 1 else []))
        check(torch.cat(rows), want[key], dtype, f"tail-decode {key}")
    assert s.manager.leaked_pages() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_portions_of_changing_size(model, dtype):
    folder, reqs, want = model
    s = session(folder, dtype, 256)
    for shift, key in enumerate(("a", "b", "c")):
        tokens, done, rows, n = reqs[key], 0, [], shift
        while done < len(tokens):
            size = PORTIONS[n % len(PORTIONS)]
            part = tokens[done:done + size]
            done += len(part)
            rows.append(s.step([entry(key, part)], [key] if done == len(tokens) else []))
            n += 1
        check(torch.cat(rows), want[key], dtype, f"portions {key}")
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
    folder, reqs, want = model
    reqs = dict(reqs, a2=reqs["a"], c2=reqs["c"])
    want = dict(want, a2=want["a"], c2=want["c"])
    # a + b + d + c live together count 256+128+64+192 = 640 tokens; the eight requests
    # together count 1216, so pages are taken again by later requests.
    s = session(folder, dtype, 640)
    used = set()

    def step_fn(entries, ends):
        out = s.step(entries, ends)
        for g in s.manager.groups:
            used.update(p for p in range(g.pool.num_pages) if g.pool.holders[p])
        s.manager.check_invariants()
        return out

    got = mixed_run(step_fn, reqs, 640)
    for key in got:
        check(got[key], want[key], dtype, f"mixed {key}")
    assert s.manager.leaked_pages() == 0
    assert len(used) <= 40


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_from_the_first_token(model, dtype):
    folder, reqs, want = model
    s = session(folder, dtype, 256)
    tokens = reqs["a"]
    rows = [s.step([entry("x", tokens[i:i + 1])], []) for i in range(len(tokens))]
    check(torch.cat(rows), want["a"], dtype, "token by token")
    # the first tokens of a sequence, each alone in its step, are right on their own
    check(torch.cat(rows[:3]), want["a"][:3], dtype, "first tokens")


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
def test_the_replay_program_itself(dtype):
    """Through bin/trace_run as a child process: whole, then chunked beside another request,
    in a pool that forces page reuse; files and `done` lines as documented."""
    folder = helpers.model_folder("A")
    weights, cfg = helpers.plain_model(folder)
    reqs = {k: helpers.random_tokens(cfg["vocab_size"], n, seed=ord(k)) for k, n in LENGTHS.items()}
    want = {k: plain.forward_logits(weights, cfg, v) for k, v in reqs.items()}
    run = helpers.TraceRun(folder, dtype, 320)
    got = run.step([entry("a", reqs["a"])], ["a"])
    check(got, want["a"], dtype, "program whole a")
    assert run.step([{"id": "b", "tokens": reqs["b"][:50], "want": []}]) is None
    out = run.step([{"id": "b", "tokens": reqs["b"][50:], "want": [46]},
                    {"id": "c", "tokens": reqs["c"], "want": [0, 149]}], ["b", "c"])
    check(out[0:1], want["b"][96:97], dtype, "program b last")
    check(out[1:3], want["c"][[0, 149]], dtype, "program c")
    got = run.step([entry("d", reqs["d"]), entry("a", reqs["a"])], ["d", "a"])
    check(got[:40], want["d"], dtype, "program d")
    check(got[40:], want["a"], dtype, "program a again")
    assert run.close() == 0
