"""Replay at the sizes the benchmark times, against the plain implementation: the 0.5B
configuration's own output head (151,936 rows, tied to the embedding), and single requests as
long as the benchmark's prompts and contexts, so that the kernels for long prompts and the
captured decode graphs beyond 4,096 tokens are reached through the step function
(the reference pins long ranges at tests/test_attention.py:84-132 and whole-model parity at
tests/test_parity.py:115-128)."""

from __future__ import annotations

import tempfile
from pathlib import Path

import pytest
import torch

from tests import helpers
from tests.plain import qwen2_plain as plain
from tests.test_gpu_replay import SIZED, bf16_cost, check, entry

pytestmark = pytest.mark.gpu

_FOLDERS: dict = {}


def folder_for(name: str, sharpen: float = 1.0, **override) -> Path:
    """Two layers of the sizes SIZED[name], written by the random-weights mode.  `sharpen`
    multiplies the query and key projections, so that the scores spread over several units and
    every query's weight sits on a few keys at arbitrary distances: with the nearly flat
    attention of small random weights a key missed far back would change nothing."""
    from safetensors.torch import load_file, save_file

    from mercury_amd.weights import write_random_model

    key = (name, sharpen, tuple(sorted(override.items())))
    if key not in _FOLDERS:
        cfg = {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
               "num_hidden_layers": 2, "rope_theta": 1000000.0,
               "max_position_embeddings": 8192, **SIZED[name], **override}
        folder = Path(tempfile.mkdtemp(prefix=f"mercury_bench_sizes_{name}_"))
        write_random_model(folder, cfg, seed=11, std=0.02, dtype=torch.bfloat16)
        if sharpen != 1.0:
            path = folder / "model.safetensors"
            tensors = load_file(str(path))
            for n in tensors:
                if ".q_proj." in n or ".k_proj." in n:
                    tensors[n] = (tensors[n].float() * sharpen).to(tensors[n].dtype)
            save_file(tensors, str(path), metadata={"format": "pt"})
        _FOLDERS[key] = folder
    return _FOLDERS[key]


def session(folder, dtype, max_tokens, page=16):
    from mercury_amd.engine.replay import ReplaySession

    return ReplaySession(folder, dtype, max_tokens, page_size=page, max_live=2)


# ---- the 0.5B configuration's head: 151,936 rows, tied

@pytest.fixture(scope="module")
def full_vocab():
    folder = folder_for("S64", vocab_size=151936)
    weights, cfg = helpers.plain_model(folder)
    reqs = {"a": helpers.random_tokens(cfg["vocab_size"], 200, seed=1),
            "d": helpers.random_tokens(cfg["vocab_size"], 40, seed=2)}
    want = {k: plain.forward_logits(weights, cfg, v) for k, v in reqs.items()}
    cost = {k: bf16_cost(folder, cfg, v, want[k]) for k, v in reqs.items()}
    return folder, reqs, want, cost


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_full_vocabulary_head_whole_and_with_a_decoded_tail(full_vocab, dtype):
    folder, reqs, want, cost = full_vocab
    s = session(folder, dtype, 512)
    assert s.model.tied_head and s.model.vocab_size == 151936
    for key, tokens in reqs.items():
        # whole: every place's logits in one step (the head over 200 and 40 rows)
        got = s.step([entry(key, tokens)], [key])
        check(got, want[key], dtype, f"full vocabulary, whole {key}", cost[key])
        # most in one step, the last 32 one by one (the head over one row, from a graph)
        head = len(tokens) - 32
        rows = [s.step([entry(key, tokens[:head])], [])]
        for i in range(head, len(tokens)):
            rows.append(s.step([entry(key, tokens[i:i + 1])], [key] if i == len(tokens) - 1 else []))
        check(torch.cat(rows), want[key], dtype, f"full vocabulary, tail {key}", cost[key])
    assert s.manager.leaked_pages() == 0


# ---- requests as long as the benchmark's prompts and contexts

def exact_logits(folder, cfg, tokens):
    """Under sharpened scores the plain implementation's own float32 rounding reaches the
    reference's bound of 1e-5 (its distance from a float64 run is about 2e-5 at 4,768
    tokens), so two float32 results cannot be held to that bound against each other.  The
    logits wanted are the float64 run's; what float32 and bfloat16 cost the plain
    implementation itself is measured and allowed on top (times the slack), the way the
    bfloat16 bound is derived everywhere."""
    exact = plain.forward_logits(plain.read_weights(folder, torch.float64), cfg, tokens)
    single = plain.forward_logits(plain.read_weights(folder), cfg, tokens)
    costs = {"bf16_cost": bf16_cost(folder, cfg, tokens, exact.float()),
             "f32_cost": float((single.double() - exact).abs().max())}
    return exact.float(), costs

LONG = [("S64", 4736, 16), ("S128", 2624, 32)]


@pytest.fixture(scope="module", params=LONG, ids=[f"{n}-{t}" for n, t, _ in LONG])
def long_case(request):
    name, head, page = request.param
    folder = folder_for(name, sharpen=3.0)
    cfg = plain.read_config(folder)
    tokens = helpers.random_tokens(cfg["vocab_size"], head + 32, seed=head)
    want, costs = exact_logits(folder, cfg, tokens)
    return name, folder, cfg, page, head, tokens, want, costs


def test_sharpened_weights_put_the_attention_on_far_keys(long_case):
    """What the long cases rest on: in the plain model, the last query's weight lies mostly on
    keys more than a thousand places back, and on few of them."""
    name, folder, cfg, page, head, tokens, want, cost = long_case
    w = plain.read_weights(folder)
    n_q, n_kv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    positions = torch.arange(len(tokens))
    cos, sin = plain.rotary_table(d, positions, cfg["rope_theta"])
    x = w["model.embed_tokens.weight"][torch.tensor(tokens)]
    p = "model.layers.0."
    x, _ = plain.rms_norm(x, w[p + "input_layernorm.weight"], cfg["rms_norm_eps"])
    q = (x[-1:] @ w[p + "self_attn.q_proj.weight"].T + w[p + "self_attn.q_proj.bias"]).view(1, n_q, d)
    k = (x @ w[p + "self_attn.k_proj.weight"].T + w[p + "self_attn.k_proj.bias"]).view(-1, n_kv, d)
    q_rot, _ = plain.apply_rotary(q, q, cos[-1:], sin[-1:])
    k_rot, _ = plain.apply_rotary(k, k, cos, sin)
    k_rot = k_rot.repeat_interleave(n_q // n_kv, dim=1)
    scores = torch.einsum("qhd,khd->hk", q_rot, k_rot) * d ** -0.5
    weight = torch.softmax(scores, dim=-1)
    far = weight[:, :len(tokens) - 1000].sum(-1)
    assert float(far.mean()) > 0.5
    assert float(weight.max(-1).values.mean()) > 0.02     # a flat row would be 1/4768 = 0.0002


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_request_whole_then_a_decoded_tail(long_case, dtype):
    from mercury_amd.hostcore import core
    from mercury_amd.kernels import ops

    name, folder, cfg, page, head, tokens, want, cost = long_case
    s = session(folder, dtype, len(tokens), page)
    if dtype == "bfloat16":
        # the kernel for long prompts is what this step launches
        plan = core.plan_attention(ops.BF16, cfg["head_dim"], page, cfg["num_attention_heads"],
                                   cfg["num_key_value_heads"], 0, [head], head, head)
        assert plan["mfma"] and plan["staged"] >= 8, plan
    rows = [s.step([entry("x", tokens[:head])], [])]
    check(rows[0], want[:head], dtype, f"{name} long, whole", **cost)
    for i in range(head, len(tokens)):
        rows.append(s.step([entry("x", tokens[i:i + 1])], ["x"] if i == len(tokens) - 1 else []))
    check(torch.cat(rows[1:]), want[head:], dtype, f"{name} long, decoded tail", **cost)
    if s.runner.use_graphs:
        # the tail went through a captured graph whose length bound covers the context
        assert any(bound >= len(tokens) for _, bound in s.runner.graphs), list(s.runner.graphs)
    assert s.manager.leaked_pages() == 0


@pytest.mark.parametrize("length,code", [(1280, 20), (3072, 24)])
def test_prompts_of_middle_lengths_through_the_other_attention_instantiations(length, code):
    """Between the short prompts of the small cases and the long ones above, the planner takes
    the 32-row attention kernel in two chains on tiles of 64 rows (1,280 tokens of 14 heads
    of 64) and in three chains on tiles of 128 (3,072): whole prompts of those lengths through
    the model, against the float64 run."""
    from mercury_amd.hostcore import core
    from mercury_amd.kernels import ops

    folder = folder_for("S64", sharpen=3.0)
    cfg = plain.read_config(folder)
    plan = core.plan_attention(ops.BF16, cfg["head_dim"], 16, cfg["num_attention_heads"],
                               cfg["num_key_value_heads"], 0, [length], length, length)
    assert plan["mfma"] and plan["staged"] == code, plan
    tokens = helpers.random_tokens(cfg["vocab_size"], length, seed=length)
    want, cost = exact_logits(folder, cfg, tokens)
    s = session(folder, "bfloat16", length, 16)
    got = s.step([entry("x", tokens)], ["x"])
    check(got, want, "bfloat16", f"S64, {length} tokens whole", **cost)
    assert s.manager.leaked_pages() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_request_in_portions_beside_a_decoding_neighbour(long_case, dtype):
    """The benchmark's serving shape: portions of 512 tokens of a long prompt beside another
    request's single decoded tokens."""
    name, folder, cfg, page, head, tokens, want, cost = long_case
    other = tokens[100:400]
    want_other, cost_other = exact_logits(folder, cfg, other)
    s = session(folder, dtype, len(tokens) + 320, page)
    s.step([{"id": "n", "tokens": other[:200], "want": []}], [])
    rows, near, done, at = [], [], 0, 200
    while done < head:
        part = tokens[done:min(done + 512, head)]
        entries = [entry("x", part)]
        if at < len(other):
            entries.append(entry("n", other[at:at + 1]))
        out = s.step(entries, [])
        rows.append(out[:len(part)])
        if at < len(other):
            near.append(out[len(part):])
            at += 1
        done += len(part)
    check(torch.cat(rows), want[:head], dtype, f"{name} long, portions of 512", **cost)
    check(torch.cat(near), want_other[200:at], dtype, f"{name} neighbour", **cost_other)
    s.step([], ["x", "n"])
    assert s.manager.leaked_pages() == 0
