"""Random requests through the whole engine under random options, in float32, against the
plain implementation's greedy tokens: shared prefixes, prompts cut into portions under small
token budgets, pools so small that requests are preempted, decode graphs and steps started
ahead; every request twice, the second time over a warm prefix cache."""

from __future__ import annotations

import random

import pytest
import torch

from tests import helpers
from tests.plain import qwen2_plain as plain

pytestmark = pytest.mark.gpu


def random_config(rng):
    n_kv, group = rng.choice([1, 2]), rng.choice([1, 2, 4])
    return {
        "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
        "hidden_size": rng.choice([64, 96, 128]), "intermediate_size": rng.choice([176, 256]),
        "num_hidden_layers": rng.randint(1, 2), "num_attention_heads": n_kv * group,
        "num_key_value_heads": n_kv, "head_dim": rng.choice([16, 32, 64]),
        "vocab_size": rng.randint(100, 600), "rope_theta": 1e4, "rms_norm_eps": 1e-6,
        "tie_word_embeddings": rng.random() < 0.5, "max_position_embeddings": 1024,
    }


# in the second row's seeds the pool is so small that requests are preempted (6, 8, 18, 6 times ...)
PREEMPTING = [106, 111, 124, 137, 141, 145, 159, 171]


@pytest.mark.parametrize("seed", [101, 102, 103, 109, 113, 120, 131, 140] + PREEMPTING)
def test_random_requests_under_random_options(seed, tmp_path):
    from mercury_amd import Engine, EngineConfig, SamplingParams
    from mercury_amd.weights import write_random_model

    rng = random.Random(seed)
    cfg = random_config(rng)
    folder = write_random_model(tmp_path / "model", cfg, seed=seed, std=0.08, dtype=torch.bfloat16)
    w, pcfg = helpers.plain_model(folder)
    vocab = cfg["vocab_size"]
    base = helpers.random_tokens(vocab, 96, seed=seed)
    prompts, max_tokens = [], []
    for i in range(rng.randint(3, 9)):
        if rng.random() < 0.5:   # shares a prefix with others
            share = rng.choice([8, 16, 24, 40, 64, 96])
            p = base[:share] + helpers.random_tokens(vocab, rng.randint(0, 30), seed=seed * 100 + i)
        else:
            p = helpers.random_tokens(vocab, rng.randint(1, 120), seed=seed * 100 + i)
        prompts.append(p)
        max_tokens.append(rng.randint(1, 24))
    page = rng.choice([8, 16, 32])
    need = -(-max(len(p) + m for p, m in zip(prompts, max_tokens)) // page) + 1
    options = dict(block_size=page, num_blocks=rng.choice([need, need + 3, 2 * need, 64]),
                   max_running=rng.choice([1, 2, 3, 8]),
                   prefill_budget=rng.choice([8, 16, 33, 64, 8192]),
                   policy=rng.choice(["fcfs", "lpm", "lpm_aging"]), max_model_len=need * page,
                   lookahead=rng.random() < 0.7, debug_invariants=True)
    want = [plain.greedy_generate(w, pcfg, p, m) for p, m in zip(prompts, max_tokens)]
    engine = Engine(EngineConfig(model=str(folder), dtype="float32", **options))
    for turn in range(2):
        events = {i: [] for i in range(len(prompts))}
        for i, (p, m) in enumerate(zip(prompts, max_tokens)):
            engine.submit(f"{turn}-{i}", p, m, events[i].append,
                          params=SamplingParams(ignore_eos=True))
        engine._take_commands()
        steps = 0
        while engine.sched.has_work():
            engine.step()
            steps += 1
            assert steps < 5000, f"the engine does not finish under {options}"
        got = [[e.token for e in events[i] if e.kind == "token"] for i in range(len(prompts))]
        assert got == want, f"turn {turn} under {options}"
        assert all(events[i][-1].kind == "done" for i in events)
        assert engine.leaked_blocks() == 0
    assert (engine.sched.stats["preemptions"] > 0) == (seed in PREEMPTING)
