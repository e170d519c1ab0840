"""Configurations drawn at random (head sizes in steps of 16, any heads and groups, widths,
intermediate sizes and vocabularies that are no multiple of anything) through replay, whole,
with a decoded tail, and mixed in a pool whose pages are used again, against the plain
implementation.  Widths that are no multiple of 8 take the float32-arithmetic kernels also in
bfloat16; head sizes the matrix-core attention does not cover likewise.  Every second seed
draws a width that is a multiple of 8 and a head size among those the matrix-core kernels
take, so that both families of kernels meet random shapes; the page size is drawn too."""

from __future__ import annotations

import random
import tempfile
from pathlib import Path

import pytest
import torch

from tests import helpers
from tests import test_gpu_replay as replay
from tests.plain import qwen2_plain as plain

pytestmark = pytest.mark.gpu


def random_config(rng: random.Random, matrix_cores: bool) -> dict:
    n_kv = rng.choice([1, 2, 3, 4])
    group = rng.choice([1, 2, 3, 4, 7])
    head_dims = [64, 96, 128] if matrix_cores else [16, 32, 48, 64, 80, 96, 112, 128]
    return {
        "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
        "head_dim": rng.choice(head_dims),
        "hidden_size": max(16, (8 if matrix_cores else rng.choice([8, 2, 1])) * rng.randint(8, 48)),
        "intermediate_size": rng.choice([8, 2]) * rng.randint(8, 90),
        "num_hidden_layers": rng.randint(1, 3),
        "num_attention_heads": n_kv * group, "num_key_value_heads": n_kv,
        "vocab_size": rng.randint(100, 3000), "rope_theta": rng.choice([1e4, 5e4, 1e6]),
        "rms_norm_eps": rng.choice([1e-6, 1e-5, 3e-6]),
        "tie_word_embeddings": rng.random() < 0.5, "max_position_embeddings": 1024,
    }


@pytest.mark.parametrize("seed", range(8))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_random_configuration(seed, dtype):
    from mercury_amd.engine.replay import ReplaySession
    from mercury_amd.weights import write_random_model

    rng = random.Random(seed)
    cfg = random_config(rng, matrix_cores=seed % 2 == 1)
    page = rng.choice([16, 32, 64] if seed % 2 else [8, 16, 32])
    folder = Path(tempfile.mkdtemp(prefix="mercury_random_"))
    write_random_model(folder, cfg, seed=seed, std=0.05, dtype=torch.bfloat16)
    weights, plain_cfg = helpers.plain_model(folder)
    lengths = {"a": rng.randint(100, 260), "b": rng.randint(2, 120), "c": rng.randint(60, 200),
               "d": rng.randint(2, 64), "e": 64, "f": 33}
    reqs = {k: helpers.random_tokens(cfg["vocab_size"], n, seed=ord(k) + seed)
            for k, n in lengths.items()}
    want = {k: plain.forward_logits(weights, plain_cfg, v) for k, v in reqs.items()}
    cost = {k: replay.bf16_cost(folder, plain_cfg, v, want[k]) for k, v in reqs.items()}
    what = f"{cfg}, pages of {page}: "
    session = lambda pool: ReplaySession(folder, dtype, pool, page_size=page)

    s = session(320)
    for key, tokens in reqs.items():
        replay.check(s.step([replay.entry(key, tokens)], [key]), want[key], dtype,
                     what + f"whole {key}", cost[key])
    tokens = reqs["a"]
    head = len(tokens) - 32
    rows = [s.step([replay.entry("a", tokens[:head])], [])]
    for i in range(head, len(tokens)):
        rows.append(s.step([replay.entry("a", tokens[i:i + 1])], ["a"] if i == len(tokens) - 1 else []))
    replay.check(torch.cat(rows), want["a"], dtype, what + "decoded tail", cost["a"])
    assert s.manager.leaked_pages() == 0

    reqs = dict(reqs, a2=reqs["a"], c2=reqs["c"])
    want = dict(want, a2=want["a"], c2=want["c"])
    pool = max(sum(replay.held(len(reqs[k])) for k in "abdc") - 64,
               max(replay.held(len(v)) for v in reqs.values()))
    s = session(pool)
    got = replay.mixed_run(lambda entries, ends: s.step(entries, ends), reqs, pool)
    for key in got:
        replay.check(got[key], want[key], dtype, what + f"mixed {key}", cost[key[0]])
    assert s.manager.leaked_pages() == 0
