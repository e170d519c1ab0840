"""Two layers of the sizes the benchmark runs (Qwen2.5-0.5B's, and a head size of 128 with
groups of 4), so that the kernels chosen for large shapes (tiled projections in every tile
configuration that a long prompt picks, prompt attention with its key groups, the fused
q/k/v projection, K-split projections, split-key decode attention, decode graphs) are
compared with the plain implementation end to end: a long prompt whole, the same prompt in
two portions beside decoded tokens of another request, and a decoded tail."""

from __future__ import annotations

import tempfile
from pathlib import Path

import pytest
import torch

from tests import helpers
from tests import test_gpu_replay as replay
from tests.plain import qwen2_plain as plain

pytestmark = pytest.mark.gpu

SHAPES = {
    "0.5b": {"hidden_size": 896, "intermediate_size": 4864, "num_attention_heads": 14,
             "num_key_value_heads": 2, "head_dim": 64, "vocab_size": 5003,
             "tie_word_embeddings": True},
    "d128": {"hidden_size": 1024, "intermediate_size": 2816, "num_attention_heads": 8,
             "num_key_value_heads": 2, "head_dim": 128, "vocab_size": 3001,
             "tie_word_embeddings": False},
}


@pytest.fixture(scope="module", params=sorted(SHAPES))
def model(request):
    from mercury_amd.weights import write_random_model

    cfg = dict({"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
                "num_hidden_layers": 2, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6,
                "max_position_embeddings": 4096}, **SHAPES[request.param])
    folder = Path(tempfile.mkdtemp(prefix=f"mercury_shape_{request.param}_"))
    write_random_model(folder, cfg, seed=3, std=0.02, dtype=torch.bfloat16)
    weights, plain_cfg = helpers.plain_model(folder)
    reqs = {"long": helpers.random_tokens(cfg["vocab_size"], 700, seed=1),
            "other": helpers.random_tokens(cfg["vocab_size"], 90, seed=2)}
    want = {k: plain.forward_logits(weights, plain_cfg, v) for k, v in reqs.items()}
    return folder, reqs, want


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_prompt_whole_in_portions_and_decoded(model, dtype):
    folder, reqs, want = model
    s = replay.session(folder, dtype, 1024)
    long, other = reqs["long"], reqs["other"]
    replay.check(s.step([replay.entry("w", long)], ["w"]), want["long"], dtype, "whole")

    # the prompt in two portions; the second beside the other request's prompt, then its last
    # 40 tokens one at a time beside the other request's decoded tokens
    rows = {"long": [], "other": []}
    rows["long"].append(s.step([replay.entry("long", long[:300])], []))
    out = s.step([replay.entry("long", long[300:660]), replay.entry("other", other[:50])], [])
    rows["long"].append(out[:360])
    rows["other"].append(out[360:])
    for i in range(40):
        last = i == 39
        out = s.step([replay.entry("long", long[660 + i:661 + i]),
                      replay.entry("other", other[50 + i:51 + i])], ["long", "other"] if last else [])
        rows["long"].append(out[:1])
        rows["other"].append(out[1:])
    replay.check(torch.cat(rows["long"]), want["long"], dtype, "portions and decoded tail")
    replay.check(torch.cat(rows["other"]), want["other"], dtype, "the request beside it")
    assert s.manager.leaked_pages() == 0
