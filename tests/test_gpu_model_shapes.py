"""Layers of the sizes the benchmark runs (two of Qwen2.5-0.5B's, two with a head size of 128
and groups of 4, one each of Qwen2.5-7B's and 32B's), so that the kernels chosen for large shapes (tiled projections in every tile
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
    # one layer of the 7B sizes: the large-matrix choices (q/k/v as partial sums with a
    # finishing kernel, the 128 x 192 gated tile for few rows, K-split o and down projections)
    "7b": {"hidden_size": 3584, "intermediate_size": 18944, "num_attention_heads": 28,
           "num_key_value_heads": 4, "head_dim": 128, "vocab_size": 2003,
           "tie_word_embeddings": False, "num_hidden_layers": 1},
    "32b": {"hidden_size": 5120, "intermediate_size": 27648, "num_attention_heads": 40,
            "num_key_value_heads": 8, "head_dim": 128, "vocab_size": 2003,
            "tie_word_embeddings": False, "num_hidden_layers": 1},
}


_MODELS: dict = {}


def model(shape):
    """The shape's model folder, its two requests and the plain implementation's logits."""
    from mercury_amd.weights import write_random_model

    if shape not in _MODELS:
        cfg = {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
               "num_hidden_layers": 2, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6,
               "max_position_embeddings": 4096, **SHAPES[shape]}
        folder = Path(tempfile.mkdtemp(prefix=f"mercury_shape_{shape}_"))
        write_random_model(folder, cfg, seed=3, std=0.02, dtype=torch.bfloat16)
        weights, plain_cfg = helpers.plain_model(folder)
        reqs = {"long": helpers.random_tokens(cfg["vocab_size"], 700, seed=1),
                "other": helpers.random_tokens(cfg["vocab_size"], 90, seed=2)}
        want = {k: plain.forward_logits(weights, plain_cfg, v) for k, v in reqs.items()}
        cost = {k: replay.bf16_cost(folder, plain_cfg, v, want[k]) for k, v in reqs.items()}
        _MODELS[shape] = (folder, reqs, want, cost)
    return _MODELS[shape]


# The 7B and 32B layers are here for the matrix-core kernels' choices at large sizes, so in
# bfloat16 only: in float32 their sums over 18,944 terms and more differ from the plain implementation's by their
# order alone by more than the bound made for the short sums of the other shapes.
CASES = [(shape, dtype) for shape in sorted(SHAPES) for dtype in ("float32", "bfloat16")
         if (shape, dtype) not in (("7b", "float32"), ("32b", "float32"))]


@pytest.mark.parametrize("shape,dtype", CASES)
def test_a_long_prompt_whole_in_portions_and_decoded(shape, dtype):
    from mercury_amd.engine.replay import ReplaySession

    folder, reqs, want, cost = model(shape)
    s = ReplaySession(folder, dtype, 1024)
    long, other = reqs["long"], reqs["other"]
    replay.check(s.step([replay.entry("w", long)], ["w"]), want["long"], dtype, "whole",
                 cost["long"])

    # the prompt in three portions: the second beside the other request's prompt, the third of
    # 40 tokens by itself (few rows over the large matrices); then its last 40 tokens one at a
    # time beside the other request's decoded tokens
    rows = {"long": [], "other": []}
    rows["long"].append(s.step([replay.entry("long", long[:300])], []))
    out = s.step([replay.entry("long", long[300:620]), replay.entry("other", other[:50])], [])
    rows["long"].append(out[:320])
    rows["other"].append(out[320:])
    rows["long"].append(s.step([replay.entry("long", long[620:660])], []))
    for i in range(40):
        last = i == 39
        out = s.step([replay.entry("long", long[660 + i:661 + i]),
                      replay.entry("other", other[50 + i:51 + i])], ["long", "other"] if last else [])
        rows["long"].append(out[:1])
        rows["other"].append(out[1:])
    replay.check(torch.cat(rows["long"]), want["long"], dtype, "portions and decoded tail",
                 cost["long"])
    replay.check(torch.cat(rows["other"]), want["other"], dtype, "the request beside it",
                 cost["other"])
    assert s.manager.leaked_pages() == 0


@pytest.mark.parametrize("shape", ["7b"])
def test_batched_decoding_through_graphs_at_large_sizes(shape):
    """Eight requests decoded together through captured graphs (the gated tile for 8 rows, the
    q/k/v projection as partial sums inside a graph): every token is the plain
    implementation's choice at its place, or within the bfloat16 bound of it."""
    from mercury_amd import Engine, EngineConfig, SamplingParams
    from tests.test_gpu_generate import plausible

    folder, _reqs, _want, _cost = model(shape)
    vocab = SHAPES[shape]["vocab_size"]
    prompts = [helpers.random_tokens(vocab, 40 + 7 * i, seed=50 + i) for i in range(8)]
    engine = Engine(EngineConfig(model=str(folder), dtype="bfloat16", num_blocks=128,
                                 max_model_len=256))
    got = engine.generate(prompts, SamplingParams(ignore_eos=True), max_tokens=10)
    assert engine.leaked_blocks() == 0
    assert any(key[0] == 8 for key in engine.runner.runner.graphs)
    assert all(len(g) == 10 for g in got)
    assert all(plausible(folder, p, g) for p, g in zip(prompts, got))
