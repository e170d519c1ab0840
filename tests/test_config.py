"""Typed configuration and the architecture registry."""

from __future__ import annotations

import json

import pytest

from mercury_amd.config import (ConfigError, EngineConfig, Qwen2Config, blocks_for_capacity,
                                build_model, known_architectures, register_architecture, resolve)
from tests.helpers import TINY_A, TINY_B, TINY_C


def test_reads_the_architecture_s_own_keys_with_the_reference_defaults():
    """(reference: mercury/config.py:45-71)"""
    raw = {"architectures": ["Qwen2ForCausalLM"], "hidden_size": 896, "intermediate_size": 4864,
           "num_hidden_layers": 24, "num_attention_heads": 14, "vocab_size": 151936}
    cfg = Qwen2Config.from_dict(raw)
    assert cfg.num_key_value_heads == 14          # defaults to the number of heads
    assert cfg.head_dim == 64                     # hidden // heads
    assert cfg.rms_norm_eps == 1e-6 and cfg.rope_theta == 10000.0
    assert cfg.max_position_embeddings == 32768 and cfg.tie_word_embeddings is False
    assert cfg.eos_token_ids == ()
    assert Qwen2Config.from_dict({**raw, "eos_token_id": 7}).eos_token_ids == (7,)
    assert Qwen2Config.from_dict({**raw, "eos_token_id": [7, 9]}).eos_token_ids == (7, 9)
    assert Qwen2Config.from_dict({**raw, "head_dim": 128}).head_dim == 128
    # 12,288 bytes of cache per token for the 0.5B shapes in 16 bits (reference: README.md:67-68)
    assert Qwen2Config.from_dict({**raw, "num_key_value_heads": 2}).kv_bytes_per_token(2) == 12288


def test_round_trip_through_config_json():
    for raw in (TINY_A, TINY_B, TINY_C):
        cfg = Qwen2Config.from_dict(raw)
        assert Qwen2Config.from_dict(json.loads(json.dumps(cfg.to_dict()))) == cfg


@pytest.mark.parametrize("change,needle", [
    ({"use_sliding_window": True}, "sliding"),
    ({"rope_scaling": {"type": "yarn", "factor": 4}}, "rope_scaling"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"num_key_value_heads": 3}, "multiple"),
    ({"head_dim": 15}, "even"),
    ({"vocab_size": 0}, "positive"),
])
def test_refuses_what_it_does_not_implement(change, needle):
    with pytest.raises(ConfigError, match=needle):
        Qwen2Config.from_dict({**TINY_A, **change})


def test_missing_key_is_named():
    raw = dict(TINY_A)
    del raw["intermediate_size"]
    with pytest.raises(ConfigError, match="intermediate_size"):
        Qwen2Config.from_dict(raw)


def test_registry_maps_the_name_to_the_model():
    assert "Qwen2ForCausalLM" in known_architectures()
    cfg, builder = resolve(TINY_B)
    model = builder(cfg)
    assert len(model.layers) == 3 and model.vocab_size == 1000 and not model.tied_head
    assert build_model(TINY_A).tied_head
    with pytest.raises(ConfigError, match="not registered"):
        resolve({**TINY_A, "architectures": ["LlamaForCausalLM"]})
    with pytest.raises(ConfigError, match="architectures"):
        resolve({k: v for k, v in TINY_A.items() if k != "architectures"})


def test_another_architecture_is_one_registration():
    @register_architecture("TestOnlyTwoLayerLM", Qwen2Config)
    def build(cfg):
        from mercury_amd.models.qwen2 import build_qwen2

        return build_qwen2(cfg)

    assert build_model({**TINY_A, "architectures": ["TestOnlyTwoLayerLM"]}).hidden_size == 64


def test_model_declares_every_checkpoint_tensor_by_name():
    specs = build_model(TINY_B).param_specs()
    assert specs["model.layers.2.self_attn.k_proj.bias"].shape == (32,)
    assert specs["model.layers.0.self_attn.q_proj.weight"].shape == (256, 256)
    assert specs["model.layers.1.mlp.down_proj.weight"].shape == (256, 704)
    assert specs["lm_head.weight"].shape == (1000, 256)
    assert "model.layers.0.self_attn.o_proj.bias" not in specs     # o has no bias
    assert "lm_head.weight" not in build_model(TINY_A).param_specs()  # tied
    assert len(specs) == 1 + 3 * 12 + 1 + 1


def test_engine_config_validation():
    """(reference: mercury/config.py:115-151)"""
    with pytest.raises(ValueError, match="policy"):
        EngineConfig(policy="sjf")
    with pytest.raises(ValueError, match="dtype"):
        EngineConfig(dtype="float16")
    with pytest.raises(ValueError, match="power of two"):
        EngineConfig(block_size=24)
    cfg = EngineConfig(num_blocks=4, block_size=16, max_model_len=128)
    with pytest.raises(ValueError, match="preempt itself"):
        cfg.validate_against(32768)
    with pytest.raises(ValueError, match="position embeddings"):
        EngineConfig(max_model_len=4096, num_blocks=512).validate_against(2048)
    assert EngineConfig(num_blocks=10).kv_capacity_tokens == 160
    assert blocks_for_capacity(33, 16) == 3 and blocks_for_capacity(0, 16) == 1
