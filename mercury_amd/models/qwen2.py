"""The Qwen2 dense decoder, put together from parts.

Every layer: RMSNorm -> attention with biased q/k/v, unbiased o, rotary positions over the
whole head, full causal softmax -> RMSNorm -> SiLU-gated MLP; a final RMSNorm; an output head
that is the embedding matrix when ``tie_word_embeddings`` is set
(reference: mercury/model/qwen2.py:45-150).  Tensor names are the checkpoint's own
(``model.layers.{i}.self_attn.q_proj.weight`` ...).
"""

from __future__ import annotations

from ..config.model_config import Qwen2Config
from ..config.registry import register_architecture
from ..parts import Attention, DecoderModel, GatedMLP, PreNormBlock, RMSNorm, RotaryPosition

PART_NAMES = {
    "mixer": "self_attn.",
    "ffn": "mlp.",
    "norm_mixer": "input_layernorm.",
    "norm_ffn": "post_attention_layernorm.",
}


@register_architecture("Qwen2ForCausalLM", Qwen2Config)
def build_qwen2(cfg: Qwen2Config) -> DecoderModel:
    layers = []
    rotary = RotaryPosition(cfg.head_dim, cfg.rope_theta)  # one angle table for all layers
    for _ in range(cfg.num_hidden_layers):
        mixer = Attention(
            hidden=cfg.hidden_size,
            n_q=cfg.num_attention_heads,
            n_kv=cfg.num_key_value_heads,
            head_dim=cfg.head_dim,
            position=rotary,
            qkv_bias=True,   # fixed by the architecture (reference: mercury/model/qwen2.py:57-60)
            o_bias=False,
            window=None,
        )
        ffn = GatedMLP(cfg.hidden_size, cfg.intermediate_size, activation="silu")
        layers.append(PreNormBlock(
            mixer, ffn,
            RMSNorm(cfg.hidden_size, cfg.rms_norm_eps),
            RMSNorm(cfg.hidden_size, cfg.rms_norm_eps),
            PART_NAMES,
        ))
    return DecoderModel(
        vocab_size=cfg.vocab_size,
        hidden_size=cfg.hidden_size,
        layers=layers,
        final_norm=RMSNorm(cfg.hidden_size, cfg.rms_norm_eps),
        tied_head=cfg.tie_word_embeddings,
        max_positions=cfg.max_position_embeddings,
        eos_token_ids=cfg.eos_token_ids,
        config=cfg,
    )
