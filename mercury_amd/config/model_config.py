"""Typed model configurations, read from an architecture's own ``config.json`` keys.

One dataclass per architecture; the registry in :mod:`mercury_amd.config.registry` maps the
``architectures[0]`` string of ``config.json`` to the dataclass and to the function that turns
it into a model description.  No size or constant that ``config.json`` gives is repeated in
code; the only defaults are the ones the reference applies when a key is absent
(reference: mercury/config.py:45-71).
"""

from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path


class ConfigError(ValueError):
    """config.json names something this engine does not implement, or lacks a key."""


def read_config_json(folder) -> dict:
    """The parsed ``config.json`` of a model folder (or the file itself, when given that)."""
    path = Path(folder)
    if path.is_dir() or path.name != "config.json":
        path = path / "config.json"
    if not path.is_file():
        raise FileNotFoundError(f"no config.json under {folder}")
    return json.loads(path.read_text())


def _require(raw: dict, key: str):
    if key not in raw:
        raise ConfigError(f"config.json has no {key!r}")
    return raw[key]


@dataclass(frozen=True)
class Qwen2Config:
    """The Qwen2 dense decoder (reference: mercury/config.py:22-71, mercury/model/qwen2.py).

    Keys and defaults follow the reference: ``num_key_value_heads`` defaults to the number of
    heads, ``head_dim`` to ``hidden_size // num_attention_heads``, ``rms_norm_eps`` to 1e-6,
    ``rope_theta`` to 10000, ``max_position_embeddings`` to 32768, ``tie_word_embeddings`` to
    false; ``eos_token_id`` may be an integer or a list.

    The reference never reads the sliding-window keys or ``rope_scaling`` or ``hidden_act``:
    its attention is always full and causal, its rotation unscaled and its activation SiLU
    (mercury/model/qwen2.py:42, mercury/model/attention.py:77-101).  A config that asks for
    anything else is refused here instead of being run with the wrong arithmetic.
    """

    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    vocab_size: int
    rms_norm_eps: float
    rope_theta: float
    max_position_embeddings: int
    tie_word_embeddings: bool
    eos_token_ids: tuple = ()
    bos_token_id: int | None = None
    architecture: str = "Qwen2ForCausalLM"

    @classmethod
    def from_dict(cls, raw: dict) -> "Qwen2Config":
        arch = (raw.get("architectures") or ["Qwen2ForCausalLM"])[0]
        heads = int(_require(raw, "num_attention_heads"))
        hidden = int(_require(raw, "hidden_size"))
        eos = raw.get("eos_token_id", [])
        if eos is None:
            eos = []
        if isinstance(eos, int):
            eos = [eos]
        if raw.get("use_sliding_window", False):
            raise ConfigError(
                "config.json sets use_sliding_window; this architecture's attention is full "
                "and causal in every layer, a windowed variant is not defined for it here"
            )
        if raw.get("rope_scaling") not in (None, {}):
            raise ConfigError(
                f"config.json sets rope_scaling={raw['rope_scaling']!r}; only unscaled rotary "
                "positions are implemented for this architecture"
            )
        if raw.get("hidden_act", "silu") != "silu":
            raise ConfigError(
                f"config.json sets hidden_act={raw['hidden_act']!r}; this architecture's "
                "feed-forward is SiLU-gated"
            )
        cfg = cls(
            hidden_size=hidden,
            intermediate_size=int(_require(raw, "intermediate_size")),
            num_hidden_layers=int(_require(raw, "num_hidden_layers")),
            num_attention_heads=heads,
            num_key_value_heads=int(raw.get("num_key_value_heads", heads)),
            head_dim=int(raw.get("head_dim") or hidden // heads),
            vocab_size=int(_require(raw, "vocab_size")),
            rms_norm_eps=float(raw.get("rms_norm_eps", 1e-6)),
            rope_theta=float(raw.get("rope_theta", 10000.0)),
            max_position_embeddings=int(raw.get("max_position_embeddings", 32768)),
            tie_word_embeddings=bool(raw.get("tie_word_embeddings", False)),
            eos_token_ids=tuple(int(t) for t in eos),
            bos_token_id=raw.get("bos_token_id"),
            architecture=arch,
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        for name in (
            "hidden_size",
            "intermediate_size",
            "num_hidden_layers",
            "num_attention_heads",
            "num_key_value_heads",
            "head_dim",
            "vocab_size",
            "max_position_embeddings",
        ):
            if getattr(self, name) <= 0:
                raise ConfigError(f"{name} must be positive, got {getattr(self, name)}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"num_attention_heads ({self.num_attention_heads}) is not a multiple of "
                f"num_key_value_heads ({self.num_key_value_heads})"
            )
        if self.head_dim % 2:
            raise ConfigError(f"head_dim ({self.head_dim}) must be even for rotary positions")
        if not self.rms_norm_eps > 0:
            raise ConfigError("rms_norm_eps must be positive")

    def to_dict(self) -> dict:
        """The ``config.json`` that reads back to this configuration."""
        out = {
            "architectures": [self.architecture],
            "model_type": "qwen2",
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "vocab_size": self.vocab_size,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "max_position_embeddings": self.max_position_embeddings,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": "silu",
            "use_sliding_window": False,
        }
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        if self.bos_token_id is not None:
            out["bos_token_id"] = self.bos_token_id
        return out

    def kv_bytes_per_token(self, elem_bytes: int = 2) -> int:
        """Bytes of keys and values one token occupies over all layers
        (reference: mercury/config.py:73-81)."""
        return (
            2 * self.num_hidden_layers * self.num_key_value_heads * self.head_dim * elem_bytes
        )
