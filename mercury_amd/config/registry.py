"""One registry from the architecture name in ``config.json`` to its model.

An architecture is a pair: a typed configuration class with ``from_dict(raw)`` that reads the
architecture's own keys, and a builder ``build(config) -> DecoderModel`` that puts the model
together from parts.  Adding an architecture is one ``register_architecture`` call; nothing
else in the engine names an architecture.
"""

from __future__ import annotations

from .model_config import ConfigError, read_config_json

_ARCHITECTURES: dict = {}


def register_architecture(name: str, config_cls):
    """Decorator: ``@register_architecture("FooForCausalLM", FooConfig)`` on the builder."""

    def decorate(builder):
        _ARCHITECTURES[name] = (config_cls, builder)
        return builder

    return decorate


def known_architectures() -> list:
    _load_builtin()
    return sorted(_ARCHITECTURES)


def _load_builtin() -> None:
    from .. import models  # noqa: F401  (registers the built-in architectures)


def architecture_of(raw: dict) -> str:
    names = raw.get("architectures")
    if not names:
        raise ConfigError("config.json has no 'architectures' entry naming the model class")
    return names[0]


def resolve(raw: dict):
    """(typed config, builder) for a parsed ``config.json``."""
    _load_builtin()
    name = architecture_of(raw)
    if name not in _ARCHITECTURES:
        raise ConfigError(
            f"architecture {name!r} is not registered; known: {sorted(_ARCHITECTURES)}"
        )
    config_cls, builder = _ARCHITECTURES[name]
    return config_cls.from_dict(raw), builder


def build_model(raw_or_folder):
    """The model described by a ``config.json`` dict or by the folder that holds one."""
    raw = raw_or_folder if isinstance(raw_or_folder, dict) else read_config_json(raw_or_folder)
    config, builder = resolve(raw)
    return builder(config)
