"""Registries of part kinds, so that an architecture can be written as data.

``register_mixer("attention")(Attention)`` makes ``build_part("mixer", "attention", **params)``
work.  Code outside this package (a test, an experiment) can register further kinds without
touching the package's files.
"""

from __future__ import annotations

_KINDS = {"mixer": {}, "ffn": {}, "norm": {}, "position": {}, "block": {}}


def _register(family: str, name: str):
    def decorate(cls):
        _KINDS[family][name] = cls
        return cls

    return decorate


def register_mixer(name):
    return _register("mixer", name)


def register_ffn(name):
    return _register("ffn", name)


def register_norm(name):
    return _register("norm", name)


def register_position(name):
    return _register("position", name)


def register_block(name):
    return _register("block", name)


def build_part(family: str, name: str, **params):
    try:
        cls = _KINDS[family][name]
    except KeyError:
        raise KeyError(
            f"no {family} of kind {name!r} is registered; known: {sorted(_KINDS.get(family, {}))}"
        ) from None
    return cls(**params)


def known(family: str) -> list:
    return sorted(_KINDS[family])
