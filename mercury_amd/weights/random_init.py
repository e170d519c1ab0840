"""Random-weights mode: draw every tensor a model declares from a seed, and write a model
folder (``config.json`` + ``model.safetensors``) that loads like any checkpoint.

Each tensor has its own generator, seeded from (seed, tensor name), so the values do not
depend on the order in which tensors are drawn.  Matrices, biases and embeddings are
N(0, std); norm weights are 1 + N(0, std).  Values are drawn in float32 and then rounded to
the storage dtype.
"""

from __future__ import annotations

import hashlib
import json
from pathlib import Path

import torch

from .safetensors_io import save_file


def _generator(seed: int, name: str, device="cpu") -> torch.Generator:
    digest = hashlib.blake2b(f"{seed}:{name}".encode(), digest_size=8).digest()
    g = torch.Generator(device=device)
    g.manual_seed(int.from_bytes(digest, "little") & (2**63 - 1))
    return g


def random_tensor(name: str, spec, seed: int, std: float, dtype: torch.dtype,
                  device="cpu") -> torch.Tensor:
    """One declared tensor.  Drawn on `device`: the values for a seed are fixed per kind of
    device (the CPU's are the ones a written model folder holds)."""
    if spec.role == "table":
        raise ValueError(f"{name}: integer tables have no random initialisation")
    if spec.init == "zeros":
        return torch.zeros(spec.shape, dtype=dtype, device=device)
    t = torch.randn(spec.shape, generator=_generator(seed, name, device), dtype=torch.float32,
                    device=device) * std
    if spec.init == "one_plus_normal":
        t += 1.0
    elif spec.init != "normal":
        raise ValueError(f"{name}: unknown initialisation {spec.init!r}")
    return t.to(dtype)


def random_state(model, seed: int, std: float = 0.02, dtype: torch.dtype = torch.bfloat16) -> dict:
    """name -> CPU tensor for every tensor the model declares."""
    return {name: random_tensor(name, spec, seed, std, dtype)
            for name, spec in model.param_specs().items()}


class RandomSource:
    """A weight source that draws each tensor when it is asked for, on `device`: random weights
    for models too large to hold twice (once on the host, once on the card)."""

    def __init__(self, model, seed: int, std: float = 0.02, dtype: torch.dtype = torch.bfloat16,
                 device="cpu"):
        self.specs = model.param_specs()
        self.seed, self.std, self.dtype, self.device = seed, std, dtype, device

    def names(self):
        return list(self.specs)

    def shape(self, name):
        return tuple(self.specs[name].shape)

    def tensor(self, name):
        return random_tensor(name, self.specs[name], self.seed, self.std, self.dtype, self.device)

    def close(self):
        pass


def write_random_model(folder, config: dict, seed: int, std: float = 0.02,
                       dtype: torch.dtype = torch.bfloat16) -> Path:
    """Write ``config.json`` (the dict as given) and ``model.safetensors`` with random weights
    for the architecture the dict names.  Returns the folder."""
    from ..config.registry import build_model

    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    model = build_model(config)
    (folder / "config.json").write_text(json.dumps(config, indent=2) + "\n")
    save_file(random_state(model, seed, std, dtype), folder / "model.safetensors",
              metadata={"format": "pt", "seed": seed, "std": std})
    return folder
