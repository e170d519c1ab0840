"""Random-weights mode: draw every tensor a model declares from a seed, and write a model
folder (``config.json`` + ``model.safetensors``) that loads like any checkpoint.

The generator is the engine's own and counter-based: element i of a tensor is a function of
(seed, tensor name, i) alone, computed by the same float32 code on the host (the host core)
and on the GPU (the fill kernel), bit for bit, so that weights drawn on the device for a model
too large to write out are the very numbers a written folder would hold.  Matrices, biases
and embeddings are N(0, std); norm weights are 1 + N(0, std).  Values are computed in float32
and then rounded to the storage dtype.
"""

from __future__ import annotations

import hashlib
import json
from pathlib import Path

import torch

from .safetensors_io import save_file

_DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1}


def stream_key(seed: int, name: str) -> int:
    """The 64-bit key of a tensor's random stream."""
    digest = hashlib.blake2b(f"{seed}:{name}".encode(), digest_size=8).digest()
    return int.from_bytes(digest, "little")


def fill_normal(out: torch.Tensor, key: int, mean: float, std: float) -> torch.Tensor:
    """out[i] = mean + std * normal(key, i) over the flattened tensor, on the host or on the
    GPU, wherever `out` lives."""
    if out.dtype not in _DTYPE_CODE or not out.is_contiguous():
        raise ValueError("random fill takes contiguous float32 or bfloat16 tensors")
    code = _DTYPE_CODE[out.dtype]
    if out.is_cuda:
        from ..kernels import lib as _lib

        lib = _lib.load("core")
        with torch.cuda.device(out.device):
            _lib.check(lib, lib.mk_fill_normal(out.data_ptr(), code, out.numel(), key, float(mean),
                                               float(std), torch.cuda.current_stream().cuda_stream),
                       "fill_normal")
    else:
        from ..hostcore import core

        core.fill_normal(out.data_ptr(), code, out.numel(), key, float(mean), float(std))
    return out


def random_tensor(name: str, spec, seed: int, std: float, dtype: torch.dtype,
                  device="cpu") -> torch.Tensor:
    """One declared tensor, drawn where it is wanted."""
    if spec.role == "table":
        raise ValueError(f"{name}: integer tables have no random initialisation")
    if spec.init == "zeros":
        return torch.zeros(spec.shape, dtype=dtype, device=device)
    if spec.init not in ("normal", "one_plus_normal"):
        raise ValueError(f"{name}: unknown initialisation {spec.init!r}")
    out = torch.empty(spec.shape, dtype=dtype, device=device)
    return fill_normal(out, stream_key(seed, name), 1.0 if spec.init == "one_plus_normal" else 0.0, std)


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
