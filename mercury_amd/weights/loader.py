"""Fill a model's parts from tensors looked up by name.

The model declares what it needs (``param_specs()``: name -> shape, role); the source offers
what a checkpoint holds.  Every disagreement is collected first and reported in one error:
tensors the model needs and the checkpoint lacks, tensors the checkpoint holds and the model
has no home for, and tensors of the wrong shape (the reference raises three separate errors
for these, mercury/model/loader.py:77-91).

Dtypes: projection matrices and the embedding go to the compute dtype (the reference casts
every tensor to the model dtype, mercury/model/loader.py:82).  Vectors (norm weights,
biases) stored in 32 bits stay float32 under bfloat16 compute; integer tables become int32.
"""

from __future__ import annotations

from pathlib import Path

import torch

from .safetensors_io import SafetensorsFile, weight_files


class WeightLoadError(RuntimeError):
    """The checkpoint does not fit the model; `.missing`, `.unexpected`, `.mismatched`."""

    def __init__(self, missing, unexpected, mismatched):
        self.missing, self.unexpected, self.mismatched = missing, unexpected, mismatched
        lines = ["checkpoint does not match the model:"]
        if missing:
            lines.append(f"  missing ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected ({len(unexpected)}): " + ", ".join(unexpected))
        if mismatched:
            lines.append(f"  wrong shape ({len(mismatched)}): " + ", ".join(
                f"{n}: checkpoint has {tuple(got)}, model expects {tuple(want)}"
                for n, got, want in mismatched))
        super().__init__("\n".join(lines))


class FolderSource:
    """The tensors of a model folder's safetensors files."""

    def __init__(self, folder):
        self.files = [SafetensorsFile(p) for p in weight_files(Path(folder))]
        self.where = {}
        for f in self.files:
            for name in f.names():
                self.where[name] = f

    def names(self):
        return list(self.where)

    def shape(self, name):
        return self.where[name].shape(name)

    def tensor(self, name):
        return self.where[name].tensor(name)

    def close(self):
        for f in self.files:
            f.close()


class DictSource:
    """Tensors already in memory (name -> tensor), e.g. freshly drawn random weights."""

    def __init__(self, tensors: dict):
        self.tensors = tensors

    def names(self):
        return list(self.tensors)

    def shape(self, name):
        return tuple(self.tensors[name].shape)

    def tensor(self, name):
        return self.tensors[name]

    def close(self):
        pass


def target_dtype(role: str, stored: torch.dtype, compute: torch.dtype) -> torch.dtype:
    if role == "table":
        return torch.int32
    if compute == torch.float32:
        return torch.float32
    if role == "vector" and stored in (torch.float32, torch.float64):
        return torch.float32
    return compute


def check_source(model, source) -> None:
    specs = model.param_specs()
    ignored = model.ignored_names()
    offered = set(source.names())
    missing = sorted(n for n, s in specs.items() if n not in offered and not s.optional)
    unexpected = sorted(n for n in offered if n not in specs and n not in ignored)
    mismatched = sorted(
        (n, source.shape(n), s.shape) for n, s in specs.items()
        if n in offered and tuple(source.shape(n)) != tuple(s.shape))
    if missing or unexpected or mismatched:
        raise WeightLoadError(missing, unexpected, mismatched)


def load_weights(model, source, dtype: torch.dtype, device) -> None:
    """Check `source` against the model, move the tensors to `device` and bind the parts."""
    check_source(model, source)
    specs = model.param_specs()
    offered = set(source.names())
    params = {}
    for name, spec in specs.items():
        if name not in offered:
            continue
        stored = source.tensor(name)
        want = target_dtype(spec.role, stored.dtype, dtype)
        params[name] = stored.to(device=device, dtype=want, copy=True).contiguous()
    model.bind(params, dtype, device)


def load_model_folder(folder, dtype: torch.dtype, device):
    """Build the model that ``config.json`` names and load its weights."""
    from ..config.registry import build_model

    model = build_model(folder)
    source = FolderSource(folder)
    try:
        load_weights(model, source, dtype, device)
    finally:
        source.close()
    return model
