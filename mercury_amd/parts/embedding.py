"""Where a step starts and where it ends: token embedding and output head."""

from __future__ import annotations

import torch

from ..hostcore import core
from ..kernels import ops
from .base import Part, TensorSpec


class TokenEmbedding(Part):
    """h[t] = table[id[t]] * scale, as the float32 residual stream
    (reference: mercury/model/qwen2.py:100, :107-108; the reference has no scale)."""

    graph_safe = True
    lowerable = True

    def __init__(self, vocab_size: int, hidden_size: int, scale: float = 1.0):
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.scale = float(scale)
        self.weight = None

    def param_specs(self) -> dict:
        return {"weight": TensorSpec((self.vocab_size, self.hidden_size))}

    def bind(self, params, dtype, device) -> None:
        self.weight = params["weight"]

    def lower(self, program) -> None:
        program.append("embed", core.embed_params(
            self.weight.data_ptr(), ops.dtype_code(self.weight.dtype), self.vocab_size, self.scale))

    def forward(self, step, out: torch.Tensor | None = None) -> torch.Tensor:
        return ops.embed(step.token_ids, self.weight, out=out, scale=self.scale)


class OutputHead(Part):
    """logits = x W^T (+ bias), optionally bounded to cap * tanh(logits / cap); float32.

    W is the part's own tensor, or, when the model ties its head, the embedding matrix, which
    the model hands over in `bind` (reference: mercury/model/qwen2.py:128-130, :145-150; the
    reference has neither bias nor cap)."""

    graph_safe = True
    lowerable = True

    def __init__(self, vocab_size: int, hidden_size: int, tied: bool = False, bias: bool = False,
                 cap: float | None = None):
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.tied, self.has_bias = bool(tied), bool(bias)
        self.cap = float(cap) if cap else 0.0
        self.weight = self.bias = None

    def param_specs(self) -> dict:
        specs = {}
        if not self.tied:
            specs["weight"] = TensorSpec((self.vocab_size, self.hidden_size))
        if self.has_bias:
            specs["bias"] = TensorSpec((self.vocab_size,), role="vector")
        return specs

    def bind(self, params, dtype, device) -> None:
        """`params["weight"]` is the embedding matrix when the head is tied."""
        self.weight = params["weight"]
        self.bias = params.get("bias")

    def weight_bytes(self) -> int:
        total = self.weight.numel() * self.weight.element_size()
        if self.bias is not None:
            total += self.bias.numel() * self.bias.element_size()
        return total

    def lower(self, program) -> None:
        bias = self.bias
        program.append("head", core.head_params(
            self.weight.data_ptr(), 0 if bias is None else bias.data_ptr(),
            ops.F32 if bias is None else ops.dtype_code(bias.dtype), self.cap))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        logits = ops.linear(x, self.weight, self.bias, out_dtype=torch.float32)
        if self.cap:
            ops.logit_cap(logits, self.cap)
        return logits
