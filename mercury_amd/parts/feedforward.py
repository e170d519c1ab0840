"""Feed-forward parts."""

from __future__ import annotations

import torch

from ..hostcore import core
from .base import FeedForward, TensorSpec
from .lowering import OneOp

ACTIVATIONS = ("silu",)
DEFAULT_NAMES = {"gate": "gate_proj", "up": "up_proj", "down": "down_proj"}


class GatedMLP(FeedForward):
    """down(act(gate(x)) * up(x)) without biases, act = SiLU
    (reference: mercury/model/qwen2.py:34-42).  `names` maps gate, up, down to the stored
    tensors' leaf names (default ``gate_proj``, ``up_proj``, ``down_proj``)."""

    graph_safe = True
    lowerable = True

    def __init__(self, hidden: int, intermediate: int, activation: str = "silu",
                 names: dict | None = None):
        if activation not in ACTIVATIONS:
            raise ValueError(f"activation {activation!r} is not implemented; known: {ACTIVATIONS}")
        self.hidden, self.intermediate = int(hidden), int(intermediate)
        self.activation = activation
        self.names = {**DEFAULT_NAMES, **(names or {})}
        self.w_gate_up = self.w_down = None
        self._alone = None

    def param_specs(self) -> dict:
        i, h, n = self.intermediate, self.hidden, self.names
        return {
            f"{n['gate']}.weight": TensorSpec((i, h)),
            f"{n['up']}.weight": TensorSpec((i, h)),
            f"{n['down']}.weight": TensorSpec((h, i)),
        }

    def bind(self, params, dtype, device) -> None:
        n = self.names
        # One projection for gate and up: rows [gate | up].
        self.w_gate_up = torch.cat(
            [params[f"{n['gate']}.weight"], params[f"{n['up']}.weight"]], dim=0
        ).contiguous()
        self.w_down = params[f"{n['down']}.weight"]
        self._alone = None

    def weight_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.w_gate_up, self.w_down))

    def lower(self, program) -> None:
        if self.activation != "silu":
            raise ValueError(f"the gated projection's kernels compute silu, not {self.activation}")
        program.append("gated_mlp", core.gated_mlp_params(
            self.w_gate_up.data_ptr(), self.w_down.data_ptr(), self.intermediate))

    def forward(self, x, step, accum):
        # the operations `lower` appends, as a program of their own
        if self._alone is None:
            self._alone = OneOp(x.dtype, self.hidden, 0, self.lower)
        _logits, _x, pending = self._alone.run(step, accum, x=x)
        return pending
