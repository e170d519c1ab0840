"""Feed-forward parts."""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import FeedForward, TensorSpec

ACTIVATIONS = ("silu",)


class GatedMLP(FeedForward):
    """down(act(gate(x)) * up(x)) without biases, act = SiLU
    (reference: mercury/model/qwen2.py:34-42).  Tensor names: ``gate_proj``, ``up_proj``,
    ``down_proj``."""

    graph_safe = True
    lowerable = True

    def __init__(self, hidden: int, intermediate: int, activation: str = "silu"):
        if activation not in ACTIVATIONS:
            raise ValueError(f"activation {activation!r} is not implemented; known: {ACTIVATIONS}")
        self.hidden, self.intermediate = int(hidden), int(intermediate)
        self.activation = activation
        self.w_gate_up = self.w_down = None

    def param_specs(self) -> dict:
        i, h = self.intermediate, self.hidden
        return {
            "gate_proj.weight": TensorSpec((i, h)),
            "up_proj.weight": TensorSpec((i, h)),
            "down_proj.weight": TensorSpec((h, i)),
        }

    def bind(self, params, dtype, device) -> None:
        # One projection for gate and up: rows [gate | up].
        self.w_gate_up = torch.cat(
            [params["gate_proj.weight"], params["up_proj.weight"]], dim=0
        ).contiguous()
        self.w_down = params["down_proj.weight"]

    def weight_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.w_gate_up, self.w_down))

    def lower(self, program) -> None:
        program.gated_mlp(self.w_gate_up.data_ptr(), self.w_down.data_ptr(), self.intermediate)

    def forward(self, x, step, accum):
        if ops.fuses_gating(x, self.w_gate_up):
            act = ops.gated_projection(x, self.w_gate_up)     # gated in the projection's epilogue
        else:
            act = ops.silu_mul(ops.linear(x, self.w_gate_up))
        if ops.wants_partials(act, self.w_down):
            return ops.linear_partials(act, self.w_down)      # the next norm adds them into accum
        ops.linear(act, self.w_down, out=accum, accumulate=True)
        return None
