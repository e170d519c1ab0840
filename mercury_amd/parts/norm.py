"""Root-mean-square normalisation over the residual stream."""

from __future__ import annotations

from ..hostcore import core
from ..kernels import ops
from .base import Norm, TensorSpec


class RMSNorm(Norm):
    """y = (x * rsqrt(mean(x^2) + eps)) * weight, statistics in float32.

    `eps` is added to the mean of squares, inside the root; the normalised value is rounded
    to the output dtype before the weight multiplies it
    (reference: mercury/model/qwen2.py:27-31).  The residual sum the reference folds into the
    norm (`x + residual`, mercury/model/qwen2.py:27-28) arrives here as `partials`: partial
    sums of the preceding projection that are added into the float32 stream in the same pass.
    """

    graph_safe = True
    lowerable = True

    def __init__(self, size: int, eps: float):
        self.size = int(size)
        self.eps = float(eps)
        self.weight = None

    def param_specs(self) -> dict:
        return {"weight": TensorSpec((self.size,), role="vector", init="one_plus_normal")}

    def bind(self, params, dtype, device) -> None:
        self.weight = params["weight"]

    def forward(self, h, out_dtype, rows=None, partials=None):
        # one kernel; its launch is the one the lowered operation makes
        return ops.rmsnorm(h, self.weight, self.eps, out_dtype, rows=rows, partials=partials)

    def lower(self, program, select_rows: bool = False) -> None:
        """`select_rows`: normalise the step's wanted rows only (before an output head)."""
        program.append("norm", core.norm_params(
            self.weight.data_ptr(), ops.dtype_code(self.weight.dtype), self.eps, select_rows))

    def weight_bytes(self) -> int:
        return self.weight.numel() * self.weight.element_size()
