"""Position encodings applied to queries and keys inside a mixer."""

from __future__ import annotations

import torch

from .base import PositionDescriptor, PositionEncoding


class RotaryPosition(PositionEncoding):
    """Rotary encoding: dims j and j + rotary_dim/2 of a head (the half-split layout; with
    `interleaved`, dims 2j and 2j + 1) form a pair that is turned by the angle
    position * theta^(-2j/rotary_dim).

    The angle table is built as the reference builds it (mercury/model/rope.py:37-47):
    inverse frequencies, positions and their outer product in float32, then cos and sin.
    The reference then casts the table to the model dtype; here it stays float32 and the
    rotation is computed in float32, whatever the activations' dtype.  Positions are absolute
    within the sequence, so keys can be cached after rotation.
    """

    def __init__(self, head_dim: int, theta: float, rotary_dim: int | None = None,
                 interleaved: bool = False):
        self.head_dim = int(head_dim)
        self.theta = float(theta)
        self.interleaved = bool(interleaved)
        self.rotary_dim = int(head_dim if rotary_dim is None else rotary_dim)
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError(f"rotary width {self.rotary_dim} must be even and within the head")
        self.cos = None
        self.sin = None

    def prepare(self, max_positions: int, device) -> None:
        if self.cos is not None and self.cos.shape[0] >= max_positions \
                and self.cos.device == torch.device(device):
            return  # a part shared by several layers is prepared once
        exponents = torch.arange(0, self.rotary_dim, 2, dtype=torch.float32) / self.rotary_dim
        inv_freq = 1.0 / (self.theta ** exponents)
        positions = torch.arange(max_positions, dtype=torch.float32)
        angles = torch.outer(positions, inv_freq)
        self.cos = angles.cos().contiguous().to(device)
        self.sin = angles.sin().contiguous().to(device)

    def describe(self) -> PositionDescriptor:
        return PositionDescriptor(self.rotary_dim, self.cos, self.sin, self.interleaved)


class NoPosition(PositionEncoding):
    """Queries and keys are used as projected."""

    def describe(self) -> PositionDescriptor:
        return PositionDescriptor()
