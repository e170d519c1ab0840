"""Position encodings applied to queries and keys inside a mixer."""

from __future__ import annotations

import torch

from .base import PositionEncoding


class RotaryPosition(PositionEncoding):
    """Rotary encoding in the half-split layout: dims j and j + rotary_dim/2 of a head form a
    pair that is turned by the angle position * theta^(-2j/rotary_dim).

    The angle table is built as the reference builds it (mercury/model/rope.py:37-47):
    inverse frequencies, positions and their outer product in float32, then cos and sin.
    The reference then casts the table to the model dtype; here it stays float32 and the
    rotation is computed in float32, whatever the activations' dtype.  Positions are absolute
    within the sequence, so keys can be cached after rotation.
    """

    def __init__(self, head_dim: int, theta: float, rotary_dim: int | None = None):
        self.head_dim = int(head_dim)
        self.theta = float(theta)
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


class NoPosition(PositionEncoding):
    """Queries and keys are used as projected."""

    rotary_dim = 0
    cos = None
    sin = None
