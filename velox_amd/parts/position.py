"""Position encodings.

``RotaryEncoding`` builds the float32 cos/sin tables the way the reference does
(``src/rope.py:45-56``): ``inv_freq[i] = 1 / theta^(2i/d)``, positions divided by a
linear scaling factor, ``cos/sin(pos * inv_freq)``, kept in float32 whatever the
run dtype (``src/rope.py:58-63``).  The rotation itself (halves paired ``(i, i + d/2)``,
``src/rope_inplace.py:25-47``) is fused into the attention mixer's cache-write kernel.
The tables are built on the host so that every run, on any device, rotates by
bit-identical angles.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from .base import PositionEncoding, register_part


class RotaryEncoding(PositionEncoding):
    def __init__(self, rotary_dim: int, theta: float, max_position: int, scaling_factor: float = 1.0) -> None:
        super().__init__("")
        if rotary_dim % 2 != 0:
            raise ValueError(f"rotary_dim must be even, got {rotary_dim}")
        self.rotary_dim = int(rotary_dim)
        self.theta = float(theta)
        self.max_position = int(max_position)
        self.scaling_factor = float(scaling_factor)
        self.cos: Optional[torch.Tensor] = None
        self.sin: Optional[torch.Tensor] = None

    def finalize(self, device, dtype) -> None:
        exponent = torch.arange(0, self.rotary_dim, 2, dtype=torch.float32) / self.rotary_dim
        inv_freq = 1.0 / (self.theta ** exponent)
        positions = torch.arange(self.max_position, dtype=torch.float32)
        if self.scaling_factor != 1.0:
            positions = positions / self.scaling_factor
        angles = torch.outer(positions, inv_freq)
        self.cos = angles.cos().contiguous().to(device)
        self.sin = angles.sin().contiguous().to(device)

    def rotary_tables(self) -> Optional[Tuple[torch.Tensor, torch.Tensor]]:
        return self.cos, self.sin


class NoPositionEncoding(PositionEncoding):
    def __init__(self) -> None:
        super().__init__("")


register_part("position", "rotary", RotaryEncoding)
register_part("position", "none", NoPositionEncoding)
