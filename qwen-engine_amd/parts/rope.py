"""Half-split rotary position encoding.  The table is built as the reference builds
it (src/models/qwen3/model.py:75-86): 32-bit inverse frequencies 1 / theta^(2i/D),
32-bit outer product with the positions, then cos and sin, row = [cos | sin]."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import Runtime, TensorInfo
from .registry import register_part


class RotaryHalf:
    fused = True   # the q/k kernel applies it from table()

    def __init__(self, spec, hidden_size: int = 0):
        self.theta = float(spec.theta)
        self.rotary_dim = int(spec.rotary_dim)
        self.max_positions = int(spec.max_positions)
        if self.rotary_dim % 2:
            raise ValueError(f"rotary_dim {self.rotary_dim} is odd")
        self._table: Optional[torch.Tensor] = None

    @staticmethod
    def expected_tensors(spec, hidden_size: int) -> Dict[str, TensorInfo]:
        return {}

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        d = self.rotary_dim
        inv_freq = 1.0 / (self.theta ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
        t = torch.arange(self.max_positions, dtype=torch.float32)
        freqs = torch.outer(t, inv_freq)
        self._table = torch.cat([torch.cos(freqs), torch.sin(freqs)], dim=-1).contiguous().to(rt.device)

    def table(self) -> torch.Tensor:
        return self._table


class RotaryPairs:
    """Rotation of neighbouring pairs (2i, 2i + 1) by position * theta^(-2i / rotary_dim).  The kernels
    that rotate form the angle, its sine and cosine in 32-bit from ``inv_freq()``; the frequencies are
    computed in 64-bit and rounded once."""

    def __init__(self, spec, hidden_size: int = 0):
        self.theta = float(spec.theta)
        self.rotary_dim = int(spec.rotary_dim)
        if self.rotary_dim % 2:
            raise ValueError(f"rotary_dim {self.rotary_dim} is odd")
        self._inv_freq: Optional[torch.Tensor] = None

    @staticmethod
    def expected_tensors(spec, hidden_size: int) -> Dict[str, TensorInfo]:
        return {}

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        d = self.rotary_dim
        i = torch.arange(0, d, 2, dtype=torch.float64)
        self._inv_freq = torch.pow(torch.tensor(self.theta, dtype=torch.float64), -i / d).to(torch.float32).to(rt.device)

    def inv_freq(self) -> torch.Tensor:
        return self._inv_freq


class RotaryHalfAngles:
    """Half-split rotation of a head's first ``rotary_dim`` numbers (number i pairs with i + rotary_dim / 2) by
    position * theta^(-2i / rotary_dim).  The kernels that rotate form the angle, its sine and cosine in 32-bit from
    ``inv_freq()``; the frequencies are computed in 64-bit, divided by the spec's scaling factor and rounded once.
    No table: no limit of positions."""

    def __init__(self, spec, hidden_size: int = 0):
        self.theta = float(spec.theta)
        self.rotary_dim = int(spec.rotary_dim)
        if self.rotary_dim % 2 or self.rotary_dim <= 0:
            raise ValueError(f"rotary_dim {self.rotary_dim} is odd or not positive")
        self.scaling_factor = float(getattr(spec, "scaling_factor", 1.0))
        if not self.scaling_factor > 0:
            raise ValueError(f"a scaling factor of {self.scaling_factor}")
        self._inv_freq: Optional[torch.Tensor] = None

    @staticmethod
    def expected_tensors(spec, hidden_size: int) -> Dict[str, TensorInfo]:
        return {}

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        d = self.rotary_dim
        i = torch.arange(0, d, 2, dtype=torch.float64)
        f = torch.pow(torch.tensor(self.theta, dtype=torch.float64), -i / d) / self.scaling_factor
        self._inv_freq = f.to(torch.float32).to(rt.device)

    def inv_freq(self) -> torch.Tensor:
        return self._inv_freq


register_part("rope_half", RotaryHalf)
register_part("rope_half_angles", RotaryHalfAngles)
register_part("rope_pairs", RotaryPairs)
