"""RMSNorm over the 32-bit residual stream, with the residual sum fused in.
Formula: src/layers/ops/layernorm.py:50-89 (all three factors in 32-bit, one rounding)."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import Runtime, TensorInfo
from .registry import register_part


class RMSNorm:
    def __init__(self, spec, size: int):
        self.eps = float(spec.eps)
        self.size = int(size)
        self.weight: Optional[torch.Tensor] = None

    @staticmethod
    def expected_tensors(spec, size: int) -> Dict[str, TensorInfo]:
        return {"weight": TensorInfo((size,), "ones", "vector")}

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        self.weight = rt.place_vector(tensors["weight"])

    def fusable_weight(self):
        """(weight, eps): this is a plain RMSNorm, which a product can take as its prologue."""
        return self.weight, self.eps

    def forward(self, h: torch.Tensor, rt: Runtime, delta: Optional[torch.Tensor] = None,
                rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        return ops.rmsnorm(h, self.weight, self.eps, rt.dtype, delta=delta, rows=rows)

    def after_sum(self, x: torch.Tensor, delta: Optional[torch.Tensor], alpha: float, rt: Runtime):
        """The norm of a post-norm block: x <- w * z / rms(z) with z = alpha * x + delta, on the 32-bit stream in
        place; returns the new x in the activation type where that is not 32-bit."""
        return ops.postnorm(x, delta, alpha, self.weight, self.eps, rt.dtype)


class ScalarRMSNorm:
    """RMS norm with one gain for all coordinates (a tensor of no dimensions, named as the part itself).
    ``forward`` is the norm interface of ``parts.base`` (the model's last norm, on the wanted rows);
    ``after_sum`` is the norm of a post-norm block: x <- g * z / rms(z) with z = alpha * x + delta, on the
    32-bit stream in place, returning the new x in the activation type where that is not 32-bit."""

    def __init__(self, spec, size: int):
        self.eps = float(spec.eps)
        self.size = int(size)
        self.gain: Optional[torch.Tensor] = None      # float32 [1]
        self.weight: Optional[torch.Tensor] = None    # the gain, once per coordinate

    @staticmethod
    def expected_tensors(spec, size: int) -> Dict[str, TensorInfo]:
        return {"": TensorInfo((), "ones", "vector")}

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        self.gain = rt.place_vector(tensors[""].reshape(1))
        self.weight = self.gain.expand(self.size).contiguous()

    def forward(self, h: torch.Tensor, rt: Runtime, delta: Optional[torch.Tensor] = None,
                rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        return ops.rmsnorm(h, self.weight, self.eps, rt.dtype, delta=delta, rows=rows)

    def after_sum(self, x: torch.Tensor, delta: Optional[torch.Tensor], alpha: float, rt: Runtime):
        return ops.postnorm(x, delta, alpha, self.gain, self.eps, rt.dtype)


class BareRMSNorm(RMSNorm):
    """RMSNorm whose weight tensor carries the part's own name (named "" inside the part)."""

    @staticmethod
    def expected_tensors(spec, size: int) -> Dict[str, TensorInfo]:
        return {"": TensorInfo((size,), "ones", "vector")}

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        self.weight = rt.place_vector(tensors[""])


class BareLayerNorm:
    """Layer norm with a weight and no bias, (v - mean) * rsqrt(mean of the squared deviations + eps) * w, the weight
    tensor named as the part itself.  The residual sum that stands before it is formed in the same kernel, as in the
    RMS norms; it is no product's prologue (no ``fusable_weight``)."""

    def __init__(self, spec, size: int):
        self.eps = float(spec.eps)
        self.size = int(size)
        self.weight: Optional[torch.Tensor] = None

    @staticmethod
    def expected_tensors(spec, size: int) -> Dict[str, TensorInfo]:
        return {"": TensorInfo((size,), "ones", "vector")}

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        self.weight = rt.place_vector(tensors[""])

    def forward(self, h: torch.Tensor, rt: Runtime, delta: Optional[torch.Tensor] = None,
                rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        return ops.rmsnorm(h, self.weight, self.eps, rt.dtype, delta=delta, rows=rows, center=True)


class StreamScale:
    """Multiplies the 32-bit stream right after the embedding by one number."""

    def __init__(self, spec, hidden_size: int = 0):
        self.scale = float(spec.scale)

    @staticmethod
    def expected_tensors(spec, hidden_size: int) -> Dict[str, TensorInfo]:
        return {}

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        pass

    def forward(self, h: torch.Tensor, ctx) -> None:
        ops.scale_(h, self.scale)


class LogitSoftcap:
    """logits <- cap * tanh(logits / cap), in place on the 32-bit logits."""

    def __init__(self, spec, hidden_size: int = 0):
        self.cap = float(spec.cap)
        if not self.cap > 0:
            raise ValueError(f"a soft cap of {self.cap}")

    @staticmethod
    def expected_tensors(spec, hidden_size: int) -> Dict[str, TensorInfo]:
        return {}

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        pass

    def forward(self, logits: torch.Tensor, ctx) -> torch.Tensor:
        return ops.unary(logits, ops.UNARY_SOFTCAP, cap=self.cap, inplace=True)


register_part("rmsnorm", RMSNorm)
register_part("logit_softcap", LogitSoftcap)
register_part("rmsnorm_bare", BareRMSNorm)
register_part("layernorm_bare", BareLayerNorm)
register_part("stream_scale", StreamScale)
register_part("rmsnorm_scalar", ScalarRMSNorm)
