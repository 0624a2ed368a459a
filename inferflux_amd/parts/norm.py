"""Norms over the float32 residual stream.

RMSNorm, fused with the residual add that precedes it:

y = x * rsqrt(mean(x^2) + eps) * w, all in float, one rounding to the activation type at the
end (runtime/backends/cuda/native/cuda_kernels.cu:15-48; with the add: 193-249, 617-671).

Layer norm with a weight and no bias: y = (x - mean) / sqrt(var + eps) * w, var the mean of the squared
deviations from the mean, all in float.  Besides the common ``forward`` it can sit on a sub-block's output
(``add_to``: stream += norm(delta)), which is how the "outnorm" block uses it.

``tensor`` names a norm's weight in full where a model file does not call it ``<name>.weight``.
"""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from ..kernels import ops
from .base import Norm, register_part
from .plan import ParamSpec


@register_part("norm", "rmsnorm")
class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, name: str, hidden_size: int, eps: float, tensor: Optional[str] = None):
        self.name, self.hidden_size, self.eps = name, int(hidden_size), float(eps)
        self.tensor = tensor or f"{name}.weight"
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {self.tensor: ParamSpec((self.hidden_size,), ("ones",))}

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.weight = tensors[self.tensor]

    def rms_params(self):
        return self.weight, self.eps

    def forward(self, residual, delta, out_dtype, rows=None):
        return ops.add_rmsnorm(residual, delta, self.weight, self.eps, out_dtype, rows)


@register_part("norm", "layernorm")
class LayerNorm(RMSNorm):
    """Mean and variance, a weight, no bias.  (Not an RMS norm: ``rms_params`` says so, and no product applies it as
    a factor per row.)"""

    def rms_params(self):
        return None

    def forward(self, residual, delta, out_dtype, rows=None):
        return ops.layernorm(residual, delta, self.weight, self.eps, out_dtype, rows)

    def add_to(self, stream, delta, cast_dtype=None):
        """stream += norm(delta) in place; returns the new stream in ``cast_dtype`` (None: nothing)."""
        return ops.add_layernorm(stream, delta, self.weight, self.eps, cast_dtype)
