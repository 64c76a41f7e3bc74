"""Norms.  RMSNorm: y = x / sqrt(mean(x^2) + eps) * (weight_offset + w), all in 32-bit.

The reference multiplies by the stored weight (llama3.rs:5244-5256), its files holding 1 + w; a
safetensors file holds w, so Gemma 2 passes weight_offset = 1.  The offset, eps and the width are
constructor arguments: another convention is another argument value.
"""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch

from ..hip import ops
from .base import NORMS, ParamSpec, Part, Precision


@NORMS.register("rmsnorm")
class RMSNorm(Part):
    graph_safe = True

    def __init__(self, precision: Precision, *, dim: int, eps: float, weight_offset: float = 0.0):
        self.precision = precision
        self.dim = dim
        self.eps = float(eps)
        self.weight_offset = float(weight_offset)
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {"weight": ParamSpec((self.dim,), init_std=0.1)}

    def assign(self, name: str, tensor: torch.Tensor) -> None:
        if name != "weight":
            raise KeyError(name)
        self.weight = tensor.contiguous()

    def fused(self) -> Optional[Tuple[torch.Tensor, float, float]]:
        """(weight, eps, offset) for the fused residual-add / norm kernel; a norm that cannot take
        part in the fusion returns None and is run through `forward`."""
        return self.weight, self.eps, self.weight_offset

    def forward(self, x: torch.Tensor, out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """x: float32 [T, dim]; with `rows` only these rows are normed (in their order)."""
        n = x.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, self.dim), dtype=out_dtype, device=x.device)
        ops.add_norm(x, None, None, self.weight, out, eps_pre=self.eps, off_pre=self.weight_offset,
                     rows=rows, full_precision=self.precision.full)
        return out
