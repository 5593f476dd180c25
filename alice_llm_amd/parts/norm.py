"""Norms.  RMSNorm: y = x / sqrt(mean(x^2) + eps) * (weight_offset + w), all in 32-bit.

The reference multiplies by the stored weight (llama3.rs:5244-5256), its files holding 1 + w; a
safetensors file holds w, so Gemma 2 passes weight_offset = 1.  The offset, eps and the width are
constructor arguments: another convention is another argument value.  `tensor_name` is the weight's local
name ("" where the tensor carries the part's own name).  `output_scale` is a constant factor of the norm's output
(a layer that adds s * norm(branch) to its stream): it is folded into the weight once, at load, in 32-bit, together
with the offset.  `keep_float32` keeps the weight in 32-bit whatever its file stores (the fused add-and-norm kernel
wants the two norms it meets in one dtype, so a design that scales some of its norms keeps them all so).
"""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch

from ..hip import ops
from .base import NORMS, ParamSpec, Part, Precision


@NORMS.register("rmsnorm")
class RMSNorm(Part):
    graph_safe = True

    def __init__(self, precision: Precision, *, dim: int, eps: float, weight_offset: float = 0.0,
                 tensor_name: str = "weight", output_scale: float = 1.0, keep_float32: bool = False):
        self.tensor_name = tensor_name
        self.precision = precision
        self.dim = dim
        self.eps = float(eps)
        self.weight_offset = float(weight_offset)
        self._stored_offset = float(weight_offset)
        self.output_scale = float(output_scale)
        self.keep_float32 = bool(keep_float32) or self.output_scale != 1.0
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {self.tensor_name: ParamSpec((self.dim,), init_std=0.1)}

    def assign(self, name: str, tensor: torch.Tensor) -> None:
        if name != self.tensor_name:
            raise KeyError(name)
        if self.output_scale != 1.0:
            # s * (offset + w) as one 32-bit weight; the kernels then see no offset
            tensor = (tensor.float() + self._stored_offset) * self.output_scale
            self.weight_offset = 0.0
        elif self.keep_float32:
            tensor = tensor.float()
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
