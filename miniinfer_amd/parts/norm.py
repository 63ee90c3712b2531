"""Weight-only RMS norm (miniinfer/layers/layernorm.py:9-42), alone or fused with the residual add."""

from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from ..kernels import ops
from .base import BuildContext, ParamSpec, Part, register_norm


class RMSNorm(Part):
  def __init__(self, spec, ctx: BuildContext):
    self.size = spec.size
    self.eps = spec.eps
    self.ctx = ctx
    self.weight: Optional[torch.Tensor] = None

  def param_specs(self) -> List[ParamSpec]:
    return [ParamSpec.single("weight", (self.size,), storage="float32", init="norm")]

  def forward(self, x: torch.Tensor) -> torch.Tensor:
    """norm(x); x [M, size] in the activation dtype or float32; result in the activation dtype."""
    out = torch.empty(x.shape, dtype=self.ctx.dtype, device=x.device)
    return ops.add_rmsnorm(x, None, self.weight, self.eps, out)

  def forward_residual(self, x: Optional[torch.Tensor], residual: torch.Tensor,
                       rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """residual += x (in place, 32-bit; x may be None), then norm(residual) in the activation dtype.
    With `rows`, only those rows are normed and the residual is left as it is."""
    M = residual.shape[0] if rows is None else rows.numel()
    out = torch.empty((M, self.size), dtype=self.ctx.dtype, device=residual.device)
    return ops.add_rmsnorm(x, residual, self.weight, self.eps, out, rows=rows,
                           write_back=(rows is None and x is not None))


register_norm("rmsnorm", RMSNorm)
