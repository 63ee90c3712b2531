"""Weight-only RMS norm (miniinfer/layers/layernorm.py:9-42), alone or fused with the residual add."""

from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from ..kernels import ops
from .base import BuildContext, ParamSpec, Part, register_norm


class DeferredNorm:
  """norm(residual + x) that has not been computed yet; x is a tensor, None, or a pending product.  A consumer
  that can fuse the add and the norm into its own first kernel takes the pieces (`linear` and `gate_up_activation`
  do, for few rows); any other calls `materialize()`.  After either, `residual` is the updated residual stream (it
  may be a new buffer, or the old one updated in place)."""

  def __init__(self, norm, x: Optional[torch.Tensor], residual: torch.Tensor):
    self.norm = norm
    self.x = x
    self.residual = residual
    self.value: Optional[torch.Tensor] = None
    self.consumed = False

  @property
  def shape(self):
    return self.residual.shape

  @property
  def dtype(self):
    return self.norm.ctx.dtype

  @property
  def device(self):
    return self.residual.device

  def materialize(self) -> torch.Tensor:
    if self.value is None:
      if self.consumed:
        raise RuntimeError("a deferred norm was fused into one product and then asked for again")
      if hasattr(self.x, "materialize"):       # a product that a part left pending
        self.x = self.x.materialize()
      self.value = self.norm.forward_residual(self.x, self.residual)
      self.consumed = True
    return self.value

  def fused(self, new_residual: torch.Tensor) -> None:
    """A consumer has done the add and the norm inside its own kernel."""
    self.residual = new_residual
    self.consumed = True


class Norm(Part):
  """Base of norm kinds: `forward(x) -> y` (x [M, size] in the activation dtype or float32, y in the activation
  dtype) and `forward_residual(x, residual, rows=None) -> y` (residual += x in place, 32-bit, x may be None, then
  the norm of the residual; with `rows`, only those rows are normed and the residual is left as it is) are the
  kind's own; `defer` hands the pieces to the consumer, who either evaluates them through those two methods or,
  for a kind that says `fusable_rms`, folds them into its own kernel."""

  fusable_rms = False

  def defer(self, x, residual: torch.Tensor) -> DeferredNorm:
    return DeferredNorm(self, x, residual)


class RMSNorm(Norm):
  # What this norm computes is exactly y = x * rsqrt(mean(x^2) + eps) * weight, with a float32 `weight` [size] and
  # `eps`: a consumer may then fold it into a kernel of its own that restates this formula (the products' kernels
  # take its two halves, the attention kernels norm heads with it).  A norm kind that computes anything else
  # (a mean taken off, a bias, 1 + weight) leaves this False, which is the default: it is then always evaluated by
  # its own `forward` / `forward_residual`, never by another part's kernel.
  fusable_rms = True

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
