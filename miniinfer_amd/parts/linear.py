"""x @ W^T (miniinfer/layers/linear.py:4-33).

In the 32-bit mode every product runs on this library's FMA kernel, so no reduced-precision
matrix mode can slip in.  In bfloat16 the product of a projection is a library routine
(hipBLASLt through torch.matmul), as the reference's projections are cuBLAS calls
(miniinfer/models/fused_qwen3.py:53-54,120-121); a 32-bit result (the logits) comes from this
library's own kernels.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops


def _fuse_norm(d, weight: torch.Tensor, gate_up: bool) -> Optional[torch.Tensor]:
  """The product of a deferred norm with `weight` in one kernel, when the shapes allow it."""
  M = d.residual.shape[0]
  if d.consumed or d.dtype != torch.bfloat16 or not ops.norm_gemm_supported(M, d.residual, d.x, weight):
    return None
  N = weight.shape[0] // 2 if gate_up else weight.shape[0]
  out = torch.empty((M, N), dtype=torch.bfloat16, device=d.device)
  new_res = torch.empty_like(d.residual) if d.x is not None else None
  ops.norm_gemm_skinny(d.residual, d.x, d.norm.weight, d.norm.eps, weight, out, residual_out=new_res,
                       gate_up=gate_up)
  d.fused(new_res if new_res is not None else d.residual)
  return out


def linear(x, weight: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
  """x: a tensor [M, K], or a DeferredNorm (the add and the norm are then fused into the product if possible)."""
  if hasattr(x, "materialize"):
    if out_dtype in (None, torch.bfloat16):
      y = _fuse_norm(x, weight, gate_up=False)
      if y is not None:
        return y
    x = x.materialize()
  out_dtype = out_dtype or x.dtype
  M, N = x.shape[0], weight.shape[0]
  if not x.is_cuda:
    raise ops.KernelError("miniinfer_amd runs on the GPU only")
  if ops.gemm_skinny_supported(x, weight):
    # few rows (decode): the time is the time to stream the weights; this library's MFMA kernel
    return ops.gemm_skinny(x, weight, torch.empty((M, N), dtype=out_dtype, device=x.device))
  if x.dtype == torch.float32 or out_dtype != x.dtype:
    out = torch.empty((M, N), dtype=out_dtype, device=x.device)
    return ops.gemm_nt(x, weight, out)
  return torch.matmul(x, weight.t())


def gate_up_activation(x: torch.Tensor, gate_up_weight: torch.Tensor) -> torch.Tensor:
  """silu(x Wg^T) * (x Wu^T) for a fused gate|up matrix [2 I, K]: one kernel for few rows (the activation is made
  from the 32-bit sums in the product's epilogue), product and activation kernels otherwise."""
  if hasattr(x, "materialize"):
    y = _fuse_norm(x, gate_up_weight, gate_up=True)
    if y is not None:
      return y
    x = x.materialize()
  M, inter = x.shape[0], gate_up_weight.shape[0] // 2
  if ops.gemm_skinny_supported(x, gate_up_weight):
    return ops.gemm_skinny(x, gate_up_weight, torch.empty((M, inter), dtype=x.dtype, device=x.device), gate_up=True)
  gu = linear(x, gate_up_weight)
  act = torch.empty((M, inter), dtype=x.dtype, device=x.device)
  ops.silu_mul(gu, act)
  return act
