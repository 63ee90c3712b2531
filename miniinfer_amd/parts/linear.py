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


class PendingLinear:
  """a @ W^T that has not been computed yet.  A part may hand this to the block instead of a tensor
  (`forward_lazy`): when a norm and another product follow, the add to the residual stream and the norm are
  split between the two products' kernels (`_fuse_norm`) and need none of their own; anyone else calls
  `materialize()`."""

  def __init__(self, a: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None):
    self.a = a
    self.weight = weight
    self.bias = bias
    self.value: Optional[torch.Tensor] = None

  @property
  def shape(self):
    return (self.a.shape[0], self.weight.shape[0])

  @property
  def dtype(self):
    return self.a.dtype

  @property
  def device(self):
    return self.a.device

  def materialize(self) -> torch.Tensor:
    if self.value is None:
      self.value = linear(self.a, self.weight, bias=self.bias)
    return self.value


def as_tensor(x) -> Optional[torch.Tensor]:
  """A tensor from what a part returned: a tensor, None, or a pending product."""
  return x.materialize() if isinstance(x, PendingLinear) else x


def _fuse_norm_around_library(d, weight: torch.Tensor) -> Optional[torch.Tensor]:
  """The gated activation of a deferred norm's product when the gate|up product itself goes to the library (more
  than 16 rows of a large matrix): the norm still needs no kernel if the branch's last product is pending and runs in
  this library's kernel, which adds to the residual stream and leaves bfloat16(residual * norm weight) and the rows'
  sums of squares; the library multiplies that operand, and the activation kernel, which follows anyway, scales
  each row by the norm's missing factor first."""
  M = d.residual.shape[0]
  p = d.x
  inter = weight.shape[0] // 2
  if not getattr(d.norm, "fusable_rms", False):
    return None
  if not (isinstance(p, PendingLinear) and p.value is None and p.bias is None and M <= ops.SKINNY_MAX_ROWS
          and inter % 4 == 0 and weight.dtype == torch.bfloat16 and weight.shape[1] == d.residual.shape[1]
          and weight.is_contiguous()):
    return None
  if not (ops.skinny_preferred(M, p.weight.shape[0], p.weight.shape[1])
          and ops.gemm_skinny_into_norm_supported(p.a, p.weight, d.residual, d.norm.weight)):
    return None
  operand, row_ss = ops.gemm_skinny_into_norm(p.a, p.weight, d.residual, d.norm.weight)
  ops.note_library_product(True)
  gu = torch.matmul(operand, weight.t())
  act = torch.empty((M, inter), dtype=torch.bfloat16, device=d.device)
  ops.silu_mul_scaled(gu, act, row_ss, d.norm.eps, weight.shape[1])
  d.fused(d.residual)
  return act


def _fuse_norm(d, weight: torch.Tensor, gate_up: bool) -> Optional[torch.Tensor]:
  """The product of a deferred norm with `weight` without a kernel for the norm, when the shapes allow it and the
  norm says that it is a weight-only RMS norm (`fusable_rms`): the kernels used here restate that formula from the
  norm's `weight` and `eps`, so a norm of any other kind is left to evaluate itself."""
  M = d.residual.shape[0]
  if d.consumed or d.dtype != torch.bfloat16 or not getattr(d.norm, "fusable_rms", False):
    return None
  if not ops.skinny_preferred(M, weight.shape[0], weight.shape[1], gate_up):
    return _fuse_norm_around_library(d, weight) if gate_up else None
  N = weight.shape[0] // 2 if gate_up else weight.shape[0]
  if isinstance(d.x, PendingLinear) and d.x.value is None and d.x.bias is not None:
    d.x = d.x.materialize()              # a product with a bias is finished by its own kernels
  if isinstance(d.x, PendingLinear) and d.x.value is None:
    # The branch's last product is still pending: its kernel adds to the residual stream in place and leaves
    # bfloat16(residual * norm weight) and partial sums of squares; this product's kernel scales its rows by them.
    p = d.x
    if ops.skinny_preferred(M, p.weight.shape[0], p.weight.shape[1]) \
        and ops.gemm_skinny_into_norm_supported(p.a, p.weight, d.residual, d.norm.weight) \
        and weight.dtype == torch.bfloat16 and weight.shape[1] == d.residual.shape[1] and weight.stride(1) == 1 \
        and weight.stride(0) % 8 == 0 and weight.data_ptr() % 16 == 0:
      operand, row_ss = ops.gemm_skinny_into_norm(p.a, p.weight, d.residual, d.norm.weight)
      out = torch.empty((M, N), dtype=torch.bfloat16, device=d.device)
      ops.gemm_skinny_scaled(operand, weight, out, row_ss, d.norm.eps, gate_up=gate_up)
      d.fused(d.residual)
      return out
    d.x = p.materialize()
  if not ops.norm_gemm_supported(M, d.residual, d.x, weight):
    return None
  out = torch.empty((M, N), dtype=torch.bfloat16, device=d.device)
  new_res = torch.empty_like(d.residual) if d.x is not None else None
  ops.norm_gemm_skinny(d.residual, d.x, d.norm.weight, d.norm.eps, weight, out, residual_out=new_res,
                       gate_up=gate_up)
  d.fused(new_res if new_res is not None else d.residual)
  return out


_MM_TAKES_OUT_DTYPE = [True]     # torch.mm(..., out_dtype=) exists in this torch (found out at the first call)


def linear(x, weight: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
           bias: Optional[torch.Tensor] = None) -> torch.Tensor:
  """x: a tensor [M, K], a pending product, or a DeferredNorm (the add and the norm are then fused into the product
  if possible).  bias [N] (of the result's dtype) is added by a kernel of its own: the architecture this engine
  serves has none, so the products' kernels carry no bias path."""
  if bias is not None:
    return ops.add_bias(linear(x, weight, out_dtype), bias)
  x = as_tensor(x)
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
  avoidable = False
  if ops.gemm_skinny_supported(x, weight):
    own = M <= ops.SKINNY_OWN_ROWS if out_dtype == torch.float32 else ops.skinny_preferred(M, N, x.shape[1])
    avoidable = out_dtype != torch.float32
    if own:
      # few rows (decode): the time is the time to stream the weights; this library's MFMA kernel
      return ops.gemm_skinny(x, weight, torch.empty((M, N), dtype=out_dtype, device=x.device))
  if out_dtype == torch.float32 and x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16:
    # 32-bit results from bfloat16 operands for more rows (the logits of many requests): the library product with
    # a 32-bit result (84 us for 64 rows of a [151936, 1024] head against 148 us for the kernel above); where the
    # library has no such product, the kernel above, 64 rows at a time
    if _MM_TAKES_OUT_DTYPE[0]:
      try:
        y = torch.mm(x, weight.t(), out_dtype=torch.float32)
        ops.note_library_product()
        return y
      except TypeError:
        _MM_TAKES_OUT_DTYPE[0] = False
    if ops.gemm_skinny_supported(x[:1], weight):
      out = torch.empty((M, N), dtype=out_dtype, device=x.device)
      for r0 in range(0, M, ops.SKINNY_MAX_ROWS):
        ops.gemm_skinny(x[r0:r0 + ops.SKINNY_MAX_ROWS], weight, out[r0:r0 + ops.SKINNY_MAX_ROWS])
      return out
  if x.dtype == torch.float32 or out_dtype != x.dtype:
    out = torch.empty((M, N), dtype=out_dtype, device=x.device)
    return ops.gemm_nt(x, weight, out)
  ops.note_library_product(avoidable)
  return torch.matmul(x, weight.t())


def gate_up_activation(x: torch.Tensor, gate_up_weight: torch.Tensor,
                       bias: Optional[torch.Tensor] = None) -> torch.Tensor:
  """silu(x Wg^T) * (x Wu^T) for a fused gate|up matrix [2 I, K]: one kernel for few rows (the activation is made
  from the 32-bit sums in the product's epilogue), product and activation kernels otherwise.  With a bias [2 I]
  (gate | up) the product, the bias and the activation are separate kernels."""
  if bias is not None:
    gu = linear(x, gate_up_weight, bias=bias)
    act = torch.empty((gu.shape[0], gu.shape[1] // 2), dtype=gu.dtype, device=gu.device)
    return ops.silu_mul(gu, act)
  x = as_tensor(x)
  if hasattr(x, "materialize"):
    y = _fuse_norm(x, gate_up_weight, gate_up=True)
    if y is not None:
      return y
    x = x.materialize()
  M, inter = x.shape[0], gate_up_weight.shape[0] // 2
  if ops.gemm_skinny_supported(x, gate_up_weight) and ops.skinny_preferred(M, 2 * inter, x.shape[1], True):
    return ops.gemm_skinny(x, gate_up_weight, torch.empty((M, inter), dtype=x.dtype, device=x.device), gate_up=True)
  gu = linear(x, gate_up_weight)
  act = torch.empty((M, inter), dtype=x.dtype, device=x.device)
  ops.silu_mul(gu, act)
  return act
