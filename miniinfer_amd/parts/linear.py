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


def linear(x: torch.Tensor, weight: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
  out_dtype = out_dtype or x.dtype
  M, N = x.shape[0], weight.shape[0]
  if not x.is_cuda:
    raise ops.KernelError("miniinfer_amd runs on the GPU only")
  if x.dtype == torch.float32 or out_dtype != x.dtype:
    out = torch.empty((M, N), dtype=out_dtype, device=x.device)
    return ops.gemm_nt(x, weight, out)
  return torch.matmul(x, weight.t())
