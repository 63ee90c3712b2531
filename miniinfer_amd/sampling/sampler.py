"""Chooses the next token of each row of logits on the GPU (one kernel, any mix of greedy and
sampled rows; the reference routes three ways by host flags: miniinfer/layers/sample.py:85-128)."""

from __future__ import annotations

from typing import List, Sequence

import torch

from ..kernels import ops
from .params import SamplingParams

_MASK63 = (1 << 63) - 1


def request_seed(engine_seed: int, request_number: int, user_seed=None) -> int:
  """A 63-bit seed per request: its own if given, else mixed from the engine's seed and its number."""
  if user_seed is not None:
    return int(user_seed) & _MASK63
  z = (engine_seed * 0x9E3779B97F4A7C15 + (request_number + 1) * 0xD1B54A32D192ED03) & ((1 << 64) - 1)
  z ^= z >> 29
  z = (z * 0xBF58476D1CE4E5B9) & ((1 << 64) - 1)
  z ^= z >> 32
  return z & _MASK63


class Sampler:
  def __init__(self, device):
    self.device = torch.device(device)

  def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams], seeds: Sequence[int],
             steps: Sequence[int]) -> List[int]:
    """logits float32 [R, V]; row r is sampled with params[r] from the stream (seeds[r], steps[r])."""
    out = torch.empty(logits.shape[0], dtype=torch.int32, device=self.device)
    return self.sample_into(logits, params, seeds, steps, out).tolist()

  def sample_into(self, logits: torch.Tensor, params: Sequence[SamplingParams], seeds: Sequence[int],
                  steps: Sequence[int], out: torch.Tensor) -> torch.Tensor:
    """The same, left on the device in `out` (int32 [R]); nothing waits for the kernel."""
    R = logits.shape[0]
    if not (len(params) == len(seeds) == len(steps) == R):
      raise ValueError("one SamplingParams, seed and step per row of logits")
    if out.numel() != R or out.dtype != torch.int32:
      raise ValueError("out must hold one int32 per row of logits")
    if all(p.temperature == 0 for p in params):
      ops.sample(logits, None, None, None, None, None, out)
      return out
    temp = torch.tensor([p.temperature for p in params], dtype=torch.float32, device=self.device)
    any_k = any(p.top_k > 0 for p in params)
    any_p = any(p.top_p < 1.0 for p in params)
    top_k = torch.tensor([p.top_k for p in params], dtype=torch.int32, device=self.device) if any_k else None
    top_p = torch.tensor([p.top_p for p in params], dtype=torch.float32, device=self.device) if any_p else None
    sd = torch.tensor(list(seeds), dtype=torch.int64, device=self.device)
    st = torch.tensor(list(steps), dtype=torch.int64, device=self.device)
    ops.sample(logits, temp, top_k, top_p, sd, st, out)
    return out
