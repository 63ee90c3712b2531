"""Chooses the next token of each row of logits on the GPU (one kernel, any mix of greedy and
sampled rows; the reference routes three ways by host flags: miniinfer/layers/sample.py:85-128)."""

from __future__ import annotations

from typing import List, Sequence

import numpy as np
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
    # per-row parameters travel in one pinned buffer and one asynchronous copy (a copy from pageable memory would
    # make the host wait for everything queued on the stream); two buffers are used in turn, since the copy of one
    # step may still be queued when the next step is laid out
    self._stage = [None, None]
    self._turn = 0

  def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams], seeds: Sequence[int],
             steps: Sequence[int]) -> List[int]:
    """logits float32 [R, V]; row r is sampled with params[r] from the stream (seeds[r], steps[r])."""
    out = torch.empty(logits.shape[0], dtype=torch.int32, device=self.device)
    return self.sample_into(logits, params, seeds, steps, out).tolist()

  def _staging(self, nbytes: int) -> torch.Tensor:
    self._turn ^= 1
    buf = self._stage[self._turn]
    if buf is None or buf.numel() < nbytes:
      buf = torch.empty(max(4096, 1 << (nbytes - 1).bit_length()), dtype=torch.uint8,
                        pin_memory=self.device.type == "cuda")
      self._stage[self._turn] = buf
    return buf

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
    # layout of the parameter block: seeds i64 [R] | steps i64 [R] | temperature f32 [R] | top_p f32 [R] | top_k i32 [R]
    Rp = (R + 3) // 4 * 4
    nbytes = Rp * (8 + 8 + 4 + 4 + 4)
    host = self._staging(nbytes)[:nbytes]
    arr = host.numpy()
    o_steps, o_temp, o_p, o_k = 8 * Rp, 16 * Rp, 20 * Rp, 24 * Rp
    arr[:8 * R].view(np.int64)[:] = seeds
    arr[o_steps:o_steps + 8 * R].view(np.int64)[:] = steps
    arr[o_temp:o_temp + 4 * R].view(np.float32)[:] = [p.temperature for p in params]
    arr[o_p:o_p + 4 * R].view(np.float32)[:] = [p.top_p for p in params]
    arr[o_k:o_k + 4 * R].view(np.int32)[:] = [p.top_k for p in params]
    dev = torch.empty(nbytes, dtype=torch.uint8, device=self.device)
    dev.copy_(host, non_blocking=True)
    any_k = any(p.top_k > 0 for p in params)
    any_p = any(p.top_p < 1.0 for p in params)
    sd = dev[:8 * R].view(torch.int64)
    st = dev[o_steps:o_steps + 8 * R].view(torch.int64)
    temp = dev[o_temp:o_temp + 4 * R].view(torch.float32)
    top_p = dev[o_p:o_p + 4 * R].view(torch.float32) if any_p else None
    top_k = dev[o_k:o_k + 4 * R].view(torch.int32) if any_k else None
    ops.sample(logits, temp, top_k, top_p, sd, st, out)
    return out
