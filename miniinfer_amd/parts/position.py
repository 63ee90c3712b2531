"""Position encodings.  A position part hands the mixer what its kernels need; the rotation
itself is fused into the mixer's per-head kernel.

Rotary (NeoX pairing): the table of cos and sin is built as the reference builds it, in 32-bit on the
host: inv_freq_j = 1 / theta^(2j/rotary_dim), angle = pos * inv_freq_j, row = cos(angle) || sin(angle)
(miniinfer/layers/position_encoding.py:29-45).  Unlike the reference, which rounds cos and sin to the
activation dtype before use (position_encoding.py:105-106), the kernel rotates in 32-bit.
"""

from __future__ import annotations

from typing import Optional

import torch

from .base import BuildContext, Part, register_position


class RotaryNeox(Part):
  def __init__(self, spec, ctx: BuildContext):
    if spec.rotary_dim % 2:
      raise ValueError(f"rotary_dim must be even, got {spec.rotary_dim}")
    self.rotary_dim = spec.rotary_dim
    self.theta = spec.theta
    self.max_positions = spec.max_positions
    inv_freq = 1.0 / (spec.theta ** (torch.arange(0, spec.rotary_dim, 2, dtype=torch.float32) / spec.rotary_dim))
    t = torch.arange(spec.max_positions, dtype=torch.float32)
    ang = torch.outer(t, inv_freq)
    self._table = torch.cat((ang.cos(), ang.sin()), dim=-1).contiguous().to(ctx.device)

  def rotary_table(self) -> Optional[torch.Tensor]:
    """[max_positions, rotary_dim] float32: cos of the rotary_dim/2 angles, then sin."""
    return self._table


class NoPosition(Part):
  def __init__(self, spec, ctx: BuildContext):
    pass

  def rotary_table(self) -> Optional[torch.Tensor]:
    return None


register_position("rope_neox", RotaryNeox)
register_position("none", NoPosition)
