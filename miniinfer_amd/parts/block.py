"""Arrangement of a mixer and a feed-forward on the residual stream.

"prenorm": x = norm1(r += h_in); a = mixer(x); x = norm2(r += a); h_out = ff(x).
The add of a branch's output is deferred into the next norm, as the reference defers it
(miniinfer/models/fused_qwen3.py:176-196); the residual stream `r` itself is kept in 32-bit.
"""

from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from .base import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, BuildContext, Part, register_block


class PreNormBlock(Part):
  def __init__(self, spec, ctx: BuildContext):
    self.spec = spec
    self.mixer_norm = NORMS.build(spec.mixer_norm, ctx)
    self.mixer = MIXERS.build(spec.mixer, ctx)
    self.ff_norm = NORMS.build(spec.feed_forward_norm, ctx)
    self.feed_forward = FEED_FORWARDS.build(spec.feed_forward, ctx)

  def children(self) -> List[Tuple[str, Part]]:
    n1, mx, n2, ff = self.spec.part_prefixes
    return [(n1, self.mixer_norm), (mx, self.mixer), (n2, self.ff_norm), (ff, self.feed_forward)]

  def cache_requirement(self):
    fn = getattr(self.mixer, "cache_requirement", None)
    return fn() if fn else None

  def forward(self, h: Optional[torch.Tensor], residual: torch.Tensor, ctx, cache):
    """h: the previous block's pending output (None for the first block); residual [T, hidden] float32.
    Returns (this block's pending output, the residual stream), which may be a new buffer.

    A part that sets `takes_deferred_norm` gets its input as a DeferredNorm and may fuse the add and the norm into
    its own first kernel; any other part gets the normed tensor.  A part that has `forward_lazy` may return its
    last product still pending (`PendingLinear`); the pending output (h, and what this returns) goes into the next
    norm as it is."""
    x = self.mixer_norm.defer(h, residual)
    if not getattr(self.mixer, "takes_deferred_norm", False):
      x.materialize()
    run = getattr(self.mixer, "forward_lazy", self.mixer.forward)
    a = run(x if getattr(self.mixer, "takes_deferred_norm", False) else x.value, ctx, cache)
    if not x.consumed:
      x.materialize()       # a mixer that ignored its input still leaves the residual updated
    residual = x.residual
    y = self.ff_norm.defer(a, residual)
    if not getattr(self.feed_forward, "takes_deferred_norm", False):
      y.materialize()
    run = getattr(self.feed_forward, "forward_lazy", self.feed_forward.forward)
    m = run(y if getattr(self.feed_forward, "takes_deferred_norm", False) else y.value, ctx)
    if not y.consumed:
      y.materialize()
    return m, y.residual


register_block("prenorm", PreNormBlock)
