"""A decoder model assembled from a `ModelSpec`: embedding, blocks run in `run_order`, final norm,
output head.  Nothing here names an architecture.

Flow of one step (miniinfer/models/fused_qwen3.py:242-259,317-344): gather the embedding rows of
the step's tokens into the 32-bit residual stream; run the blocks; add the last pending output,
keep only the rows whose logits are wanted, norm them; logits = rows @ head^T in 32-bit.

What varies between architectures in this frame is data of the spec: a factor on the embedding
rows, a learned table of absolute positions added to them, a factor and a soft cap on the logits.
A frame of another shape altogether is another class under its own `ModelSpec.kind`
(`register_frame`).
"""

from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from ..config.spec import ModelSpec
from ..kernels import ops
from .base import BLOCKS, NORMS, BuildContext, ParamSpec, Part, Source, register_frame
from .linear import as_tensor, linear


class DecoderModel(Part):
  def __init__(self, spec: ModelSpec, ctx: BuildContext):
    self.spec = spec
    self.ctx = ctx
    self.blocks = [BLOCKS.build(ls, ctx) for ls in spec.layers]
    for i in spec.run_order:
      if not 0 <= i < len(self.blocks):
        raise ValueError(f"run_order names layer {i}, the model has {len(self.blocks)}")
    self.final_norm = NORMS.build(spec.final_norm, ctx)
    if spec.logit_softcap is not None and not spec.logit_softcap > 0:
      raise ValueError(f"logit_softcap must be positive, got {spec.logit_softcap}")
    self.embedding: Optional[torch.Tensor] = None
    self.head: Optional[torch.Tensor] = None
    self.position_table: Optional[torch.Tensor] = None

  # ------------------------------------------------------------------ tensors
  def param_specs(self) -> List[ParamSpec]:
    V, H = self.spec.vocab_size, self.spec.hidden_size
    out = [ParamSpec("embedding", (V, H), (Source(self.spec.embedding_name, V),)),
           ParamSpec("head", (V, H), (Source(self.spec.head_name, V),))]
    if self.spec.position_table_name is not None:
      P = self.spec.max_positions
      out.append(ParamSpec("position_table", (P, H), (Source(self.spec.position_table_name, P),)))
    return out

  def children(self) -> List[Tuple[str, Part]]:
    out = [(ls.prefix, b) for ls, b in zip(self.spec.layers, self.blocks)]
    out.append((self.spec.final_norm_prefix, self.final_norm))
    return out

  def cache_needs(self) -> List[object]:
    """Per run of `run_order`: what that run's mixer keeps between steps.  A layer that is run twice keeps a cache
    per run; a layer that borrows another layer's cache keeps nothing."""
    needs = []
    for li in self.spec.run_order:
      ls, b = self.spec.layers[li], self.blocks[li]
      needs.append(None if ls.cache_of is not None else b.cache_requirement())
    for li in self.spec.run_order:
      ls = self.spec.layers[li]
      if ls.cache_of is None:
        continue
      if not 0 <= ls.cache_of < len(self.blocks) or self.spec.layers[ls.cache_of].cache_of is not None:
        raise ValueError(f"layer {li} borrows the cache of layer {ls.cache_of}, which has none of its own")
      if ls.cache_of not in self.spec.run_order[:self.spec.run_order.index(li)]:
        raise ValueError(f"layer {li} borrows the cache of layer {ls.cache_of}, which has not run before it")
      if self.blocks[ls.cache_of].cache_requirement() != self.blocks[li].cache_requirement():
        raise ValueError(f"layer {li} borrows the cache of layer {ls.cache_of}, whose geometry differs")
    return needs

  def cache_index(self, run: int) -> int:
    """Which run's cache the run at position `run` of `run_order` uses."""
    co = self.spec.layers[self.spec.run_order[run]].cache_of
    return run if co is None else self.spec.run_order.index(co)

  # ------------------------------------------------------------------ one step
  def forward(self, ctx) -> torch.Tensor:
    """ctx: StepContext.  Returns float32 logits [len(ctx.logit_rows), vocab]."""
    T, H = ctx.num_tokens, self.spec.hidden_size
    residual = torch.empty((T, H), dtype=torch.float32, device=self.ctx.device)
    ops.embed(self.embedding, ctx.token_ids, residual, future=getattr(ctx, "future_tokens", None),
              scale=self.spec.embedding_scale, pos_table=self.position_table, positions=ctx.positions)
    h = None
    for run, li in enumerate(self.spec.run_order):
      h, residual = self.blocks[li].forward(h, residual, ctx, ctx.layer_cache(self.cache_index(run)))
    R = ctx.num_logit_rows
    if R == 0:
      return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=self.ctx.device)
    x = self.final_norm.forward_residual(as_tensor(h), residual, rows=ctx.logit_rows)
    logits = linear(x, self.head if self.head is not None else self.embedding, out_dtype=torch.float32)
    if self.spec.logit_scale != 1.0 or self.spec.logit_softcap is not None:
      ops.logit_transform(logits, self.spec.logit_scale, self.spec.logit_softcap or 0.0)
    return logits


register_frame("decoder", DecoderModel)
