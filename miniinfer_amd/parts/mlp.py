"""Dense gated feed-forward: down( silu(x Wg^T) * (x Wu^T) ) with gate and up fused into one matrix,
gate rows first (miniinfer/models/fused_qwen3.py:111-138; miniinfer/loader/weight.py:87-93)."""

from __future__ import annotations

from typing import List, Optional

import torch

from .base import BuildContext, ParamSpec, Part, Source, register_feed_forward
from .linear import PendingLinear, gate_up_activation


class GatedMLP(Part):
  takes_deferred_norm = True

  def __init__(self, spec, ctx: BuildContext):
    if spec.activation != "silu":
      raise ValueError(f"activation {spec.activation!r} is not supported, only 'silu'")
    self.spec = spec
    self.hidden = spec.hidden_size
    self.inter = spec.intermediate_size
    self.gate_up_weight: Optional[torch.Tensor] = None
    self.down_weight: Optional[torch.Tensor] = None
    self.gate_up_bias: Optional[torch.Tensor] = None     # only when the spec asks for them
    self.down_bias: Optional[torch.Tensor] = None

  def param_specs(self) -> List[ParamSpec]:
    g, u, d = self.spec.tensor_names
    out = [
      ParamSpec("gate_up_weight", (2 * self.inter, self.hidden),
                (Source(g + ".weight", self.inter), Source(u + ".weight", self.inter))),
      ParamSpec("down_weight", (self.hidden, self.inter), (Source(d + ".weight", self.hidden),)),
    ]
    if getattr(self.spec, "bias", False):
      out.append(ParamSpec("gate_up_bias", (2 * self.inter,),
                           (Source(g + ".bias", self.inter), Source(u + ".bias", self.inter))))
      out.append(ParamSpec("down_bias", (self.hidden,), (Source(d + ".bias", self.hidden),)))
    return out

  def products(self):
    return [(self.gate_up_weight, True), (self.down_weight, False)]

  def forward(self, x, ctx) -> torch.Tensor:
    return self.forward_lazy(x, ctx).materialize()

  def forward_lazy(self, x, ctx) -> PendingLinear:
    """The same with the down projection left pending, so that the block can fold the add and the next norm into it."""
    return PendingLinear(gate_up_activation(x, self.gate_up_weight, self.gate_up_bias), self.down_weight, self.down_bias)


register_feed_forward("gated_mlp", GatedMLP)
