"""Interfaces of the parts a model is put together from, and the registries that name them.

A model is a list of blocks; a block arranges a mixer and a feed-forward, each behind a norm,
on a residual stream; a mixer may use a position encoding.  Every part is built from its own
spec (sizes and constants only) and a `BuildContext` (device, dtype); no part knows which
architecture it is in.  A spec's `kind` selects the class through the registries below, so a
model can have different mixers and feed-forwards in different layers, and code outside the
framework can add kinds (`register_mixer("my_kind", MyMixer)`).

What each kind of part must provide
-----------------------------------
every part      `param_specs()`   the tensors it owns (name, shape, storage class, the checkpoint
                                  tensors that fill it);
                `children()`      sub-parts with their name prefix;
                tensors arrive through `set_param(name, tensor)`.
Norm            `forward(x) -> y`,  `forward_residual(x, residual) -> (y, new_residual)`
                where new_residual = x + residual (32-bit) and y = norm(new_residual).
Position        `tables()` device tensors the mixer's kernels read (e.g. cos/sin rows).
Mixer           `cache_requirement()` -> PagedKV | FixedState | None;
                `forward(x [T, hidden], ctx: StepContext, cache: LayerCache) -> [T, hidden]`.
FeedForward     `forward(x [T, hidden], ctx) -> [T, hidden]`.
Block           `forward(h, residual, ctx, cache) -> (h, residual)`.
Frame           the whole model around the blocks (`ModelSpec.kind`): `forward(ctx) -> float32 logits
                [wanted rows, vocab]`, `cache_needs()`, `cache_index(run)`, `spec`, `ctx`.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Dict, Iterator, List, Optional, Tuple

import torch


# ----------------------------------------------------------------------------- parameters

@dataclass(frozen=True)
class Source:
  """A checkpoint tensor (name relative to the part's prefix) that fills `rows` rows of a parameter."""
  name: str
  rows: int


@dataclass(frozen=True)
class ParamSpec:
  """A tensor a part owns.

  storage: "compute" = the engine's dtype (bfloat16 or float32); "float32" = always 32-bit
  (norm weights and the like: a tensor stored in 32-bit stays so, one stored in 16-bit is widened,
  which is exact); "int32" = integer tables.
  sources: the checkpoint tensors that are laid one after the other along dim 0 to form it
  (q, k, v projections into one fused matrix; gate and up likewise).
  init: "normal" = N(0, std); "norm" = 1 + N(0, 0.1); used by the random-weights mode."""
  name: str
  shape: Tuple[int, ...]
  sources: Tuple[Source, ...]
  storage: str = "compute"
  init: str = "normal"

  @staticmethod
  def single(name: str, shape, storage="compute", init="normal") -> "ParamSpec":
    return ParamSpec(name=name, shape=tuple(shape), sources=(Source(name, shape[0]),), storage=storage, init=init)


# ----------------------------------------------------------------------------- cache needs

@dataclass(frozen=True)
class PagedKV:
  """Keys and values of every past token (or of the last `window` tokens) in pages.  Layers whose needs are equal
  in every field share a group: one pool of pages, one free list, one block table per request.
  page_size: tokens per page of this group (a power of two), None = the engine's; dtype: of the pages, None = the
  engine's.  A group with a window is given only as many pages as its requests can hold at once."""
  num_kv_heads: int
  head_dim: int
  window: Optional[int] = None
  page_size: Optional[int] = None
  dtype: Optional[torch.dtype] = None


@dataclass(frozen=True)
class FixedState:
  """Per-request state of fixed size, kept in a slot for as long as the request lives;
  zero when the request is admitted.  `dtype` None = the engine's dtype."""
  shape: Tuple[int, ...]
  dtype: Optional[torch.dtype] = None


# ----------------------------------------------------------------------------- build context

@dataclass
class BuildContext:
  device: torch.device
  dtype: torch.dtype            # torch.bfloat16 or torch.float32

  @property
  def exact(self) -> bool:
    """True in the 32-bit mode: no reduced-precision matrix product anywhere."""
    return self.dtype == torch.float32


class Part:
  """Base of every part: owns tensors, may have children."""

  # Whether the part's forward pass can be recorded into a HIP graph: everything it does is queued on the current
  # stream from values the host already has.  A part that reads device values on the host (`.tolist()`, `.item()`),
  # or launches a number of kernels that depends on them, sets this to False; steps of a model that holds such a
  # part are never captured.
  capturable = True

  def is_capturable(self) -> bool:
    return bool(self.capturable) and all(child.is_capturable() for _, child in self.children())

  def param_specs(self) -> List[ParamSpec]:
    return []

  def children(self) -> List[Tuple[str, "Part"]]:
    return []

  def set_param(self, name: str, tensor: torch.Tensor) -> None:
    setattr(self, name.replace(".", "_"), tensor)

  def named_params(self, prefix: str = "") -> Iterator[Tuple[str, "Part", ParamSpec]]:
    for ps in self.param_specs():
      yield prefix, self, ps
    for sub, child in self.children():
      yield from child.named_params(prefix + sub)

  def products(self) -> List[Tuple[torch.Tensor, bool]]:
    """(matrix, whether it is a fused gate|up matrix) of every product this part and its children run on a step's
    rows through `linear` / `gate_up_activation`; an engine times the candidates for them once
    (`kernels.tuning.tune_products`)."""
    out: List[Tuple[torch.Tensor, bool]] = []
    for _, child in self.children():
      out.extend(child.products())
    return out

  def finalize(self) -> None:
    """Called once after all tensors have arrived."""
    for _, child in self.children():
      child.finalize()


# ----------------------------------------------------------------------------- registries

class Registry:
  def __init__(self, what: str):
    self.what = what
    self._classes: Dict[str, Callable[..., Part]] = {}

  def register(self, kind: str, cls) -> None:
    self._classes[kind] = cls

  def build(self, spec: Any, ctx: BuildContext, **kw) -> Part:
    kind = getattr(spec, "kind", None)
    if kind not in self._classes:
      raise KeyError(f"no {self.what} of kind {kind!r} is registered; known: {sorted(self._classes)}")
    return self._classes[kind](spec, ctx, **kw)

  def known(self) -> List[str]:
    return sorted(self._classes)


NORMS = Registry("norm")
POSITIONS = Registry("position encoding")
MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed-forward")
BLOCKS = Registry("block")
FRAMES = Registry("model frame")


def register_norm(kind, cls): NORMS.register(kind, cls)
def register_position(kind, cls): POSITIONS.register(kind, cls)
def register_mixer(kind, cls): MIXERS.register(kind, cls)
def register_feed_forward(kind, cls): FEED_FORWARDS.register(kind, cls)
def register_block(kind, cls): BLOCKS.register(kind, cls)
def register_frame(kind, cls): FRAMES.register(kind, cls)
