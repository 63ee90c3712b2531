"""Architecture-independent description of a model: which parts, with which sizes, in which order.

An architecture's configuration (e.g. `Qwen3Config`) is translated into a `ModelSpec`.
Everything below the registry (parts, loader, cache manager, step function) reads only
the `ModelSpec`; none of it knows which architecture it serves.  A spec is plain data:
a `kind` string that names the part class in the part registry, and that part's sizes
and constants.  New kinds of parts bring their own spec dataclass; the only thing the
framework asks of a spec is the `kind` attribute.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Optional, Tuple


@dataclass(frozen=True)
class NormSpec:
  """Weight-only RMS normalisation over the last `size` elements."""
  size: int
  eps: float
  kind: str = "rmsnorm"


@dataclass(frozen=True)
class RotarySpec:
  """Rotary position encoding: pairs (j, j + rotary_dim/2) of the first `rotary_dim`
  elements of a head are rotated by pos * theta^(-2j/rotary_dim)."""
  rotary_dim: int
  theta: float
  max_positions: int
  kind: str = "rope_neox"


@dataclass(frozen=True)
class NoPositionSpec:
  kind: str = "none"


@dataclass(frozen=True)
class AttentionSpec:
  """Causal grouped-query attention over a paged cache of keys and values."""
  hidden_size: int
  num_heads: int
  num_kv_heads: int
  head_dim: int
  scale: float
  position: Any                      # RotarySpec | NoPositionSpec | another registered kind
  qk_norm: Optional[NormSpec] = None  # per-head norm of q and k before the rotation
  window: Optional[int] = None       # a query at p sees keys p-window < j <= p; None = all
  shares_kv: bool = False            # no k/v projections of its own: reads the keys and values of the layer
                                     # named by LayerSpec.cache_of
  # checkpoint names of the q, k, v and output projections and of the q and k norms
  tensor_names: Tuple[str, ...] = ("q_proj", "k_proj", "v_proj", "o_proj", "q_norm", "k_norm")
  qkv_bias: bool = False             # "<name>.bias" tensors beside the q, k, v projections' weights
  o_bias: bool = False               # and beside the output projection's
  kind: str = "paged_attention"


@dataclass(frozen=True)
class GatedMLPSpec:
  """down( act(x Wg^T) * (x Wu^T) )."""
  hidden_size: int
  intermediate_size: int
  activation: str = "silu"
  tensor_names: Tuple[str, ...] = ("gate_proj", "up_proj", "down_proj")
  bias: bool = False                 # "<name>.bias" tensors beside the three weights
  kind: str = "gated_mlp"


@dataclass(frozen=True)
class LayerSpec:
  """One block: a mixer and a feed-forward, each behind its own norm, on a residual stream.

  `prefix` is the checkpoint-name prefix of the block's tensors.  `cache_of` lets a layer read the
  cache of another layer (by index into `ModelSpec.layers`; the cache of that layer's first run)
  instead of owning one."""
  prefix: str
  mixer: Any
  feed_forward: Any
  mixer_norm: Any
  feed_forward_norm: Any
  cache_of: Optional[int] = None
  # name prefixes, below `prefix`, of the mixer's norm, the mixer, the feed-forward's norm, the feed-forward
  part_prefixes: Tuple[str, ...] = ("input_layernorm.", "self_attn.", "post_attention_layernorm.", "mlp.")
  kind: str = "prenorm"


@dataclass(frozen=True)
class ModelSpec:
  architecture: str
  vocab_size: int
  hidden_size: int
  layers: Tuple[LayerSpec, ...]
  run_order: Tuple[int, ...]          # indices into `layers`; a layer may be named twice (each run has a
                                      # cache of its own unless the layer borrows one)
  final_norm: Any
  embedding_name: str = "model.embed_tokens.weight"
  final_norm_prefix: str = "model.norm."
  head_name: str = "lm_head.weight"
  head_optional: bool = True          # head tensor absent in the checkpoint: the embedding table is the head
  random_writes_head: bool = True     # whether a random-weights folder holds a head tensor of its own
  optional_name_prefix: str = "model."  # checkpoints may leave this prefix out
  max_positions: int = 0
  init_std: float = 0.02
  # The frame around the blocks is data too.  `kind` names the frame class in the frame registry; the default
  # frame (embedding -> blocks -> final norm -> head) takes the variations below as plain numbers and names.
  embedding_scale: float = 1.0        # h = E[ids] * embedding_scale
  position_table_name: Optional[str] = None   # a learned table [max_positions, hidden] whose row of the token's
                                      # position is added to the embedding (absolute positions)
  logit_scale: float = 1.0            # logits = (x . head) * logit_scale
  logit_softcap: Optional[float] = None   # then cap * tanh(logits / cap)
  kind: str = "decoder"
