"""Typed configuration of Qwen3 dense, read from the keys of its own config.json.

Reference: miniinfer/config/model/qwen3.py:16-63 (keys and defaults),
miniinfer/config/model/base.py:62-71 (config.json is read from the model folder),
miniinfer/models/fused_qwen3.py:29-75 (which keys the model uses).  Where the
reference parses a key and then ignores it (`attention_bias`, `rope_scaling`),
a value this engine cannot honour is an error here instead of a silent wrong result.
"""

from __future__ import annotations

from dataclasses import dataclass, asdict
from typing import Any, Dict, Optional, Tuple

from .spec import (AttentionSpec, GatedMLPSpec, LayerSpec, ModelSpec, NormSpec, RotarySpec)


class ConfigError(ValueError):
  pass


@dataclass(frozen=True)
class Qwen3Config:
  vocab_size: int
  hidden_size: int
  intermediate_size: int
  num_hidden_layers: int
  num_attention_heads: int
  num_key_value_heads: int
  head_dim: int
  max_position_embeddings: int
  rms_norm_eps: float
  rope_theta: float
  hidden_act: str = "silu"
  tie_word_embeddings: bool = True
  attention_bias: bool = False
  initializer_range: float = 0.02
  # per layer: None = every key, an int = that many most recent keys
  layer_windows: Tuple[Optional[int], ...] = ()
  eos_token_id: Optional[int] = None
  bos_token_id: Optional[int] = None
  torch_dtype: str = "bfloat16"

  architecture = "Qwen3ForCausalLM"
  model_type = "qwen3"

  # ------------------------------------------------------------------ reading
  @classmethod
  def from_dict(cls, raw: Dict[str, Any]) -> "Qwen3Config":
    def need(key):
      if key not in raw or raw[key] is None:
        raise ConfigError(f"config.json: required key '{key}' is missing")
      return raw[key]

    nq = int(need("num_attention_heads"))
    nkv = raw.get("num_key_value_heads")
    nkv = nq if nkv is None else int(nkv)          # qwen3.py:46-48
    hidden = int(need("hidden_size"))
    head_dim = raw.get("head_dim")
    head_dim = hidden // nq if head_dim is None else int(head_dim)   # qwen3.py:75-79
    layers = int(need("num_hidden_layers"))

    rope_theta = raw.get("rope_theta")
    rope_params = raw.get("rope_parameters") or {}
    if rope_theta is None:
      rope_theta = rope_params.get("rope_theta", 1000000.0)
    scaling = raw.get("rope_scaling")
    if scaling is None and rope_params.get("rope_type", "default") not in ("default", None):
      scaling = rope_params
    if scaling is not None and scaling.get("rope_type", scaling.get("type", "default")) != "default":
      raise ConfigError(f"config.json: rope_scaling={scaling!r} is not supported (plain rotary positions only)")

    eos = raw.get("eos_token_id")
    if isinstance(eos, (list, tuple)):
      eos = eos[0] if eos else None

    cfg = cls(
      vocab_size=int(need("vocab_size")),
      hidden_size=hidden,
      intermediate_size=int(need("intermediate_size")),
      num_hidden_layers=layers,
      num_attention_heads=nq,
      num_key_value_heads=nkv,
      head_dim=head_dim,
      max_position_embeddings=int(need("max_position_embeddings")),
      rms_norm_eps=float(raw.get("rms_norm_eps", 1e-6)),
      rope_theta=float(rope_theta),
      hidden_act=str(raw.get("hidden_act", "silu")),
      tie_word_embeddings=bool(raw.get("tie_word_embeddings", True)),
      attention_bias=bool(raw.get("attention_bias", False)),
      initializer_range=float(raw.get("initializer_range", 0.02)),
      layer_windows=cls._windows(raw, layers),
      eos_token_id=None if eos is None else int(eos),
      bos_token_id=raw.get("bos_token_id"),
      torch_dtype=str(raw.get("torch_dtype", raw.get("dtype", "bfloat16"))),
    )
    cfg.validate()
    return cfg

  @staticmethod
  def _windows(raw: Dict[str, Any], layers: int) -> Tuple[Optional[int], ...]:
    window = raw.get("sliding_window")
    types = raw.get("layer_types")
    if types is not None:
      if len(types) != layers:
        raise ConfigError(f"config.json: layer_types has {len(types)} entries for {layers} layers")
      out = []
      for t in types:
        if t == "full_attention":
          out.append(None)
        elif t == "sliding_attention":
          if window is None:
            raise ConfigError("config.json: layer_types names sliding_attention but sliding_window is null")
          out.append(int(window))
        else:
          raise ConfigError(f"config.json: unknown layer type {t!r}")
      return tuple(out)
    if raw.get("use_sliding_window", False) and window is not None:
      first = int(raw.get("max_window_layers", layers))
      return tuple(int(window) if i >= first else None for i in range(layers))
    return tuple(None for _ in range(layers))

  def validate(self) -> None:
    def positive(name):
      if getattr(self, name) <= 0:
        raise ConfigError(f"config.json: {name} must be positive, got {getattr(self, name)}")

    for n in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads",
              "num_key_value_heads", "head_dim", "max_position_embeddings", "rope_theta", "rms_norm_eps"):
      positive(n)
    if self.num_attention_heads % self.num_key_value_heads != 0:
      raise ConfigError(f"config.json: num_attention_heads={self.num_attention_heads} is not a multiple of "
                        f"num_key_value_heads={self.num_key_value_heads}")
    if self.head_dim % 2 != 0:
      raise ConfigError(f"config.json: head_dim={self.head_dim} must be even for rotary positions")
    if self.hidden_act != "silu":
      # miniinfer/models/fused_qwen3.py:122-123
      raise ConfigError(f"config.json: hidden_act={self.hidden_act!r} is not supported, only 'silu'")
    if self.attention_bias:
      raise ConfigError("config.json: attention_bias=true is not supported (Qwen3 projections carry no bias)")
    if len(self.layer_windows) != self.num_hidden_layers:
      raise ConfigError("layer_windows must have one entry per layer")
    for w in self.layer_windows:
      if w is not None and w <= 0:
        raise ConfigError(f"config.json: sliding_window must be positive, got {w}")

  # ------------------------------------------------------------------ writing
  def to_dict(self) -> Dict[str, Any]:
    d = asdict(self)
    windows = d.pop("layer_windows")
    d["architectures"] = [self.architecture]
    d["model_type"] = self.model_type
    d["rope_scaling"] = None
    d["use_cache"] = True
    distinct = {w for w in windows if w is not None}
    if distinct:
      if len(distinct) > 1:
        raise ConfigError("config.json can hold one sliding_window size")
      d["sliding_window"] = distinct.pop()
      d["use_sliding_window"] = True
      d["layer_types"] = ["full_attention" if w is None else "sliding_attention" for w in windows]
    else:
      d["sliding_window"] = None
      d["use_sliding_window"] = False
    return d

  # ------------------------------------------------------------------ the model this describes
  def build_spec(self) -> ModelSpec:
    """miniinfer/models/fused_qwen3.py:141-196 (block), :29-75 (attention), :111-124 (MLP)."""
    rope = RotarySpec(rotary_dim=self.head_dim, theta=self.rope_theta, max_positions=self.max_position_embeddings)
    head_norm = NormSpec(size=self.head_dim, eps=self.rms_norm_eps)
    block_norm = NormSpec(size=self.hidden_size, eps=self.rms_norm_eps)
    layers = []
    for i in range(self.num_hidden_layers):
      mixer = AttentionSpec(
        hidden_size=self.hidden_size, num_heads=self.num_attention_heads, num_kv_heads=self.num_key_value_heads,
        head_dim=self.head_dim, scale=self.head_dim ** -0.5, position=rope, qk_norm=head_norm,
        window=self.layer_windows[i])
      ff = GatedMLPSpec(hidden_size=self.hidden_size, intermediate_size=self.intermediate_size,
                        activation=self.hidden_act)
      layers.append(LayerSpec(prefix=f"model.layers.{i}.", mixer=mixer, feed_forward=ff,
                              mixer_norm=block_norm, feed_forward_norm=block_norm))
    return ModelSpec(
      architecture=self.architecture, vocab_size=self.vocab_size, hidden_size=self.hidden_size,
      layers=tuple(layers), run_order=tuple(range(self.num_hidden_layers)), final_norm=block_norm,
      # the head is lm_head.weight when the checkpoint has it, else the embedding table:
      # miniinfer/layers/embedding.py:41-48 decides by the key's presence, not by the flag
      head_optional=True, random_writes_head=not self.tie_word_embeddings,
      max_positions=self.max_position_embeddings, init_std=self.initializer_range)
