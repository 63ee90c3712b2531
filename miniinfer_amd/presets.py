"""Named Qwen3 shapes for random-weight runs (sizes of the published Qwen3 dense checkpoints' config.json,
and the two tiny test shapes)."""

from .config import Qwen3Config


def _q(**kw):
  base = dict(hidden_act="silu", attention_bias=False, initializer_range=0.02, torch_dtype="bfloat16")
  base.update(kw)
  L = base["num_hidden_layers"]
  base.setdefault("layer_windows", tuple(None for _ in range(L)))
  return Qwen3Config(**base)


PRESETS = {
  "tiny-a": lambda: _q(vocab_size=256, hidden_size=64, intermediate_size=128, num_hidden_layers=2,
                       num_attention_heads=4, num_key_value_heads=2, head_dim=16, max_position_embeddings=128,
                       rms_norm_eps=1e-6, rope_theta=10000.0, tie_word_embeddings=True),
  "tiny-b": lambda: _q(vocab_size=384, hidden_size=96, intermediate_size=160, num_hidden_layers=3,
                       num_attention_heads=8, num_key_value_heads=2, head_dim=32, max_position_embeddings=256,
                       rms_norm_eps=1e-5, rope_theta=1000000.0, tie_word_embeddings=False),
  "qwen3-0.6b": lambda: _q(vocab_size=151936, hidden_size=1024, intermediate_size=3072, num_hidden_layers=28,
                           num_attention_heads=16, num_key_value_heads=8, head_dim=128,
                           max_position_embeddings=40960, rms_norm_eps=1e-6, rope_theta=1000000.0,
                           tie_word_embeddings=True),
  "qwen3-8b": lambda: _q(vocab_size=151936, hidden_size=4096, intermediate_size=12288, num_hidden_layers=36,
                         num_attention_heads=32, num_key_value_heads=8, head_dim=128,
                         max_position_embeddings=40960, rms_norm_eps=1e-6, rope_theta=1000000.0,
                         tie_word_embeddings=False),
  "qwen3-32b": lambda: _q(vocab_size=151936, hidden_size=5120, intermediate_size=25600, num_hidden_layers=64,
                          num_attention_heads=64, num_key_value_heads=8, head_dim=128,
                          max_position_embeddings=40960, rms_norm_eps=1e-6, rope_theta=1000000.0,
                          tie_word_embeddings=False),
}


def preset(name: str, num_hidden_layers=None) -> Qwen3Config:
  if name not in PRESETS:
    raise KeyError(f"unknown preset {name!r}; known: {sorted(PRESETS)}")
  cfg = PRESETS[name]()
  if num_hidden_layers is not None:
    from dataclasses import replace
    cfg = replace(cfg, num_hidden_layers=num_hidden_layers, layer_windows=tuple(None for _ in range(num_hidden_layers)))
  return cfg
