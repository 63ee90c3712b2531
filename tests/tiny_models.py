"""Tiny Qwen3 configurations and random weights for tests, written with the safetensors library
(not with the engine's own writer), so that the engine's reader is checked against an independent
file.  The three configurations differ in every size and option."""

import json
import os

import torch

TINY_A = dict(  # 2 layers, tied head, theta 1e4
  architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=256, hidden_size=64, intermediate_size=128,
  num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, head_dim=16, hidden_act="silu",
  max_position_embeddings=128, rms_norm_eps=1e-6, rope_theta=10000.0, tie_word_embeddings=True,
  attention_bias=False, rope_scaling=None)
TINY_B = dict(  # 3 layers, GQA 4:1, q width 256 != hidden, untied head, theta 1e6, eps 1e-5
  architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=384, hidden_size=96, intermediate_size=160,
  num_hidden_layers=3, num_attention_heads=8, num_key_value_heads=2, head_dim=32, hidden_act="silu",
  max_position_embeddings=256, rms_norm_eps=1e-5, rope_theta=1000000.0, tie_word_embeddings=False,
  attention_bias=False, rope_scaling=None)
TINY_C = dict(  # no size a power of two: 3 kv heads, head 48, vocab 500, long positions
  architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=500, hidden_size=80, intermediate_size=112,
  num_hidden_layers=2, num_attention_heads=6, num_key_value_heads=3, head_dim=48, hidden_act="silu",
  max_position_embeddings=2048, rms_norm_eps=3e-6, rope_theta=500000.0, tie_word_embeddings=False,
  attention_bias=False, rope_scaling=None)
TINY_D = dict(  # sliding windows in the two middle layers, one kv head, head 64, tied head
  architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=320, hidden_size=128, intermediate_size=96,
  num_hidden_layers=4, num_attention_heads=4, num_key_value_heads=1, head_dim=64, hidden_act="silu",
  max_position_embeddings=512, rms_norm_eps=1e-6, rope_theta=50000.0, tie_word_embeddings=True,
  attention_bias=False, rope_scaling=None, sliding_window=40, use_sliding_window=True,
  layer_types=["full_attention", "sliding_attention", "sliding_attention", "full_attention"])
PAGE_SIZE = {"A": 16, "B": 8, "C": 16, "D": 8}
CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D}


def random_weights(cfg: dict, seed: int, dtype=torch.float32, std=0.02, norm_std=0.1):
  """Linear and embedding N(0, std), norm weights 1 + N(0, norm_std)."""
  g = torch.Generator().manual_seed(seed)
  H, I, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
  nq, nkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]

  def mat(*shape):
    return (torch.randn(*shape, generator=g) * std).to(dtype)

  def norm(n):
    return (1.0 + norm_std * torch.randn(n, generator=g)).to(dtype)

  w = {"model.embed_tokens.weight": mat(V, H), "model.norm.weight": norm(H)}
  for i in range(cfg["num_hidden_layers"]):
    p = f"model.layers.{i}."
    w[p + "input_layernorm.weight"] = norm(H)
    w[p + "post_attention_layernorm.weight"] = norm(H)
    w[p + "self_attn.q_proj.weight"] = mat(nq * d, H)
    w[p + "self_attn.k_proj.weight"] = mat(nkv * d, H)
    w[p + "self_attn.v_proj.weight"] = mat(nkv * d, H)
    w[p + "self_attn.o_proj.weight"] = mat(H, nq * d)
    w[p + "self_attn.q_norm.weight"] = norm(d)
    w[p + "self_attn.k_norm.weight"] = norm(d)
    w[p + "mlp.gate_proj.weight"] = mat(I, H)
    w[p + "mlp.up_proj.weight"] = mat(I, H)
    w[p + "mlp.down_proj.weight"] = mat(H, I)
  if not cfg.get("tie_word_embeddings", True):
    w["lm_head.weight"] = mat(V, H)
  return w


def write_model(folder: str, cfg: dict, weights: dict) -> str:
  from safetensors.torch import save_file
  os.makedirs(folder, exist_ok=True)
  with open(os.path.join(folder, "config.json"), "w") as f:
    json.dump(cfg, f)
  save_file({k: v.contiguous() for k, v in weights.items()}, os.path.join(folder, "model.safetensors"))
  return folder


def make_model(folder: str, name: str, seed: int = 0, dtype=torch.float32, std=0.02, sharpen: float = 1.0):
  """sharpen: factor on the per-head norm weights of q and k; scores grow with its square, so attention picks
  few keys and a key wrongly seen or missed (a window's edge, a page) moves the logits."""
  cfg = CONFIGS[name]
  w = random_weights(cfg, seed, dtype=dtype, std=std)
  if sharpen != 1.0:
    for k in w:
      if k.endswith("q_norm.weight") or k.endswith("k_norm.weight"):
        w[k] = (w[k].float() * sharpen).to(dtype)
  write_model(folder, cfg, w)
  return cfg, w


def random_tokens(cfg: dict, n: int, seed: int):
  g = torch.Generator().manual_seed(seed)
  return torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist()
