"""Plain, slow Qwen3-dense forward pass: whole sequences, no cache, no batching.

One function per part, written from the formulas of tom-jerr/MiniInfer (each
function cites the file and lines it restates).  It shares no code with the
`miniinfer_amd` package: it reads `config.json` with `json`, weights with the
`safetensors` library, and computes with ordinary torch tensor arithmetic on the
CPU in the dtype it is given (float32 by default, float64 for tighter bounds).

All arithmetic is done in one dtype.  The reference rounds to fp16 between some
operations (norm output before the weight multiply, the residual add); in a
single-precision run those roundings are the identity, so the formulas below are
the reference's with "activation dtype" = the compute dtype.
"""

from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional

import torch


# ----------------------------------------------------------------------------
# configuration and weights (plain dicts)
# ----------------------------------------------------------------------------

def read_config(model_dir: str) -> dict:
  """config.json keys as the reference's Qwen3Config reads them
  (miniinfer/config/model/qwen3.py:16-63, defaults included)."""
  with open(os.path.join(model_dir, "config.json")) as f:
    raw = json.load(f)
  cfg = dict(raw)
  if cfg.get("num_key_value_heads") is None:
    # miniinfer/config/model/qwen3.py:46-48
    cfg["num_key_value_heads"] = cfg["num_attention_heads"]
  if cfg.get("head_dim") is None:
    # miniinfer/config/model/qwen3.py:75-79
    cfg["head_dim"] = cfg["hidden_size"] // cfg["num_attention_heads"]
  cfg.setdefault("rms_norm_eps", 1e-6)
  cfg.setdefault("rope_theta", 1000000.0)
  return cfg


def read_weights(model_dir: str, dtype=torch.float32) -> Dict[str, torch.Tensor]:
  """Every tensor of every *.safetensors file in the folder, by name
  (miniinfer/loader/weight.py:109-113,140-158)."""
  from safetensors import safe_open

  out: Dict[str, torch.Tensor] = {}
  for fn in sorted(os.listdir(model_dir)):
    if not fn.endswith(".safetensors"):
      continue
    with safe_open(os.path.join(model_dir, fn), framework="pt", device="cpu") as f:
      for k in f.keys():
        out[k] = f.get_tensor(k).to(dtype)
  return out


# ----------------------------------------------------------------------------
# parts
# ----------------------------------------------------------------------------

def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
  """x * rsqrt(mean(x^2) + eps) * w over the last dim; the weight multiplies
  directly (not 1+w).  miniinfer/layers/layernorm.py:22-32."""
  var = (x * x).mean(dim=-1, keepdim=True)
  return w * (x * torch.rsqrt(var + eps))


def rope_angles(positions: torch.Tensor, rotary_dim: int, theta: float, dtype) -> torch.Tensor:
  """ang[p, j] = pos_p * theta^(-2j/rotary_dim), j = 0 .. rotary_dim/2 - 1.
  miniinfer/layers/position_encoding.py:29-45."""
  j = torch.arange(0, rotary_dim, 2, dtype=dtype)
  inv_freq = 1.0 / (theta ** (j / rotary_dim))
  return positions.to(dtype)[:, None] * inv_freq[None, :]


def apply_rope_neox(x: torch.Tensor, ang: torch.Tensor) -> torch.Tensor:
  """NeoX / rotate-half rotation of x [T, heads, d] by ang [T, d/2]:
  o1 = x1*cos - x2*sin, o2 = x2*cos + x1*sin with x1 = x[..., :d/2], x2 = x[..., d/2:].
  miniinfer/layers/position_encoding.py:91-117 (is_neox_style branch)."""
  cos = ang.cos()[:, None, :]
  sin = ang.sin()[:, None, :]
  half = x.shape[-1] // 2
  x1, x2 = x[..., :half], x[..., half:]
  return torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin), dim=-1)


def causal_mask(L: int, S: int, dtype=torch.float32, window: Optional[int] = None) -> torch.Tensor:
  """Additive mask [L, S], bottom-right aligned: query i sees keys j <= i + (S - L).
  miniinfer/layers/attention.py:112-128.  With `window` (no counterpart in the reference, which reads no
  sliding-window key of config.json) the query at position p = i + (S - L) sees the `window` keys
  p - window < j <= p, itself included."""
  i = torch.arange(L)[:, None]
  j = torch.arange(S)[None, :]
  m = torch.zeros(L, S, dtype=dtype)
  m[j > i + (S - L)] = -math.inf
  if window is not None:
    m[j <= i + (S - L) - window] = -math.inf
  return m


def layer_window(cfg: dict, i: int) -> Optional[int]:
  """The window of layer i from the config.json keys `layer_types` ("full_attention" | "sliding_attention") and
  `sliding_window`, or from `use_sliding_window` + `max_window_layers` (layers from that index on slide).
  The reference ignores these keys (miniinfer/config/model/qwen3.py:16-63 reads none of them)."""
  types = cfg.get("layer_types")
  if types is not None:
    return int(cfg["sliding_window"]) if types[i] == "sliding_attention" else None
  if cfg.get("use_sliding_window") and cfg.get("sliding_window") is not None:
    return int(cfg["sliding_window"]) if i >= int(cfg.get("max_window_layers", cfg["num_hidden_layers"])) else None
  return None


def grouped_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                      mask: Optional[torch.Tensor]) -> torch.Tensor:
  """q [L, nq, d], k and v [S, nkv, d] -> [L, nq, d].  Query head h reads kv head
  h // (nq/nkv); scores = scale * q.k + mask; softmax over keys; weighted sum of v.
  miniinfer/layers/attention.py:131-191."""
  L, nq, d = q.shape
  S, nkv, _ = k.shape
  assert nq % nkv == 0
  rep = nq // nkv
  out = torch.empty_like(q)
  for h in range(nq):
    g = h // rep
    s = (q[:, h, :] @ k[:, g, :].T) * scale
    if mask is not None:
      s = s + mask
    p = torch.softmax(s, dim=-1)
    out[:, h, :] = p @ v[:, g, :]
  return out


def swiglu(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor) -> torch.Tensor:
  """down( silu(x Wg^T) * (x Wu^T) ); silu(g) = g * sigmoid(g).
  miniinfer/models/fused_qwen3.py:134-138; kernels/triton/silu_mul.py:33-37."""
  g = x @ w_gate.T
  u = x @ w_up.T
  return ((g * torch.sigmoid(g)) * u) @ w_down.T


def attention_block(x: torch.Tensor, positions: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str,
                    cfg: dict, window: Optional[int] = None) -> torch.Tensor:
  """QKV projection (no bias), per-head RMSNorm of q and k before the rotation, rotation
  of q and k, causal grouped attention with scale d^-1/2, output projection.
  miniinfer/models/fused_qwen3.py:46-58,95-107."""
  T = x.shape[0]
  nq, nkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
  eps = cfg["rms_norm_eps"]
  q = (x @ w[prefix + "q_proj.weight"].T).reshape(T, nq, d)
  k = (x @ w[prefix + "k_proj.weight"].T).reshape(T, nkv, d)
  v = (x @ w[prefix + "v_proj.weight"].T).reshape(T, nkv, d)
  q = rms_norm(q, w[prefix + "q_norm.weight"], eps)
  k = rms_norm(k, w[prefix + "k_norm.weight"], eps)
  ang = rope_angles(positions, d, cfg["rope_theta"], x.dtype)
  q = apply_rope_neox(q, ang)
  k = apply_rope_neox(k, ang)
  o = grouped_attention(q, k, v, d ** -0.5, causal_mask(T, T, x.dtype, window))
  return o.reshape(T, nq * d) @ w[prefix + "o_proj.weight"].T


def decoder_block(h: torch.Tensor, positions: torch.Tensor, w: Dict[str, torch.Tensor], i: int, cfg: dict,
                  p: str) -> torch.Tensor:
  """Pre-norm block on the summed residual stream `h`:
  h += attn(norm_in(h)); h += mlp(norm_post(h)).  The reference carries (hidden, residual)
  separately and adds inside the next norm (miniinfer/models/fused_qwen3.py:176-196,245-259);
  summed up that is this."""
  pre = f"{p}layers.{i}."
  eps = cfg["rms_norm_eps"]
  a = attention_block(rms_norm(h, w[pre + "input_layernorm.weight"], eps), positions, w, pre + "self_attn.", cfg,
                      layer_window(cfg, i))
  h = h + a
  m = swiglu(rms_norm(h, w[pre + "post_attention_layernorm.weight"], eps),
             w[pre + "mlp.gate_proj.weight"], w[pre + "mlp.up_proj.weight"], w[pre + "mlp.down_proj.weight"])
  return h + m


def qwen3_logits(token_ids: List[int], w: Dict[str, torch.Tensor], cfg: dict, start_pos: int = 0) -> torch.Tensor:
  """Logits [T, V] at every position of one whole sequence.
  Embedding gather without scaling, the blocks, final norm, head = lm_head.weight or, when the
  checkpoint has none, the embedding table (miniinfer/models/fused_qwen3.py:242-259,285-294,344;
  miniinfer/layers/embedding.py:27,41-52).  Positions are start_pos + i
  (miniinfer/scheduler/scheduler_batch.py:450-470)."""
  p = "model." if "model.embed_tokens.weight" in w else ""
  emb = w[p + "embed_tokens.weight"]
  ids = torch.tensor(token_ids, dtype=torch.long)
  h = emb[ids]
  positions = torch.arange(len(token_ids)) + start_pos
  for i in range(cfg["num_hidden_layers"]):
    h = decoder_block(h, positions, w, i, cfg, p)
  h = rms_norm(h, w[p + "norm.weight"], cfg["rms_norm_eps"])
  head = w["lm_head.weight"] if "lm_head.weight" in w else emb
  return h @ head.T


def greedy_generate(prompt: List[int], n: int, w: Dict[str, torch.Tensor], cfg: dict) -> List[int]:
  """n greedy tokens, recomputing the whole sequence each time (the reference's own
  way of checking its cache: tests/test_memory_pressure.py:97-113).  Ties go to the lowest id
  (torch.argmax, miniinfer/layers/sample.py:111-112)."""
  ids = list(prompt)
  out = []
  for _ in range(n):
    nxt = int(torch.argmax(qwen3_logits(ids, w, cfg)[-1]))
    out.append(nxt)
    ids.append(nxt)
  return out


# ----------------------------------------------------------------------------
# sampling (plain statements of the distributions the engine samples from)
# ----------------------------------------------------------------------------

def sampling_distribution(logits: torch.Tensor, temperature: float, top_k: int = 0, top_p: float = 1.0) -> torch.Tensor:
  """The distribution a token is drawn from: softmax(logits / T); keep the top_k most probable
  (0 = all) and renormalise; then keep the smallest most-probable set whose mass reaches top_p and
  renormalise (top-k first, as the reference's fused call applies them).
  temperature 0 is argmax.  miniinfer/layers/sample.py:107-128; utils/sampling_params.py:5-23."""
  x = logits.to(torch.float64)
  V = x.numel()
  if temperature <= 0:
    p = torch.zeros(V, dtype=torch.float64)
    p[int(torch.argmax(x))] = 1.0
    return p
  p = torch.softmax(x / temperature, dim=-1)
  if top_k and top_k < V:
    kth = torch.sort(p, descending=True).values[top_k - 1]
    p = torch.where(p >= kth, p, torch.zeros_like(p))
    p = p / p.sum()
  if top_p < 1.0:
    sp, order = torch.sort(p, descending=True, stable=True)
    before = torch.cumsum(sp, 0) - sp  # mass strictly ahead of each token
    keep = torch.zeros(V, dtype=torch.bool)
    keep[order[before < top_p]] = True
    p = torch.where(keep, p, torch.zeros_like(p))
  return p / p.sum()
