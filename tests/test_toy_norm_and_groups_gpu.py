"""Two more freedoms of the parts, shown with toy parts that live only in this file:

  * a norm of another kind, mean-centred with a weight and a bias, registered from here and used as block norm, as
    final norm and as the per-head norm of q and k.  It carries `weight` and `eps` attributes like the built-in
    norm, but it does not say `fusable_rms`, so neither the product kernels (which fold a weight-only RMS norm into
    themselves for steps of few rows) nor the attention kernels (which norm heads that way) may take it over: it
    has to be evaluated by its own methods, in steps of 1 to 16 rows as in any other;
  * an attention layer whose cache group names a page size of its own beside layers that take the engine's, one of
    them with a window: each group's pool, block table and token slots follow its own page size.
"""

import json
import os
from dataclasses import dataclass
from typing import List, Optional

import numpy as np
import pytest
import torch

import plain_qwen3 as plain
import trace_tools as tt



@dataclass(frozen=True)
class CenteredNormSpec:
  size: int
  eps: float
  kind: str = "toy_centered_norm"


@dataclass(frozen=True)
class Toy3:
  vocab_size: int = 190
  hidden_size: int = 48
  num_heads: int = 4
  num_kv_heads: int = 2
  head_dim: int = 32
  intermediate_size: int = 80
  eps: float = 1e-5
  theta: float = 20000.0
  max_positions: int = 300
  window: int = 37
  own_page_size: int = 32
  centered: bool = True


def _register():
  from miniinfer_amd.config import (AttentionSpec, GatedMLPSpec, LayerSpec, ModelSpec, NormSpec, RotarySpec,
                                    register_architecture)
  from miniinfer_amd.parts import MIXERS, Norm, PagedKV, ParamSpec, register_mixer, register_norm
  from miniinfer_amd.parts.attention import PagedAttention

  class CenteredNorm(Norm):
    """y = (x - mean(x)) * rsqrt(var(x) + eps) * weight + bias, in 32-bit.  Plain torch: a toy, not a kernel."""

    def __init__(self, spec, ctx):
      self.size, self.eps, self.ctx = spec.size, spec.eps, ctx
      self.weight = self.bias = None

    def param_specs(self):
      return [ParamSpec.single("weight", (self.size,), storage="float32", init="norm"),
              ParamSpec.single("bias", (self.size,), storage="float32")]

    def forward(self, x):
      y = torch.nn.functional.layer_norm(x.float(), (self.size,), self.weight, self.bias, self.eps)
      return y.to(self.ctx.dtype)

    def forward_residual(self, x, residual, rows=None):
      if rows is not None:
        r = residual.index_select(0, rows.long())
        return self.forward(r if x is None else r + x.float().index_select(0, rows.long()))
      if x is not None:
        residual.add_(x.float())
      return self.forward(residual)

  register_norm("toy_centered_norm", CenteredNorm)

  class OwnPagesAttention(PagedAttention):
    """The built-in attention with a page size of its own for its cache group."""

    def cache_requirement(self):
      return PagedKV(num_kv_heads=self.nkv, head_dim=self.d, window=self.window, page_size=self.spec.page_size)

  register_mixer("toy_own_pages_attention", OwnPagesAttention)

  @dataclass(frozen=True)
  class OwnPagesSpec(AttentionSpec):
    page_size: int = 32
    kind: str = "toy_own_pages_attention"

  class Toy3Config(Toy3):
    @classmethod
    def from_dict(cls, raw):
      return cls(**{k: raw[k] for k in Toy3.__dataclass_fields__ if k in raw})

    def build_spec(self):
      H, d = self.hidden_size, self.head_dim
      mk = (lambda n: CenteredNormSpec(n, self.eps)) if self.centered else (lambda n: NormSpec(n, self.eps))
      rope = RotarySpec(rotary_dim=d, theta=self.theta, max_positions=self.max_positions)
      common = dict(hidden_size=H, num_heads=self.num_heads, num_kv_heads=self.num_kv_heads, head_dim=d,
                    scale=d ** -0.5, position=rope, qk_norm=mk(d))
      mixers = (AttentionSpec(**common), OwnPagesSpec(**common, page_size=self.own_page_size),
                AttentionSpec(**common, window=self.window))
      layers = tuple(LayerSpec(prefix=f"model.layers.{i}.", mixer=m,
                               feed_forward=GatedMLPSpec(hidden_size=H, intermediate_size=self.intermediate_size),
                               mixer_norm=mk(H), feed_forward_norm=mk(H)) for i, m in enumerate(mixers))
      return ModelSpec(architecture="Toy3ForCausalLM", vocab_size=self.vocab_size, hidden_size=H, layers=layers,
                       run_order=(0, 1, 2), final_norm=mk(H), max_positions=self.max_positions)

  register_architecture("Toy3ForCausalLM", Toy3Config)


def _weights(c: Toy3, seed=0, std=0.08):
  g = torch.Generator().manual_seed(seed)
  H, V, nq, nkv, d, I = c.hidden_size, c.vocab_size, c.num_heads, c.num_kv_heads, c.head_dim, c.intermediate_size
  mat = lambda *s: torch.randn(*s, generator=g) * std
  w = {}

  def norm(name, n):
    w[name + ".weight"] = 1 + 0.1 * torch.randn(n, generator=g)
    if c.centered:
      w[name + ".bias"] = 0.3 * torch.randn(n, generator=g)

  w["model.embed_tokens.weight"] = mat(V, H) + 0.05          # a mean that the centred norm must take off
  norm("model.norm", H)
  w["lm_head.weight"] = mat(V, H)
  for i in range(3):
    p = f"model.layers.{i}."
    norm(p + "input_layernorm", H)
    norm(p + "post_attention_layernorm", H)
    for n, shape in (("q_proj", (nq * d, H)), ("k_proj", (nkv * d, H)), ("v_proj", (nkv * d, H)), ("o_proj", (H, nq * d))):
      w[p + f"self_attn.{n}.weight"] = mat(*shape)
    norm(p + "self_attn.q_norm", d)
    norm(p + "self_attn.k_norm", d)
    for n, shape in (("gate_proj", (I, H)), ("up_proj", (I, H)), ("down_proj", (H, I))):
      w[p + f"mlp.{n}.weight"] = mat(*shape)
  return w


def _plain_toy3(tokens: List[int], w, c: Toy3) -> torch.Tensor:
  """Whole sequence, no cache, float64: the Qwen3 block of the plain implementation with the norm replaced."""
  w = {k: v.double() for k, v in w.items()}
  T, nq, nkv, d = len(tokens), c.num_heads, c.num_kv_heads, c.head_dim

  def norm(x, name):
    if not c.centered:
      return plain.rms_norm(x, w[name + ".weight"], c.eps)
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + c.eps) * w[name + ".weight"] + w[name + ".bias"]

  pos = torch.arange(T)
  ang = plain.rope_angles(pos, d, c.theta, torch.float64)
  h = w["model.embed_tokens.weight"][torch.tensor(tokens)]
  for i in range(3):
    p = f"model.layers.{i}."
    x = norm(h, p + "input_layernorm")
    q = norm((x @ w[p + "self_attn.q_proj.weight"].T).reshape(T, nq, d), p + "self_attn.q_norm")
    k = norm((x @ w[p + "self_attn.k_proj.weight"].T).reshape(T, nkv, d), p + "self_attn.k_norm")
    v = (x @ w[p + "self_attn.v_proj.weight"].T).reshape(T, nkv, d)
    q, k = plain.apply_rope_neox(q, ang), plain.apply_rope_neox(k, ang)
    mask = plain.causal_mask(T, T, torch.float64, c.window if i == 2 else None)
    o = plain.grouped_attention(q, k, v, d ** -0.5, mask)
    h = h + o.reshape(T, nq * d) @ w[p + "self_attn.o_proj.weight"].T
    x = norm(h, p + "post_attention_layernorm")
    h = h + plain.swiglu(x, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
  return norm(h, "model.norm") @ w["lm_head.weight"].T


def test_the_centred_norm_of_the_plain_statement_is_the_library_routine():
  """What pins the toy norm's plain statement: it is torch's layer_norm, and, unlike an RMS norm, a shift of the
  input leaves it alone."""
  g = torch.Generator().manual_seed(1)
  c = Toy3()
  H = c.hidden_size
  x = torch.randn(7, H, generator=g, dtype=torch.float64) + 0.5
  w = {k: v.double() for k, v in _weights(c).items()}
  wt, b = w["model.norm.weight"], w["model.norm.bias"]
  mu = x.mean(-1, keepdim=True)
  stated = (x - mu) / torch.sqrt(((x - mu) ** 2).mean(-1, keepdim=True) + c.eps) * wt + b
  torch.testing.assert_close(torch.nn.functional.layer_norm(x, (H,), wt, b, c.eps), stated, rtol=1e-12, atol=1e-12)
  torch.testing.assert_close(torch.nn.functional.layer_norm(x + 3.0, (H,), wt, b, c.eps), stated, rtol=1e-9, atol=1e-9)
  assert not torch.allclose(plain.rms_norm(x + 3.0, wt, c.eps), plain.rms_norm(x, wt, c.eps))


def _folder(tmp_path, c: Toy3, w, file_dtype):
  from safetensors.torch import save_file
  d = tmp_path / "toy3"
  os.makedirs(d, exist_ok=True)
  with open(d / "config.json", "w") as f:
    json.dump(dict(architectures=["Toy3ForCausalLM"], **c.__dict__), f)
  save_file({k: v.to(file_dtype).contiguous() for k, v in w.items()}, str(d / "model.safetensors"))
  return str(d)


def _few_rows_plans(requests):
  """Three ways of cutting in which every step has at most 16 rows, the steps in which a weight-only RMS norm is
  folded into the products' kernels: small portions; portions of 16 and then the last 32 tokens one by one; mixed."""
  small = tt.portions(requests, sizes=(2, 3, 7, 2, 16, 5, 1, 9))
  tail = []
  for r, t in requests.items():
    head = max(1, len(t) - 32)
    for i in list(range(0, head, 16)):
      n = min(16, head - i)
      tail.append({"entries": [{"id": r, "tokens": t[i:i + n], "want": list(range(n))}], "end": []})
    for i in range(head, len(t)):
      tail.append({"entries": [{"id": r, "tokens": t[i:i + 1], "want": [0]}], "end": []})
    tail[-1]["end"] = [r]
  for i, s in enumerate(tail):
    s["step"] = i
  return {"small portions": small, "tail decoded": tail, "mixed": tt.mixed(requests, max_live=3, seed=2, max_portion=5)}


@pytest.mark.gpu
@pytest.mark.parametrize("centered", [True, False])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_norm_of_another_kind_and_groups_with_their_own_page_size(tmp_path, dtype, centered, monkeypatch):
  _register()
  from miniinfer_amd.engine.replay import Replayer
  from miniinfer_amd.kernels import ops
  c = Toy3(centered=centered)
  file_dtype = torch.float32 if dtype == "float32" else torch.bfloat16
  w = {k: v.to(file_dtype) for k, v in _weights(c, seed=3).items()}
  g = torch.Generator().manual_seed(8)
  requests = {f"r{i}": torch.randint(0, c.vocab_size, (n,), generator=g).tolist() for i, n in enumerate((70, 33, 5, 120, 41))}
  want = {r: _plain_toy3(t, {k: v.float() for k, v in w.items()}, c).float().numpy() for r, t in requests.items()}
  folder = _folder(tmp_path, c, w, file_dtype)
  took_norm_over = []
  for name in ("gemm_skinny_into_norm", "norm_gemm_skinny", "gemm_skinny_scaled"):
    real = getattr(ops, name)
    monkeypatch.setattr(ops, name, (lambda real, name: lambda *a, **k: (took_norm_over.append(name), real(*a, **k))[1])(real, name))
  real_front = ops.attn_decode_front
  monkeypatch.setattr(ops, "attn_decode_front",
                      lambda *a, **k: (took_norm_over.append("attn_decode_front") if a[17] is not None else None,
                                       real_front(*a, **k))[1])
  for name, steps in _few_rows_plans(requests).items():
    print(f"toy norm (centred {centered}) {dtype} {name}: {len(steps)} steps", flush=True)
    rp = Replayer(folder, dtype, tt.peak_tokens(steps, requests), page_size=8)
    groups = rp.cache.paged
    assert [g_.page_size for g_ in groups] == [8, c.own_page_size, 8] and [g_.layers for g_ in groups] == [[0], [1], [2]]
    assert groups[2].need.window == c.window and groups[2].pool.num_pages <= groups[0].pool.num_pages
    assert groups[1].pool.num_pages * c.own_page_size >= groups[0].pool.num_pages * 8
    outs = []
    for st in steps:
      if name != "mixed":
        assert sum(len(e["tokens"]) for e in st["entries"]) <= 16
      outs.append(rp.step(st))
      rp.cache.check()
    assert rp.cache.all_pages_free()
    got = tt.gather(steps, outs, requests, c.vocab_size)
    for r in requests:
      err = np.abs(got[r] - want[r]).max()
      scale = np.abs(want[r]).max()
      assert err <= (1e-4 if dtype == "float32" else 3e-2 * scale), \
          f"{name}, request {r}: max err {err:.3g} (scale {scale:.3g}); kernels that took a norm over: {sorted(set(took_norm_over))}"
  if dtype == "bfloat16":
    # the built-in norm is folded into the products' and the attention's kernels; the toy norm never is
    assert bool(took_norm_over) == (not centered), sorted(set(took_norm_over))
