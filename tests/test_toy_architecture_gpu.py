"""Generality of the parts: a toy architecture, defined here and registered from outside the framework, with
  * a mixer with fixed-size state of its own (a decayed running sum per request, kept in a state slot),
  * attention layers with a window (pages of their own, given back as the window passes),
  * a layer that is run twice (each run has its own cache),
  * a layer that borrows another layer's keys and values,
and a model frame that scales the embedding, adds a learned table of absolute positions and caps the logits,
is built from a config.json, loaded by tensor name, and stepped through the engine's step function in portions and
mixed batches; its logits must equal a plain whole-sequence statement of the same toy model.  The same architecture
then generates through the entry point with so few pages that a request that owns a state slot is preempted and
recomputed, and a variant whose stateful mixer can be recorded into a graph decodes from captured steps.  No
framework file knows about any of it."""

import json
import math
import os
from dataclasses import dataclass
from typing import List, Optional

import numpy as np
import pytest
import torch

import plain_qwen3 as plain
import trace_tools as tt

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


# ----------------------------------------------------------------------------- the toy parts (test-only code)

@dataclass(frozen=True)
class DecaySumSpec:
  hidden_size: int
  decay: float
  kind: str = "toy_decay_sum"      # or "toy_decay_sum_graph": the same mixer, recordable into a graph


def _register():
  from miniinfer_amd.config import (AttentionSpec, GatedMLPSpec, LayerSpec, ModelSpec, NormSpec, RotarySpec,
                                    register_architecture)
  from miniinfer_amd.parts import FixedState, ParamSpec, Part, register_mixer

  class DecaySum(Part):
    """y_t = W (s_t), s_t = decay * s_{t-1} + x_t: a recurrent mixer whose state s lives in the request's slot."""

    capturable = False      # forward() reads the state slots on the host

    def __init__(self, spec, ctx):
      self.H, self.decay, self.ctx = spec.hidden_size, spec.decay, ctx
      self.weight = None

    def param_specs(self):
      return [ParamSpec.single("weight", (self.H, self.H))]

    def cache_requirement(self):
      return FixedState(shape=(self.H,), dtype=torch.float32)

    def forward(self, x, ctx, cache):
      out = torch.empty_like(x)
      cu = [0]
      for n in ctx.q_lens:
        cu.append(cu[-1] + n)
      slots = ctx.req_slots.tolist()
      for b, n in enumerate(ctx.q_lens):          # plain torch: this is a toy, not a kernel
        xs = x[cu[b]:cu[b + 1]].float()
        s = cache.state[slots[b]]
        states = []
        for t in range(n):
          s = self.decay * s + xs[t]
          states.append(s)
        cache.state[slots[b]] = s
        out[cu[b]:cu[b + 1]] = (torch.stack(states) @ self.weight.float().T).to(x.dtype)
      return out

  register_mixer("toy_decay_sum", DecaySum)

  class DecaySumForGraphs(DecaySum):
    """The same mixer; a step of single tokens is done with tensor operations only (no value comes back to the
    host), so it can be recorded into a graph and replayed with other slots."""
    capturable = True

    def forward(self, x, ctx, cache):
      if ctx.num_multi > 0:
        return super().forward(x, ctx, cache)
      idx = ctx.req_slots.long()
      s = self.decay * cache.state.index_select(0, idx) + x.float()
      cache.state.index_copy_(0, idx, s)
      return (s @ self.weight.float().T).to(x.dtype)

  register_mixer("toy_decay_sum_graph", DecaySumForGraphs)

  @dataclass(frozen=True)
  class ToyConfig:
    vocab_size: int
    hidden_size: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    intermediate_size: int
    window: int
    decay: float
    eps: float
    theta: float
    max_positions: int
    embedding_scale: float
    logit_scale: float
    logit_softcap: float
    state_mixer: str = "toy_decay_sum"
    eos_token_id = None

    @classmethod
    def from_dict(cls, raw):
      return cls(**{k: raw[k] for k in cls.__dataclass_fields__ if k in raw})

    def build_spec(self):
      H = self.hidden_size
      rope = RotarySpec(rotary_dim=self.head_dim, theta=self.theta, max_positions=self.max_positions)
      norm = NormSpec(size=H, eps=self.eps)

      def attn(window=None, shares_kv=False, qk_norm=True):
        return AttentionSpec(hidden_size=H, num_heads=self.num_heads, num_kv_heads=self.num_kv_heads,
                             head_dim=self.head_dim, scale=self.head_dim ** -0.5, position=rope,
                             qk_norm=NormSpec(self.head_dim, self.eps) if qk_norm else None, window=window,
                             shares_kv=shares_kv)

      ff = GatedMLPSpec(hidden_size=H, intermediate_size=self.intermediate_size)
      layer = lambda i, mixer, **kw: LayerSpec(prefix=f"toy.layers.{i}.", mixer=mixer, feed_forward=ff,
                                               mixer_norm=norm, feed_forward_norm=norm, **kw)
      layers = (layer(0, attn()),                                   # full attention
                layer(1, DecaySumSpec(H, self.decay, kind=self.state_mixer)),   # stateful mixer
                layer(2, attn(window=self.window, qk_norm=False)),  # windowed attention without per-head norm
                layer(3, attn(shares_kv=True), cache_of=0))         # reads layer 0's keys and values
      return ModelSpec(architecture="ToyForCausalLM", vocab_size=self.vocab_size, hidden_size=H, layers=layers,
                       run_order=(0, 1, 2, 1, 3, 2), final_norm=norm, embedding_name="toy.embed.weight",
                       final_norm_prefix="toy.norm.", head_name="toy.head.weight", head_optional=False,
                       optional_name_prefix="", max_positions=self.max_positions,
                       # the frame's options: h = E[id] * scale + P[position]; logits scaled, then capped
                       embedding_scale=self.embedding_scale, position_table_name="toy.positions.weight",
                       logit_scale=self.logit_scale, logit_softcap=self.logit_softcap)

  register_architecture("ToyForCausalLM", ToyConfig)
  return ToyConfig


TOY = dict(architectures=["ToyForCausalLM"], vocab_size=300, hidden_size=48, num_heads=4, num_kv_heads=2, head_dim=16,
           intermediate_size=80, window=21, decay=0.8, eps=1e-5, theta=10000.0, max_positions=512,
           embedding_scale=3.0, logit_scale=0.5, logit_softcap=2.5)


def _toy_weights(seed=0, std=0.08):
  g = torch.Generator().manual_seed(seed)
  H, I, V, nq, nkv, d = 48, 80, 300, 4, 2, 16
  mat = lambda *s: torch.randn(*s, generator=g) * std
  norm = lambda n: 1 + 0.1 * torch.randn(n, generator=g)
  w = {"toy.embed.weight": mat(V, H), "toy.head.weight": mat(V, H) * 8, "toy.norm.weight": norm(H),
       "toy.positions.weight": mat(TOY["max_positions"], H)}
  for i in range(4):
    p = f"toy.layers.{i}."
    w[p + "input_layernorm.weight"] = norm(H)
    w[p + "post_attention_layernorm.weight"] = norm(H)
    for n, shape in (("gate_proj", (I, H)), ("up_proj", (I, H)), ("down_proj", (H, I))):
      w[p + f"mlp.{n}.weight"] = mat(*shape)
    if i == 1:
      w[p + "self_attn.weight"] = mat(H, H) * 3
      continue
    w[p + "self_attn.q_proj.weight"] = mat(nq * d, H)
    w[p + "self_attn.o_proj.weight"] = mat(H, nq * d)
    if i != 3:
      w[p + "self_attn.k_proj.weight"] = mat(nkv * d, H)
      w[p + "self_attn.v_proj.weight"] = mat(nkv * d, H)
    if i != 2:
      w[p + "self_attn.q_norm.weight"] = norm(d)
      if i != 3:
        w[p + "self_attn.k_norm.weight"] = norm(d)
  return w


def _plain_toy(tokens: List[int], w) -> torch.Tensor:
  """Whole sequence, no cache, plain torch (float64): the same toy model written from its definition."""
  w = {k: v.double() for k, v in w.items()}
  c = TOY
  T = len(tokens)
  nq, nkv, d = c["num_heads"], c["num_kv_heads"], c["head_dim"]
  pos = torch.arange(T)
  ang = plain.rope_angles(pos, d, c["theta"], torch.float64)
  h = w["toy.embed.weight"][torch.tensor(tokens)] * c["embedding_scale"] + w["toy.positions.weight"][pos]
  kv0 = None
  for li in (0, 1, 2, 1, 3, 2):
    p = f"toy.layers.{li}."
    x = plain.rms_norm(h, w[p + "input_layernorm.weight"], c["eps"])
    if li == 1:
      s = torch.zeros(c["hidden_size"], dtype=torch.float64)
      states = []
      for t in range(T):
        s = c["decay"] * s + x[t]
        states.append(s)
      a = torch.stack(states) @ w[p + "self_attn.weight"].T
    else:
      q = (x @ w[p + "self_attn.q_proj.weight"].T).reshape(T, nq, d)
      if li != 2:
        q = plain.rms_norm(q, w[p + "self_attn.q_norm.weight"], c["eps"])
      q = plain.apply_rope_neox(q, ang)
      if li == 3:
        k, v = kv0
      else:
        k = (x @ w[p + "self_attn.k_proj.weight"].T).reshape(T, nkv, d)
        v = (x @ w[p + "self_attn.v_proj.weight"].T).reshape(T, nkv, d)
        if li != 2:
          k = plain.rms_norm(k, w[p + "self_attn.k_norm.weight"], c["eps"])
        k = plain.apply_rope_neox(k, ang)
        if li == 0:
          kv0 = (k, v)
      mask = plain.causal_mask(T, T, torch.float64)
      if li == 2:
        i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
        mask = mask.clone()
        mask[j <= i - c["window"]] = -math.inf
      o = plain.grouped_attention(q, k, v, d ** -0.5, mask)
      a = o.reshape(T, nq * d) @ w[p + "self_attn.o_proj.weight"].T
    h = h + a
    x = plain.rms_norm(h, w[p + "post_attention_layernorm.weight"], c["eps"])
    h = h + plain.swiglu(x, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
  logits = plain.rms_norm(h, w["toy.norm.weight"], c["eps"]) @ w["toy.head.weight"].T
  return c["logit_softcap"] * torch.tanh(logits * c["logit_scale"] / c["logit_softcap"])


def _write_toy(folder, dtype, **config_changes):
  from safetensors.torch import save_file
  _register()
  w = _toy_weights()
  file_dtype = torch.float32 if dtype == "float32" else torch.bfloat16
  w = {k: v.to(file_dtype) for k, v in w.items()}
  os.makedirs(folder)
  with open(os.path.join(folder, "config.json"), "w") as f:
    json.dump(dict(TOY, **config_changes), f)
  save_file({k: v.contiguous() for k, v in w.items()}, os.path.join(folder, "model.safetensors"))
  return w


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_is_registered_built_and_stepped(tmp_path, dtype):
  from miniinfer_amd.engine.replay import Replayer
  w = _write_toy(str(tmp_path / "toy"), dtype)
  g = torch.Generator().manual_seed(1)
  requests = {f"r{i}": torch.randint(0, 300, (n,), generator=g).tolist() for i, n in enumerate((70, 33, 5, 120, 48))}
  want = {r: _plain_toy(t, {k: v.float() for k, v in w.items()}).float().numpy() for r, t in requests.items()}
  for steps in (tt.whole(requests), tt.portions(requests), tt.mixed(requests, max_live=3, seed=5)):
    rp = Replayer(str(tmp_path / "toy"), dtype, tt.peak_tokens(steps, requests), page_size=8)
    # what the cache manager made of the layers: full attention (runs 0), windowed attention (runs 2 and 5, a cache
    # each), the state of the mixer that is run twice (runs 1 and 3, a slot row each); the borrowing run has none
    assert len(rp.cache.paged) == 2 and len(rp.cache.states) == 1
    assert rp.cache.paged[0].layers == [0] and rp.cache.paged[1].layers == [2, 5] and rp.cache.states[0].layers == [1, 3]
    outs = []
    for st in steps:
      outs.append(rp.step(st))
      rp.cache.check()
    assert rp.cache.all_pages_free()
    got = tt.gather(steps, outs, requests, 300)
    for r in requests:
      err = np.abs(got[r] - want[r]).max()
      scale = np.abs(want[r]).max()
      assert err <= (2e-4 if dtype == "float32" else 4e-2 * scale), f"request {r}: max err {err:.3g} (scale {scale:.3g})"


def _plain_toy_greedy(prompt, n, w):
  ids, out = list(prompt), []
  for _ in range(n):
    out.append(int(torch.argmax(_plain_toy(ids, w)[-1])))
    ids.append(out[-1])
  return out


@pytest.mark.parametrize("overlap", [False, True])
def test_toy_architecture_generates_through_the_entry_point_and_survives_preemption(tmp_path, overlap):
  """The scheduler, the cache manager and the entry point know nothing of the toy parts: requests that hold a state
  slot and pages in two groups are admitted, cut into portions, preempted when pages run out (slot and pages
  given back, state zeroed at the next admission) and recomputed, with the tokens of the plain statement."""
  from miniinfer_amd import LLMEngine, SamplingParams
  w = _write_toy(str(tmp_path / "toy"), "float32")
  g = torch.Generator().manual_seed(4)
  prompts = [torch.randint(0, 300, (n,), generator=g).tolist() for n in (30, 41, 25, 37)]
  want = [_plain_toy_greedy(p, 24, w) for p in prompts]
  with LLMEngine(model=str(tmp_path / "toy"), dtype="float32", page_size=8, num_pages=20, max_num_seqs=3,
                 max_num_batched_tokens=48, enable_overlap=overlap) as eng:
    assert not eng.runner.use_graphs, "a mixer that reads its slots on the host must keep its steps out of graphs"
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=24, ignore_eos=True), use_tqdm=False)
    assert eng.scheduler.num_preemptions > 0, "the test is meant to run out of pages"
    eng.cache.check()
    assert eng.cache.all_pages_free() and eng.cache.num_free_slots() == 3
  assert [o["token_ids"] for o in outs] == want


def test_stateful_mixer_in_captured_steps_leaves_live_state_slots_alone(tmp_path):
  """Decode steps of a recordable stateful mixer replayed from graphs at a padded batch size (3 requests in a graph
  for 4) while state slot 0 belongs to a live request: padding entries, and the warm-up and capture runs that
  consist of padding only, must use the scratch state row.  Logits equal the eager steps' and the plain
  statement's."""
  from miniinfer_amd.engine.replay import Replayer
  from miniinfer_amd.engine.runner import ModelRunner
  w = _write_toy(str(tmp_path / "toy"), "float32", state_mixer="toy_decay_sum_graph")
  g = torch.Generator().manual_seed(6)
  requests = {f"r{i}": torch.randint(0, 300, (n,), generator=g).tolist() for i, n in enumerate((29, 12, 21))}
  want = {r: _plain_toy(t, w).float().numpy() for r, t in requests.items()}
  tail = 9
  steps = [{"step": 0, "entries": [{"id": r, "tokens": t[:-tail], "want": []} for r, t in requests.items()], "end": []}]
  for i in range(tail):
    steps.append({"step": 1 + i, "end": list(requests) if i == tail - 1 else [],
                  "entries": [{"id": r, "tokens": [t[len(t) - tail + i]], "want": [0]} for r, t in requests.items()]})
  results = {}
  for graphs in (False, True):
    rp = Replayer(str(tmp_path / "toy"), "float32", 256, page_size=8)
    assert rp.model.is_capturable()
    rp.runner = ModelRunner(rp.model, rp.cache, use_graphs=graphs)
    outs = [rp.step(st) for st in steps]
    results[graphs] = outs
    if graphs:
      assert list(rp.runner._graphs) == [(4, 16)], "three single tokens replay the graph for four"
  for i in range(1, len(steps)):
    for b, r in enumerate(requests):
      p = len(requests[r]) - tail + i - 1
      assert np.abs(results[True][i][b] - want[r][p]).max() <= 2e-4, f"graph step {i} request {r}"
      assert np.abs(results[True][i][b] - results[False][i][b]).max() <= 2e-5


def test_recordable_toy_architecture_generates_from_graphs(tmp_path):
  """The same through the entry point with graphs on: decode steps of the stateful toy come from captured steps,
  requests are preempted and recomputed, tokens equal the plain statement's."""
  from miniinfer_amd import LLMEngine, SamplingParams
  w = _write_toy(str(tmp_path / "toy"), "float32", state_mixer="toy_decay_sum_graph")
  g = torch.Generator().manual_seed(8)
  prompts = [torch.randint(0, 300, (n,), generator=g).tolist() for n in (30, 41, 25, 37)]
  want = [_plain_toy_greedy(p, 20, w) for p in prompts]
  with LLMEngine(model=str(tmp_path / "toy"), dtype="float32", page_size=8, num_pages=20, max_num_seqs=3,
                 max_num_batched_tokens=48) as eng:
    assert eng.runner.use_graphs
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=20, ignore_eos=True), use_tqdm=False)
    assert eng.scheduler.num_preemptions > 0 and len(eng.runner._graphs) > 0
    assert eng.cache.all_pages_free()
  assert [o["token_ids"] for o in outs] == want
