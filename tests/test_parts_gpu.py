"""Each part of the model alone against its plain statement: norm, rotary table, the attention mixer (whole
prompt, and the same prompt in two steps from the cache), the gated feed-forward, the block, embedding and head."""

from types import SimpleNamespace

import pytest
import torch

import plain_qwen3 as plain
import tiny_models as tm

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
DTYPES = [torch.float32, torch.bfloat16]


def _ctx_builder(cache):
  from miniinfer_amd.engine.runner import ModelRunner
  stub = SimpleNamespace(ctx=SimpleNamespace(device=DEV), spec=SimpleNamespace(vocab_size=1 << 30))
  return ModelRunner(stub, cache)


def _close(got, want, dtype, scale=None):
  got, want = got.double().cpu(), want.double().cpu()
  s = float(want.abs().max()) if scale is None else scale
  tol = 2e-5 if dtype == torch.float32 else 2.5e-2
  assert float((got - want).abs().max()) <= tol * max(s, 1e-6), f"max err {(got - want).abs().max():.3g} vs scale {s:.3g}"


@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_part(dtype):
  from miniinfer_amd.config import NormSpec
  from miniinfer_amd.parts import NORMS, BuildContext
  n = NORMS.build(NormSpec(size=80, eps=3e-6), BuildContext(DEV, dtype))
  assert [p.name for p in n.param_specs()] == ["weight"] and n.param_specs()[0].storage == "float32"
  w = 1 + 0.1 * torch.randn(80)
  n.set_param("weight", w.to(DEV))
  x = torch.randn(9, 80).to(dtype)
  r = torch.randn(9, 80)
  _close(n.forward(x.to(DEV)), plain.rms_norm(x.float(), w, 3e-6), dtype)
  rd = r.to(DEV).clone()
  y = n.forward_residual(x.to(DEV), rd)
  _close(rd, r + x.float(), torch.float32)
  _close(y, plain.rms_norm(r + x.float(), w, 3e-6), dtype)


def test_rotary_table_is_the_reference_table():
  from miniinfer_amd.config import RotarySpec
  from miniinfer_amd.parts import POSITIONS, BuildContext
  rope = POSITIONS.build(RotarySpec(rotary_dim=48, theta=5e5, max_positions=300), BuildContext(DEV, torch.bfloat16))
  t = rope.rotary_table().cpu()
  ang = plain.rope_angles(torch.arange(300), 48, 5e5, torch.float32)
  assert t.dtype == torch.float32 and t.shape == (300, 48)
  torch.testing.assert_close(t[:, :24], ang.cos(), rtol=0, atol=1e-6)
  torch.testing.assert_close(t[:, 24:], ang.sin(), rtol=0, atol=1e-6)


def _attention_part(cfg, dtype, w, layer=0):
  from miniinfer_amd.config import Qwen3Config, model_spec_of
  from miniinfer_amd.parts import MIXERS, BuildContext
  spec = model_spec_of(Qwen3Config.from_dict(cfg)).layers[layer].mixer
  part = MIXERS.build(spec, BuildContext(DEV, dtype))
  p = f"model.layers.{layer}.self_attn."
  part.set_param("qkv_weight", torch.cat([w[p + "q_proj.weight"], w[p + "k_proj.weight"], w[p + "v_proj.weight"]]).to(dtype).to(DEV))
  part.set_param("o_weight", w[p + "o_proj.weight"].to(dtype).to(DEV))
  part.q_norm.set_param("weight", w[p + "q_norm.weight"].float().to(DEV))
  part.k_norm.set_param("weight", w[p + "k_norm.weight"].float().to(DEV))
  return part, p


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["B", "C"])
def test_attention_mixer_alone(name, dtype):
  from miniinfer_amd.cache import CacheManager
  from miniinfer_amd.engine.runner import StepEntry
  cfg = dict(tm.CONFIGS[name])
  w = {k: v.to(dtype).float() for k, v in tm.random_weights(cfg, 3, std=0.08).items()}
  part, p = _attention_part(cfg, dtype, w)
  T, H = 75, cfg["hidden_size"]
  x = torch.randn(T, H, generator=torch.Generator().manual_seed(1)).to(dtype)
  want = plain.attention_block(x.float(), torch.arange(T), w, p, cfg)
  cache = CacheManager([part.cache_requirement()], page_size=tm.PAGE_SIZE[name], num_pages=24, max_requests=2,
                       max_model_len=256, dtype=dtype, device=DEV)
  builder = _ctx_builder(cache)
  toks = [0] * T
  # whole, in one step
  cache.admit("a")
  ctx, _, kv = builder.build_context([StepEntry("a", toks, [])])
  got = part.forward(x.to(DEV), ctx, cache.layer_cache(0))
  cache.commit("a", kv[0])
  _close(got, want, dtype)
  # the same in three steps, the last a single token: later steps read the earlier keys from the cache
  cache.admit("b")
  outs = []
  for lo, hi in ((0, 41), (41, 74), (74, 75)):
    ctx, _, kv = builder.build_context([StepEntry("b", toks[lo:hi], [])])
    outs.append(part.forward(x[lo:hi].to(DEV), ctx, cache.layer_cache(0)))
    cache.commit("b", kv[0])
  _close(torch.cat(outs), want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_gated_mlp_alone(dtype):
  from miniinfer_amd.config import GatedMLPSpec
  from miniinfer_amd.parts import FEED_FORWARDS, BuildContext
  ff = FEED_FORWARDS.build(GatedMLPSpec(hidden_size=80, intermediate_size=112), BuildContext(DEV, dtype))
  g = torch.Generator().manual_seed(2)
  wg, wu, wd = (torch.randn(112, 80, generator=g) * 0.1).to(dtype), (torch.randn(112, 80, generator=g) * 0.1).to(dtype), \
      (torch.randn(80, 112, generator=g) * 0.1).to(dtype)
  ff.set_param("gate_up_weight", torch.cat([wg, wu]).to(DEV))
  ff.set_param("down_weight", wd.to(DEV))
  for T in (5, 100):     # few rows (the decode kernels) and many
    x = torch.randn(T, 80, generator=g).to(dtype)
    _close(ff.forward(x.to(DEV), None), plain.swiglu(x.float(), wg.float(), wu.float(), wd.float()), dtype)
  # gate rows first: swapping the halves of the fused matrix changes the result
  ff.set_param("gate_up_weight", torch.cat([wu, wg]).to(DEV))
  x = torch.randn(5, 80, generator=g).to(dtype)
  assert not torch.allclose(ff.forward(x.to(DEV), None).float().cpu(),
                            plain.swiglu(x.float(), wg.float(), wu.float(), wd.float()), atol=1e-3)


@pytest.mark.parametrize("library_products", [False, True])
@pytest.mark.parametrize("dtype", DTYPES)
def test_block_alone(dtype, library_products, monkeypatch):
  """One block on a residual stream: r += attn(norm(r)); r += mlp(norm(r)) with the adds deferred into the norms.
  With `library_products`, products of more than 16 rows go the way they go for large matrices: to the library,
  with norm and activation kernels of their own."""
  from miniinfer_amd.kernels import ops
  if library_products:
    monkeypatch.setattr(ops, "SKINNY_OWN_ELEMENTS", 0)
    assert ops.skinny_preferred(16, 64, 64) and not ops.skinny_preferred(17, 64, 64)
    assert not ops.skinny_preferred(65, 64, 64)
  from miniinfer_amd.cache import CacheManager
  from miniinfer_amd.config import Qwen3Config, model_spec_of
  from miniinfer_amd.engine.runner import StepEntry
  from miniinfer_amd.parts import BLOCKS, BuildContext
  from miniinfer_amd.parts.linear import as_tensor
  from miniinfer_amd.weights.loader import expected_tensors
  cfg = dict(tm.TINY_B)
  w = {k: v.to(dtype).float() for k, v in tm.random_weights(cfg, 5, std=0.08).items()}
  spec = model_spec_of(Qwen3Config.from_dict(cfg))
  block = BLOCKS.build(spec.layers[1], BuildContext(DEV, dtype))
  for prefix, part, ps in block.named_params(spec.layers[1].prefix):
    t = torch.cat([w[prefix + s.name] for s in ps.sources])
    part.set_param(ps.name, t.to(torch.float32 if ps.storage == "float32" else dtype).to(DEV))
  for T in (6, 50):
    h0 = torch.randn(T, cfg["hidden_size"], generator=torch.Generator().manual_seed(T))
    want = plain.decoder_block(h0, torch.arange(T), w, 1, cfg, "model.")
    cache = CacheManager([block.cache_requirement()], page_size=8, num_pages=16, max_requests=1, max_model_len=128,
                         dtype=dtype, device=DEV)
    cache.admit(0)
    ctx, _, kv = _ctx_builder(cache).build_context([StepEntry(0, [0] * T, [])])
    residual = h0.to(DEV).clone()
    h, residual = block.forward(None, residual, ctx, cache.layer_cache(0))
    h = as_tensor(h)              # the block may leave its last product pending for the next norm to absorb
    _close(residual + h.float(), want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_and_head(dtype, tmp_path):
  """Embedding rows are gathered unscaled; the head is lm_head.weight, or the table when the file has none."""
  from miniinfer_amd.cache import CacheManager
  from miniinfer_amd.engine.runner import ModelRunner, StepEntry
  from miniinfer_amd.weights import load_model
  file_dtype = dtype
  for name in ("A", "B"):
    cfg, w = tm.make_model(str(tmp_path / name), name, seed=8, dtype=file_dtype, std=0.05)
    model, _ = load_model(str(tmp_path / name), dtype, DEV)
    assert (model.head is None) == (name == "A")
    cache = CacheManager(model.cache_needs(), page_size=8, num_pages=8, max_requests=1, max_model_len=64, dtype=dtype,
                         device=DEV)
    cache.admit(0)
    toks = tm.random_tokens(cfg, 7, 1)
    got = ModelRunner(model, cache).step([StepEntry(0, toks, list(range(7)))])
    assert got.dtype == torch.float32
    want = plain.qwen3_logits(toks, {k: v.float() for k, v in w.items()}, dict(cfg))
    _close(got, want, dtype)
