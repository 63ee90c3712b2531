"""The layer sizes that the benchmark runs (Qwen3-0.6B: width 1024, 16 query and 8 kv heads of 128, feed-forward
3072, a vocabulary of 151,936 with a tied head), two layers of them, held to the plain implementation as a whole.

At these sizes the engine takes other kernel instances than at the tiny ones: head size 128 in the prefill and
decode attention, the norm split between two products at 1,024 columns, the many-token norm and rotation kernel,
library products of 1,024 to 6,144 columns, the wide output head with a 32-bit result, and captured decode steps
with timed kernel choices.  The four ways of cutting the work are replayed in 32-bit and in bfloat16; greedy
generation runs through the entry point with graphs, overlap and timed product kernels on.
"""

import numpy as np
import pytest
import torch

import plain_qwen3 as plain
import tiny_models as tm
import trace_tools as tt

pytestmark = pytest.mark.gpu

SHAPE = dict(
  architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=151936, hidden_size=1024, intermediate_size=3072,
  num_hidden_layers=2, num_attention_heads=16, num_key_value_heads=8, head_dim=128, hidden_act="silu",
  max_position_embeddings=40960, rms_norm_eps=1e-6, rope_theta=1000000.0, tie_word_embeddings=True,
  attention_bias=False, rope_scaling=None)
LENGTHS = [70, 200, 37, 130]
FP32_TOL = 1e-4


# factor on the per-head norm weights of q and k: in 32-bit, attention that picks few keys shows a misplaced one;
# in bfloat16 the rounding of queries and keys would grow with the scores (3.8% of the largest logit at 2.0), so
# the weights stay as drawn there
SHARPEN = {"float32": 2.0, "bfloat16": 1.0}


@pytest.fixture(scope="module")
def shape_model(tmp_path_factory):
  """Weights drawn once as bfloat16 values (so that both precisions read numbers they can hold), and per dtype the
  model folder and the plain logits of every request."""
  base = tm.random_weights(SHAPE, seed=3, dtype=torch.bfloat16, std=0.03)
  requests = {f"r{i}": tm.random_tokens(SHAPE, n, seed=300 + i) for i, n in enumerate(LENGTHS)}
  out = dict(requests=requests, weights={}, want={}, folders={})
  for name, dt in (("float32", torch.float32), ("bfloat16", torch.bfloat16)):
    w = dict(base)
    for k in w:
      if k.endswith("q_norm.weight") or k.endswith("k_norm.weight"):
        w[k] = (w[k].float() * SHARPEN[name]).to(torch.bfloat16)
    wf = {k: v.float() for k, v in w.items()}
    out["weights"][name] = wf
    out["want"][name] = {rid: plain.qwen3_logits(toks, wf, dict(SHAPE)).numpy() for rid, toks in requests.items()}
    out["folders"][name] = str(tmp_path_factory.mktemp("shape06b") / name)
    tm.write_model(out["folders"][name], SHAPE, {k: v.to(dt) for k, v in w.items()})
  return out


REGIMES = {
  "whole": lambda r: tt.whole(r),
  "tail_decoded": lambda r: tt.tail_decoded(r, 32),
  "portions": lambda r: tt.portions(r),
  "mixed": lambda r: tt.mixed(r, max_live=4, seed=5),
}

# largest errors seen on an MI355X against the plain logits (scale = the largest plain logit of the request):
# bfloat16 max 1.1% and mean 0.15% of the scale (the max is over 151,936 logits a position); the bounds are about
# twice what was seen
BF16_MAX, BF16_MEAN = 0.025, 0.003


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_benchmark_shape_under_every_way_of_cutting(shape_model, dtype):
  from miniinfer_amd.engine.replay import Replayer
  requests, want = shape_model["requests"], shape_model["want"][dtype]
  plans = {name: make(requests) for name, make in REGIMES.items()}
  rp = Replayer(shape_model["folders"][dtype], dtype, max(tt.peak_tokens(p, requests) for p in plans.values()),
                page_size=16)
  worst = {}
  for name, steps in plans.items():
    print(f"0.6B shape {dtype} {name}: {len(steps)} steps", flush=True)
    outs = []
    for st in steps:
      outs.append(rp.step(st))
      rp.cache.check()
    assert rp.cache.all_pages_free() and not rp.cache.live_requests()
    got = tt.gather(steps, outs, requests, SHAPE["vocab_size"])
    for rid in requests:
      assert not np.isnan(got[rid]).any()
      err = np.abs(got[rid] - want[rid])
      scale = np.abs(want[rid]).max()
      worst[name] = max(worst.get(name, (0.0, 0.0)), (float(err.max() / scale), float(err.mean() / scale)))
      if dtype == "float32":
        assert err.max() <= FP32_TOL, f"{name} request {rid}: max abs err {err.max():.3g}"
      else:
        assert err.max() <= BF16_MAX * scale, f"{name} request {rid}: max err {err.max():.4g} of scale {scale:.4g}"
        assert err.mean() <= BF16_MEAN * scale, f"{name} request {rid}: mean err {err.mean():.4g} of scale {scale:.4g}"
  print(f"0.6B shape {dtype}: largest (max, mean) error / largest logit by regime: {worst}", flush=True)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_benchmark_shape_generates_through_the_entry_point(shape_model, dtype):
  """Greedy tokens through `LLMEngine` as the benchmark runs it: captured decode steps, the next step launched
  before the last one's tokens are read, product kernels chosen by timing, prompts cut by a small token budget.
  In 32-bit the tokens are the plain implementation's; in bfloat16 each token is one that the plain
  implementation, given the engine's own history, all but ties for."""
  from miniinfer_amd import LLMEngine, SamplingParams
  w, cfg = shape_model["weights"][dtype], dict(SHAPE)
  prompts = [tm.random_tokens(SHAPE, n, seed=400 + n) for n in (9, 75, 40)]
  n_new = 8
  with LLMEngine(model=shape_model["folders"][dtype], dtype=dtype, page_size=16, num_pages=64, max_num_seqs=4,
                 max_model_len=512, max_num_batched_tokens=64) as eng:
    assert eng.runner.use_graphs and eng.config.enable_overlap and eng.config.tune_products
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=n_new, ignore_eos=True), use_tqdm=False)
    assert len(eng.runner._graphs) > 0, "decode steps were meant to come from captured graphs"
    assert eng.cache.all_pages_free()
  for p, o in zip(prompts, outs):
    if dtype == "float32":
      assert o["token_ids"] == plain.greedy_generate(p, n_new, w, cfg)
      continue
    hist = list(p)
    for tok in o["token_ids"]:
      lg = plain.qwen3_logits(hist, w, cfg)[-1]
      assert lg[tok] >= lg.max() - BF16_MAX * lg.abs().max(), f"token {tok} is not near the plain top"
      hist.append(tok)
