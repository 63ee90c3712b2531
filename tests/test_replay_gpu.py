"""The engine against the plain implementation, under every way of cutting the work.

The same requests are replayed whole; with the last 32 tokens decoded one by one; in portions of
changing size down to two tokens; and mixed, up to four live requests with portions of some beside
decoded tokens of others and so few pages that they are used again.  In 32-bit the logits must
agree with the plain implementation to 1e-4; in bfloat16 to the rounding of bfloat16 activations.
"""

import numpy as np
import pytest
import torch

import plain_qwen3 as plain
import tiny_models as tm
import trace_tools as tt

pytestmark = pytest.mark.gpu

LENGTHS = {"A": [5, 17, 33, 100, 128, 64], "B": [1, 9, 40, 64, 100, 200, 33], "C": [300, 77, 513, 2, 150],
           "D": [130, 45, 300, 7, 81]}
# The configuration with sliding windows, in 32-bit: attention that picks few keys shows a window's edge.  (In
# bfloat16 the rounding of queries and keys grows with the scores too, 17% of the largest logit at this factor;
# there the plain weights stand, with which a window that is off by one key still moves the logits by 9%.)
SHARPEN = {("D", "float32"): 2.5}
FP32_TOL = 1e-4


def _requests(name, cfg):
  return {f"r{i}": tm.random_tokens(cfg, n, seed=100 + i) for i, n in enumerate(LENGTHS[name])}


def _plain_logits(cfg_dict, weights, requests):
  pc = dict(cfg_dict)
  w = {k: v.float() for k, v in weights.items()}
  return {rid: plain.qwen3_logits(toks, w, pc).numpy() for rid, toks in requests.items()}


def _replay(folder, dtype, steps, requests, page_size, max_tokens):
  from miniinfer_amd.engine.replay import Replayer
  rp = Replayer(str(folder), dtype, max_tokens, page_size=page_size)
  outs = []
  for st in steps:
    outs.append(rp.step(st))
    rp.cache.check()
  assert rp.cache.all_pages_free(), "pages were not all given back"
  assert not rp.cache.live_requests()
  return outs


_SEEN = {"max": 0.0, "mean": 0.0}


def _bf16_check(got, want, what):
  scale = np.abs(want).max()
  err = np.abs(got - want)
  _SEEN["max"], _SEEN["mean"] = max(_SEEN["max"], err.max() / scale), max(_SEEN["mean"], err.mean() / scale)
  print(f"bf16 {what}: max {err.max() / scale:.5f} mean {err.mean() / scale:.5f} of the largest logit; "
        f"worst so far {_SEEN['max']:.5f} / {_SEEN['mean']:.5f}", flush=True)
  # seen on an MI355X over all configurations and regimes: at most 0.8% (max) and 0.13% (mean) of the largest logit
  assert err.max() <= 0.015 * scale, f"{what}: max err {err.max():.4g} vs scale {scale:.4g}"
  assert err.mean() <= 0.0025 * scale, f"{what}: mean err {err.mean():.4g} vs scale {scale:.4g}"
  # the top token agrees wherever the plain margin is clear
  top = want.argmax(-1)
  srt = np.sort(want, -1)
  clear = (srt[:, -1] - srt[:, -2]) > 0.08 * scale
  assert (got.argmax(-1)[clear] == top[clear]).all(), f"{what}: top token differs at a clear margin"


REGIMES = {
  "whole": lambda r: tt.whole(r),
  "tail_decoded": lambda r: tt.tail_decoded(r, 32),
  "portions": lambda r: tt.portions(r),
  "mixed": lambda r: tt.mixed(r, max_live=4, seed=3),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
@pytest.mark.parametrize("regime", list(REGIMES))
def test_regime(tmp_path, name, dtype, regime):
  file_dtype = torch.float32 if dtype == "float32" else torch.bfloat16
  cfg, w = tm.make_model(str(tmp_path / "m"), name, seed=7, dtype=file_dtype, std=0.05, sharpen=SHARPEN.get((name, dtype), 1.0))
  requests = _requests(name, cfg)
  want = _plain_logits(cfg, w, requests)
  steps = REGIMES[regime](requests)
  max_tokens = tt.peak_tokens(steps, requests)
  print(f"config {name} {dtype} {regime}: {len(steps)} steps, pool for {max_tokens} tokens", flush=True)
  outs = _replay(tmp_path / "m", dtype, steps, requests, tm.PAGE_SIZE[name], max_tokens)
  got = tt.gather(steps, outs, requests, cfg["vocab_size"])
  for rid in requests:
    assert not np.isnan(got[rid]).any()
    if dtype == "float32":
      err = np.abs(got[rid] - want[rid]).max()
      assert err <= FP32_TOL, f"{name} {regime} request {rid}: max abs err {err:.3g}"
    else:
      _bf16_check(got[rid], want[rid], f"{name} {regime} request {rid}")


@pytest.mark.parametrize("name", ["B", "C", "D"])
def test_prefill_variant_for_long_prompts_through_the_engine(tmp_path, name, monkeypatch):
  """The prefill attention's instance with two blocks of query columns per wave is chosen for steps with thousands of
  workgroups; with the threshold lowered to one, the tiny configurations run through it, whole and mixed."""
  from miniinfer_amd.kernels import ops
  monkeypatch.setattr(ops, "PREFILL_WIDE_WORKGROUPS_PER_UNIT", 0)
  seen = []
  real = ops.attn_prefill
  monkeypatch.setattr(ops, "attn_prefill", lambda *a, **k: (seen.append(k.get("variant")), real(*a, **k))[1])
  cfg, w = tm.make_model(str(tmp_path / "m"), name, seed=7, dtype=torch.bfloat16, std=0.05)
  requests = _requests(name, cfg)
  want = _plain_logits(cfg, w, requests)
  for regime in ("whole", "mixed"):
    steps = REGIMES[regime](requests)
    outs = _replay(tmp_path / "m", "bfloat16", steps, requests, tm.PAGE_SIZE[name], tt.peak_tokens(steps, requests))
    got = tt.gather(steps, outs, requests, cfg["vocab_size"])
    for rid in requests:
      _bf16_check(got[rid], want[rid], f"{name} wide prefill {regime} request {rid}")
  assert seen and all(v == "wide" for v in seen)


def _drawn_config(rng):
  """A Qwen3 configuration with every size drawn: head sizes that are and are not multiples of 16, any number of heads
  and groups, widths and vocabularies that are no powers of two, windows in some layers."""
  d = rng.choice([8, 16, 24, 32, 40, 48, 64, 80, 96, 112, 128])
  nkv = rng.choice([1, 2, 3, 4, 5])
  nq = nkv * rng.choice([1, 2, 3, 4, 6, 8])
  layers = rng.choice([1, 2, 3])
  cfg = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=rng.choice([97, 256, 333, 500, 1031]),
             hidden_size=rng.choice([40, 64, 72, 96, 104, 136, 200, 256]),
             intermediate_size=rng.choice([48, 88, 112, 160, 200, 264]), num_hidden_layers=layers,
             num_attention_heads=nq, num_key_value_heads=nkv, head_dim=d, hidden_act="silu",
             max_position_embeddings=rng.choice([512, 1024]), rms_norm_eps=rng.choice([1e-6, 1e-5, 3e-6]),
             rope_theta=rng.choice([1e4, 5e5, 1e6]), tie_word_embeddings=rng.random() < 0.5, attention_bias=False,
             rope_scaling=None)
  if rng.random() < 0.4:
    cfg.update(sliding_window=rng.choice([5, 17, 40, 64, 100]), use_sliding_window=True,
               layer_types=[rng.choice(["full_attention", "sliding_attention"]) for _ in range(layers)])
  return cfg


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("draw", range(12))
def test_drawn_configurations(tmp_path, draw, dtype):
  """Twelve drawn configurations, page sizes and sets of requests, replayed in portions and mixed.  In bfloat16 the
  bound is 3% of the largest logit: over 64 such draws and all four regimes up to 2.0% was seen, the same whether a
  request ran whole or cut (which is what rounding does and a fault of the cache or the batch does not)."""
  import random
  rng = random.Random(4000 + draw)
  cfg = _drawn_config(rng)
  page = rng.choice([8, 16, 32])
  lens = [rng.choice([1, 2, 7, 33, 64, 65, 100, 129, 200, 257, 400]) for _ in range(rng.choice([3, 4, 5]))]
  w = tm.random_weights(cfg, 4000 + draw, std=0.05)
  tm.write_model(str(tmp_path / "m"), cfg, w)
  requests = {f"r{i}": tm.random_tokens(cfg, n, seed=11 * draw + i) for i, n in enumerate(lens)}
  want = _plain_logits(cfg, w, requests)
  for regime, steps in (("portions", tt.portions(requests)), ("mixed", tt.mixed(requests, max_live=4, seed=draw))):
    print(f"draw {draw} {dtype} {regime}: {cfg} page {page} lengths {lens}", flush=True)
    outs = _replay(tmp_path / "m", dtype, steps, requests, page, tt.peak_tokens(steps, requests, granule=max(64, page)))
    got = tt.gather(steps, outs, requests, cfg["vocab_size"])
    for rid in requests:
      err = np.abs(got[rid] - want[rid]).max()
      bound = FP32_TOL if dtype == "float32" else 0.03 * np.abs(want[rid]).max()
      assert err <= bound, f"draw {draw} {regime} request {rid}: max abs err {err:.3g}, bound {bound:.3g}"


def test_first_tokens_and_single_token_prompt(tmp_path):
  """The first tokens of a sequence: position 0 sees one key; a one-token prompt; a two-token portion first."""
  cfg, w = tm.make_model(str(tmp_path / "m"), "B", seed=11, dtype=torch.float32, std=0.05)
  requests = {"a": tm.random_tokens(cfg, 1, 1), "b": tm.random_tokens(cfg, 2, 2), "c": tm.random_tokens(cfg, 3, 3)}
  want = _plain_logits(cfg, w, requests)
  steps = [{"step": 0, "entries": [{"id": r, "tokens": t, "want": list(range(len(t)))} for r, t in requests.items()],
            "end": list(requests)}]
  outs = _replay(tmp_path / "m", "float32", steps, requests, 8, 256)
  got = tt.gather(steps, outs, requests, cfg["vocab_size"])
  for rid in requests:
    assert np.abs(got[rid] - want[rid]).max() <= FP32_TOL


def test_long_decoding(tmp_path):
  """A short prompt and then hundreds of single-token steps, across many page edges."""
  cfg, w = tm.make_model(str(tmp_path / "m"), "C", seed=5, dtype=torch.float32, std=0.05)
  toks = tm.random_tokens(cfg, 700, 9)
  requests = {"long": toks}
  want = _plain_logits(cfg, w, requests)
  steps = tt.tail_decoded(requests, tail=690)
  outs = _replay(tmp_path / "m", "float32", steps, requests, 16, 704)
  got = tt.gather(steps, outs, requests, cfg["vocab_size"])
  assert np.abs(got["long"] - want["long"]).max() <= FP32_TOL


def test_wanted_rows_only(tmp_path):
  """`want` picks places; an empty `want` writes nothing; the rest of the step is unchanged."""
  cfg, w = tm.make_model(str(tmp_path / "m"), "A", seed=2, dtype=torch.float32, std=0.05)
  toks = tm.random_tokens(cfg, 40, 4)
  want = _plain_logits(cfg, w, {"a": toks})["a"]
  from miniinfer_amd.engine.replay import Replayer
  rp = Replayer(str(tmp_path / "m"), "float32", 64, page_size=16)
  assert rp.step({"step": 0, "entries": [{"id": "a", "tokens": toks[:10], "want": []}], "end": []}) is None
  out = rp.step({"step": 1, "entries": [{"id": "a", "tokens": toks[10:40], "want": [29, 0, 7]}], "end": ["a"]})
  assert out.shape == (3, cfg["vocab_size"])
  for r, p in enumerate([39, 10, 17]):
    assert np.abs(out[r] - want[p]).max() <= FP32_TOL


def test_trace_run_program(tmp_path):
  """bin/trace_run as a user calls it: JSON lines on stdin, <step>.f32 files, `done <step>` lines."""
  import json
  import os
  import subprocess
  import sys
  cfg, w = tm.make_model(str(tmp_path / "m"), "A", seed=3, dtype=torch.float32, std=0.05)
  requests = {"x": tm.random_tokens(cfg, 50, 1), "y": tm.random_tokens(cfg, 21, 2)}
  want = _plain_logits(cfg, w, requests)
  steps = tt.mixed(requests, max_live=2, seed=1)
  root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
  inp = "".join(json.dumps(s) + "\n" for s in steps)
  out_dir = tmp_path / "out"
  proc = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(tmp_path / "m"),
                         "--dtype", "float32", "--out", str(out_dir), "--max-tokens", "128"],
                        input=inp, capture_output=True, text=True, timeout=300)
  assert proc.returncode == 0, proc.stderr[-2000:]
  assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {s['step']}" for s in steps]
  outs = []
  for s in steps:
    n = sum(len(e["want"]) for e in s["entries"])
    arr = np.fromfile(out_dir / f"{s['step']}.f32", dtype="<f4").reshape(n, cfg["vocab_size"]) if n else None
    outs.append(arr)
  got = tt.gather(steps, outs, requests, cfg["vocab_size"])
  for rid in requests:
    assert np.abs(got[rid] - want[rid]).max() <= FP32_TOL
