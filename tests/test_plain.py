"""Pins the plain implementation by what fixes it beside the reference's text: library routines for special
cases, vectors the reference's own tests hold, and invariants, each chosen so that a plausible mistake fails."""

import math

import pytest
import torch

import plain_qwen3 as plain
import tiny_models as tm


def test_rms_norm_equals_library_routine():
  # the reference's own check: tests/unittests/test_norm_mlp.py:13-25 (100 inputs [100, 111], eps 1e-5)
  g = torch.Generator().manual_seed(0)
  for _ in range(10):
    x = torch.randn(100, 111, generator=g)
    w = torch.randn(111, generator=g)
    torch.testing.assert_close(plain.rms_norm(x, w, 1e-5), torch.nn.functional.rms_norm(x, (111,), w, 1e-5))


def test_rms_norm_unit_rms_and_scale_invariance():
  x = torch.randn(7, 64, dtype=torch.float64)
  y = plain.rms_norm(x, torch.ones(64, dtype=torch.float64), 0.0)
  torch.testing.assert_close(y.pow(2).mean(-1), torch.ones(7, dtype=torch.float64))
  torch.testing.assert_close(plain.rms_norm(3.7 * x, torch.ones(64, dtype=torch.float64), 0.0), y)
  # the weight multiplies directly, it is not (1 + w)
  assert torch.equal(plain.rms_norm(x, torch.zeros(64, dtype=torch.float64), 1e-6), torch.zeros_like(x))


def test_rope_is_complex_multiplication_on_half_split_pairs():
  # the reference's test helper states the rotation as complex multiplication: tests/utils.py:12-17,65-116
  d, theta = 16, 10000.0
  x = torch.randn(9, 3, d, dtype=torch.float64)
  pos = torch.arange(9) + 5
  ang = plain.rope_angles(pos, d, theta, torch.float64)
  freqs = 1.0 / (theta ** (torch.arange(0, d, 2, dtype=torch.float64)[: d // 2] / d))
  cis = torch.polar(torch.ones(9, d // 2, dtype=torch.float64), torch.outer(pos.double(), freqs))
  z = torch.complex(x[..., : d // 2], x[..., d // 2:]) * cis[:, None, :]
  want = torch.cat((z.real, z.imag), -1)
  torch.testing.assert_close(plain.apply_rope_neox(x, ang), want)
  # an interleaved pairing (x[0], x[1]), a wrong sign, or a wrong frequency exponent all fail this


def test_rope_invariants():
  d, theta = 32, 1e6
  q = torch.randn(1, 1, d, dtype=torch.float64)
  k = torch.randn(1, 1, d, dtype=torch.float64)
  rot = lambda x, p: plain.apply_rope_neox(x, plain.rope_angles(torch.tensor([p]), d, theta, torch.float64))
  # position 0 is the identity
  torch.testing.assert_close(rot(q, 0), q)
  # norms of pairs are kept
  r = rot(q, 77)
  torch.testing.assert_close(r[..., : d // 2] ** 2 + r[..., d // 2:] ** 2, q[..., : d // 2] ** 2 + q[..., d // 2:] ** 2)
  # <rope(q, m), rope(k, n)> depends on m - n only
  a = (rot(q, 10) * rot(k, 3)).sum()
  b = (rot(q, 110) * rot(k, 103)).sum()
  c = (rot(q, 11) * rot(k, 3)).sum()
  torch.testing.assert_close(a, b)
  assert abs(a - c) > 1e-6


def test_causal_mask_vectors_of_the_reference():
  # tests/unittests/test_gqa.py:105-148
  ninf = -math.inf
  assert torch.equal(plain.causal_mask(3, 3), torch.tensor([[0, ninf, ninf], [0, 0, ninf], [0, 0, 0]]))
  assert torch.equal(plain.causal_mask(3, 5),
                     torch.tensor([[0, 0, 0, ninf, ninf], [0, 0, 0, 0, ninf], [0, 0, 0, 0, 0]]))


def test_attention_reduces_to_library_routine():
  # plain attention without rotation: equals scaled_dot_product_attention with repeated kv heads
  g = torch.Generator().manual_seed(1)
  L, nq, nkv, d = 7, 6, 2, 8
  q, k, v = (torch.randn(L, n, d, generator=g) for n in (nq, nkv, nkv))
  got = plain.grouped_attention(q, k, v, d ** -0.5, plain.causal_mask(L, L))
  rep = nq // nkv
  want = torch.nn.functional.scaled_dot_product_attention(
    q.transpose(0, 1)[None], k.repeat_interleave(rep, 1).transpose(0, 1)[None],
    v.repeat_interleave(rep, 1).transpose(0, 1)[None], is_causal=True, scale=d ** -0.5)[0].transpose(0, 1)
  torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-6)
  # no mask, scale 0.8, the shapes of the reference's grouped test (tests/unittests/test_gqa.py:18-88: 18/6 heads)
  q, k, v = torch.randn(3, 18, 5, generator=g), torch.randn(7, 6, 5, generator=g), torch.randn(7, 6, 5, generator=g)
  got = plain.grouped_attention(q, k, v, 0.8, None)
  want = torch.nn.functional.scaled_dot_product_attention(
    q.transpose(0, 1)[None], k.repeat_interleave(3, 1).transpose(0, 1)[None],
    v.repeat_interleave(3, 1).transpose(0, 1)[None], scale=0.8)[0].transpose(0, 1)
  torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-6)


def test_attention_head_mapping_and_single_key():
  # query head h reads kv head h // (nq / nkv): make the kv heads differ
  nq, nkv, d = 4, 2, 4
  q = torch.randn(1, nq, d)
  k = torch.randn(1, nkv, d)
  v = torch.stack([torch.full((d,), 1.0), torch.full((d,), 2.0)])[None]   # [1, nkv, d]
  out = plain.grouped_attention(q, k, v, 0.5, None)
  assert torch.equal(out[0, :, 0], torch.tensor([1.0, 1.0, 2.0, 2.0]))   # a single key: the output is its value


def test_swiglu_equals_library_and_gate_up_order():
  g = torch.Generator().manual_seed(2)
  x, wg, wu, wd = torch.randn(5, 12, generator=g), torch.randn(20, 12, generator=g), torch.randn(20, 12, generator=g), \
      torch.randn(12, 20, generator=g)
  want = (torch.nn.functional.silu(x @ wg.T) * (x @ wu.T)) @ wd.T
  torch.testing.assert_close(plain.swiglu(x, wg, wu, wd), want)
  assert torch.equal(plain.swiglu(x, wg, torch.zeros_like(wu), wd), torch.zeros(5, 12))
  assert torch.equal(plain.swiglu(x, torch.zeros_like(wg), wu, wd), torch.zeros(5, 12))   # silu(0) = 0
  assert not torch.allclose(plain.swiglu(x, wu, wg, wd), want)   # swapping gate and up changes the result


def test_model_position_shift_changes_nothing_but_rounding():
  """Only distances count: the logits of a whole sequence do not depend on where its positions start."""
  cfg = dict(tm.TINY_B)
  w = {k: v.double() for k, v in tm.random_weights(cfg, 3, std=0.05).items()}
  toks = tm.random_tokens(cfg, 12, 1)
  a = plain.qwen3_logits(toks, w, cfg, start_pos=0)
  b = plain.qwen3_logits(toks, w, cfg, start_pos=100)
  torch.testing.assert_close(a, b, rtol=1e-9, atol=1e-9)


def test_model_causality_and_one_layer_by_hand():
  cfg = dict(tm.TINY_A)
  w = tm.random_weights(cfg, 4, std=0.05)
  toks = tm.random_tokens(cfg, 10, 2)
  full = plain.qwen3_logits(toks, w, cfg)
  torch.testing.assert_close(plain.qwen3_logits(toks[:6], w, cfg), full[:6], rtol=1e-5, atol=1e-6)
  # tied head: logits = h E^T; deleting lm_head from an untied model gives the tied behaviour
  cfgb = dict(tm.TINY_B)
  wb = tm.random_weights(cfgb, 5, std=0.05)
  tb = tm.random_tokens(cfgb, 5, 3)
  untied = plain.qwen3_logits(tb, wb, cfgb)
  wb2 = dict(wb)
  head = wb2.pop("lm_head.weight")
  tied = plain.qwen3_logits(tb, wb2, cfgb)
  assert not torch.allclose(untied, tied)
  wb2["lm_head.weight"] = wb2["model.embed_tokens.weight"]
  torch.testing.assert_close(plain.qwen3_logits(tb, wb2, cfgb), tied)


def test_fused_projection_split():
  # split(x W_qkv^T) == (x Wq^T, x Wk^T, x Wv^T): tests/unittests/test_weight_loader.py:34
  x, wq, wk, wv = torch.randn(3, 8), torch.randn(6, 8), torch.randn(4, 8), torch.randn(4, 8)
  fused = x @ torch.cat([wq, wk, wv]).T
  q, k, v = fused.split([6, 4, 4], -1)
  torch.testing.assert_close(q, x @ wq.T)
  torch.testing.assert_close(k, x @ wk.T)
  torch.testing.assert_close(v, x @ wv.T)


def test_sampling_distribution():
  lg = torch.tensor([2.0, 1.0, 0.0, -1.0])
  p = plain.sampling_distribution(lg, 1.0)
  torch.testing.assert_close(p, torch.softmax(lg.double(), -1))
  assert plain.sampling_distribution(lg, 0.0).tolist() == [1, 0, 0, 0]
  p = plain.sampling_distribution(lg, 1.0, top_k=2)
  assert p[2] == 0 and p[3] == 0 and abs(p.sum() - 1) < 1e-12
  # top_p: the smallest set of most probable tokens whose mass reaches p
  p = plain.sampling_distribution(lg, 1.0, top_p=0.7)   # 0.644 < 0.7 <= 0.644 + 0.237
  assert (p > 0).tolist() == [True, True, False, False]
  p = plain.sampling_distribution(lg, 0.01)
  assert p[0] > 0.999999


def test_window_mask_reduces_to_the_causal_mask_and_to_one_key():
  """A window at least as long as the sequence changes nothing; a window of one key leaves each query its own
  key, so attention returns that key's value; in between, query p sees exactly keys p - window + 1 .. p."""
  L, S = 5, 9
  assert torch.equal(plain.causal_mask(L, S, window=S), plain.causal_mask(L, S))
  m = plain.causal_mask(L, S, window=3)
  for i in range(L):
    p = i + S - L
    assert [j for j in range(S) if m[i, j] == 0] == [j for j in range(p - 2, p + 1) if j >= 0]
  g = torch.Generator().manual_seed(3)
  q, k, v = (torch.randn(6, 2, 8, generator=g) for _ in range(3))
  out = plain.grouped_attention(q, k, v, 0.3, plain.causal_mask(6, 6, window=1))
  assert torch.allclose(out, v, atol=1e-6)


def test_layer_windows_follow_the_config_keys():
  cfg = dict(tm.TINY_D)
  assert [plain.layer_window(cfg, i) for i in range(4)] == [None, 40, 40, None]
  old = dict(tm.TINY_A, use_sliding_window=True, sliding_window=7, max_window_layers=1)
  assert [plain.layer_window(old, i) for i in range(2)] == [None, 7]
  assert plain.layer_window(dict(tm.TINY_A), 0) is None
  # a sliding layer changes the logits only from the first position that has more keys than the window
  w = tm.random_weights(cfg, 1, std=0.05)
  toks = tm.random_tokens(cfg, 60, 2)
  a = plain.qwen3_logits(toks, w, cfg)
  b = plain.qwen3_logits(toks, w, dict(cfg, layer_types=["full_attention"] * 4))
  assert torch.allclose(a[:40], b[:40], atol=1e-5) and (a[40:] - b[40:]).abs().max() > 1e-3


def test_plain_attention_key_ranges():
  """The one-wave-per-head kernel's key ranges: whole for prompt portions and short contexts, cut for few tokens
  over many keys, never shorter than one tile, never more than 64."""
  from miniinfer_amd.parts.attention import plain_splits
  assert plain_splits(2048 * 16, 2048) == 1
  assert plain_splits(8 * 16, 100) == 2
  assert plain_splits(8 * 16, 2048) == 32 and plain_splits(8 * 8, 2048) == 32
  assert plain_splits(1, 700) == 11
  assert plain_splits(1, 1 << 20) == 64
  assert plain_splits(4096, 1 << 20) == 1
  # the kernel with four lanes a key holds 8 waves a compute unit: 8 requests x 8 kv heads get 32 ranges of 2,100 keys'
  # 33 tiles (a 33rd range would start a second round of waves), and it takes 8 query heads of a kv head as 2 waves
  import torch
  from miniinfer_amd.kernels import ops
  assert ops.plain_attention_geometry(torch.float32, 16, 8, 128, 16) == (2, 8)
  assert ops.plain_attention_geometry(torch.float32, 16, 2, 64, 32) == (4, 8)
  assert ops.plain_attention_geometry(torch.float32, 16, 2, 48, 16) == (8, 16)      # head size without the kernel
  assert ops.plain_attention_geometry(torch.float32, 16, 8, 128, 8) == (2, 16)      # pages too small for it
  assert ops.plain_attention_geometry(torch.bfloat16, 15, 5, 128, 16) == (1, 16)
  assert plain_splits(8 * 8, 2100, 8 * 256) == 32
