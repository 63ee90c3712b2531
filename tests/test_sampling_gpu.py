"""The sampling kernel against the plain statement of the distribution it draws from."""

import numpy as np
import pytest
import torch

import plain_qwen3 as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _draws(logits_row, temperature, top_k, top_p, n):
  """n draws from one row of logits with seeds 0..n-1."""
  from miniinfer_amd.kernels import ops
  V = logits_row.numel()
  logits = logits_row.to(DEV).float().expand(n, V).contiguous()
  out = torch.empty(n, dtype=torch.int32, device=DEV)
  f = lambda v, dt: torch.full((n,), v, dtype=dt, device=DEV)
  ops.sample(logits, f(temperature, torch.float32), f(top_k, torch.int32), f(top_p, torch.float32),
             torch.arange(n, dtype=torch.int64, device=DEV) * 7919 + 13, f(5, torch.int64), out)
  return out.cpu().numpy()


def test_greedy_lowest_index_wins_ties():
  from miniinfer_amd.kernels import ops
  g = torch.Generator().manual_seed(0)
  logits = torch.randn(7, 1531, generator=g)
  logits[3, 100] = logits[3, 900] = 50.0
  out = torch.empty(7, dtype=torch.int32, device=DEV)
  ops.sample(logits.to(DEV), None, None, None, None, None, out)
  want = logits.argmax(-1)
  want[3] = 100
  assert out.cpu().tolist() == want.tolist()
  # temperature 0 in a mixed batch is argmax too (the pitfall the reference hit with a fused softmax:
  # docs/Logger_Loader_MoE_与采样器乱码修复.md:167-182)
  temp = torch.tensor([0, 1, 0, 0, 2, 0, 0], dtype=torch.float32, device=DEV)
  z = torch.zeros(7, dtype=torch.int64, device=DEV)
  ops.sample(logits.to(DEV), temp, None, None, z, z, out)
  got = out.cpu().tolist()
  assert [got[i] for i in (0, 2, 3, 5, 6)] == [want.tolist()[i] for i in (0, 2, 3, 5, 6)]


@pytest.mark.parametrize("temperature,top_k,top_p", [(1.0, 0, 1.0), (0.7, 0, 1.0), (1.3, 5, 1.0), (1.0, 0, 0.6),
                                                     (0.9, 8, 0.8)])
def test_frequencies_match_distribution(temperature, top_k, top_p):
  g = torch.Generator().manual_seed(1)
  V = 37
  row = torch.randn(V, generator=g) * 1.5
  want = plain.sampling_distribution(row, temperature, top_k, top_p).numpy()
  n = 40000
  got = np.bincount(_draws(row, temperature, top_k, top_p, n), minlength=V) / n
  assert (got[want == 0] == 0).all(), "a filtered token was drawn"
  # chi-square against the plain distribution
  keep = want > 0
  chi2 = n * ((got[keep] - want[keep]) ** 2 / want[keep]).sum()
  dof = keep.sum() - 1
  assert chi2 < dof + 5 * np.sqrt(2 * dof) + 10, f"chi2={chi2:.1f} for {dof} degrees of freedom"


def test_low_temperature_is_argmax_and_large_vocab():
  g = torch.Generator().manual_seed(2)
  row = torch.randn(151936, generator=g)
  assert (_draws(row, 1e-3, 0, 1.0, 16) == int(row.argmax())).all()
  # top_k = 1 is argmax at any temperature
  assert (_draws(row, 2.0, 1, 1.0, 16) == int(row.argmax())).all()


def test_same_stream_same_token_whatever_the_batch():
  from miniinfer_amd.kernels import ops
  g = torch.Generator().manual_seed(3)
  logits = torch.randn(5, 777, generator=g).to(DEV)
  temp = torch.full((5,), 0.9, device=DEV)
  seeds = torch.tensor([11, 22, 33, 44, 55], dtype=torch.int64, device=DEV)
  steps = torch.tensor([0, 3, 9, 1, 2], dtype=torch.int64, device=DEV)
  out = torch.empty(5, dtype=torch.int32, device=DEV)
  ops.sample(logits, temp, None, None, seeds, steps, out)
  one = torch.empty(1, dtype=torch.int32, device=DEV)
  for r in range(5):
    ops.sample(logits[r:r + 1].contiguous(), temp[r:r + 1].contiguous(), None, None, seeds[r:r + 1].contiguous(),
               steps[r:r + 1].contiguous(), one)
    assert int(one) == int(out[r])
