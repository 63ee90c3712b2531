"""The attention kernels at the sequence lengths that the measurements quote: prompts of 2,048 and 8,192 new
tokens, 1,000 new tokens over 7,000 cached ones, decoding over 8,192 and 32,768 keys with the number of key ranges
that the engine's own rule picks.  Each against a plain torch statement in 64-bit, computed in blocks of queries.

Random keys make every softmax nearly flat, so a key wrongly left out moves the result by 1/keys only; each case
therefore also plants keys that stand out for a few queries (their scores far above the rest), at places chosen
where an indexing fault would hide: the very first key, the last key of a macro tile, the first key of a page far
into the block table, a key just past a power of two.  The output at those queries must be the planted key's value.
"""

import math

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _ref_blockwise(q, k, v, scale, window, first_pos, block=512):
  """q [L, nq, d] at positions first_pos + i over keys k, v [S, nkv, d]; 64-bit, `block` queries at a time."""
  L, nq, d = q.shape
  S, nkv, _ = k.shape
  rep = nq // nkv
  kk = k.double().repeat_interleave(rep, dim=1)
  vv = v.double().repeat_interleave(rep, dim=1)
  out = torch.empty(L, nq, d, dtype=torch.float64)
  jj = torch.arange(S)[None, :]
  for l0 in range(0, L, block):
    l1 = min(L, l0 + block)
    pos = first_pos + torch.arange(l0, l1)[:, None]
    s = torch.einsum("lhd,shd->hls", q[l0:l1].double(), kk) * scale
    mask = jj > pos
    if window:
      mask = mask | (jj <= pos - window)
    s = s.masked_fill(mask[None], -math.inf)
    out[l0:l1] = torch.einsum("hls,shd->lhd", torch.softmax(s, -1), vv)
  return out


def _pages_of(k, v, P, gen, dtype):
  """Keys and values [S, nkv, d] laid into pages in a random order: key pages [n + 1, nkv, P, d], transposed value
  pages [n + 1, nkv, d, P], and the block table row."""
  S, nkv, d = k.shape
  n = -(-S // P)
  order = (torch.randperm(n, generator=gen) + 1)
  kp = torch.zeros(n + 1, nkv, P, d, dtype=dtype)
  vp = torch.zeros(n + 1, nkv, d, P, dtype=dtype)
  pad = n * P - S
  kk = torch.cat((k, torch.zeros(pad, nkv, d, dtype=k.dtype)), 0).view(n, P, nkv, d).to(dtype)
  vv = torch.cat((v, torch.zeros(pad, nkv, d, dtype=v.dtype)), 0).view(n, P, nkv, d).to(dtype)
  kp[order] = kk.permute(0, 2, 1, 3)
  vp[order] = vv.permute(0, 2, 3, 1)
  return kp, vp, order.to(torch.int32)


def _plant(q, k, rows_and_keys, nq, nkv, strength=6.0):
  """Makes key `j` stand out for query row `i` (all heads): the key becomes the query's direction, scaled."""
  rep = nq // nkv
  for i, j in rows_and_keys:
    for g in range(nkv):
      qh = q[i, g * rep].float()
      k[j, g] = (qh / qh.norm() * strength * math.sqrt(q.shape[-1])).to(k.dtype)
      for h in range(g * rep, (g + 1) * rep):       # the group's other heads look the same way
        q[i, h] = q[i, g * rep]


PREFILL_CASES = [  # (cached, new tokens)
  (0, 2048), (0, 8192), (7000, 1000)]


_CASES = {}


def _prefill_case(nq, nkv, d, P, past, new):
  """Queries, paged keys and values (values a bfloat16 can hold, so that both precisions read the same numbers) and
  the plain result; made once for all kernel variants."""
  key = (nq, nkv, d, P, past, new)
  if key not in _CASES:
    g = torch.Generator().manual_seed(past + new + d)
    S = past + new
    q = torch.randn(new, nq, d, generator=g).bfloat16()
    k = torch.randn(S, nkv, d, generator=g).bfloat16()
    v = torch.randn(S, nkv, d, generator=g).bfloat16()
    # (query row, key): the first key seen from the last row; the last key of a 64-key tile seen from a middle row;
    # a row's own key; the first key of a page past 256 table entries (when the sequence is that long)
    plants = [(new - 1, 0), (new // 2, ((past + new // 2) // 64) * 64 - 1), (new - 7, past + new - 7)]
    if S > 257 * P + 3:
      plants.append((new - 3, 257 * P))
    _plant(q, k, plants, nq, nkv)
    want = _ref_blockwise(q, k, v, d ** -0.5, 0, past)
    for i, j in plants:          # the plain statement itself finds the planted keys
      torch.testing.assert_close(want[i, 0], v[j, 0].double(), rtol=0, atol=5e-2)
    kp, vp, order = _pages_of(k, v, P, g, torch.bfloat16)
    _CASES[key] = (q, kp, vp, order, want)
  return _CASES[key]


@pytest.mark.parametrize("variant", ["two_tiles", "dense", "wide", "plain", "plain32"])
@pytest.mark.parametrize("past,new", PREFILL_CASES)
@pytest.mark.parametrize("nq,nkv,d,P", [(4, 2, 128, 16), (3, 1, 64, 8)])
def test_prefill_attention_at_benchmark_lengths(nq, nkv, d, P, past, new, variant):
  from miniinfer_amd.kernels import ops
  print(f"prefill attention {variant}: heads {nq}/{nkv} of {d}, page {P}, {new} new tokens over {past}", flush=True)
  dtype = torch.float32 if variant == "plain32" else torch.bfloat16
  S = past + new
  q, kp, vp, order, want = _prefill_case(nq, nkv, d, P, past, new)
  i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
  qd = q.reshape(new, nq * d).to(dtype).to(DEV)
  kp, vp = kp.to(dtype).to(DEV), vp.to(dtype).to(DEV)
  out = torch.zeros(new, nq * d, dtype=dtype, device=DEV)
  table = order.view(1, -1).to(DEV)
  if variant.startswith("plain"):
    ops.paged_attention(qd, nq, nkv, d, out, kp, vp, table, torch.zeros(new, dtype=torch.int32, device=DEV),
                        i32([0, new]), i32([S]), d ** -0.5, 0)
  else:
    tpb = ops.attn_prefill_tokens_per_block(nq, nkv, d, wide=variant == "wide")
    work = [(0, b) for b in range(-(-new // tpb))]
    ops.attn_prefill(qd, nq, nkv, d, out, kp, vp, table, i32(work), i32([0, new]), i32([S]), d ** -0.5, 0,
                     variant=variant)
  got = out.double().cpu().view(new, nq, d)
  if dtype == torch.float32:
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-5)
  else:
    torch.testing.assert_close(got, want, rtol=1.6e-2, atol=1e-2)


@pytest.mark.parametrize("front", [False, True])
@pytest.mark.parametrize("lens", [[8192], [32768], [32768, 8191, 100, 8193, 20000, 1, 4097, 12000]])
def test_decode_attention_at_long_contexts_with_the_engines_own_split_counts(lens, front):
  """Qwen3-0.6B's head geometry (16 query heads, 8 kv heads of 128, pages of 16): one request of 8,192 and of 32,768
  keys, and eight requests of mixed lengths, cut into as many key ranges as `decode_splits` gives the engine."""
  from miniinfer_amd.kernels import ops
  from miniinfer_amd.parts.attention import decode_splits
  nq, nkv, d, P = 16, 8, 128, 16
  B = len(lens)
  tile_keys, waves = ops.attn_decode_geometry(d)
  splits = decode_splits(B * nkv, max(lens), tile_keys, waves)
  print(f"decode attention: {B} requests of {lens} keys, {splits} key ranges, fused front {front}", flush=True)
  assert splits == ({8192: 32, 32768: 64}[lens[0]] if B == 1 else 8)
  g = torch.Generator().manual_seed(sum(lens))
  qs, kps, vps, rows, wants = [], [], [], [], []
  base = 0
  eps = 1e-6
  for b, S in enumerate(lens):
    q = torch.randn(1, nq, d, generator=g).bfloat16()
    k = torch.randn(S, nkv, d, generator=g).bfloat16()
    v = torch.randn(S, nkv, d, generator=g).bfloat16()
    # a far key stands out: the first key of the sequence for even requests, the first key of the last-but-one key
    # range for odd ones
    far = 0 if b % 2 == 0 else max(0, (S // splits) * (splits - 2))
    if S > 1:
      _plant(q, k, [(0, far)], nq, nkv)
    wants.append(_ref_blockwise(q, k, v, d ** -0.5, 0, S - 1).view(1, nq * d))
    if S > 1:
      torch.testing.assert_close(wants[-1][0, :d], v[far, 0].double(), rtol=0, atol=5e-2)
    kp, vp, order = _pages_of(k, v, P, g, torch.bfloat16)
    qs.append(q.view(1, nq * d))
    kps.append(kp[1:])
    vps.append(vp[1:])
    rows.append(order + base)
    base += kp.shape[0] - 1
  W = max(r.numel() for r in rows)
  table = torch.zeros(B, W, dtype=torch.int32)
  for b, r in enumerate(rows):
    table[b, :r.numel()] = r
  kp = torch.cat([torch.zeros(1, nkv, P, d, dtype=torch.bfloat16)] + kps, 0).to(DEV)
  vp = torch.cat([torch.zeros(1, nkv, d, P, dtype=torch.bfloat16)] + vps, 0).to(DEV)
  i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
  want = torch.cat(wants, 0)
  out = torch.zeros(B, nq * d, dtype=torch.bfloat16, device=DEV)
  part_o = torch.empty(B * nq * splits * d, dtype=torch.float32, device=DEV)
  part_ml = torch.empty(B * nq * splits * 2, dtype=torch.float32, device=DEV)
  cu, kv = i32(list(range(B + 1))), i32(lens)
  if not front:
    ops.attn_decode(torch.cat(qs, 0).to(DEV), nq, nkv, d, out, kp, vp, table.to(DEV), cu, kv, 0, B, splits, part_o,
                    part_ml, d ** -0.5, 0)
  else:
    # the raw projection: the kernel itself norms nothing here (no weights) and rotates nothing (no table), but it
    # takes the new key and value from the projection's row and writes them to the cache slot of the last position
    qkv = torch.zeros(B, (nq + 2 * nkv) * d, dtype=torch.bfloat16)
    slots = []
    for b, S in enumerate(lens):
      page = int(table[b, (S - 1) // P])
      slot = page * P + (S - 1) % P
      slots.append(slot)
      qkv[b, :nq * d] = qs[b][0]
      qkv[b, nq * d:(nq + nkv) * d] = kp[page, :, (S - 1) % P, :].reshape(-1).cpu()
      qkv[b, (nq + nkv) * d:] = vp[page, :, :, (S - 1) % P].reshape(-1).cpu()
      kp[page, :, (S - 1) % P, :] = 0        # the cache does not hold the new token yet
      vp[page, :, :, (S - 1) % P] = 0
    ops.attn_decode_front(qkv.to(DEV), nq, nkv, d, out, kp, vp, table.to(DEV), cu, kv, 0, B, splits, part_o, part_ml,
                          d ** -0.5, 0, None, None, eps, None, i32([s - 1 for s in lens]), i32(slots))
  torch.testing.assert_close(out.double().cpu(), want, rtol=1.6e-2, atol=1e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_plain_decode_attention_over_32768_keys(dtype):
  """The one-wave-per-head kernel (the 32-bit path's attention) with the key ranges `plain_splits` gives a single
  decoding request of 32,768 keys."""
  from miniinfer_amd.kernels import ops
  from miniinfer_amd.parts.attention import plain_splits
  nq, nkv, d, P, S = 6, 3, 48, 16, 32768
  splits = plain_splits(nq, S)
  assert splits > 1
  g = torch.Generator().manual_seed(5)
  q = torch.randn(1, nq, d, generator=g).to(dtype)
  k = torch.randn(S, nkv, d, generator=g).to(dtype)
  v = torch.randn(S, nkv, d, generator=g).to(dtype)
  _plant(q, k, [(0, 4096)], nq, nkv)
  want = _ref_blockwise(q, k, v, d ** -0.5, 0, S - 1).view(1, nq * d)
  torch.testing.assert_close(want[0, :d], v[4096, 0].double(), rtol=0, atol=5e-2)
  kp, vp, order = _pages_of(k, v, P, g, dtype)
  i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
  out = torch.zeros(1, nq * d, dtype=dtype, device=DEV)
  part_o = torch.empty(nq * splits * d, dtype=torch.float32, device=DEV)
  part_ml = torch.empty(nq * splits * 2, dtype=torch.float32, device=DEV)
  ops.paged_attention(q.view(1, nq * d).to(DEV), nq, nkv, d, out, kp.to(DEV), vp.to(DEV), order.view(1, -1).to(DEV),
                      i32([0]), i32([0, 1]), i32([S]), d ** -0.5, 0, splits, part_o, part_ml)
  tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1.6e-2, atol=1e-2)
  torch.testing.assert_close(out.double().cpu(), want, **tol)
