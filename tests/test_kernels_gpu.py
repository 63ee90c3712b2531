"""Each HIP kernel alone against a plain torch statement of the same operation, at sizes other than
the engine tests use (odd widths, vocabularies and head counts that are no power of two)."""

import math

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def _tol(dtype):
  return dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1.6e-2, atol=1e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("V,H,T", [(500, 80, 7), (1000, 1024, 33), (37, 3, 1)])
def test_embed(dtype, V, H, T):
  from miniinfer_amd.kernels import ops
  g = torch.Generator().manual_seed(0)
  table = torch.randn(V, H, generator=g).to(dtype).to(DEV)
  ids = torch.randint(0, V, (T,), generator=g).to(torch.int32).to(DEV)
  out = torch.empty(T, H, dtype=torch.float32, device=DEV)
  ops.embed(table, ids, out)
  assert torch.equal(out, table.float()[ids.long()])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,N", [(5, 80), (3, 1024), (17, 111), (2, 5120), (4, 7)])
def test_add_rmsnorm(dtype, M, N):
  from miniinfer_amd.kernels import ops
  g = torch.Generator().manual_seed(1)
  x = (torch.randn(M, N, generator=g) * 3).to(dtype).to(DEV)
  r = (torch.randn(M, N, generator=g) * 3).to(DEV)
  w = (1 + 0.1 * torch.randn(N, generator=g)).to(DEV)
  eps = 1e-5
  want_r = r + x.float()
  want = torch.nn.functional.rms_norm(want_r, (N,), w, eps)
  out = torch.empty(M, N, dtype=dtype, device=DEV)
  r2 = r.clone()
  ops.add_rmsnorm(x, r2, w, eps, out, write_back=True)
  torch.testing.assert_close(r2, want_r, rtol=1e-6, atol=1e-6)
  torch.testing.assert_close(out.float(), want, **_tol(dtype))
  # plain norm of x alone, the reference's own check (tests/unittests/test_norm_mlp.py:13-25)
  out2 = torch.empty(M, N, dtype=dtype, device=DEV)
  ops.add_rmsnorm(x, None, w, eps, out2)
  torch.testing.assert_close(out2.float(), torch.nn.functional.rms_norm(x.float(), (N,), w, eps), **_tol(dtype))
  # selected rows, residual untouched
  rows = torch.tensor([M - 1, 0], dtype=torch.int32, device=DEV)
  out3 = torch.empty(2, N, dtype=dtype, device=DEV)
  r3 = r.clone()
  ops.add_rmsnorm(x, r3, w, eps, out3, rows=rows)
  assert torch.equal(r3, r)
  torch.testing.assert_close(out3.float(), want[rows.long()], **_tol(dtype))


def test_rmsnorm_large_values_do_not_overflow():
  """bfloat16 inputs of magnitude 1e3 (the reference checks fp16 this way: tests/unittests/test_norm_mlp.py:30-43)."""
  from miniinfer_amd.kernels import ops
  x = (torch.randn(4, 256) * 1000).to(torch.bfloat16).to(DEV)
  w = torch.ones(256, device=DEV)
  out = torch.empty_like(x)
  ops.add_rmsnorm(x, None, w, 1e-6, out)
  rms = out.float().pow(2).mean(-1).sqrt()
  torch.testing.assert_close(rms, torch.ones_like(rms), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,I", [(3, 112), (9, 3072), (1, 5)])
def test_silu_mul(dtype, M, I):
  from miniinfer_amd.kernels import ops
  g = torch.Generator().manual_seed(2)
  gu = (torch.randn(M, 2 * I, generator=g) * 2).to(dtype).to(DEV)
  out = torch.empty(M, I, dtype=dtype, device=DEV)
  ops.silu_mul(gu, out)
  want = torch.nn.functional.silu(gu.float()[:, :I]) * gu.float()[:, I:]
  torch.testing.assert_close(out.float(), want, **_tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,N,K", [(1, 500, 80), (7, 130, 96), (65, 64, 17), (33, 1000, 1024), (128, 257, 300),
                                   (5, 1100, 2048), (8, 2049, 512), (3, 4096, 1024)])
def test_gemm_nt(dtype, M, N, K):
  from miniinfer_amd.kernels import ops
  g = torch.Generator().manual_seed(3)
  a = torch.randn(M, K, generator=g).to(dtype).to(DEV)
  w = torch.randn(N, K, generator=g).to(dtype).to(DEV)
  want = a.double() @ w.double().T
  out32 = torch.empty(M, N, dtype=torch.float32, device=DEV)
  ops.gemm_nt(a, w, out32)
  torch.testing.assert_close(out32.double(), want, rtol=1e-5, atol=1e-4)
  out = torch.empty(M, N, dtype=dtype, device=DEV)
  ops.gemm_nt(a, w, out)
  torch.testing.assert_close(out.double(), want, rtol=1e-5 if dtype == torch.float32 else 1e-2,
                             atol=1e-4 if dtype == torch.float32 else 1e-1)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N,K", [(130, 96), (1000, 1030), (48, 17), (1027, 1024), (4096, 768), (601, 3072)])
def test_gemm_nt_rows_do_not_depend_on_the_batch(dtype, N, K):
  """Few rows go to kernels of their own, many to the tiled one: all add a result element's products in the same
  order, so a row's result is the same bits whichever kernel ran it.  (Up to 8 rows in 32-bit with k a multiple of 256
  and row groups for half to all of the compute units take both operands through LDS: the last three shapes, with 4,
  16 and 4 rows of the matrix per workgroup and a last workgroup that is not full.)"""
  from miniinfer_amd.kernels import ops
  g = torch.Generator().manual_seed(4)
  a = torch.randn(40, K, generator=g).to(dtype).to(DEV)
  w = torch.randn(N, K, generator=g).to(dtype).to(DEV)
  many = ops.gemm_nt(a, w, torch.empty(40, N, dtype=torch.float32, device=DEV))
  for rows in (1, 7, 16):
    few = ops.gemm_nt(a[:rows], w, torch.full((rows, N), float("nan"), dtype=torch.float32, device=DEV))
    assert torch.equal(few, many[:rows])


def _rope_ref(x, pos, theta, rotary_dim):
  """Complex multiplication by e^{i pos theta^(-2j/rd)} on pairs (j, j + rd/2): the statement of the
  reference's test helper (tests/utils.py:12-17,65-116)."""
  j = torch.arange(0, rotary_dim, 2, dtype=torch.float32)
  ang = pos.float()[:, None] * (1.0 / theta ** (j / rotary_dim))[None, :]
  cis = torch.polar(torch.ones_like(ang), ang)[:, None, :]
  half = rotary_dim // 2
  z = torch.complex(x[..., :half], x[..., half:rotary_dim]) * cis
  return torch.cat((z.real, z.imag, x[..., rotary_dim:]), dim=-1)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T", [11, 75])
@pytest.mark.parametrize("nq,nkv,d,rd,P", [(6, 3, 48, 48, 16), (4, 4, 128, 128, 8), (5, 1, 16, 16, 4), (2, 2, 80, 32, 16),
                                           (3, 1, 72, 72, 8), (2, 1, 256, 256, 16), (7, 1, 32, 32, 16)])
def test_qk_norm_rope_cache(dtype, nq, nkv, d, rd, P, T):
  _check_qk_norm_rope_cache(dtype, nq, nkv, d, rd, P, T, 0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("offset", [1, 4, 8])
def test_qk_norm_rope_cache_of_a_view(dtype, offset):
  """The many-token kernel reads 4 elements a lane, which it can where the projection lies on a multiple of as many
  bytes, and leaves anything else to the kernel that reads single elements: a projection that starts 1, 4 or 8
  elements into a wider buffer."""
  _check_qk_norm_rope_cache(dtype, 4, 2, 64, 64, 16, 75, offset)


def _check_qk_norm_rope_cache(dtype, nq, nkv, d, rd, P, T, offset):
  from miniinfer_amd.kernels import ops
  g = torch.Generator().manual_seed(4)
  pages, max_pos, theta, eps = 12 + 2 * T // P, 300, 12345.0, 1e-5
  qkv = torch.randn(T, (nq + 2 * nkv) * d, generator=g).to(dtype)
  qw = 1 + 0.1 * torch.randn(d, generator=g)
  kw = 1 + 0.1 * torch.randn(d, generator=g)
  pos = torch.randint(0, max_pos, (T,), generator=g)
  slots = torch.randperm(pages * P, generator=g)[:T] + P   # never page 0
  if T > 32:
    # like a prompt's portion: runs of consecutive slots (16 tokens that fill slots from a multiple of 16 on, a run
    # that starts in the middle of a page, one that starts with a page but not with a block of 16 tokens), then
    # scattered ones
    slots[:16] = torch.arange(16) + 3 * P
    second = ((3 * P + 16) // P + 2) * P + 5
    slots[16:45] = torch.arange(29) + second
    slots[45:66] = torch.arange(21) + ((second + 29) // P + 2) * P
    rest = [x for x in range(P, (pages + 1) * P) if x not in set(slots[:66].tolist())]
    slots[66:] = torch.tensor(rest)[torch.randperm(len(rest), generator=g)[:T - 66]]
  assert len(set(slots.tolist())) == T
  j = torch.arange(0, rd, 2, dtype=torch.float32)
  ang = torch.outer(torch.arange(max_pos, dtype=torch.float32), 1.0 / theta ** (j / rd))
  table = torch.cat((ang.cos(), ang.sin()), -1)

  x = qkv.float().view(T, nq + 2 * nkv, d)
  q, k, v = x[:, :nq], x[:, nq:nq + nkv], x[:, nq + nkv:]
  qn = torch.nn.functional.rms_norm(q, (d,), qw, eps)
  kn = torch.nn.functional.rms_norm(k, (d,), kw, eps)
  q_want, k_want = _rope_ref(qn, pos, theta, rd), _rope_ref(kn, pos, theta, rd)

  wide = torch.zeros(T, qkv.shape[1] + 16, dtype=dtype, device=DEV)
  dq = wide[:, offset:offset + qkv.shape[1]]
  dq.copy_(qkv)
  kp = torch.zeros(pages + 1, nkv, P, d, dtype=dtype, device=DEV)
  vp = torch.zeros(pages + 1, nkv, d, P, dtype=dtype, device=DEV)   # value pages are stored transposed
  ops.qk_norm_rope_cache(dq, nq, nkv, d, qw.to(DEV), kw.to(DEV), eps, table.to(DEV), pos.to(torch.int32).to(DEV),
                         kp, vp, slots.to(torch.int32).to(DEV), P)
  got = dq.float().cpu().view(T, nq + 2 * nkv, d)
  torch.testing.assert_close(got[:, :nq], q_want, **_tol(dtype))
  torch.testing.assert_close(got[:, nq:nq + nkv], k_want, **_tol(dtype))
  assert torch.equal(got[:, nq + nkv:], v)
  kc, vc = kp.float().cpu(), vp.float().cpu().transpose(2, 3)
  for t in range(T):
    page, off = int(slots[t]) // P, int(slots[t]) % P
    assert torch.equal(kc[page, :, off], got[t, nq:nq + nkv])
    assert torch.equal(vc[page, :, off], v[t])
  # nothing else was written
  assert int((kc.abs().sum(-1) > 0).sum()) == T * nkv
  assert not wide[:, :offset].any() and not wide[:, offset + qkv.shape[1]:].any()


def _attention_ref(q, k, v, scale, window):
  """q [L, nq, d], k, v [S, nkv, d]; bottom-right aligned causal mask; float64."""
  L, nq, d = q.shape
  S, nkv, _ = k.shape
  rep = nq // nkv
  kk = k.repeat_interleave(rep, dim=1).double()
  vv = v.repeat_interleave(rep, dim=1).double()
  s = torch.einsum("lhd,shd->hls", q.double(), kk) * scale
  i = torch.arange(L)[:, None] + (S - L)
  jj = torch.arange(S)[None, :]
  mask = jj > i
  if window:
    mask = mask | (jj <= i - window)
  s = s.masked_fill(mask[None], -math.inf)
  return torch.einsum("hls,shd->lhd", torch.softmax(s, -1), vv)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("splits", [1, 2, 3, 7])
@pytest.mark.parametrize("nq,nkv,d,P,window", [(6, 3, 48, 16, 0), (8, 2, 128, 8, 0), (4, 4, 16, 4, 0), (5, 1, 80, 32, 0),
                                               (4, 2, 64, 16, 37), (16, 8, 256, 16, 0), (4, 2, 64, 16, 150),
                                               (8, 2, 128, 16, 0), (8, 1, 96, 64, 0), (16, 8, 128, 32, 101)])
def test_paged_attention(dtype, nq, nkv, d, P, window, splits):
  """Key ranges cut into parts (some of them empty for the short requests) give the same result as whole ones.  In
  32-bit the head sizes 64, 80, 96 and 128 with pages of 16 keys or more run on the kernel with four lanes a key (1,
  2 and 4 query heads a wave, 8 as two waves of 4; windows whose edge is no multiple of 16), the others on the
  kernel with a key a lane."""
  from miniinfer_amd.kernels import ops
  g = torch.Generator().manual_seed(5)
  # requests: (keys already cached, new tokens)
  reqs = [(0, 70), (129, 1), (40, 3), (0, 1), (63, 2), (200, 1), (447, 2)]
  B = len(reqs)
  kv_lens = [a + n for a, n in reqs]
  T = sum(n for _, n in reqs)
  W = max(-(-kv // P) for kv in kv_lens)
  n_pages = sum(-(-kv // P) for kv in kv_lens)
  perm = (torch.randperm(n_pages, generator=g) + 1).tolist()
  kp = torch.randn(n_pages + 1, nkv, P, d, generator=g).to(dtype)
  vp = torch.randn(n_pages + 1, nkv, P, d, generator=g).to(dtype)      # [page, head, key, dim]; the kernel gets it transposed
  q = torch.randn(T, nq * d, generator=g).to(dtype)
  table = torch.zeros(B, W, dtype=torch.int32)
  cu = [0]
  token_req = []
  want = []
  for b, (past, n) in enumerate(reqs):
    npg = -(-kv_lens[b] // P)
    pages = [perm.pop() for _ in range(npg)]
    table[b, :npg] = torch.tensor(pages, dtype=torch.int32)
    kk = torch.cat([kp[p].transpose(0, 1) for p in pages], 0)[:kv_lens[b]]   # [S, nkv, d]
    vv = torch.cat([vp[p].transpose(0, 1) for p in pages], 0)[:kv_lens[b]]
    qq = q[cu[-1]:cu[-1] + n].view(n, nq, d)
    want.append(_attention_ref(qq.float(), kk.float(), vv.float(), d ** -0.5, window).reshape(n, nq * d))
    token_req += [b] * n
    cu.append(cu[-1] + n)
  want = torch.cat(want, 0)
  out = torch.empty(T, nq * d, dtype=dtype, device=DEV)
  i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
  part_o = torch.full((T * nq * splits * d,), float("nan"), device=DEV) if splits > 1 else None
  part_ml = torch.full((T * nq * splits * 2,), float("nan"), device=DEV) if splits > 1 else None
  ops.paged_attention(q.to(DEV), nq, nkv, d, out, kp.to(DEV), vp.transpose(2, 3).contiguous().to(DEV), table.to(DEV),
                      i32(token_req), i32(cu), i32(kv_lens), d ** -0.5, window, splits, part_o, part_ml)
  torch.testing.assert_close(out.double().cpu(), want, **(_tol(dtype) if dtype == torch.bfloat16
                                                           else dict(rtol=1e-5, atol=1e-5)))


def test_attention_one_key_returns_its_value():
  """A single visible key: softmax is 1 and the output is that key's value row, for every head of its group."""
  from miniinfer_amd.kernels import ops
  nq, nkv, d, P = 4, 2, 32, 8
  kp = torch.randn(3, nkv, P, d, device=DEV)
  vp = torch.randn(3, nkv, d, P, device=DEV)
  q = torch.randn(1, nq * d, device=DEV)
  out = torch.empty(1, nq * d, device=DEV)
  i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
  ops.paged_attention(q, nq, nkv, d, out, kp, vp, i32([[2]]), i32([0]), i32([0, 1]), i32([1]), d ** -0.5, 0)
  for h in range(nq):
    torch.testing.assert_close(out[0, h * d:(h + 1) * d], vp[2, h // 2, :, 0])


def _paged_case(reqs, nq, nkv, d, P, window, seed):
  """Random pages and queries for requests (keys already cached, new tokens); returns device tensors, the plain
  result, and the host lists."""
  g = torch.Generator().manual_seed(seed)
  B = len(reqs)
  kv_lens = [a + n for a, n in reqs]
  T = sum(n for _, n in reqs)
  W = max(-(-kv // P) for kv in kv_lens)
  n_pages = sum(-(-kv // P) for kv in kv_lens)
  perm = (torch.randperm(n_pages, generator=g) + 1).tolist()
  kp = torch.randn(n_pages + 1, nkv, P, d, generator=g).bfloat16()
  vp = torch.randn(n_pages + 1, nkv, P, d, generator=g).bfloat16()
  q = torch.randn(T, (nq + 2 * nkv) * d, generator=g).bfloat16()     # a fused qkv buffer: q is its first part
  table = torch.zeros(B, W, dtype=torch.int32)
  cu, token_req, want = [0], [], []
  for b, (past, n) in enumerate(reqs):
    npg = -(-kv_lens[b] // P)
    pages = [perm.pop() for _ in range(npg)]
    table[b, :npg] = torch.tensor(pages, dtype=torch.int32)
    kk = torch.cat([kp[p].transpose(0, 1) for p in pages], 0)[:kv_lens[b]]
    vv = torch.cat([vp[p].transpose(0, 1) for p in pages], 0)[:kv_lens[b]]
    qq = q[cu[-1]:cu[-1] + n, :nq * d].reshape(n, nq, d)
    want.append(_attention_ref(qq.float(), kk.float(), vv.float(), d ** -0.5, window).reshape(n, nq * d))
    token_req += [b] * n
    cu.append(cu[-1] + n)
  i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
  return dict(q=q.to(DEV), kp=kp.to(DEV), vp=vp.transpose(2, 3).contiguous().to(DEV), table=table.to(DEV),
              cu=i32(cu), kv=i32(kv_lens), token_req=i32(token_req), want=torch.cat(want, 0), T=T, B=B, q_lens=[n for _, n in reqs])


MFMA_SHAPES = [(16, 8, 128, 16, 0), (6, 3, 48, 16, 0), (8, 2, 32, 8, 0), (4, 4, 16, 8, 0), (5, 1, 80, 32, 0),
               (16, 1, 64, 16, 0), (12, 4, 96, 64, 0), (4, 2, 256, 16, 0), (8, 4, 128, 16, 50), (6, 2, 64, 8, 17)]


@pytest.mark.parametrize("variant", ["two_tiles", "dense", "wide"])
@pytest.mark.parametrize("nq,nkv,d,P,window", MFMA_SHAPES)
def test_mfma_prefill_attention(nq, nkv, d, P, window, variant):
  from miniinfer_amd.kernels import ops
  reqs = [(0, 70), (129, 2), (40, 33), (0, 2), (63, 17), (300, 5), (0, 200), (190, 130)]
  c = _paged_case(reqs, nq, nkv, d, P, window, seed=6)
  tpb = ops.attn_prefill_tokens_per_block(nq, nkv, d, wide=variant == "wide")
  if tpb == 0:
    assert variant == "wide" and d > 128       # head sizes above 128 have no instance with two column blocks
    with pytest.raises(ops.KernelError):
      ops.attn_prefill(c["q"], nq, nkv, d, torch.zeros(c["T"], nq * d, dtype=torch.bfloat16, device=DEV), c["kp"],
                       c["vp"], c["table"], torch.zeros(1, 2, dtype=torch.int32, device=DEV), c["cu"], c["kv"],
                       d ** -0.5, window, variant=variant)
    return
  work = [(b, i) for b, n in enumerate(c["q_lens"]) for i in range(-(-n // tpb))]
  out = torch.zeros(c["T"], nq * d, dtype=torch.bfloat16, device=DEV)
  ops.attn_prefill(c["q"], nq, nkv, d, out, c["kp"], c["vp"], c["table"],
                   torch.tensor(work, dtype=torch.int32, device=DEV), c["cu"], c["kv"], d ** -0.5, window, variant=variant)
  torch.testing.assert_close(out.double().cpu(), c["want"], rtol=1.6e-2, atol=1e-2)


@pytest.mark.parametrize("splits", [1, 3, 16, 29, 40])
@pytest.mark.parametrize("nq,nkv,d,P,window", MFMA_SHAPES)
def test_mfma_decode_attention_any_number_of_splits(nq, nkv, d, P, window, splits):
  from miniinfer_amd.kernels import ops
  # two multi-token entries first (skipped by the decode kernel), then single-token entries
  reqs = [(5, 3), (0, 2), (129, 1), (0, 1), (15, 1), (16, 1), (700, 1), (63, 1)]
  c = _paged_case(reqs, nq, nkv, d, P, window, seed=7)
  first, n = 2, 6
  out = torch.zeros(c["T"], nq * d, dtype=torch.bfloat16, device=DEV)
  part_o = torch.empty(n * nq * splits * d, dtype=torch.float32, device=DEV)
  part_ml = torch.empty(n * nq * splits * 2, dtype=torch.float32, device=DEV)
  ops.attn_decode(c["q"], nq, nkv, d, out, c["kp"], c["vp"], c["table"], c["cu"], c["kv"], first, n, splits, part_o,
                  part_ml, d ** -0.5, window)
  torch.testing.assert_close(out.double().cpu()[5:], c["want"][5:], rtol=1.6e-2, atol=1e-2)
  assert float(out[:5].abs().sum()) == 0.0       # rows of the multi-token entries are not touched
  # the keys and values read with nontemporal loads (as launches over many keys do): the same arithmetic
  streamed = torch.zeros_like(out)
  ops.attn_decode(c["q"], nq, nkv, d, streamed, c["kp"], c["vp"], c["table"], c["cu"], c["kv"], first, n, splits,
                  part_o, part_ml, d ** -0.5, window, stream_keys=True)
  assert torch.equal(streamed, out)
  # workgroups of twice the waves (as launches of many workgroups get): the macro tiles go to other waves, so the
  # sums are rounded elsewhere; held to the same reference
  wide = torch.zeros_like(out)
  ops.attn_decode(c["q"], nq, nkv, d, wide, c["kp"], c["vp"], c["table"], c["cu"], c["kv"], first, n, splits, part_o,
                  part_ml, d ** -0.5, window, wide=True)
  torch.testing.assert_close(wide.double().cpu()[5:], c["want"][5:], rtol=1.6e-2, atol=1e-2)
  assert float(wide[:5].abs().sum()) == 0.0


@pytest.mark.parametrize("splits", [1, 5])
@pytest.mark.parametrize("P,long_kv", [(8, 2100), (16, 4200), (16, 4090)])
def test_mfma_decode_attention_with_long_block_tables(P, long_kv, splits):
  """Requests of thousands of keys beside short ones: block tables of 263 and of exactly 256 entries."""
  from miniinfer_amd.kernels import ops
  nq, nkv, d = 4, 2, 32
  reqs = [(long_kv - 1, 1), (300, 1), (0, 1)]
  c = _paged_case(reqs, nq, nkv, d, P, 0, seed=12)
  assert (c["table"].shape[1] > 256) == (long_kv != 4090)
  out = torch.zeros(c["T"], nq * d, dtype=torch.bfloat16, device=DEV)
  part_o = torch.empty(3 * nq * splits * d, dtype=torch.float32, device=DEV)
  part_ml = torch.empty(3 * nq * splits * 2, dtype=torch.float32, device=DEV)
  ops.attn_decode(c["q"], nq, nkv, d, out, c["kp"], c["vp"], c["table"], c["cu"], c["kv"], 0, 3, splits, part_o,
                  part_ml, d ** -0.5, 0)
  torch.testing.assert_close(out.double().cpu(), c["want"], rtol=1.6e-2, atol=1e-2)


def test_mfma_attention_finds_a_far_key_and_respects_the_window_edge():
  """One key among hundreds is made to stand out (its score is far above the rest): the output must be its value.
  With a window that just excludes it, it must vanish; with one that just includes it, it is back."""
  from miniinfer_amd.kernels import ops
  nq, nkv, d, P = 4, 2, 64, 16
  kv, far = 600, 37
  c = _paged_case([(kv - 1, 1)], nq, nkv, d, P, 0, seed=8)
  q = c["q"].clone()
  kp, vp, table = c["kp"].clone(), c["vp"].clone(), c["table"]
  page, off = int(table[0, far // P]), far % P
  qh = q[0, :nq * d].float().view(nq, d)
  for g in range(nkv):
    kp[page, g, off] = (qh[g * 2] * 4).bfloat16()        # aligned with the first head of each group
  out = torch.empty(1, nq * d, dtype=torch.bfloat16, device=DEV)
  po = torch.empty(nq * 8 * d, dtype=torch.float32, device=DEV)
  pm = torch.empty(nq * 8 * 2, dtype=torch.float32, device=DEV)
  run = lambda w: ops.attn_decode(q, nq, nkv, d, out, kp, vp, table, c["cu"], c["kv"], 0, 1, 8, po, pm, d ** -0.5, w)
  run(0)
  for g in range(nkv):
    torch.testing.assert_close(out[0, g * 2 * d:(g * 2 + 1) * d].float(), vp[page, g, :, off].float(), rtol=2e-2, atol=2e-2)
  run(kv - 1 - far)          # sees keys far+1 .. kv-1: the far key is just outside
  assert (out[0, :d].float() - vp[page, 0, :, off].float()).abs().max() > 0.5
  run(kv - far)              # just inside
  torch.testing.assert_close(out[0, :d].float(), vp[page, 0, :, off].float(), rtol=2e-2, atol=2e-2)


# whole rows of the result per workgroup / k split across workgroups / whole rows, left operand staged through LDS /
# whole rows, weights fetched in whole memory lines / both / both operands staged through LDS / the rows of the left
# operand shared out across workgroups too
@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4, 5, 6])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("M,N,K", [(1, 1024, 1024), (8, 4096, 1024), (16, 1024, 3072), (17, 500, 80), (64, 6144, 1024),
                                   (3, 151936, 256), (33, 48, 2048), (5, 130, 88), (64, 1000, 40), (7, 2050, 64),
                                   (16, 1001, 512), (48, 1024, 4360), (64, 100, 12288), (20, 2064, 1000),
                                   (9, 1024, 2048), (13, 520, 3072), (30, 1000, 6144), (64, 272, 1024), (4, 2050, 4096),
                                   (6, 600, 192), (16, 5120, 2560), (5, 300, 6400), (64, 40, 4224), (2, 2000, 128),
                                   (64, 30001, 256)])
def test_gemm_skinny(M, N, K, out_dtype, variant):
  from miniinfer_amd.kernels import ops
  g = torch.Generator().manual_seed(9)
  a = torch.randn(M, K, generator=g).bfloat16().to(DEV)
  w = (torch.randn(N, K, generator=g) * 0.1).bfloat16().to(DEV)
  out = torch.full((M, N), float("nan"), dtype=out_dtype, device=DEV)
  ops.gemm_skinny(a, w, out, variant=variant)
  want = a.double() @ w.double().T
  if out_dtype == torch.float32:
    torch.testing.assert_close(out.double(), want, rtol=1e-4, atol=1e-4 * K ** 0.5)
  else:
    torch.testing.assert_close(out.double(), want, rtol=1e-2, atol=1e-2)
  if variant in (2, 4, 5):      # the staged operands change where the operands come from, not one sum
    other = {2: 0, 4: 3, 5: 0}[variant]
    same = torch.empty_like(out)
    ops.gemm_skinny(a, w, same, variant=other)
    # (with two row blocks, 16 waves' pieces of both operands do not fit a unit's LDS: that form then runs fewer
    # waves, which cut k into other slices)
    if ops.gemm_skinny_waves(variant, M, N, K) == ops.gemm_skinny_waves(other, M, N, K):
      assert torch.equal(out, same)
    else:
      assert variant == 5 and (M, N, K) == (16, 5120, 2560)


@pytest.mark.parametrize("M,N,K,gate_up", [(8, 4096, 1024, False), (64, 3072, 1024, True), (40, 1000, 2048, False),
                                          (33, 12288, 512, True), (16, 5120, 2560, False)])
def test_gemm_skinny_nontemporal_build_gives_the_same_bits(M, N, K, gate_up):
  """The build of the product kernels whose weight loads are nontemporal (for matrices too large to stay in the caches,
  and for every matrix while the table in use says `stream_weights`) does the same arithmetic: equal results in every
  form."""
  from miniinfer_amd.kernels import ops
  g = torch.Generator().manual_seed(12)
  a = torch.randn(M, K, generator=g).bfloat16().to(DEV)
  w = (torch.randn(2 * N if gate_up else N, K, generator=g) * 0.1).bfloat16().to(DEV)
  table = ops.ProductChoices()
  for variant in (0, 1, 2, 3, 4, 5, 6):
    plain = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    streamed = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.gemm_skinny(a, w, plain, gate_up=gate_up, variant=variant)
    with table:
      table.stream_weights = True
      ops.gemm_skinny(a, w, streamed, gate_up=gate_up, variant=variant)
    assert torch.equal(plain, streamed), variant
  assert ("gemm_skinny", (("SKINNY_NT", 1),)) in ops._libs and ("gemm_skinny", ()) in ops._libs


def test_gemm_skinny_drawn_shapes():
  """Every form of the weight-streaming product on shapes drawn at random (rows 1 to 64, k a multiple of 8 from 8 to
  6,400, 1 to 5,000 columns, left operands with a row stride of their own, a third of them gate|up), against 64-bit
  arithmetic; and the forms that only change where the operands come from give the very same sums."""
  import random
  from miniinfer_amd.kernels import ops
  rng = random.Random(3)
  for it in range(48):
    M = rng.choice([1, 2, 3, 4, 5, 7, 8, 9, 12, 15, 16, 17, 24, 31, 32, 33, 47, 48, 63, 64])
    K = 8 * rng.choice([1, 3, 4, 5, 8, 9, 12, 16, 24, 31, 32, 40, 64, 72, 100, 128, 192, 264, 320, 512, 800])
    N = rng.choice([1, 3, 5, 16, 17, 33, 64, 100, 129, 256, 500, 1000, 2050, 5000])
    gate_up = rng.random() < 0.3
    if gate_up and rng.random() < 0.7:
      N = (N + 3) // 4 * 4
    g = torch.Generator().manual_seed(it)
    a = torch.randn(M, K + rng.choice([0, 0, 8, 16, 64]), generator=g).bfloat16().to(DEV)[:, :K]
    w = (torch.randn(2 * N if gate_up else N, K, generator=g) * 0.1).bfloat16().to(DEV)
    want = a.double() @ w.double().T
    if gate_up:
      want = torch.nn.functional.silu(want[:, :N]) * want[:, N:]
    outs = {}
    for variant in (0, 1, 2, 3, 4, 5, 6):
      if variant == 1 and gate_up and N % 4:
        continue
      out = torch.full((M, N), float("nan"), dtype=torch.float32, device=DEV)
      ops.gemm_skinny(a, w, out, gate_up=gate_up, variant=variant)
      torch.testing.assert_close(out.double(), want, rtol=2e-4, atol=2e-4 * K ** 0.5,
                                 msg=lambda m: f"variant {variant}, {M} x [{N}, {K}] gate_up={gate_up}: {m}")
      outs[variant] = out
    assert torch.equal(outs[2], outs[0]) and torch.equal(outs[4], outs[3]), (M, N, K)
    rows_w = 2 * N if gate_up else N
    if ops.gemm_skinny_waves(5, M, rows_w, K, gate_up) == ops.gemm_skinny_waves(0, M, rows_w, K, gate_up):
      assert torch.equal(outs[5], outs[0]), (M, N, K)


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4, 5, 6])
@pytest.mark.parametrize("M,I,K", [(8, 3072, 1024), (1, 112, 80), (40, 160, 96), (64, 100, 256), (33, 1028, 2200),
                                   (8, 1536, 4096), (16, 516, 2048), (48, 260, 1024), (3, 200, 5120), (20, 36, 448),
                                   (64, 12288, 512), (5, 11012, 256)])      # k split: unsplit, the kernel's own ending
def test_gemm_skinny_gate_up_activation(M, I, K, variant):
  from miniinfer_amd.kernels import ops
  g = torch.Generator().manual_seed(10)
  x = torch.randn(M, K, generator=g).bfloat16().to(DEV)
  w = (torch.randn(2 * I, K, generator=g) * 0.1).bfloat16().to(DEV)
  out = torch.full((M, I), float("nan"), dtype=torch.bfloat16, device=DEV)
  ops.gemm_skinny(x, w, out, gate_up=True, variant=variant)
  gu = x.double() @ w.double().T
  want = torch.nn.functional.silu(gu[:, :I]) * gu[:, I:]
  torch.testing.assert_close(out.double(), want, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("M,N,K,with_x,gate_up", [(8, 4096, 1024, True, False), (1, 500, 80, False, False),
                                                   (16, 3072, 1024, True, True), (5, 112, 88, True, True),
                                                   (3, 151936, 256, False, False)])
def test_norm_gemm_skinny(M, N, K, with_x, gate_up):
  from miniinfer_amd.kernels import ops
  g = torch.Generator().manual_seed(11)
  r = (torch.randn(M, K, generator=g) * 2).to(DEV)
  x = torch.randn(M, K, generator=g).bfloat16().to(DEV) if with_x else None
  nw = (1 + 0.1 * torch.randn(K, generator=g)).to(DEV)
  w = (torch.randn(2 * N if gate_up else N, K, generator=g) * 0.1).bfloat16().to(DEV)
  out = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
  r_out = torch.empty_like(r) if with_x else None
  ops.norm_gemm_skinny(r, x, nw, 1e-5, w, out, residual_out=r_out, gate_up=gate_up)
  v = r.double() + (x.double() if with_x else 0)
  if with_x:
    torch.testing.assert_close(r_out.double(), v, rtol=1e-6, atol=1e-6)
  # the kernel's own rounding points: the left operand is bfloat16(r' * w); the row's rstd scales the 32-bit sums
  rstd = torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + 1e-5)
  y = ((v * nw.double()).bfloat16().double() @ w.double().T) * rstd
  torch.testing.assert_close(y, torch.nn.functional.rms_norm(v, (K,), nw.double(), 1e-5) @ w.double().T, rtol=3e-2,
                             atol=3e-2 * float(y.abs().max()))
  want = torch.nn.functional.silu(y[:, :N]) * y[:, N:] if gate_up else y
  torch.testing.assert_close(out.double(), want, rtol=1e-2, atol=1e-2)
  # rows picked by index, residual untouched
  rows = torch.tensor([M - 1, 0], dtype=torch.int32, device=DEV)
  out2 = torch.empty(2, N, dtype=torch.bfloat16, device=DEV)
  ops.norm_gemm_skinny(r, x, nw, 1e-5, w, out2, rows=rows, gate_up=gate_up)
  torch.testing.assert_close(out2.double(), want[rows.long()], rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("splits", [1, 4])
@pytest.mark.parametrize("with_norm,rd_of", [(True, 1.0), (False, 1.0), (True, 0.5), (True, 0.0)])
@pytest.mark.parametrize("nq,nkv,d,P,window", MFMA_SHAPES)
def test_mfma_decode_with_fused_norm_rotation_and_cache_write(nq, nkv, d, P, window, with_norm, rd_of, splits):
  """The decode kernel that takes the raw projection: against head norm, rotation and attention done one after the
  other in 32-bit on the host, with the new key rounded to bfloat16 as the cache holds it.  The slot of the new
  token holds stale numbers before the call and the new key and value after it."""
  from miniinfer_amd.kernels import ops
  reqs = [(129, 1), (0, 1), (15, 1), (16, 1), (700, 1), (63, 1), (1, 1)]
  c = _paged_case(reqs, nq, nkv, d, P, window, seed=9)
  g = torch.Generator().manual_seed(10)
  B, max_pos, theta, eps = len(reqs), 800, 5000.0, 2e-6
  rd = int(d * rd_of) // 2 * 2
  qw = (1 + 0.1 * torch.randn(d, generator=g)) if with_norm else None
  kw = (1 + 0.1 * torch.randn(d, generator=g)) if with_norm else None
  pos = torch.tensor([past for past, _ in reqs])
  table_host = c["table"].cpu()
  slots = torch.tensor([int(table_host[b, past // P]) * P + past % P for b, (past, _) in enumerate(reqs)])
  cos_sin = None
  if rd:
    j = torch.arange(0, rd, 2, dtype=torch.float32)
    ang = torch.outer(torch.arange(max_pos, dtype=torch.float32), 1.0 / theta ** (j / rd))
    cos_sin = torch.cat((ang.cos(), ang.sin()), -1).to(DEV)

  raw = c["q"].float().cpu().view(B, nq + 2 * nkv, d)
  q, k, v = raw[:, :nq], raw[:, nq:nq + nkv], raw[:, nq + nkv:]
  if with_norm:
    q = torch.nn.functional.rms_norm(q, (d,), qw, eps)
    k = torch.nn.functional.rms_norm(k, (d,), kw, eps)
  if rd:
    q, k = _rope_ref(q, pos, theta, rd), _rope_ref(k, pos, theta, rd)
  q, k = q.bfloat16().float(), k.bfloat16().float()
  kp, vp = c["kp"].clone(), c["vp"].clone()
  kc, vc = kp.float().cpu(), vp.float().cpu().transpose(2, 3)      # [pages, nkv, P, d]
  want = []
  for b, (past, _) in enumerate(reqs):
    pages = table_host[b, :past // P + 1].tolist()
    kk = torch.cat([kc[p].transpose(0, 1) for p in pages], 0)[:past]
    vv = torch.cat([vc[p].transpose(0, 1) for p in pages], 0)[:past]
    kk, vv = torch.cat((kk, k[b][None]), 0), torch.cat((vv, v[b][None]), 0)
    want.append(_attention_ref(q[b][None], kk, vv, d ** -0.5, window).reshape(1, nq * d))
  want = torch.cat(want, 0)

  out = torch.zeros(B, nq * d, dtype=torch.bfloat16, device=DEV)
  part_o = torch.empty(B * nq * splits * d, dtype=torch.float32, device=DEV)
  part_ml = torch.empty(B * nq * splits * 2, dtype=torch.float32, device=DEV)
  before = c["q"].clone()
  if 0 < rd < d:                                         # a partly rotated head is refused, not miscomputed
    with pytest.raises(ops.KernelError, match="whole heads"):
      ops.attn_decode_front(c["q"], nq, nkv, d, out, kp, vp, c["table"], c["cu"], c["kv"], 0, B, splits, part_o,
                            part_ml, d ** -0.5, window, None, None, eps, cos_sin, pos.to(torch.int32).to(DEV),
                            slots.to(torch.int32).to(DEV))
    return
  ops.attn_decode_front(c["q"], nq, nkv, d, out, kp, vp, c["table"], c["cu"], c["kv"], 0, B, splits, part_o, part_ml,
                        d ** -0.5, window, qw.to(DEV) if with_norm else None, kw.to(DEV) if with_norm else None, eps,
                        cos_sin, pos.to(torch.int32).to(DEV), slots.to(torch.int32).to(DEV))
  torch.testing.assert_close(out.double().cpu(), want.double(), rtol=1.6e-2, atol=1e-2)
  assert torch.equal(c["q"], before)                     # the projection is read only
  kp2, vp2, streamed = c["kp"].clone(), c["vp"].clone(), torch.zeros_like(out)
  ops.attn_decode_front(c["q"], nq, nkv, d, streamed, kp2, vp2, c["table"], c["cu"], c["kv"], 0, B, splits, part_o,
                        part_ml, d ** -0.5, window, qw.to(DEV) if with_norm else None, kw.to(DEV) if with_norm else None,
                        eps, cos_sin, pos.to(torch.int32).to(DEV), slots.to(torch.int32).to(DEV), stream_keys=True)
  assert torch.equal(streamed, out) and torch.equal(kp2, kp) and torch.equal(vp2, vp)   # nontemporal loads: same bits
  kp3, vp3, wide = c["kp"].clone(), c["vp"].clone(), torch.zeros_like(out)          # workgroups of twice the waves
  ops.attn_decode_front(c["q"], nq, nkv, d, wide, kp3, vp3, c["table"], c["cu"], c["kv"], 0, B, splits, part_o,
                        part_ml, d ** -0.5, window, qw.to(DEV) if with_norm else None, kw.to(DEV) if with_norm else None,
                        eps, cos_sin, pos.to(torch.int32).to(DEV), slots.to(torch.int32).to(DEV), wide=True)
  torch.testing.assert_close(wide.double().cpu(), want.double(), rtol=1.6e-2, atol=1e-2)
  assert torch.equal(kp3, kp) and torch.equal(vp3, vp)                                # the same cache writes
  k_after, v_after = kp.float().cpu(), vp.float().cpu().transpose(2, 3)
  changed_k = (k_after != kc).any(-1)
  for b in range(B):
    page, off = int(slots[b]) // P, int(slots[b]) % P
    torch.testing.assert_close(k_after[page, :, off], k[b], rtol=1e-2, atol=1e-2)
    assert torch.equal(v_after[page, :, off], v[b])
    changed_k[page, :, off] = False
  assert not bool(changed_k.any())                       # no other slot was written


@pytest.mark.parametrize("M,N,K,N2,gate_up", [(8, 1024, 2048, 6144, True), (1, 80, 96, 112, False), (16, 1024, 3072, 4096, False),
                                               (40, 136, 264, 200, True), (64, 1024, 2048, 3072, False), (5, 88, 40, 24, False),
                                               (12, 2056, 96, 160, True), (64, 1024, 3072, 4096, False),
                                               (33, 520, 2304, 132, True), (40, 1024, 256, 11008, True)])
@pytest.mark.parametrize("variants", [(0, 0), (1, 0), (0, 1), (1, 1), (2, 2), (2, 1), (4, 3), (3, 4), (5, 5), (6, 6), (6, 1)])
def test_norm_split_between_two_products(M, N, K, N2, gate_up, variants):
  """residual += a W1^T; y = rmsnorm(residual) * w; out = y W2^T (or the gated activation of it), the add and the
  norm done half in the first product's kernel and half in the second's.  Against 64-bit arithmetic with the
  kernels' rounding points restated: the second product's left operand is bfloat16(residual * w), and the row's
  rsqrt(mean square + eps) scales its 32-bit sums."""
  from miniinfer_amd.kernels import ops
  g = torch.Generator().manual_seed(31)
  eps = 3e-6
  a = torch.randn(M, K, generator=g).bfloat16().to(DEV)
  w1 = (torch.randn(N, K, generator=g) * 0.05).bfloat16().to(DEV)
  r = (torch.randn(M, N, generator=g) * 2).to(DEV)
  nw = (1 + 0.1 * torch.randn(N, generator=g)).to(DEV)
  w2 = (torch.randn(2 * N2 if gate_up else N2, N, generator=g) * 0.1).bfloat16().to(DEV)
  want_r = r.double() + a.double() @ w1.double().T
  r_dev = r.clone()
  operand, row_ss = ops.gemm_skinny_into_norm(a, w1, r_dev, nw, variant=variants[0])
  torch.testing.assert_close(r_dev.double(), want_r, rtol=1e-5, atol=1e-4)
  torch.testing.assert_close(operand.double(), (r_dev.double() * nw.double()).bfloat16().double(), rtol=1e-2, atol=1e-6)
  torch.testing.assert_close(row_ss[:, :M].sum(0).double(), r_dev.double().pow(2).sum(-1), rtol=1e-5, atol=1e-5)
  out = torch.empty(M, N2, dtype=torch.bfloat16, device=DEV)
  ops.gemm_skinny_scaled(operand, w2, out, row_ss, eps, gate_up=gate_up, variant=variants[1])
  rstd = torch.rsqrt(r_dev.double().pow(2).mean(-1, keepdim=True) + eps)
  y = (operand.double() @ w2.double().T) * rstd
  # ... which is the norm followed by the product, up to the operand's rounding
  torch.testing.assert_close(y, torch.nn.functional.rms_norm(want_r, (N,), nw.double(), eps) @ w2.double().T,
                             rtol=3e-2, atol=3e-2 * float(y.abs().max()))
  want = torch.nn.functional.silu(y[:, :N2]) * y[:, N2:] if gate_up else y
  torch.testing.assert_close(out.double(), want, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,N", [(7, 136), (1, 5), (130, 1000)])
def test_add_bias(dtype, M, N):
  from miniinfer_amd.kernels import ops
  g = torch.Generator().manual_seed(M + N)
  y = torch.randn(M, N, generator=g).to(dtype)
  b = torch.randn(N, generator=g).to(dtype)
  want = (y.float() + b.float()).to(dtype)
  got = ops.add_bias(y.clone().to(DEV), b.to(DEV))
  assert torch.equal(got.cpu(), want)
  with pytest.raises(ops.KernelError):
    ops.add_bias(y.to(DEV), b[:-1].to(DEV))


def test_microbench_commands_run_at_small_sizes(capsys):
  """The measuring tool that the profile summaries cite: each command runs and prints its line."""
  from miniinfer_amd.kernels import microbench
  assert microbench.main(["product", "--rows", "4", "--n", "256", "--k", "128", "--calls", "4", "--copies", "2"]) == 0
  assert microbench.main(["product", "--rows", "20", "--n", "64", "--k", "256", "--gate-up", "--calls", "4"]) == 0
  assert microbench.main(["prefill-attention", "--tokens", "200", "--heads", "4", "--kv-heads", "2", "--head-dim", "64",
                          "--calls", "2"]) == 0
  assert microbench.main(["decode-attention", "--batch", "3", "--context", "300", "--heads", "4", "--kv-heads", "2",
                          "--head-dim", "64", "--calls", "4"]) == 0
  assert microbench.main(["prompt-front", "--tokens", "100", "--heads", "4", "--kv-heads", "2", "--head-dim", "64",
                          "--calls", "4"]) == 0
  out = capsys.readouterr().out
  # every line ends in a time and a rate that a kernel of these sizes can have: more than a launch costs nothing,
  # less than a millisecond, and no more bytes or flops a second than the machine has
  import re
  times = [float(x) for x in re.findall(r"([0-9.]+) us", out)]
  assert len(times) >= 20 and all(0.3 < t < 1000.0 for t in times), times
  rates = [float(x) for x in re.findall(r"([0-9.]+) TB/s", out)]
  assert rates and all(0.0 < r < 8.0 for r in rates), rates
  flops = [float(x) for x in re.findall(r"([0-9.]+) TFLOP/s", out)]
  assert all(0.0 < f < 2500.0 for f in flops), flops
  assert "qk_norm_rope_cache: 100 tokens" in out
  assert out.count("gemm_skinny:") == 2 and out.count("gemm_skinny with k split:") == 2
  assert out.count("gemm_skinny with the rows of the left operand shared out:") == 2
  assert out.count("gemm_skinny with the left operand staged and the weights in whole lines:") == 2
  assert out.count("gemm_skinny with both operands staged:") == 2
  assert out.count("gemm_skinny with the left operand staged:") == 2 and "attn_prefill dense" in out and "attn_decode_front" in out


def test_measured_peaks_are_plausible():
  from miniinfer_amd.kernels import ops
  gbs, tflops = ops.measured_peaks(stream_bytes=1 << 30)
  # an MI355X: 8 TB/s and 2.5 PFLOP/s on the data sheet; the bare loops have reached 5.8 to 6.3 TB/s and 2.1 PFLOP/s
  assert 4000 < gbs < 8000 and 1500 < tflops < 2500, (gbs, tflops)
  assert ops.measured_peaks() == (gbs, tflops)      # measured once per process and device


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,I,parts,ss_row", [(5, 112, 3, 16), (40, 1028, 256, 64), (64, 36, 1, 64), (1, 4096, 17, 16)])
def test_silu_mul_scaled(dtype, M, I, parts, ss_row):
  """The activation kernel that also applies an RMS norm's missing row factor, from the rows' partial sums of
  squares, against the statement in 64-bit."""
  from miniinfer_amd.kernels import ops
  g = torch.Generator().manual_seed(M + I)
  gu = torch.randn(M, 2 * I, generator=g).to(dtype)
  row_ss = torch.rand(parts, ss_row, generator=g) * 50
  eps, K = 1e-5, 96
  rstd = torch.rsqrt(row_ss.double().sum(0)[:M] / K + eps)[:, None]
  want = torch.nn.functional.silu(gu[:, :I].double() * rstd) * (gu[:, I:].double() * rstd)
  out = ops.silu_mul_scaled(gu.to(DEV), torch.empty(M, I, dtype=dtype, device=DEV), row_ss.to(DEV), eps, K)
  torch.testing.assert_close(out.double().cpu(), want, **_tol(dtype))
  with pytest.raises(ops.KernelError):
    ops.silu_mul_scaled(gu.to(DEV), torch.empty(M, I, dtype=dtype, device=DEV), row_ss[:, :0].contiguous().to(DEV), eps, K)
