"""The decode attention entry point that allocates nothing (`mi_attn_decode_static`), called through ctypes.

It runs the kernels of `mi_attn_decode` with the key splits' partial results in a device array of the shared
object instead of a workspace the caller brings.  Its output must equal `mi_attn_decode`'s on two calls in a row,
the second with a smaller input (the array then still holds the first call's partials), and a launch whose
partials do not fit the array must be refused with a message.  At another head size, with a window and with entries
that do not start at the first one, it is also held to a plain torch statement of the attention itself.
"""

import math

import ctypes
from ctypes import c_float, c_int, c_int64, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu
D = 64


def _load(d=D):
  from miniinfer_amd.kernels import jit
  lib = ctypes.CDLL(jit.compile_module("attention_mfma", (("HEAD_DIM", d),)))
  common = [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int,
            c_int, c_int]
  tail = [c_int, c_int, c_int, c_float, c_int, c_void_p]
  lib.mi_attn_decode.argtypes = common + [c_void_p, c_void_p] + tail[:-1] + [c_int, c_int, c_void_p]   # + stream_keys, wide
  lib.mi_attn_decode_static.argtypes = common + tail
  for f in (lib.mi_attn_decode, lib.mi_attn_decode_static, lib.mi_attn_static_scratch_floats):
    f.restype = c_int
  lib.mi_last_error.restype = ctypes.c_char_p
  return lib


def _case(entries, nq, nkv, P, kv_lens, seed, D=D):
  """Random queries and paged keys and values for `entries` requests of one new token each."""
  dev = torch.device("cuda:0")
  g = torch.Generator().manual_seed(seed)
  W = max(-(-n // P) for n in kv_lens)
  pages = 1 + entries * W
  k = (torch.randn(pages, nkv, P, D, generator=g) * 0.5).bfloat16().to(dev)
  v = (torch.randn(pages, nkv, D, P, generator=g) * 0.5).bfloat16().to(dev)
  perm = (torch.randperm(pages - 1, generator=g) + 1).to(torch.int32)
  table = torch.zeros(entries, W, dtype=torch.int32)
  for b in range(entries):
    n = -(-kv_lens[b] // P)
    table[b, :n] = perm[b * W:b * W + n]
  q = (torch.randn(entries, nq * D, generator=g)).bfloat16().to(dev)
  cu = torch.arange(entries + 1, dtype=torch.int32, device=dev)
  kv = torch.tensor(kv_lens, dtype=torch.int32, device=dev)
  return dict(q=q, k=k, v=v, table=table.to(dev), cu=cu, kv=kv, W=W)


def _run(lib, c, entries, nq, nkv, P, splits, static, D=D, window=0, first=0):
  """Entries first .. entries - 1 of the case; the rows of the entries before `first` stay NaN."""
  out = torch.full((entries, nq * D), float("nan"), dtype=torch.bfloat16, device=c["q"].device)
  stream = torch.cuda.current_stream().cuda_stream
  args = [c["q"].data_ptr(), c["q"].stride(0), out.data_ptr(), out.stride(0), c["k"].data_ptr(), c["v"].data_ptr(),
          c["table"].data_ptr(), c["W"], c["cu"].data_ptr(), c["kv"].data_ptr(), first, entries - first, splits]
  tail = [nq, nkv, P, D ** -0.5, window, stream]
  if static:
    rc = lib.mi_attn_decode_static(*args, *tail)
  else:
    need = (entries - first) * nq * splits
    part_o = torch.empty(need * D, dtype=torch.float32, device=out.device)
    part_ml = torch.empty(need * 2, dtype=torch.float32, device=out.device)
    rc = lib.mi_attn_decode(*args, part_o.data_ptr(), part_ml.data_ptr(), *tail[:-1], 0, 0, stream)
  assert rc == 0, lib.mi_last_error().decode()
  torch.cuda.synchronize()
  return out


def test_decode_attention_from_the_static_scratch_equals_the_workspace_form():
  lib = _load()
  assert lib.mi_attn_static_scratch_floats() == 1 << 20
  nq, nkv, P = 8, 2, 16
  # first a larger launch (6 requests, 8 key splits), then a smaller one (2 requests, 3 splits, shorter contexts)
  for entries, splits, kv_lens, seed in ((6, 8, [700, 1500, 64, 1, 333, 2048], 1), (2, 3, [200, 517], 2)):
    c = _case(entries, nq, nkv, P, kv_lens, seed)
    print(f"static decode attention: {entries} entries, {splits} splits", flush=True)
    want = _run(lib, c, entries, nq, nkv, P, splits, static=False)
    got = _run(lib, c, entries, nq, nkv, P, splits, static=True)
    assert not torch.isnan(got.float()).any()
    assert torch.equal(got, want)
  # one split needs no partials at all
  c = _case(3, nq, nkv, P, [90, 30, 55], 3)
  assert torch.equal(_run(lib, c, 3, nq, nkv, P, 1, static=True), _run(lib, c, 3, nq, nkv, P, 1, static=False))


def _plain(c, entries, nq, nkv, P, window, D):
  """softmax(q . K / sqrt(D)) V per entry and head over the entry's own keys (the last `window` of them), float64."""
  out = torch.zeros(entries, nq * D, dtype=torch.float64)
  k, v, table, kv = c["k"].double().cpu(), c["v"].double().cpu(), c["table"].cpu(), c["kv"].cpu().tolist()
  q = c["q"].double().cpu().view(entries, nq, D)
  for b in range(entries):
    S = kv[b]
    pages = table[b, :-(-S // P)].long()
    keys = k[pages].permute(0, 2, 1, 3).reshape(-1, nkv, D)[:S]          # [S, nkv, D]
    vals = v[pages].permute(0, 3, 1, 2).reshape(-1, nkv, D)[:S]          # value pages are [.., D, P]
    lo = max(0, S - window) if window else 0
    for h in range(nq):
      g = h // (nq // nkv)
      p = torch.softmax(keys[lo:, g] @ q[b, h] / math.sqrt(D), dim=0)
      out[b, h * D:(h + 1) * D] = p @ vals[lo:, g]
  return out


def test_static_scratch_at_another_head_size_with_a_window_and_a_first_entry_against_plain_torch():
  """Head size 80, 3 entries x 5 heads x 7 splits (an odd number of partials), a window of 300 keys, and the
  launch starting at the second entry; two calls in a row, the second smaller."""
  d = 80
  lib = _load(d)
  nq, nkv, P = 5, 1, 16
  for entries, first, splits, kv_lens, window, seed in ((4, 1, 7, [50, 900, 301, 1234], 300, 5), (2, 0, 3, [411, 77], 0, 6)):
    c = _case(entries, nq, nkv, P, kv_lens, seed, D=d)
    print(f"static decode attention, head size {d}: entries {first}..{entries - 1}, {splits} splits, window {window}", flush=True)
    got = _run(lib, c, entries, nq, nkv, P, splits, static=True, D=d, window=window, first=first)
    want = _run(lib, c, entries, nq, nkv, P, splits, static=False, D=d, window=window, first=first)
    assert torch.isnan(got[:first].float()).all() and not torch.isnan(got[first:].float()).any()
    assert torch.equal(got[first:], want[first:])
    torch.testing.assert_close(got[first:].double().cpu(), _plain(c, entries, nq, nkv, P, window, d)[first:],
                               rtol=1.6e-2, atol=1e-2)


def test_a_launch_beyond_the_static_scratch_is_refused():
  lib = _load()
  nq, nkv, P = 16, 2, 16
  entries, splits = 64, 32                     # 64 * 16 * 32 * (64 + 2) floats = 2.1 M > 1 M
  c = _case(entries, nq, nkv, P, [40] * entries, 4)
  out = torch.zeros((entries, nq * D), dtype=torch.bfloat16, device=c["q"].device)
  rc = lib.mi_attn_decode_static(c["q"].data_ptr(), c["q"].stride(0), out.data_ptr(), out.stride(0), c["k"].data_ptr(),
                                 c["v"].data_ptr(), c["table"].data_ptr(), c["W"], c["cu"].data_ptr(),
                                 c["kv"].data_ptr(), 0, entries, splits, nq, nkv, P, D ** -0.5, 0,
                                 torch.cuda.current_stream().cuda_stream)
  assert rc != 0
  msg = lib.mi_last_error().decode()
  assert "static scratch" in msg and "2162688" in msg, msg
  torch.cuda.synchronize()
  assert float(out.float().abs().max()) == 0.0     # nothing was launched
