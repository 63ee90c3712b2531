"""Causal grouped-query attention over the paged cache (the mixer of Qwen3).

Order of operations, as miniinfer/models/fused_qwen3.py:95-107: one fused QKV projection
(rows q | k | v, no bias), per-head RMS norm of q and k, rotation of q and k, the new keys and
values written to their cache slots before attention (flashinfer_backend.py:341-348), attention
of the new tokens over all cached keys of their request, output projection.
"""

from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from ..kernels import ops
from .base import (BuildContext, NORMS, POSITIONS, PagedKV, ParamSpec, Part, Source, register_mixer)
from .linear import PendingLinear, linear


class PagedAttention(Part):
  takes_deferred_norm = True    # the input goes straight into `linear`, which can fuse the norm

  def __init__(self, spec, ctx: BuildContext):
    if spec.num_heads % spec.num_kv_heads:
      raise ValueError(f"{spec.num_heads} query heads are no multiple of {spec.num_kv_heads} kv heads")
    if spec.head_dim % 8 or spec.head_dim > 256:
      raise ValueError(f"head_dim={spec.head_dim} is not supported: the attention kernels take multiples of 8 up to 256")
    self.spec = spec
    self.ctx = ctx
    self.nq, self.nkv, self.d = spec.num_heads, spec.num_kv_heads, spec.head_dim
    self.hidden = spec.hidden_size
    self.scale = float(spec.scale)
    self.window = spec.window
    self.position = POSITIONS.build(spec.position, ctx)
    self.q_norm = NORMS.build(spec.qk_norm, ctx) if spec.qk_norm is not None else None
    self.k_norm = NORMS.build(spec.qk_norm, ctx) if spec.qk_norm is not None else None
    # The attention kernels norm the heads themselves, restating a weight-only RMS norm from `weight` and `eps`.
    # A head norm of another kind (one that does not say `fusable_rms`) is evaluated by its own `forward` on the
    # heads as rows [tokens * heads, head_dim], and the kernels are then given no norm to do.
    self.heads_norm_fused = self.q_norm is None or bool(getattr(self.q_norm, "fusable_rms", False))
    self.shares_kv = bool(getattr(spec, "shares_kv", False))
    self.qkv_weight: Optional[torch.Tensor] = None   # q rows only when the keys and values are borrowed
    self.o_weight: Optional[torch.Tensor] = None
    self.qkv_bias: Optional[torch.Tensor] = None     # only when the spec asks for them
    self.o_bias: Optional[torch.Tensor] = None

  # ------------------------------------------------------------------ tensors
  def param_specs(self) -> List[ParamSpec]:
    qn, kn, vn, on = self.spec.tensor_names[:4]
    nq, nkv, d, H = self.nq, self.nkv, self.d, self.hidden
    if self.shares_kv:
      qkv = ParamSpec("qkv_weight", (nq * d, H), (Source(qn + ".weight", nq * d),))
    else:
      qkv = ParamSpec("qkv_weight", ((nq + 2 * nkv) * d, H),
                      (Source(qn + ".weight", nq * d), Source(kn + ".weight", nkv * d), Source(vn + ".weight", nkv * d)))
    out = [qkv, ParamSpec("o_weight", (H, nq * d), (Source(on + ".weight", H),))]
    if getattr(self.spec, "qkv_bias", False):
      srcs = (Source(qn + ".bias", nq * d),) if self.shares_kv else \
          (Source(qn + ".bias", nq * d), Source(kn + ".bias", nkv * d), Source(vn + ".bias", nkv * d))
      out.append(ParamSpec("qkv_bias", (sum(s.rows for s in srcs),), srcs, init="normal"))
    if getattr(self.spec, "o_bias", False):
      out.append(ParamSpec("o_bias", (H,), (Source(on + ".bias", H),), init="normal"))
    return out

  def children(self) -> List[Tuple[str, Part]]:
    if self.q_norm is None:
      return []
    out = [(self.spec.tensor_names[4] + ".", self.q_norm)]
    if not self.shares_kv:
      out.append((self.spec.tensor_names[5] + ".", self.k_norm))
    return out

  def products(self):
    return [(self.qkv_weight, False), (self.o_weight, False)]

  def cache_requirement(self):
    return PagedKV(num_kv_heads=self.nkv, head_dim=self.d, window=self.window)

  # ------------------------------------------------------------------ one step
  def forward(self, x, ctx, cache) -> torch.Tensor:
    return self.forward_lazy(x, ctx, cache).materialize()

  def forward_lazy(self, x, ctx, cache) -> PendingLinear:
    """The same with the output projection left pending, so that the block can fold the add and the next norm
    into it."""
    T = x.shape[0]
    qkv = linear(x, self.qkv_weight, bias=self.qkv_bias)
    table = self.position.rotary_table()
    q_weight = k_weight = None
    eps = 0.0
    if self.q_norm is not None and self.heads_norm_fused:
      q_weight, eps = self.q_norm.weight, self.q_norm.eps
      k_weight = self.k_norm.weight if not self.shares_kv else None
    elif self.q_norm is not None:
      self._norm_heads(qkv)
    if ctx.num_multi == 0 and self.heads_norm_fused and not self.shares_kv and (table is None or table.shape[1] == self.d) and \
        ops.mfma_attention_supported(qkv.dtype, self.nq, self.nkv, self.d, cache.page_size):
      # a step of decoded tokens only: the attention kernel norms, rotates and caches by itself
      out = torch.empty((T, self.nq * self.d), dtype=qkv.dtype, device=qkv.device)
      self._attend_decode(qkv, out, ctx, cache, 0, ctx.num_requests, front=(table, eps, q_weight, k_weight))
      return PendingLinear(out, self.o_weight, self.o_bias)
    if self.shares_kv:
      # only queries of its own: they are normed and rotated; the borrowed pages are read, never written
      ops.qk_norm_rope_cache(qkv, self.nq, 0, self.d, q_weight, None, eps, table, ctx.positions, None, None, None,
                             cache.page_size)
    else:
      ops.qk_norm_rope_cache(qkv, self.nq, self.nkv, self.d, q_weight, k_weight, eps, table, ctx.positions,
                             cache.k, cache.v, ctx.slots[cache.group], cache.page_size)
    out = torch.empty((T, self.nq * self.d), dtype=qkv.dtype, device=qkv.device)
    self._attend(qkv, out, ctx, cache)
    return PendingLinear(out, self.o_weight, self.o_bias)

  def _norm_heads(self, qkv: torch.Tensor) -> None:
    """The head norms by the norm parts' own `forward`, in place on the q and k columns of the fused projection."""
    T = qkv.shape[0]
    nq, nkv, d = self.nq, self.nkv, self.d
    q = qkv[:, :nq * d]
    q.copy_(self.q_norm.forward(q.reshape(T * nq, d)).view(T, nq * d))
    if not self.shares_kv:
      k = qkv[:, nq * d:(nq + nkv) * d]
      k.copy_(self.k_norm.forward(k.reshape(T * nkv, d)).view(T, nkv * d))

  def _attend(self, qkv: torch.Tensor, out: torch.Tensor, ctx, cache) -> None:
    nq, nkv, d, window = self.nq, self.nkv, self.d, self.window or 0
    table = ctx.block_tables[cache.group]
    if not ops.mfma_attention_supported(qkv.dtype, nq, nkv, d, cache.page_size):
      T = qkv.shape[0]
      heads_a_wave, waves_a_unit = ops.plain_attention_geometry(qkv.dtype, nq, nkv, d, cache.page_size)
      splits = plain_splits(T * (nq // heads_a_wave), min(ctx.max_kv_len, window) if window else ctx.max_kv_len,
                            waves_a_unit * ops.compute_units())
      part_o = part_ml = None
      if splits > 1:
        part_o = ctx.scratch("attn_part_o", T * nq * splits * d, torch.float32)
        part_ml = ctx.scratch("attn_part_ml", T * nq * splits * 2, torch.float32)
      ops.paged_attention(qkv, nq, nkv, d, out, cache.k, cache.v, table, ctx.token_req, ctx.cu_q, ctx.kv_len,
                          self.scale, window, splits, part_o, part_ml)
      return
    # entries with several tokens come first, single tokens last
    if ctx.num_multi > 0:
      wide = ops.attn_prefill_wide_pays(ctx.q_lens[:ctx.num_multi], nq, nkv, d)
      work = ctx.prefill_work(wide or ops.attn_prefill_tokens_per_block(nq, nkv, d))
      ops.attn_prefill(qkv, nq, nkv, d, out, cache.k, cache.v, table, work, ctx.cu_q, ctx.kv_len, self.scale, window,
                       variant="wide" if wide else "auto")
    n_single = ctx.num_requests - ctx.num_multi
    if n_single > 0:
      self._attend_decode(qkv, out, ctx, cache, ctx.num_multi, n_single)

  def _attend_decode(self, qkv, out, ctx, cache, first: int, count: int, front=None) -> None:
    """Entries first .. first + count - 1, one token each.  With `front` = (rotation table, eps, q norm weight, k norm
    weight) the projection is still raw and the kernel does the head norms, the rotation and the cache write too."""
    nq, nkv, d, window = self.nq, self.nkv, self.d, self.window or 0
    table = ctx.block_tables[cache.group]
    tile_keys, waves = ops.attn_decode_geometry(d)
    splits, wide = decode_launch(count * nkv, min(ctx.max_kv_len, window) if window else ctx.max_kv_len, tile_keys,
                                 waves, 2 * ops.compute_units())
    need = count * nq * splits
    part_o = ctx.scratch("attn_part_o", need * d, torch.float32)
    part_ml = ctx.scratch("attn_part_ml", need * 2, torch.float32)
    streams = ops.decode_streams_keys(count, nkv, d, min(ctx.max_kv_len, window) if window else ctx.max_kv_len)
    if front is None:
      ops.attn_decode(qkv, nq, nkv, d, out, cache.k, cache.v, table, ctx.cu_q, ctx.kv_len, first, count, splits,
                      part_o, part_ml, self.scale, window, streams, wide)
    else:
      ops.attn_decode_front(qkv, nq, nkv, d, out, cache.k, cache.v, table, ctx.cu_q, ctx.kv_len, first, count, splits,
                            part_o, part_ml, self.scale, window, front[2], front[3], front[1], front[0],
                            ctx.positions, ctx.slots[cache.group], streams, wide)


def decode_splits(num_head_entries: int, max_keys: int, tile_keys: int = 64, waves: int = 4,
                  resident_workgroups: int = 512) -> int:
  """Into how many key ranges (workgroups of `waves` waves, each taking macro tiles of `tile_keys` keys in turn) a
  decoding request is cut.  `resident_workgroups` run on the chip at once (two per compute unit, whatever the head
  size; the default is an MI355X's 2 x 256, the attention part passes its device's): the ranges are as many as still fit in one such round, since a second round that is nearly empty costs as
  much as a full one (96 kv-head entries: 5 ranges take 27 us, 6 take 32); when one range per entry would leave
  more than a fifth of the round empty, two are used (384 entries: 77 against 82 us).  At most 64 (one request of
  32,768 keys: 34.4 us with 32 ranges, 32.2 with 64, 34.0 with 128; beyond 32 ranges the merge is a kernel of four
  waves per head, whose loads are all on their way at once), and at least one macro tile per wave."""
  tiles = -(-max_keys // tile_keys)
  n = max(1, num_head_entries)
  want = max(1, resident_workgroups // n)
  if want == 1 and n < resident_workgroups and 5 * n <= 4 * resident_workgroups:
    want = 2
  return int(max(1, min(want, max(1, tiles // waves), 64)))


def decode_launch(num_head_entries: int, max_keys: int, tile_keys: int = 64, waves: int = 4,
                  resident_workgroups: int = 512):
  """(key ranges, wide) of a decode launch: `decode_splits`' ranges with workgroups of `waves` waves, or half the
  ranges with workgroups of twice the waves (`wide`): half as many workgroups to hand out, fewer heads a wave for the
  norms and the rotation, half the partials to merge or none at all.  Wide workgroups pay where they are a single
  round of one a compute unit and still half a round (or, where they need no merge, a quarter): requests x us with
  the merge, 2,048 keys each, wide against not: 4 x 14.1 / 14.5, 8 x 19.2 / 20.5, 16 x 30.1 / 32.4, 24 x 40.0 / 46.0,
  32 x 50.2 / 53.8; 512 keys each: 8 x 10.5 / 12.3, 32 x 17.1 / 21.5; but 1 x 12.8 / 11.5 (too few workgroups), 12 x
  33.8 / 26.6 and 48 x 82.1 / 77.4 (a second round)."""
  splits = decode_splits(num_head_entries, max_keys, tile_keys, waves, resident_workgroups)
  units = resident_workgroups // 2
  half = (splits + 1) // 2
  groups = max(1, num_head_entries) * half
  if splits >= 2 and groups <= units and (2 * groups >= units or (half == 1 and 4 * groups >= units)):
    return half, True
  return splits, False


def plain_splits(num_waves: int, max_keys: int, resident_waves: int = 4096) -> int:
  """Into how many key ranges the plain kernel (one wave per token and group of query heads) cuts each token's keys:
  as many as fill the chip's wave slots once (`resident_waves`: 8 or 16 on each compute unit, by the kernel that
  runs, `ops.plain_attention_geometry`; the default is 16 x 256; one wave more than fit costs a second round: 40
  against 31.5 us for 8 requests of 2,048 keys in 33 against 32 ranges), each range at least one tile of 64 keys, at
  most 64 ranges: a wave takes its tiles one after the other, so few tokens over many keys are as quick as their
  longest range.  Prompt portions have waves enough and stay whole."""
  want = resident_waves // max(1, num_waves)
  tiles = -(-max_keys // 64)
  return int(max(1, min(want, tiles, 64)))


register_mixer("paged_attention", PagedAttention)
