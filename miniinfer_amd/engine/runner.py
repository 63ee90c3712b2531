"""The step function: one batch of (request, its next tokens) through the model, from the cache.

A step takes any mix of prompt portions and single decoded tokens, cut anywhere.  It runs only
the tokens it is given: their keys and values are written to the requests' pages, attention
reads everything earlier from the cache, and logits come back only for the positions asked for.

The reference's counterpart is `ModelRunner.forward(ForwardBatch)` with its three batch modes
(miniinfer/engine/model_runner.py:123-139, miniinfer/scheduler/scheduler_batch.py:235-441,
miniinfer/kvcache/kv_cache_manager.py:211-328,330-599,601-662).  Here there is one mode: every
entry is `(request, start position, n tokens >= 1)`; positions are start + i
(scheduler_batch.py:450-470), a decode is the case n = 1 (kv_cache_manager.py:384-385).  All
index arrays are built on the host with numpy and reach the device in one copy.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheManager, LayerCache
from ..parts import DecoderModel


@dataclass
class StepEntry:
  req: Hashable
  tokens: Sequence[int]
  want: Sequence[int] = ()      # indices into `tokens` whose logits are wanted


class StepContext:
  """Device-side description of one step, shared by all layers."""

  def __init__(self):
    self.num_tokens = 0
    self.num_requests = 0
    self.num_logit_rows = 0
    self.token_ids: torch.Tensor = None      # [T] int32
    self.positions: torch.Tensor = None      # [T] int32
    self.token_req: torch.Tensor = None      # [T] int32, index of the token's request in this step
    self.cu_q: torch.Tensor = None           # [B+1] int32, first token of each request
    self.kv_len: torch.Tensor = None         # [B] int32, keys per request after this step
    self.req_slots: torch.Tensor = None      # [B] int32, state slot of each request
    self.logit_rows: torch.Tensor = None     # [R] int32, flattened token rows whose logits are wanted
    self.slots: List[torch.Tensor] = []      # per paged group: [T] int32, page * page_size + offset
    self.block_tables: List[torch.Tensor] = []   # per paged group: [B, W] int32
    # host copies
    self.q_lens: List[int] = []
    self.kv_lens: List[int] = []
    self.num_multi = 0                       # requests with more than one token come first
    self.max_q_len = 0
    self.max_kv_len = 0
    self._cache: CacheManager = None
    self._device = None
    self._work: Dict[int, torch.Tensor] = {}
    self._scratch: Dict[str, torch.Tensor] = {}

  def layer_cache(self, layer: int) -> LayerCache:
    return self._cache.layer_cache(layer)

  def prefill_work(self, tokens_per_block: int) -> torch.Tensor:
    """[n, 2] int32 = (entry, block of `tokens_per_block` query tokens within it) for every multi-token entry;
    built once per step and granule, shared by all layers."""
    w = self._work.get(tokens_per_block)
    if w is None:
      items = [(b, i) for b in range(self.num_multi) for i in range(-(-self.q_lens[b] // tokens_per_block))]
      # the blocks with the most keys first: they take longest
      items.sort(key=lambda it: -(self.kv_lens[it[0]] - self.q_lens[it[0]] + (it[1] + 1) * tokens_per_block))
      w = torch.tensor(items, dtype=torch.int32).reshape(-1, 2).to(self._device, non_blocking=True)
      self._work[tokens_per_block] = w
    return w

  def scratch(self, name: str, numel: int, dtype: torch.dtype) -> torch.Tensor:
    """A device buffer that lives for this step (reused by every layer that asks under the same name)."""
    t = self._scratch.get(name)
    if t is None or t.numel() < numel or t.dtype != dtype:
      t = torch.empty(numel, dtype=dtype, device=self._device)
      self._scratch[name] = t
    return t


class ModelRunner:
  def __init__(self, model: DecoderModel, cache: CacheManager):
    self.model = model
    self.cache = cache
    self.device = model.ctx.device
    self.vocab_size = model.spec.vocab_size
    self._staging: Optional[torch.Tensor] = None

  # ------------------------------------------------------------------ host side of a step
  def _stage(self, n: int) -> torch.Tensor:
    if self._staging is None or self._staging.numel() < n:
      cap = max(4096, 1 << (n - 1).bit_length())
      self._staging = torch.empty(cap, dtype=torch.int32, pin_memory=(self.device.type == "cuda"))
    return self._staging

  def build_context(self, entries: Sequence[StepEntry]):
    """Grows the requests' page tables and lays the step out.  Returns (ctx, order, new lengths)."""
    cache = self.cache
    P = cache.page_size
    if not entries:
      raise ValueError("a step needs at least one entry")
    seen = set()
    for e in entries:
      if e.req in seen:
        raise ValueError(f"request {e.req!r} appears twice in one step")
      seen.add(e.req)
      if len(e.tokens) == 0:
        raise ValueError(f"request {e.req!r} brings no tokens")
      if not cache.has(e.req):
        raise KeyError(f"request {e.req!r} was not admitted to the cache")
      for w in e.want:
        if not 0 <= w < len(e.tokens):
          raise IndexError(f"request {e.req!r}: wanted place {w} is outside its {len(e.tokens)} tokens")
    # multi-token entries first, single tokens last (stable), so kernels that treat the two
    # kinds differently get contiguous ranges
    order = sorted(range(len(entries)), key=lambda i: 0 if len(entries[i].tokens) > 1 else 1)
    B = len(entries)
    q_lens = [len(entries[i].tokens) for i in order]
    starts = [cache.length(entries[i].req) for i in order]
    kv_lens = [s + n for s, n in zip(starts, q_lens)]
    T = sum(q_lens)
    # all or nothing: check the whole step's need before any table grows
    need = sum(cache.pages_needed(entries[i].req, kv) for i, kv in zip(order, kv_lens))
    if need > cache.num_free_pages():
      from ..cache.manager import OutOfPages
      raise OutOfPages(f"step needs {need} new pages, {cache.num_free_pages()} are free")
    for i, kv in zip(order, kv_lens):
      cache.grow(entries[i].req, kv)

    cu_q = np.zeros(B + 1, dtype=np.int32)
    np.cumsum(q_lens, out=cu_q[1:])
    token_ids = np.empty(T, dtype=np.int32)
    positions = np.empty(T, dtype=np.int32)
    token_req = np.empty(T, dtype=np.int32)
    for b, i in enumerate(order):
      lo, hi = cu_q[b], cu_q[b + 1]
      token_ids[lo:hi] = np.asarray(entries[i].tokens, dtype=np.int64)
      positions[lo:hi] = np.arange(starts[b], kv_lens[b], dtype=np.int32)
      token_req[lo:hi] = b
    if T and (token_ids.min() < 0 or token_ids.max() >= self.vocab_size):
      raise ValueError(f"token id outside [0, {self.vocab_size})")
    # logit rows in the order of the entries as given, then of `want`
    first_row = {i: int(cu_q[b]) for b, i in enumerate(order)}
    rows = [first_row[i] + w for i, e in enumerate(entries) for w in e.want]
    R = len(rows)
    req_slots = np.asarray([cache.slot(entries[i].req) for i in order], dtype=np.int32)

    G = len(cache.paged)
    W = max(1, max(-(-kv // P) for kv in kv_lens))
    tables = np.zeros((G, B, W), dtype=np.int32)
    slots = np.empty((G, T), dtype=np.int32)
    for g in range(G):
      for b, i in enumerate(order):
        tab = cache.table(g, entries[i].req)
        n = min(len(tab), W)
        tables[g, b, :n] = tab[:n]
        pos = positions[cu_q[b]:cu_q[b + 1]]
        slots[g, cu_q[b]:cu_q[b + 1]] = tables[g, b, pos // P] * P + pos % P

    parts = [token_ids, positions, token_req, cu_q, np.asarray(kv_lens, dtype=np.int32), req_slots,
             np.asarray(rows, dtype=np.int32), slots.reshape(-1), tables.reshape(-1)]
    total = sum(p.size for p in parts)
    stage = self._stage(total)
    host = stage.numpy()
    offs = []
    o = 0
    for p in parts:
      host[o:o + p.size] = p
      offs.append(o)
      o += p.size
    dev = torch.empty(total, dtype=torch.int32, device=self.device)
    dev.copy_(stage[:total], non_blocking=False)

    ctx = StepContext()
    ctx._cache = cache
    ctx._device = self.device
    ctx.num_tokens, ctx.num_requests, ctx.num_logit_rows = T, B, R
    ctx.token_ids = dev[offs[0]:offs[0] + T]
    ctx.positions = dev[offs[1]:offs[1] + T]
    ctx.token_req = dev[offs[2]:offs[2] + T]
    ctx.cu_q = dev[offs[3]:offs[3] + B + 1]
    ctx.kv_len = dev[offs[4]:offs[4] + B]
    ctx.req_slots = dev[offs[5]:offs[5] + B]
    ctx.logit_rows = dev[offs[6]:offs[6] + R]
    ctx.slots = [dev[offs[7] + g * T:offs[7] + (g + 1) * T] for g in range(G)]
    ctx.block_tables = [dev[offs[8] + g * B * W:offs[8] + (g + 1) * B * W].view(B, W) for g in range(G)]
    ctx.q_lens, ctx.kv_lens = q_lens, kv_lens
    ctx.num_multi = sum(1 for n in q_lens if n > 1)
    ctx.max_q_len, ctx.max_kv_len = max(q_lens), max(kv_lens)
    return ctx, order, kv_lens

  # ------------------------------------------------------------------ the step
  @torch.no_grad()
  def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
    """Runs the entries as one batch.  Returns float32 logits [number of wanted places, vocab] on the
    device, in the order of the entries and of each entry's `want`."""
    ctx, order, kv_lens = self.build_context(entries)
    logits = self.model.forward(ctx)
    for i, kv in zip(order, kv_lens):
      self.cache.commit(entries[i].req, kv)
    return logits
