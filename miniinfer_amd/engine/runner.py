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

import logging
import warnings
from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheManager, LayerCache
from ..kernels import ops
from ..parts import DecoderModel

log = logging.getLogger("miniinfer_amd")


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
    self.future_tokens: Optional[torch.Tensor] = None   # int32: a token id -(r + 1) stands for future_tokens[r]
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
    self._spare_host: Optional[torch.Tensor] = None   # pinned int32 room behind the step's arrays (work lists)
    self._spare_used = 0
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
      n = 2 * len(items)
      if self._spare_host is not None and self._spare_used + n <= self._spare_host.numel():
        # from the step's pinned staging buffer, so that the copy is queued like the rest of the step's inputs
        host = self._spare_host[self._spare_used:self._spare_used + n]
        self._spare_used += n
        host.copy_(torch.tensor(items, dtype=torch.int32).reshape(-1))
        w = torch.empty(n, dtype=torch.int32, device=self._device)
        w.copy_(host, non_blocking=True)
        w = w.view(-1, 2)
      else:
        w = torch.tensor(items, dtype=torch.int32).reshape(-1, 2).to(self._device, non_blocking=True)
      self._work[tokens_per_block] = w
    return w

  def scratch(self, name: str, numel: int, dtype: torch.dtype, zero: bool = False) -> torch.Tensor:
    """A device buffer that lives for this step (reused by every layer that asks under the same name).
    zero: the buffer is all zero when it is made, and every user leaves it all zero."""
    t = self._scratch.get(name)
    if t is None or t.numel() < numel or t.dtype != dtype:
      t = (torch.zeros if zero else torch.empty)(numel, dtype=dtype, device=self._device)
      self._scratch[name] = t
    return t


class _Layout:
  """Host-side arrays of one step (numpy int32), in the order the device buffer holds them."""
  FIELDS = ("token_ids", "positions", "token_req", "cu_q", "kv_len", "req_slots", "logit_rows", "slots", "tables")

  def __init__(self, T, B, R, G, W):
    self.T, self.B, self.R, self.G, self.W = T, B, R, G, W
    self.sizes = dict(token_ids=T, positions=T, token_req=T, cu_q=B + 1, kv_len=B, req_slots=B, logit_rows=R,
                      slots=G * T, tables=G * B * W)
    self.offsets = {}
    o = 0
    for f in self.FIELDS:
      self.offsets[f] = o
      o += self.sizes[f]
    self.total = o

  def views(self, buf):
    """Slices of a flat int32 buffer (numpy array or torch tensor), one per field."""
    return {f: buf[self.offsets[f]:self.offsets[f] + self.sizes[f]] for f in self.FIELDS}

  def context(self, dev: torch.Tensor, cache: CacheManager, device) -> StepContext:
    v = self.views(dev)
    ctx = StepContext()
    ctx._cache, ctx._device = cache, device
    ctx.num_tokens, ctx.num_requests, ctx.num_logit_rows = self.T, self.B, self.R
    ctx.token_ids, ctx.positions, ctx.token_req = v["token_ids"], v["positions"], v["token_req"]
    ctx.cu_q, ctx.kv_len, ctx.req_slots, ctx.logit_rows = v["cu_q"], v["kv_len"], v["req_slots"], v["logit_rows"]
    ctx.slots = [v["slots"][g * self.T:(g + 1) * self.T] for g in range(self.G)]
    ctx.block_tables = [v["tables"][g * self.B * self.W:(g + 1) * self.B * self.W].view(self.B, self.W)
                        for g in range(self.G)]
    return ctx


class _DecodeGraph:
  """One captured decode step for `B` single-token entries and block tables `W` pages wide.
  Its integer inputs live in one static device buffer that a step refreshes with one copy."""

  def __init__(self, runner: "ModelRunner", B: int, W: int):
    self.B, self.W = B, W
    cache = runner.cache
    self.scratch_slot = cache.scratch_slot
    G = len(cache.paged)
    self.layout = _Layout(T=B, B=B, R=B, G=G, W=W)
    # two pinned staging buffers, used in turn: the copy of one step may still be queued on the stream while the
    # host lays out the next step (the engine reads a step's tokens only after it has launched the next one)
    self.stages = [torch.zeros(self.layout.total, dtype=torch.int32, pin_memory=True) for _ in range(2)]
    self.hosts = [self.layout.views(st.numpy()) for st in self.stages]
    self.turn = 0
    for self.host in self.hosts:
      # what never changes: one token per entry, every row's logits
      self.host["token_req"][:] = np.arange(B, dtype=np.int32)
      self.host["cu_q"][:] = np.arange(B + 1, dtype=np.int32)
      self.host["logit_rows"][:] = np.arange(B, dtype=np.int32)
      self.fill_padding(0)
    self.stage = self.stages[0]
    self.dev = torch.zeros(self.layout.total, dtype=torch.int32, device=runner.device)
    self.dev.copy_(self.stage)
    ctx = self.layout.context(self.dev, cache, runner.device)
    ctx.q_lens, ctx.kv_lens = [1] * B, [W * cache.min_page_size] * B   # host-side sizes the kernels are tuned for
    ctx.num_multi, ctx.max_q_len, ctx.max_kv_len = 0, 1, W * cache.min_page_size
    ctx.future_tokens = runner.future_tokens
    self.ctx = ctx
    # every entry is padding while warming up and capturing: it reads and writes the scratch page only
    runner.set_weight_streaming(B * W * cache.min_page_size)
    before, off_rule = ops.library_products_run(), ops.off_rule_products_run()
    self.graph, self.logits = self._capture(runner, ctx)
    self.ok = True
    after = ops.library_products_run()
    library, avoidable = after[0] != before[0], after[1] != before[1]
    # Which kernel runs a product was measured on each product alone (or follows a rule).  Inside a step that can
    # still lose: to this library's own kernels, which need no norm and activation kernels beside them, where a
    # product went to the library; or to the rule's choices, where the measurement chose otherwise (at 48 requests
    # of the Qwen3-8B shape by 4% of the step).  Such a step is captured those ways too and the quickest graph kept.
    others = []
    self.kept = "as chosen"
    if avoidable and runner.compare_captures:
      with ops.own_products_only():
        others.append(self._capture(runner, ctx) + ((after[0] - before[0]) > (after[1] - before[1]), "own kernels only"))
    if ops.off_rule_products_run() != off_rule and runner.compare_captures:
      mark = ops.library_products_run()
      with ops.rule_products_only():
        others.append(self._capture(runner, ctx) + (ops.library_products_run()[0] != mark[0], "by rule"))
    if others:
      best = self._replay_ms(self.graph)
      timings = [f"as chosen {best * 1e3:.0f} us"]
      for graph, logits, uses_library, how in others:
        ms = self._replay_ms(graph)
        timings.append(f"{how} {ms * 1e3:.0f} us")
        if ms <= best:
          best, self.graph, self.logits, library, self.kept = ms, graph, logits, uses_library, how
      log.info("decode graph for %d entries, tables of %d pages: %s -> kept %s", B, W, ", ".join(timings), self.kept)
    if library and runner.check_graphs:
      # What a library records into a graph is its own affair (clears of a workspace have replayed wrongly): the
      # graph is replayed a few times, with eager work in between, against the eager result of the same (padding)
      # inputs, and a graph that does not reproduce it is not used.  A library may choose another kernel under
      # capture than it does eagerly, which moves the result by a rounding of bfloat16 (0.4% of the largest logit
      # has been seen): the replays must agree with the eager result to within 1.5% of the largest logit, and
      # with one another exactly, which a stale workspace would not.
      want = runner.model.forward(ctx).clone()
      bound = 1.5e-2 * max(float(want.abs().max()), 1e-6)
      first = None
      for _ in range(3):
        self.graph.replay()
        got = self.logits.clone()
        torch.cuda.synchronize()
        if first is None:
          first = got
        if float((got - want).abs().max()) > bound or not torch.equal(got, first):
          self.ok = False
          warnings.warn(f"the captured decode step for {B} entries does not reproduce the eager step; "
                        "such steps run without a graph")
          break
        want = runner.model.forward(ctx).clone()

  @staticmethod
  def _capture(runner: "ModelRunner", ctx):
    side = ops.side_stream(runner.device)
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
      runner.model.forward(ctx)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    # one memory pool for all captured steps of a runner: they never run side by side, so what one holds while it
    # runs can be another's; only each graph's logits stay its own
    with torch.cuda.graph(graph, pool=runner.graph_pool()):
      logits = runner.model.forward(ctx)
    return graph, logits

  @staticmethod
  def _replay_ms(graph) -> float:
    graph.replay()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best = float("inf")
    for _ in range(3):
      start.record()
      graph.replay()
      end.record()
      torch.cuda.synchronize()
      best = min(best, start.elapsed_time(end))
    return best

  def fill_padding(self, first: int) -> None:
    """Entries first.. are padding: token 0 at position 0 of a request of one key in the scratch page, whose
    fixed-size state is the scratch row that no request ever holds."""
    h = self.host
    h["token_ids"][first:] = 0
    h["positions"][first:] = 0
    h["kv_len"][first:] = 1
    h["req_slots"][first:] = self.scratch_slot
    G, B, W = self.layout.G, self.B, self.W
    h["slots"].reshape(G, B)[:, first:] = 0
    h["tables"].reshape(G, B, W)[:, first:, :] = 0

  def next_host(self):
    """The staging views to lay the next step out in."""
    self.turn ^= 1
    self.stage, self.host = self.stages[self.turn], self.hosts[self.turn]
    return self.host

  def run(self) -> torch.Tensor:
    self.dev.copy_(self.stage, non_blocking=True)
    self.graph.replay()
    return self.logits


_GRAPH_BATCHES = (1, 2, 4, 8, 12, 16, 24, 32, 48, 64, 96, 128, 192, 256)


def graph_bucket_rows(max_requests: int, max_tokens: int, page_size: int):
  """(rows of all batch buckets that steps of up to `max_requests` single tokens can fall into, number of
  table-width buckets up to `max_tokens` tokens a request): what the captured decode steps of an engine with these
  limits keep alive at most, one row of logits per bucket row and width."""
  top = next((b for b in _GRAPH_BATCHES if b >= max_requests), _GRAPH_BATCHES[-1])
  rows = sum(b for b in _GRAPH_BATCHES if b <= top)
  W = max(1, -(-max_tokens // page_size))
  widths = max(1, (max(16, 1 << (W - 1).bit_length()) // 16).bit_length())
  return rows, widths


class ModelRunner:
  def __init__(self, model: DecoderModel, cache: CacheManager, use_graphs: bool = False,
               choices: Optional[ops.ProductChoices] = None, compare_captures: bool = True):
    """use_graphs: replay steps that hold only single decoded tokens (at most 256 of them) from HIP graphs,
    captured on demand per (batch bucket, block-table width bucket).  choices: the table that says which kernel
    runs a product of few rows; it is this runner's own (a new, empty one by default: every product by rule) and is
    the current one while the runner steps.  compare_captures: a step whose products could go more than one way
    is captured each way and the quickest graph kept; off, it is captured once, as the table says."""
    self.model = model
    self.choices = choices if choices is not None else ops.ProductChoices()
    self.compare_captures = compare_captures
    self.cache = cache
    self.device = model.ctx.device
    self.vocab_size = model.spec.vocab_size
    # a part that cannot be recorded into a graph (one that reads device values on the host, say) declares
    # `capturable = False`; the steps of a model that holds such a part always run eagerly
    self.use_graphs = use_graphs and self.device.type == "cuda" and model.is_capturable()
    self.check_graphs = True      # replay every captured step against its eager result before it is used
    # two pinned staging buffers for eager steps, used in turn, each with the event of the copy that last read it:
    # a step's copy may still be queued on the stream while the host lays out the next step
    self._staging: List[Optional[torch.Tensor]] = [None, None]
    self._staging_done: List[Optional[torch.cuda.Event]] = [None, None]
    self._staging_turn = 0
    self._allow_future = False
    self._graphs: Dict[tuple, _DecodeGraph] = {}
    self._graph_pool = None
    # Tokens of the last step's sampling output, by row.  A token id -(r + 1) in a step's entries stands for
    # future_tokens[r] as it is when the step's embedding kernel runs: whoever samples writes here, and may
    # launch the next step before reading the tokens back.
    self.future_tokens = torch.zeros(max(1, cache.max_requests), dtype=torch.int32, device=self.device)
    if self.device.type == "cuda":
      from ..kernels import prepare
      prepare(cache.dtype, [g.need.head_dim for g in cache.paged])      # what is not built yet, side by side

  def graph_pool(self):
    if self._graph_pool is None:
      self._graph_pool = torch.cuda.graph_pool_handle()
    return self._graph_pool

  # ------------------------------------------------------------------ host side of a step
  def _stage(self, n: int) -> torch.Tensor:
    """The pinned buffer to lay the next eager step out in: the one of the two that was not used last, once the
    copy that last read it is done (that copy was queued two steps back, so the host practically never waits)."""
    self._staging_turn ^= 1
    t = self._staging_turn
    if self._staging_done[t] is not None:
      self._staging_done[t].synchronize()
      self._staging_done[t] = None
    if self._staging[t] is None or self._staging[t].numel() < n:
      cap = max(4096, 1 << (n - 1).bit_length())
      self._staging[t] = torch.empty(cap, dtype=torch.int32, pin_memory=(self.device.type == "cuda"))
    return self._staging[t]

  def _plan(self, entries: Sequence[StepEntry]):
    """Checks the entries, grows the requests' page tables (all or nothing), and orders the entries: those
    with several tokens first, single tokens last (stable), so kernels that treat the two kinds differently
    get contiguous ranges.  Returns (order, q_lens, starts, kv_lens)."""
    cache = self.cache
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
      for t in e.tokens:
        if not (0 <= t < self.vocab_size or (self._allow_future and -self.future_tokens.numel() <= t < 0)):
          raise ValueError(f"request {e.req!r}: token id {t} is outside [0, {self.vocab_size})")
    order = sorted(range(len(entries)), key=lambda i: 0 if len(entries[i].tokens) > 1 else 1)
    q_lens = [len(entries[i].tokens) for i in order]
    starts = [cache.length(entries[i].req) for i in order]
    kv_lens = [s + n for s, n in zip(starts, q_lens)]
    room = cache.room()
    for i, kv in zip(order, kv_lens):
      if not cache.take(room, entries[i].req, kv):
        from ..cache.manager import OutOfPages
        raise OutOfPages(f"the step's requests need more pages than are free (request {entries[i].req!r} growing to "
                         f"{kv} tokens; free pages per cache group: {cache.room()})")
    for i, kv in zip(order, kv_lens):
      cache.grow(entries[i].req, kv)
    return order, q_lens, starts, kv_lens

  def _fill(self, host, lay: _Layout, entries, order, q_lens, starts, kv_lens) -> None:
    """Writes the step's integer arrays into `host` (views of a flat buffer laid out by `lay`).  Only the first
    len(order) entries are written; a wider layout's tail belongs to the caller."""
    cache = self.cache
    B, T, G, W = len(order), sum(q_lens), lay.G, lay.W
    cu = np.zeros(B + 1, dtype=np.int64)
    np.cumsum(q_lens, out=cu[1:])
    host["cu_q"][:B + 1] = cu
    host["kv_len"][:B] = kv_lens
    tables = host["tables"].reshape(G, lay.B, W)
    slots = host["slots"].reshape(G, lay.T)
    for b, i in enumerate(order):
      lo, hi = int(cu[b]), int(cu[b + 1])
      host["token_ids"][lo:hi] = entries[i].tokens
      pos = np.arange(starts[b], kv_lens[b], dtype=np.int32)
      host["positions"][lo:hi] = pos
      host["token_req"][lo:hi] = b
      host["req_slots"][b] = cache.slot(entries[i].req)
      for g in range(G):
        tab = cache.table(g, entries[i].req)
        P = cache.paged[g].page_size
        n = min(len(tab), W)
        tables[g, b, :n] = tab[:n]
        tables[g, b, n:] = 0
        slots[g, lo:hi] = tables[g, b, pos // P] * P + pos % P

  def build_context(self, entries: Sequence[StepEntry]):
    """Grows the requests' page tables and lays the step out on the device.  Returns (ctx, order, new lengths)."""
    cache = self.cache
    order, q_lens, starts, kv_lens = self._plan(entries)
    B, T = len(order), sum(q_lens)
    # logit rows in the order of the entries as given, then of `want`
    first = np.zeros(B, dtype=np.int64)
    first[1:] = np.cumsum(q_lens)[:-1]
    first_row = {i: int(first[b]) for b, i in enumerate(order)}
    rows = [first_row[i] + w for i, e in enumerate(entries) for w in e.want]
    W = max(1, max(-(-kv // cache.min_page_size) for kv in kv_lens))
    lay = _Layout(T=T, B=B, R=len(rows), G=len(cache.paged), W=W)
    spare = 2 * (T // 4 + B + 1)           # room for a list of (entry, block of >= 4 query tokens)
    stage = self._stage(lay.total + spare)
    host = lay.views(stage.numpy())
    self._fill(host, lay, entries, order, q_lens, starts, kv_lens)
    host["logit_rows"][:] = rows
    dev = torch.empty(lay.total, dtype=torch.int32, device=self.device)
    dev.copy_(stage[:lay.total], non_blocking=True)
    if self.device.type == "cuda":
      self._staging_done[self._staging_turn] = torch.cuda.Event()
      self._staging_done[self._staging_turn].record()
    ctx = lay.context(dev, cache, self.device)
    ctx.q_lens, ctx.kv_lens = q_lens, kv_lens
    ctx.num_multi = sum(1 for n in q_lens if n > 1)
    ctx.max_q_len, ctx.max_kv_len = max(q_lens), max(kv_lens)
    ctx.future_tokens = self.future_tokens
    if self.device.type == "cuda":
      ctx._spare_host = stage[lay.total:lay.total + spare]
    return ctx, order, kv_lens

  # ------------------------------------------------------------------ the step
  @torch.no_grad()
  def step(self, entries: Sequence[StepEntry], allow_future: bool = False) -> torch.Tensor:
    """Runs the entries as one batch.  Returns float32 logits [number of wanted places, vocab] on the
    device, in the order of the entries and of each entry's `want`.  With `allow_future`, a token id -(r + 1)
    is taken from `future_tokens[r]` on the device."""
    self._allow_future = allow_future
    with self.choices:
      if self.use_graphs and len(entries) <= _GRAPH_BATCHES[-1] and all(len(e.tokens) == 1 for e in entries):
        return self._step_from_graph(entries)
      return self._step_eager(entries)

  def graph_buckets(self, num_requests: int, num_tokens: int):
    """(batch bucket, block-table width bucket) of the graph that a step of `num_requests` single tokens replays
    when the longest of them holds `num_tokens` tokens."""
    cache = self.cache
    Bb = next(b for b in _GRAPH_BATCHES if b >= num_requests)
    W = max(1, -(-num_tokens // cache.min_page_size))
    Wb = max(16, 1 << (W - 1).bit_length())
    return Bb, min(Wb, max(cache.max_pages_per_request, W))

  @torch.no_grad()
  def capture_graphs(self, max_requests: int, max_tokens: int) -> int:
    """Captures, ahead of their first use, the graphs of every batch bucket up to `max_requests` and every width
    bucket up to `max_tokens` tokens (the reference captures its graphs when the engine starts:
    miniinfer/engine/llm_engine.py:281-313).  Returns how many graphs there are."""
    if not self.use_graphs:
      return 0
    P = self.cache.min_page_size
    widths = sorted({self.graph_buckets(1, n)[1] for n in
                     [P * (16 << i) for i in range(32) if P * (16 << i) < max_tokens] + [max_tokens]})
    with self.choices:
      for b in _GRAPH_BATCHES:
        if b > max(1, max_requests) and b != self.graph_buckets(max(1, max_requests), 1)[0]:
          continue
        for w in widths:
          if (b, w) not in self._graphs:
            self._graphs[(b, w)] = _DecodeGraph(self, b, w)
    return len(self._graphs)

  def set_weight_streaming(self, cached_tokens_bound: int) -> None:
    """Says, for the step that follows, whether the weights are kept out of the last-level cache: they are where
    the keys and values of the step's requests (at most `cached_tokens_bound` tokens) can stay there instead."""
    self.choices.stream_weights = ops.weights_stream_past_cache(cached_tokens_bound * self.cache.token_bytes())

  def _step_eager(self, entries: Sequence[StepEntry]) -> torch.Tensor:
    ctx, order, kv_lens = self.build_context(entries)
    self.set_weight_streaming(sum(kv_lens))
    logits = self.model.forward(ctx)
    if ctx._spare_used:                     # further copies out of the staging buffer were queued by the layers
      self._staging_done[self._staging_turn].record()
    for i, kv in zip(order, kv_lens):
      self.cache.commit(entries[i].req, kv)
    return logits

  def _step_from_graph(self, entries: Sequence[StepEntry]) -> torch.Tensor:
    """A step of single tokens only, replayed from the graph of its batch and table-width buckets."""
    cache = self.cache
    order, q_lens, starts, kv_lens = self._plan(entries)     # all single tokens: order is the given order
    B = len(entries)
    Bb, Wb = self.graph_buckets(B, max(kv_lens))
    g = self._graphs.get((Bb, Wb))
    if g is None:
      g = _DecodeGraph(self, Bb, Wb)
      self._graphs[(Bb, Wb)] = g
    if not g.ok:
      return self._step_eager(entries)
    self._fill(g.next_host(), g.layout, entries, order, q_lens, starts, kv_lens)
    g.fill_padding(B)
    logits = g.run()
    for i, kv in zip(order, kv_lens):
      cache.commit(entries[i].req, kv)
    rows = [b for b, e in enumerate(entries) for w in e.want]
    if rows == list(range(B)):
      return logits[:B]
    if not rows:
      return logits[:0]
    return logits.index_select(0, torch.tensor(rows, dtype=torch.int64, device=self.device))
