"""The cache manager: pages of keys and values with a block table per request, and slots of
fixed-size per-request state.

Layers are put into groups by what they need.  All layers that keep every key with the same
geometry form one group; layers that keep a window of keys form another; each group has a page
pool, a free list and block tables of its own, because its pages come back at other times (a
window group gives a page back as soon as the window has passed it).  Layers whose mixer keeps
a state of fixed size get a row in a state tensor, indexed by the request's slot.

Everything here is host-side bookkeeping on Python lists; the only device memory is the page
and state storage itself.  The reference keeps a token-granular table on the device and derives
page tables from it at every step (miniinfer/kvcache/memory_pool.py:245-499,
miniinfer/kvcache/kv_cache_manager.py:211-328,601-662); the rules kept from it are: a new page is
opened exactly when a token crosses a page edge (memory_pool.py:217-242), a partial page is filled
before a new one is opened, page 0 is never handed out (memory_pool.py:422-426), and a finished
request gives everything back (kv_cache_manager.py:718-750).
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import torch

from ..parts.base import FixedState, PagedKV


class OutOfPages(RuntimeError):
  pass


class OutOfSlots(RuntimeError):
  pass


class CacheError(RuntimeError):
  pass


SPREAD_EVERY = 33


class PagePool:
  """Free list of page ids 1..num_pages (page 0 is a scratch page that is never handed out).
  Pages freed last are handed out first, so reuse shows early."""

  def __init__(self, num_pages: int):
    if num_pages <= 0:
      raise ValueError("a page pool needs at least one page")
    self.num_pages = num_pages
    # Ascending, but every SPREAD_EVERY-th page only after all the others: requests of the same power-of-two length
    # (benchmarks love 2,048 tokens) would otherwise lie a power of two apart in memory, and the workgroups of a
    # decode step, which walk their requests' pages side by side, would ask the same few memory channels at the same
    # time (64 requests of 2,048 tokens of the 0.6B shape: 17,300 -> 17,830 tok/s with 33, 17,600 with 17, 17,700 with
    # 129; the attention kernel over the engine's own tables 96.3 us a layer, 91.5 with their pages shuffled).
    first = [p for p in range(1, num_pages + 1) if p % SPREAD_EVERY]
    last = [p for p in range(1, num_pages + 1) if p % SPREAD_EVERY == 0]
    self._free: List[int] = (first + last)[::-1]
    self._held = bytearray(num_pages + 1)

  @property
  def num_free(self) -> int:
    return len(self._free)

  def alloc(self, n: int) -> List[int]:
    if n > len(self._free):
      raise OutOfPages(f"{n} pages wanted, {len(self._free)} free of {self.num_pages}")
    out = [self._free.pop() for _ in range(n)]
    for p in out:
      if self._held[p]:
        raise CacheError(f"page {p} was on the free list while held")
      self._held[p] = 1
    return out

  def free(self, pages: Sequence[int]) -> None:
    for p in pages:
      if p <= 0 or p > self.num_pages:
        raise CacheError(f"page id {p} does not exist")
      if not self._held[p]:
        raise CacheError(f"page {p} freed twice")
      self._held[p] = 0
      self._free.append(p)

  def held(self) -> List[int]:
    return [p for p in range(1, self.num_pages + 1) if self._held[p]]


@dataclass
class PagedGroup:
  need: PagedKV
  layers: List[int]
  pool: PagePool
  page_size: int                       # tokens per page of this group
  dtype: torch.dtype
  k: Optional[torch.Tensor] = None     # [len(layers), pages + 1, nkv, page_size, d]
  v: Optional[torch.Tensor] = None     # [len(layers), pages + 1, nkv, d, page_size] (transposed pages)
  tables: Dict[Hashable, List[int]] = field(default_factory=dict)   # per request: page id per page index, 0 = given back


@dataclass
class StateGroup:
  need: FixedState
  layers: List[int]
  state: Optional[torch.Tensor] = None  # [len(layers), max_requests + 1, *shape]; the last row is scratch


@dataclass
class LayerCache:
  """What one layer's mixer sees of the cache."""
  kind: str                              # "paged" | "state" | "none"
  group: int = -1
  k: Optional[torch.Tensor] = None       # [pages + 1, nkv, page_size, d]
  v: Optional[torch.Tensor] = None       # [pages + 1, nkv, d, page_size]
  state: Optional[torch.Tensor] = None   # [max_requests + 1, *shape]; row max_requests is scratch
  page_size: int = 0
  window: Optional[int] = None


def _check_page_size(page_size: int) -> None:
  if page_size <= 0 or page_size & (page_size - 1):
    raise ValueError(f"page_size must be a power of two, got {page_size}")


class CacheManager:
  def __init__(self, layer_needs: Sequence[object], page_size: int, num_pages: int, max_requests: int,
               max_model_len: int, dtype: torch.dtype, device, allocate: bool = True,
               max_step_tokens: Optional[int] = None):
    """layer_needs[i] is the PagedKV / FixedState / None of layer i.

    page_size, dtype: of every group that names none of its own.  num_pages: pages of `page_size` tokens, i.e. a
    group that keeps every key has room for num_pages * page_size tokens, whatever its own page size; a group
    with a window has at most that, and no more than its requests can hold at once (`window_pool_pages`).
    max_step_tokens: the most new tokens one step brings (default: max_model_len); it only bounds window pools."""
    _check_page_size(page_size)
    self.page_size = page_size
    self.num_pages = num_pages
    self.max_requests = max_requests
    self.max_model_len = max_model_len
    self.max_step_tokens = max_step_tokens if max_step_tokens is not None else max_model_len
    self.dtype = dtype
    self.device = torch.device(device)
    self.paged: List[PagedGroup] = []
    self.states: List[StateGroup] = []
    self._layer_map: List[Tuple[str, int, int]] = []
    for i, need in enumerate(layer_needs):
      if need is None:
        self._layer_map.append(("none", -1, -1))
      elif isinstance(need, PagedKV):
        for gi, g in enumerate(self.paged):
          if g.need == need:
            break
        else:
          gi = len(self.paged)
          P = need.page_size or page_size
          _check_page_size(P)
          pages = self.group_pages(need, page_size, num_pages, max_requests, self.max_step_tokens)
          self.paged.append(PagedGroup(need=need, layers=[], pool=PagePool(pages), page_size=P,
                                       dtype=need.dtype or dtype))
        self._layer_map.append(("paged", gi, len(self.paged[gi].layers)))
        self.paged[gi].layers.append(i)
      elif isinstance(need, FixedState):
        for si, s in enumerate(self.states):
          if s.need == need:
            break
        else:
          si = len(self.states)
          self.states.append(StateGroup(need=need, layers=[]))
        self._layer_map.append(("state", si, len(self.states[si].layers)))
        self.states[si].layers.append(i)
      else:
        raise TypeError(f"layer {i}: unknown cache need {need!r}")
    # the finest page of any group: block tables are at most this many entries wide
    self.min_page_size = min((g.page_size for g in self.paged), default=page_size)
    self.max_pages_per_request = -(-max_model_len // self.min_page_size)
    self._free_slots: List[int] = list(range(max_requests - 1, -1, -1))
    # The state row that no request ever gets: padding entries of captured steps read and write it, as they
    # read and write page 0 of the paged groups.
    self.scratch_slot = max_requests
    self._slot: Dict[Hashable, int] = {}
    self._length: Dict[Hashable, int] = {}
    if allocate:
      self._allocate()

  # ------------------------------------------------------------------ sizes
  @staticmethod
  def window_pool_pages(window: int, page_size: int, max_requests: int, max_step_tokens: int) -> int:
    """Pages that `max_requests` requests of a group with a window can hold at once.  Between steps a request
    keeps the pages that its next token can still see, at most ceil(window / P) + 1; inside a step it also holds
    the pages of the step's new tokens, ceil(n / P) + 1 more for n of them, and a step brings at most
    `max_step_tokens` in all."""
    per_request = -(-window // page_size) + 3
    return max_requests * per_request + -(-max_step_tokens // page_size)

  @classmethod
  def group_pages(cls, need: PagedKV, page_size: int, num_pages: int, max_requests: int, max_step_tokens: int) -> int:
    """Pages (of its own size) in the pool of the group with this need."""
    P = need.page_size or page_size
    pages = -(-num_pages * page_size // P)
    if need.window is not None:
      pages = min(pages, cls.window_pool_pages(need.window, P, max_requests, max_step_tokens))
    return max(1, pages)

  @classmethod
  def storage_bytes(cls, layer_needs: Sequence[object], page_size: int, num_pages: int, max_requests: int,
                    max_step_tokens: int, dtype: torch.dtype) -> int:
    """Device bytes of the page pools for `num_pages` (scratch pages included)."""
    total = 0
    for n in layer_needs:
      if isinstance(n, PagedKV):
        P = n.page_size or page_size
        esize = torch.empty((), dtype=n.dtype or dtype).element_size()
        pages = cls.group_pages(n, page_size, num_pages, max_requests, max_step_tokens) + 1
        total += 2 * n.num_kv_heads * n.head_dim * P * esize * pages
    return total

  @staticmethod
  def bytes_per_page(layer_needs: Sequence[object], page_size: int, dtype: torch.dtype) -> int:
    """Device bytes that room for `page_size` more tokens costs in every layer (window pools, which are bounded,
    counted as if they grew too)."""
    return sum(2 * n.num_kv_heads * n.head_dim * page_size * torch.empty((), dtype=n.dtype or dtype).element_size()
               for n in layer_needs if isinstance(n, PagedKV))

  def token_bytes(self) -> int:
    """Bytes of keys and values that one cached token holds in all layers (window groups counted like the others)."""
    return sum(len(g.layers) * 2 * g.need.num_kv_heads * g.need.head_dim * torch.empty((), dtype=g.dtype).element_size()
               for g in self.paged)

  def _allocate(self) -> None:
    for g in self.paged:
      n, h, d, P = len(g.layers), g.need.num_kv_heads, g.need.head_dim, g.page_size
      # keys [.., page_size, d]; values transposed [.., d, page_size]: the MFMA kernels read runs of keys per dim
      g.k = torch.zeros((n, g.pool.num_pages + 1, h, P, d), dtype=g.dtype, device=self.device)
      g.v = torch.zeros((n, g.pool.num_pages + 1, h, d, P), dtype=g.dtype, device=self.device)
    for s in self.states:
      shape = (len(s.layers), self.max_requests + 1) + tuple(s.need.shape)
      s.state = torch.zeros(shape, dtype=s.need.dtype or self.dtype, device=self.device)

  def layer_cache(self, layer: int) -> LayerCache:
    kind, gi, li = self._layer_map[layer]
    if kind == "paged":
      g = self.paged[gi]
      return LayerCache(kind="paged", group=gi, k=None if g.k is None else g.k[li], v=None if g.v is None else g.v[li],
                        page_size=g.page_size, window=g.need.window)
    if kind == "state":
      s = self.states[gi]
      return LayerCache(kind="state", group=gi, state=None if s.state is None else s.state[li])
    return LayerCache(kind="none")

  # ------------------------------------------------------------------ requests
  def has(self, req) -> bool:
    return req in self._slot

  def num_free_slots(self) -> int:
    return len(self._free_slots)

  def num_free_pages(self) -> int:
    """Free pages of the tightest group (in pages of that group's own size)."""
    return min((g.pool.num_free for g in self.paged), default=self.num_pages)

  def all_pages_free(self) -> bool:
    return all(g.pool.num_free == g.pool.num_pages for g in self.paged)

  def length(self, req) -> int:
    return self._length[req]

  def slot(self, req) -> int:
    return self._slot[req]

  def admit(self, req) -> int:
    """A slot for a new request; its fixed-size state starts at zero."""
    if req in self._slot:
      raise CacheError(f"request {req!r} is admitted already")
    if not self._free_slots:
      raise OutOfSlots(f"all {self.max_requests} request slots are taken")
    slot = self._free_slots.pop()
    self._slot[req] = slot
    self._length[req] = 0
    for g in self.paged:
      g.tables[req] = []
    for s in self.states:
      if s.state is not None:
        s.state[:, slot].zero_()
    return slot

  def _first_needed_page(self, g: PagedGroup, next_pos: int) -> int:
    """Index of the first page that the token at `next_pos` can still see."""
    if g.need.window is None:
      return 0
    lo = max(0, next_pos - g.need.window + 1)
    return lo // g.page_size

  def held_pages(self, req, group: int = 0) -> int:
    """Page indices `req` has been given so far in a group (0 for a request that is not admitted)."""
    if group >= len(self.paged) or req not in self.paged[group].tables:
      return 0
    return len(self.paged[group].tables[req])

  # ---- room: what the groups can still hand out.  A scheduler takes a copy (`room`), books its plan against it
  # (`take`) and so never plans a step that `grow` would refuse; groups differ in page size, pool size and in when
  # pages come back, so the books are kept per group.
  def room(self) -> List[int]:
    """Free pages per paged group (a copy to plan against)."""
    return [g.pool.num_free for g in self.paged]

  def _needs(self, req, new_len: int) -> List[int]:
    return [max(0, -(-new_len // g.page_size) - len(g.tables.get(req, ()))) for g in self.paged]

  def fits(self, room: Sequence[int], req, new_len: int, spare: int = 0) -> bool:
    """Whether `req` (admitted or not) can grow to `new_len` tokens out of `room`, leaving `spare` pages in every group."""
    return all(n + spare <= r for n, r in zip(self._needs(req, new_len), room))

  def take(self, room: List[int], req, new_len: int) -> bool:
    """Books growing `req` to `new_len` tokens against `room` (in place); False, and nothing booked, if it does not fit."""
    needs = self._needs(req, new_len)
    if any(n > r for n, r in zip(needs, room)):
      return False
    for i, n in enumerate(needs):
      room[i] -= n
    return True

  def tokens_that_fit(self, room: Sequence[int], req) -> int:
    """The longest `req` can become out of `room`."""
    if not self.paged:
      return self.max_model_len
    return min((len(g.tables.get(req, ())) + r) * g.page_size for g, r in zip(self.paged, room))

  def never_fits(self, num_tokens: int) -> Optional[str]:
    """Why a request of `num_tokens` tokens could not be held even with every page free, or None if it could."""
    for gi, g in enumerate(self.paged):
      if g.need.window is None:
        need = -(-num_tokens // g.page_size)
      else:
        need = min(-(-num_tokens // g.page_size), -(-g.need.window // g.page_size) + 2)
      if need > g.pool.num_pages:
        return (f"{num_tokens} tokens need {need} pages of {g.page_size} tokens in cache group {gi}, "
                f"which has {g.pool.num_pages}")
    return None

  def pages_needed(self, req, new_len: int) -> int:
    """The most pages any group must still hand out so that `req` can hold new_len tokens."""
    return max(self._needs(req, new_len), default=0)

  def can_grow(self, req, new_len: int) -> bool:
    return self.fits(self.room(), req, new_len)

  def grow(self, req, new_len: int) -> None:
    """Make room for tokens up to position new_len - 1 in every group (all or nothing)."""
    if new_len > self.max_model_len:
      raise CacheError(f"request {req!r}: {new_len} tokens exceed max_model_len={self.max_model_len}")
    if new_len < self._length[req]:
      raise CacheError(f"request {req!r} cannot shrink from {self._length[req]} to {new_len}")
    needs = self._needs(req, new_len)
    for gi, (g, n) in enumerate(zip(self.paged, needs)):
      if n > g.pool.num_free:
        raise OutOfPages(f"request {req!r} needs {n} more pages in cache group {gi}, {g.pool.num_free} are free")
    for g, n in zip(self.paged, needs):
      g.tables[req].extend(g.pool.alloc(n))

  def commit(self, req, new_len: int) -> None:
    """The step that wrote tokens up to new_len - 1 is done: record the length and give back
    the pages of window groups that no later token can see."""
    for g in self.paged:
      if new_len > len(g.tables[req]) * g.page_size:
        raise CacheError(f"request {req!r}: commit of {new_len} tokens beyond its pages")
    self._length[req] = new_len
    for g in self.paged:
      if g.need.window is None:
        continue
      table = g.tables[req]
      first = min(self._first_needed_page(g, new_len), len(table))
      gone = [p for p in table[:first] if p != 0]
      if gone:
        g.pool.free(gone)
        for i in range(first):
          table[i] = 0

  def release(self, req) -> None:
    """Everything the request holds comes back: its pages in every group and its slot."""
    if req not in self._slot:
      raise CacheError(f"request {req!r} is not admitted (released twice?)")
    for g in self.paged:
      g.pool.free([p for p in g.tables.pop(req) if p != 0])
    self._free_slots.append(self._slot.pop(req))
    del self._length[req]

  def table(self, group: int, req) -> List[int]:
    return self.paged[group].tables[req]

  def live_requests(self) -> List[Hashable]:
    return list(self._slot)

  # ------------------------------------------------------------------ invariants (tests, debug)
  def check(self) -> None:
    """No page lost, none held twice, none both free and held; slots likewise."""
    for gi, g in enumerate(self.paged):
      held = [p for t in g.tables.values() for p in t if p != 0]
      if len(held) != len(set(held)):
        raise CacheError(f"group {gi}: a page is in two block tables")
      if sorted(held) != g.pool.held():
        raise CacheError(f"group {gi}: tables hold {sorted(held)}, the pool says {g.pool.held()}")
      if len(held) + g.pool.num_free != g.pool.num_pages:
        raise CacheError(f"group {gi}: {len(held)} held + {g.pool.num_free} free != {g.pool.num_pages}")
      if len(set(g.pool._free)) != len(g.pool._free) or set(g.pool._free) & set(held):
        raise CacheError(f"group {gi}: free list is inconsistent")
    slots = list(self._slot.values())
    if len(slots) != len(set(slots)) or set(slots) & set(self._free_slots):
      raise CacheError("a request slot is held twice")
    if len(slots) + len(self._free_slots) != self.max_requests:
      raise CacheError("a request slot was lost")
