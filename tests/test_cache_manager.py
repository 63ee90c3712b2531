"""The cache manager on the host: no page lost, held twice or freed twice, under random orders of requests;
groups with a window give pages back as the window passes; state slots start at zero."""

import random

import pytest
import torch

from miniinfer_amd.cache import CacheError, CacheManager, OutOfPages, OutOfSlots, PagePool
from miniinfer_amd.parts import FixedState, PagedKV


def _mgr(needs=None, P=16, pages=8, slots=4, max_len=4096):
  needs = needs if needs is not None else [PagedKV(2, 8)] * 2
  return CacheManager(needs, page_size=P, num_pages=pages, max_requests=slots, max_model_len=max_len,
                      dtype=torch.float32, device="cpu")


def test_pool_never_hands_out_page_zero_and_catches_double_free():
  pool = PagePool(5)
  got = pool.alloc(5)
  assert sorted(got) == [1, 2, 3, 4, 5]
  with pytest.raises(OutOfPages):
    pool.alloc(1)
  pool.free([3])
  with pytest.raises(CacheError, match="twice"):
    pool.free([3])
  with pytest.raises(CacheError):
    pool.free([0])
  assert pool.alloc(1) == [3]        # freed last, handed out first: reuse shows early


def test_pages_open_exactly_at_page_edges():
  # the reference's rules (tests/unittests/test_kv_cache_manager.py:300-373): a partial page is filled before a new
  # one opens; decoding opens a page exactly when it crosses an edge
  m = _mgr(P=16, pages=8)
  m.admit("a")
  m.grow("a", 10); m.commit("a", 10)
  assert m.held_pages("a") == 1
  m.grow("a", 16); m.commit("a", 16)
  assert m.held_pages("a") == 1 and m.pages_needed("a", 16) == 0 and m.pages_needed("a", 17) == 1
  m.grow("a", 17); m.commit("a", 17)
  assert m.held_pages("a") == 2
  # numbers of the reference's backend test (test_flashinfer_backend.py:50-71): lengths 10 and 20 at P=16 -> 1 and 2 pages
  m.admit("b"); m.grow("b", 20)
  assert m.held_pages("b") == 2
  m.check()
  m.release("a"); m.release("b")
  assert m.num_free_pages() == 8 and m.num_free_slots() == 4
  with pytest.raises(CacheError, match="not admitted"):
    m.release("a")


def test_grow_is_all_or_nothing_and_errors_are_typed():
  m = _mgr(P=8, pages=4, slots=2)
  m.admit(1); m.admit(2)
  with pytest.raises(OutOfSlots):
    m.admit(3)
  m.grow(1, 24)
  with pytest.raises(OutOfPages):
    m.grow(2, 17)
  assert m.held_pages(2) == 0 and m.num_free_pages() == 1


def test_max_model_len_is_enforced():
  m = _mgr(max_len=32)
  m.admit("x")
  with pytest.raises(CacheError, match="max_model_len"):
    m.grow("x", 33)


def test_groups_have_pages_of_their_own_and_windows_give_pages_back():
  full, win = PagedKV(2, 8), PagedKV(2, 8, window=20)
  m = _mgr(needs=[full, win, full, win, FixedState((4,), torch.float32)], P=8, pages=10)
  assert len(m.paged) == 2 and m.paged[0].layers == [0, 2] and m.paged[1].layers == [1, 3]
  assert m.paged[0].k.shape == (2, 11, 2, 8, 8) and m.paged[0].v.shape == (2, 11, 2, 8, 8)
  assert m.layer_cache(3).group == 1 and m.layer_cache(3).window == 20 and m.layer_cache(4).kind == "state"
  m.admit("r")
  m.grow("r", 40); m.commit("r", 40)
  # next token is at 40 and sees keys 21..40: pages 0 and 1 (keys 0..15) of the window group are gone
  assert len(m.table(0, "r")) == 5 and all(p > 0 for p in m.table(0, "r"))
  assert m.table(1, "r")[:2] == [0, 0] and all(p > 0 for p in m.table(1, "r")[2:])
  assert m.paged[0].pool.num_free == 5 and m.paged[1].pool.num_free == 7
  m.check()
  for n in range(41, 80):
    m.grow("r", n); m.commit("r", n); m.check()
  assert sum(1 for p in m.table(1, "r") if p) <= 4      # a window of 20 keys touches at most 4 pages of 8
  m.release("r")
  assert m.paged[0].pool.num_free == 10 and m.paged[1].pool.num_free == 10


def test_state_slots_are_zero_on_admission():
  m = _mgr(needs=[FixedState((3,), torch.float32), PagedKV(1, 8)], slots=2)
  s = m.admit("a")
  m.states[0].state[0, s] = 7.0
  m.release("a")
  s2 = m.admit("b")
  assert s2 == s and float(m.states[0].state[0, s2].abs().sum()) == 0.0


@pytest.mark.parametrize("seed", range(5))
def test_random_orders_keep_the_books(seed):
  rnd = random.Random(seed)
  m = _mgr(needs=[PagedKV(1, 8), PagedKV(1, 8, window=24)], P=8, pages=24, slots=5, max_len=400)
  live = {}
  next_id = 0
  for _ in range(600):
    op = rnd.random()
    if op < 0.25 and m.num_free_slots() > 0:
      m.admit(next_id); live[next_id] = 0; next_id += 1
    elif op < 0.85 and live:
      r = rnd.choice(list(live))
      new_len = min(400, live[r] + rnd.choice([1, 1, 1, 2, 7, 30]))
      if m.can_grow(r, new_len):
        m.grow(r, new_len); m.commit(r, new_len); live[r] = new_len
      else:
        with pytest.raises(OutOfPages):
          m.grow(r, new_len)
    elif live:
      r = rnd.choice(list(live))
      m.release(r); del live[r]
    m.check()
    for r, n in live.items():
      assert m.length(r) == n and m.held_pages(r) == -(-n // 8)
  for r in list(live):
    m.release(r)
  m.check()
  assert m.num_free_pages() == 24 and m.num_free_slots() == 5


def test_groups_may_have_page_sizes_dtypes_and_pool_sizes_of_their_own():
  """A group names its own page size and dtype; a group with a window gets only the pages its requests can hold at
  once; a group that keeps every key has room for num_pages * page_size tokens whatever its own page size."""
  full, coarse = PagedKV(2, 8), PagedKV(1, 16, page_size=32, dtype=torch.float32)
  win = PagedKV(2, 8, window=20, page_size=4)
  m = CacheManager([full, coarse, win, full], page_size=8, num_pages=64, max_requests=3, max_model_len=512,
                   dtype=torch.bfloat16, device="cpu", max_step_tokens=40)
  assert [g.page_size for g in m.paged] == [8, 32, 4] and [g.layers for g in m.paged] == [[0, 3], [1], [2]]
  assert m.paged[0].pool.num_pages == 64 and m.paged[1].pool.num_pages == 16      # 512 tokens each
  # window 20 in pages of 4: (5 + 3) pages a request, 10 pages for a step's 40 new tokens
  assert m.paged[2].pool.num_pages == CacheManager.window_pool_pages(20, 4, 3, 40) == 3 * 8 + 10
  assert m.paged[0].k.shape == (2, 65, 2, 8, 8) and m.paged[0].k.dtype == torch.bfloat16
  assert m.paged[1].v.shape == (1, 17, 1, 16, 32) and m.paged[1].k.dtype == torch.float32
  assert m.paged[2].k.shape == (1, 35, 2, 4, 8)
  assert m.layer_cache(1).page_size == 32 and m.layer_cache(2).page_size == 4 and m.layer_cache(0).page_size == 8
  assert m.min_page_size == 4 and m.max_pages_per_request == 128
  want = 2 * 2 * 2 * 8 * 8 * 2 * 65 + 2 * 1 * 16 * 32 * 4 * 17 + 2 * 2 * 8 * 4 * 2 * 35
  assert CacheManager.storage_bytes([full, coarse, win, full], 8, 64, 3, 40, torch.bfloat16) == want
  assert sum(t.numel() * t.element_size() for g in m.paged for t in (g.k, g.v)) == want
  m.admit("a")
  m.grow("a", 33); m.commit("a", 33)
  assert [len(m.table(g, "a")) for g in range(3)] == [5, 2, 9]
  # the next token, at 33, sees keys 14..33: the window group's pages 0..2 (keys 0..11) are gone
  assert m.table(2, "a")[:3] == [0, 0, 0] and all(p > 0 for p in m.table(2, "a")[3:])
  m.check()
  m.release("a")
  assert m.all_pages_free()


def test_room_is_booked_per_group():
  full, coarse = PagedKV(1, 8), PagedKV(1, 8, page_size=16)
  m = CacheManager([full, coarse], page_size=4, num_pages=16, max_requests=4, max_model_len=64, dtype=torch.float32,
                   device="cpu")
  assert m.room() == [16, 4]
  m.admit("a"); m.admit("b")
  m.grow("a", 17); m.commit("a", 17)                 # 5 fine pages, 2 coarse ones
  room = m.room()
  assert room == [11, 2]
  assert m.tokens_that_fit(room, "a") == min((5 + 11) * 4, (2 + 2) * 16) == 64
  assert m.tokens_that_fit(room, "b") == 32           # the coarse group is the tighter one for a new request
  assert m.fits(room, "b", 32) and not m.fits(room, "b", 33) and not m.fits(room, "b", 32, spare=1)
  assert m.take(room, "b", 20) and room == [6, 0]
  assert m.take(room, "a", 24) and room == [5, 0]     # one more fine page, no coarse one
  assert not m.take(room, "a", 33) and room == [5, 0]   # refused: nothing booked
  assert m.room() == [11, 2]                          # the manager's own books are untouched by a plan
  assert m.pages_needed("b", 20) == 5 and m.can_grow("b", 32) and not m.can_grow("b", 33)
  with pytest.raises(OutOfPages):
    m.grow("b", 33)
  assert m.held_pages("b") == 0                       # all or nothing
  assert m.never_fits(64) is None and "group 0" in m.never_fits(65)
  w = CacheManager([PagedKV(1, 8, window=8)], page_size=4, num_pages=6, max_requests=1, max_model_len=4096,
                   dtype=torch.float32, device="cpu")
  assert w.never_fits(4000) is None                   # a window needs the pages of its window only
  assert CacheManager([PagedKV(1, 8, window=64)], page_size=4, num_pages=6, max_requests=1, max_model_len=4096,
                      dtype=torch.float32, device="cpu").never_fits(4000) is not None


@pytest.mark.parametrize("seed", range(4))
def test_random_orders_keep_the_books_of_unlike_groups(seed):
  rnd = random.Random(100 + seed)
  needs = [PagedKV(1, 8), PagedKV(1, 8, page_size=16), PagedKV(1, 8, window=24, page_size=4), PagedKV(2, 8, window=9)]
  m = CacheManager(needs, page_size=8, num_pages=24, max_requests=5, max_model_len=400, dtype=torch.float32,
                   device="cpu", max_step_tokens=30)
  live = {}
  next_id = 0
  for _ in range(800):
    op = rnd.random()
    if op < 0.25 and m.num_free_slots() > 0:
      m.admit(next_id); live[next_id] = 0; next_id += 1
    elif op < 0.85 and live:
      # one step: several requests grow together, planned against one copy of the room, within the step's tokens
      room, plan, left = m.room(), [], 30
      for r in rnd.sample(list(live), k=min(len(live), rnd.choice([1, 2, 3]))):
        n = min(left, rnd.choice([1, 1, 1, 2, 7, 30]), 400 - live[r])
        if n > 0 and m.take(room, r, live[r] + n):
          plan.append((r, live[r] + n))
          left -= n
      for r, new_len in plan:
        m.grow(r, new_len)                              # never refused: the plan was booked
      for r, new_len in plan:
        m.commit(r, new_len); live[r] = new_len
    elif live:
      r = rnd.choice(list(live))
      m.release(r); del live[r]
    m.check()
    for r, n in live.items():
      assert m.length(r) == n and [m.held_pages(r, g) for g in range(4)] == [-(-n // 8), -(-n // 16), -(-n // 4), -(-n // 8)]
  for r in list(live):
    m.release(r)
  m.check()
  assert m.all_pages_free() and m.num_free_slots() == 5


def test_token_bytes_and_the_rule_that_keeps_weights_out_of_the_last_level_cache():
  """A cached token's bytes over all layers; weights are streamed past the cache while a step's keys and values
  (an upper bound) stay within twice its size, and never for a step without any."""
  import torch
  from miniinfer_amd.cache.manager import CacheManager
  from miniinfer_amd.kernels import ops
  from miniinfer_amd.parts import PagedKV
  needs = [PagedKV(8, 128)] * 28
  cm = CacheManager(needs, 16, 64, 4, 1024, torch.bfloat16, torch.device("cpu"), allocate=False)
  assert cm.token_bytes() == 28 * 2 * 8 * 128 * 2 == 114688
  mixed = CacheManager([PagedKV(2, 64), PagedKV(2, 64, window=32), PagedKV(4, 32, dtype=torch.float32)], 16, 64, 4,
                       1024, torch.bfloat16, torch.device("cpu"), allocate=False)
  assert mixed.token_bytes() == 2 * (2 * 2 * 64 * 2) + 2 * 4 * 32 * 4
  tb = cm.token_bytes()
  assert ops.weights_stream_past_cache(1 * 4096 * tb) and ops.weights_stream_past_cache(2 * 2048 * tb)
  assert not ops.weights_stream_past_cache(4 * 2048 * tb) and not ops.weights_stream_past_cache(0)
