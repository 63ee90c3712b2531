"""The scheduler's decisions on the host, with the real cache manager and a fake model whose next token is a
function of the request's whole history (so recomputation after a preemption must give the same tokens)."""

import random

import pytest
import torch

from miniinfer_amd.cache import CacheManager
from miniinfer_amd.engine.scheduler import Request, Scheduler
from miniinfer_amd.parts import PagedKV
from miniinfer_amd.sampling import SamplingParams

V = 1000


def fake_next(tokens):
  h = 1469598103934665603
  for t in tokens:
    h = ((h ^ t) * 1099511628211) & ((1 << 64) - 1)
  return h % V


def make(pages, P=8, max_seqs=4, budget=32, max_len=512, chunked=True, eos=None):
  cache = CacheManager([PagedKV(1, 8)], page_size=P, num_pages=pages, max_requests=max_seqs, max_model_len=max_len,
                       dtype=torch.float32, device="cpu")
  return cache, Scheduler(cache, max_num_seqs=max_seqs, max_num_batched_tokens=budget, max_model_len=max_len,
                          enable_chunked_prefill=chunked, eos_token_id=eos)


def run(cache, sched, reqs, max_steps=100000, on_step=None):
  """Drives the scheduler like the engine does; the 'model' checks that it is fed contiguous portions."""
  for r in reqs:
    sched.add(r)
  steps = 0
  while sched.has_unfinished():
    plan = sched.schedule()
    assert plan is not None and plan.entries
    assert plan.num_tokens <= sched.max_num_batched_tokens
    assert len({id(e.request) for e in plan.entries}) == len(plan.entries)
    sampled = {}
    for e in plan.entries:
      r = e.request
      assert e.start == r.num_computed == cache.length(r.number), "a portion must continue where the cache ends"
      assert 1 <= e.num_tokens <= r.remaining
      cache.grow(r.number, e.start + e.num_tokens)       # what runner.step does
      cache.commit(r.number, e.start + e.num_tokens)
      assert e.samples == (e.start + e.num_tokens == r.num_tokens)
      if e.samples:
        sampled[r.number] = fake_next(r.tokens)
    if on_step:
      on_step(plan)
    sched.update(plan, sampled)
    cache.check()
    steps += 1
    assert steps < max_steps
  return steps


def expected(prompt, n):
  toks = list(prompt)
  for _ in range(n):
    toks.append(fake_next(toks))
  return toks[len(prompt):]


def _req(i, n_prompt, max_tokens, seed=0, **kw):
  rnd = random.Random(seed * 1000 + i)
  return Request(number=i, request_id=f"r{i}", prompt=[rnd.randrange(V) for _ in range(n_prompt)],
                 params=SamplingParams(temperature=0.0, max_tokens=max_tokens, ignore_eos=True, **kw))


def test_prompts_are_cut_under_the_budget_and_decodes_ride_along():
  cache, sched = make(pages=100, budget=32)
  reqs = [_req(0, 70, 5), _req(1, 9, 8), _req(2, 40, 3)]
  seen = []
  run(cache, sched, reqs, on_step=lambda p: seen.append([(e.request.number, e.start, e.num_tokens) for e in p.entries]))
  assert seen[0] == [(0, 0, 32)]                       # first portion takes the whole budget
  assert seen[1] == [(0, 32, 32)]
  assert seen[2] == [(0, 64, 6), (1, 0, 9), (2, 0, 17)]  # the rest of r0, all of r1, the start of r2
  assert seen[3][:2] == [(0, 70, 1), (1, 9, 1)]          # decodes first, then r2's next portion
  assert seen[3][2] == (2, 17, 23)
  for r in reqs:
    assert r.outputs == expected(r.prompt, r.params.max_tokens) and r.finish_reason == "max_tokens"
  assert cache.num_free_pages() == 100 and cache.num_free_slots() == 4


def test_without_chunked_prefill_prompts_run_whole():
  cache, sched = make(pages=100, budget=64, chunked=False)
  reqs = [_req(0, 40, 4), _req(1, 30, 4), _req(2, 20, 4)]
  seen = []
  run(cache, sched, reqs, on_step=lambda p: seen.append([(e.request.number, e.num_tokens) for e in p.entries]))
  assert seen[0] == [(0, 40), (2, 20)] or seen[0] == [(0, 40)]   # r1 does not fit beside r0; nothing is cut
  assert all(n in (1, 40, 30, 20) for step in seen for _, n in step)
  with pytest.raises(ValueError, match="chunked"):
    sched.add(_req(9, 100, 4))


def test_batch_size_cap_and_fcfs():
  cache, sched = make(pages=200, max_seqs=2, budget=64)
  reqs = [_req(i, 10, 6) for i in range(5)]
  live = []
  run(cache, sched, reqs, on_step=lambda p: live.append(len(sched.running)))
  assert max(live) <= 2
  order = [r.number for r in sched.finished]
  assert order == sorted(order)


def test_pages_run_out_newest_is_preempted_and_recomputes():
  # 4 requests that each grow to 30 + 50 = 80 tokens (10 pages) in a pool of 22 pages
  cache, sched = make(pages=22, P=8, max_seqs=4, budget=48)
  reqs = [_req(i, 30, 50) for i in range(4)]
  preempted = []
  run(cache, sched, reqs, on_step=lambda p: preempted.extend(r.number for r in p.preempted))
  assert sched.num_preemptions > 0 and preempted
  for r in reqs:
    assert len(r.outputs) == 50 and r.outputs == expected(r.prompt, 50)     # exactly max_tokens, same tokens
  assert reqs[0].num_preemptions == 0                  # the oldest running request is never the victim
  assert cache.num_free_pages() == 22


@pytest.mark.parametrize("seed", range(4))
def test_starvation_level_pools_still_finish_everything(seed):
  rnd = random.Random(seed)
  P = 8
  reqs = [_req(i, rnd.randint(1, 60), rnd.randint(1, 40), seed=seed) for i in range(12)]
  biggest = max(-(-(len(r.prompt) + r.params.max_tokens) // P) for r in reqs)
  cache, sched = make(pages=biggest + rnd.randint(0, 3), P=P, max_seqs=3, budget=rnd.choice([8, 16, 64]))
  run(cache, sched, reqs)
  for r in reqs:
    assert r.outputs == expected(r.prompt, r.params.max_tokens)
  assert cache.num_free_pages() == cache.num_pages and cache.num_free_slots() == 3


def test_requests_that_can_never_fit_are_refused_when_added():
  cache, sched = make(pages=4, P=8, max_len=64)
  with pytest.raises(ValueError, match="never fit"):
    sched.add(_req(0, 30, 10))
  with pytest.raises(ValueError, match="max_model_len"):
    sched.add(_req(1, 60, 10))
  with pytest.raises(ValueError, match="at least one"):
    sched.add(Request(number=2, request_id="e", prompt=[], params=SamplingParams()))


def test_eos_and_length_finish():
  cache, sched = make(pages=50, eos=None)
  r = _req(0, 5, 20)
  want = expected(r.prompt, 20)
  cache2, sched2 = make(pages=50, eos=want[3])
  r2 = Request(number=0, request_id="x", prompt=list(r.prompt), params=SamplingParams(temperature=0.0, max_tokens=20))
  run(cache2, sched2, [r2])
  assert r2.outputs == want[:want.index(want[3]) + 1] and r2.finish_reason == "eos"
  r3 = Request(number=1, request_id="y", prompt=list(r.prompt),
               params=SamplingParams(temperature=0.0, max_tokens=20, ignore_eos=True))
  run(cache2, sched2, [r3])
  assert r3.outputs == want and r3.finish_reason == "max_tokens"


# ---------------------------------------------------------------------------- results that arrive one step late

def run_pipelined(cache, sched, reqs, max_steps=100000):
  """Drives the scheduler like the engine does when it launches a step before it has read the tokens of the
  step before: schedule, 'launch' (advance), then resolve the previous step.  The fake model looks a placeholder
  token -(row + 1) up in the previous step's sampling output, as the embedding kernel does."""
  for r in reqs:
    sched.add(r)
  pending = None          # (plan, tokens by row) of the launched step
  future = []             # tokens by row of the last launched step
  steps = 0
  while sched.has_unfinished():
    plan = sched.schedule()
    launched = None
    if plan is not None:
      rows = []
      for e in plan.entries:
        r = e.request
        assert e.start == r.num_computed == cache.length(r.number)
        cache.grow(r.number, e.start + e.num_tokens)
        cache.commit(r.number, e.start + e.num_tokens)
        if e.samples:
          toks = [t if t >= 0 else future[-(t + 1)] for t in r.tokens]
          assert all(t >= 0 for t in toks), "a placeholder may only name a row of the step before"
          rows.append((r.number, fake_next(toks)))
      sched.advance(plan)
      launched = (plan, rows)
    if pending is not None:
      sched.resolve(pending[0], dict(pending[1]))
    cache.check()
    if launched is not None:
      future = [t for _, t in launched[1]]
    pending = launched
    steps += 1
    assert steps < max_steps
  assert pending is None
  return steps


def test_placeholders_stand_for_tokens_until_they_are_resolved():
  cache, sched = make(pages=100, budget=32)
  r = _req(0, 5, 4)
  sched.add(r)
  plan = sched.schedule()
  cache.grow(0, 5)
  cache.commit(0, 5)
  sched.advance(plan)
  assert r.outputs == [-1] and r.pending == 1 and r.num_computed == 5 and sched.has_unfinished()
  nxt = sched.schedule()                                   # the next step is planned against the placeholder
  assert [(e.start, e.num_tokens, e.samples) for e in nxt.entries] == [(5, 1, True)]
  assert r.tokens[5:6] == [-1]
  assert sched.resolve(plan, {0: 77}) == []
  assert r.outputs == [77] and r.tokens[-1] == 77 and r.pending == 0


@pytest.mark.parametrize("seed", range(4))
def test_late_results_give_the_same_tokens_and_leave_no_page_behind(seed):
  rnd = random.Random(100 + seed)
  P = 8
  reqs = [_req(i, rnd.randint(1, 60), rnd.randint(1, 40), seed=seed) for i in range(10)]
  biggest = max(-(-(len(r.prompt) + r.params.max_tokens) // P) for r in reqs)
  cache, sched = make(pages=biggest + rnd.randint(0, 6), P=P, max_seqs=3, budget=rnd.choice([8, 16, 64]))
  run_pipelined(cache, sched, reqs)
  for r in reqs:
    assert r.outputs == expected(r.prompt, r.params.max_tokens) and r.pending == 0
  assert cache.num_free_pages() == cache.num_pages and cache.num_free_slots() == 3
  assert sorted(r.number for r in sched.finished) == list(range(10))


def test_an_end_of_sequence_token_found_late_drops_the_token_launched_after_it():
  prompt = [3, 1, 4, 1, 5]
  want = expected(prompt, 6)
  eos = want[2]
  stop = want.index(eos) + 1
  cache, sched = make(pages=100, eos=eos)
  r = Request(number=0, request_id="r0", prompt=list(prompt), params=SamplingParams(temperature=0.0, max_tokens=6))
  other = _req(1, 7, 9)
  run_pipelined(cache, sched, [r, other])
  assert r.outputs == want[:stop] and r.finish_reason == "eos" and r.pending == 0
  assert other.outputs == expected(other.prompt, 9)
  assert cache.num_free_pages() == 100 and cache.num_free_slots() == 4
  assert [q.number for q in sched.finished].count(0) == 1


def test_a_decode_short_of_a_page_waits_for_a_finished_request_instead_of_preempting():
  """Results arrive one step late.  Request a reaches max_tokens while its last token is still outstanding, so its
  pages come back one call later; request b needs a new page for its next decoded token and none is free.  b must
  sit the step out, not be preempted and recomputed."""
  P = 8
  cache, sched = make(pages=4, P=P, max_seqs=2, budget=64)
  a = _req(0, 8, 2)           # one page; its 2nd token (the 9th) opens a second one
  b = _req(1, 15, 4)          # two pages; its 2nd decoded token (the 17th) needs a third
  sched.add(a)
  sched.add(b)

  def launch():
    plan = sched.schedule()
    if plan is None:
      return None
    for e in plan.entries:
      cache.grow(e.request.number, e.start + e.num_tokens)
      cache.commit(e.request.number, e.start + e.num_tokens)
    sched.advance(plan)
    return plan

  def settle(plan):
    # by now every earlier placeholder of the request has been written in
    sched.resolve(plan, {e.request.number: fake_next(e.request.tokens[:e.start + e.num_tokens])
                         for e in plan.entries if e.samples})
    cache.check()

  p0 = launch()
  assert sorted((e.request.number, e.num_tokens) for e in p0.entries) == [(0, 8), (1, 15)]
  assert cache.num_free_pages() == 1
  p1 = launch()               # launched against placeholders: a's 9th token takes the last page, b's 16th fits
  assert cache.num_free_pages() == 0 and a.finish_reason == "max_tokens" and a not in sched.running
  settle(p0)
  p2 = launch()               # b's 17th token needs a page; the only pages to come are a's, one call from now
  assert p2 is None and sched.num_preemptions == 0 and b in sched.running and b.num_computed == 16
  settle(p1)                  # a's last token is in: its two pages are free
  assert cache.num_free_pages() == 2
  p3 = launch()
  assert [(e.request.number, e.start, e.num_tokens) for e in p3.entries] == [(1, 16, 1)]
  settle(p3)
  while sched.has_unfinished():
    settle(launch())
  assert sched.num_preemptions == 0 and b.num_preemptions == 0
  assert a.outputs == expected(a.prompt, 2) and b.outputs == expected(b.prompt, 4)
  assert cache.num_free_pages() == 4 and cache.num_free_slots() == 2


def test_stop_token_ids_end_a_request_and_several_eos_ids_are_honoured():
  prompt = [2, 7, 1, 8]
  want = expected(prompt, 8)
  cache, sched = make(pages=50, eos=[want[5], 999999])
  r = Request(number=0, request_id="r0", prompt=list(prompt),
              params=SamplingParams(temperature=0.0, max_tokens=8, stop_token_ids=[want[3]]))
  run(cache, sched, [r])
  assert r.outputs == want[:want.index(want[3]) + 1] and r.finish_reason == "stop"
  r = Request(number=1, request_id="r1", prompt=list(prompt), params=SamplingParams(temperature=0.0, max_tokens=8))
  run(cache, sched, [r])
  assert r.outputs == want[:want.index(want[5]) + 1] and r.finish_reason == "eos"
  # ignore_eos switches the end-of-sequence ids off, not the request's own stop ids
  r = Request(number=2, request_id="r2", prompt=list(prompt),
              params=SamplingParams(temperature=0.0, max_tokens=8, ignore_eos=True, stop_token_ids=[want[6]]))
  run(cache, sched, [r])
  assert r.outputs == want[:want.index(want[6]) + 1] and r.finish_reason == "stop"
  assert sched.num_finished == 3 and cache.num_free_pages() == 50


def test_the_log_of_finished_requests_is_bounded():
  cache, sched = make(pages=50)
  n = sched.finished.maxlen + 10
  for i in range(0, n, 4):
    run(cache, sched, [_req(j, 3, 1) for j in range(i, min(n, i + 4))])
  assert sched.num_finished == n and len(sched.finished) == sched.finished.maxlen
