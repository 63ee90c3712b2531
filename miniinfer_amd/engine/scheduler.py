"""The scheduler: admits requests, cuts prompts into portions under a token budget, decodes, finishes
and frees.  Host-only; it talks to the cache manager through a handful of calls, so tests drive it
with the real manager on the CPU.

Policy (Sarathi-style, like the reference with `enable_chunked_prefill`,
miniinfer/scheduler/scheduler.py:242-286,417-434): every step carries one token for each running
request that is decoding, and the rest of the token budget is filled with prompt portions, first of
requests already running, then of waiting requests in arrival order
(miniinfer/scheduler/prefill_adder.py:39-421 plays this role there, with page-rounded chunks; here a
portion is any length >= 1).

When pages run out (the reference retracts from the tail of the running list and drops the generated
tokens, scheduler.py:519-610): the most recently admitted running request is preempted: its pages
and slot are given back and it returns to the head of the waiting queue, keeping its generated tokens;
when it is admitted again it recomputes prompt + outputs as one prompt.  Admission of new requests
stops while running requests cannot grow.  A request that could never fit the pool alone is refused
when it is added.

Results come back in two halves, so that the engine can launch the next step before it has read the
tokens of the last one (the reference's overlap mode schedules step N+1 against placeholders for step N's
tokens too: miniinfer/engine/future_map.py:1-206, llm_engine.py:559-700): `advance` moves the lengths on
and appends a placeholder for each token to come (a negative id that names the row of the step's sampling
output), `resolve` writes the tokens in and finishes requests.  `update` is both at once.
"""

from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, Iterable, List, Optional, Sequence, Union

from ..sampling.params import SamplingParams


@dataclass
class Request:
  number: int                     # arrival order; also the handle in the cache manager
  request_id: str
  prompt: List[int]
  params: SamplingParams
  seed: int = 0
  outputs: List[int] = field(default_factory=list)
  num_computed: int = 0           # tokens whose keys and values are in the cache
  finish_reason: Optional[str] = None
  num_preemptions: int = 0
  pending: int = 0                # sampled tokens that are still placeholders
  _tokens: Optional[List[int]] = field(default=None, repr=False, compare=False)

  @property
  def tokens(self) -> List[int]:
    """prompt + outputs, kept as one list (it is sliced every step)."""
    if self._tokens is None or len(self._tokens) != len(self.prompt) + len(self.outputs):
      self._tokens = self.prompt + self.outputs
    return self._tokens

  def append_output(self, tok: int) -> None:
    toks = self.tokens
    self.outputs.append(tok)
    toks.append(tok)

  def set_output(self, index: int, tok: int) -> None:
    toks = self.tokens
    self.outputs[index] = tok
    toks[len(self.prompt) + index] = tok

  def truncate_outputs(self, count: int) -> None:
    del self.outputs[count:]
    self._tokens = None

  @property
  def num_tokens(self) -> int:
    return len(self.prompt) + len(self.outputs)

  @property
  def remaining(self) -> int:
    return self.num_tokens - self.num_computed

  @property
  def finished(self) -> bool:
    return self.finish_reason is not None


@dataclass
class ScheduledEntry:
  request: Request
  start: int                      # position of the first token of this portion
  num_tokens: int
  samples: bool                   # the portion ends the known tokens: its last logits pick the next token
  output_index: int = -1          # where in the request's outputs its sampled token goes (set by `advance`)


@dataclass
class ScheduledStep:
  entries: List[ScheduledEntry]
  preempted: List[Request] = field(default_factory=list)

  @property
  def num_tokens(self) -> int:
    return sum(e.num_tokens for e in self.entries)

  @property
  def num_decode_tokens(self) -> int:
    return sum(1 for e in self.entries if e.num_tokens == 1 and e.start > 0)

  @property
  def num_prefill_tokens(self) -> int:
    return self.num_tokens - self.num_decode_tokens


class Scheduler:
  def __init__(self, cache, max_num_seqs: int, max_num_batched_tokens: int, max_model_len: int,
               enable_chunked_prefill: bool = True, eos_token_id: Union[int, Iterable[int], None] = None):
    self.cache = cache
    self.max_num_seqs = max_num_seqs
    self.max_num_batched_tokens = max_num_batched_tokens
    self.max_model_len = max_model_len
    self.enable_chunked_prefill = enable_chunked_prefill
    self.eos_token_id = eos_token_id
    self.waiting: Deque[Request] = deque()
    self.running: List[Request] = []      # in order of admission
    self.finished: Deque[Request] = deque(maxlen=1024)   # the last requests that finished (a log, not a queue)
    self.num_finished = 0
    self.num_preemptions = 0
    self.num_unresolved = 0               # sampled tokens launched and not yet written in
    self._draining: List[Request] = []    # finished, pages still held until their last token is written in
    self._retired_unadmitted: List[Request] = []

  @property
  def eos_token_id(self):
    """One id, several, or None; any of them ends a request that does not ignore it (a generation_config.json
    may list more than one)."""
    return self._eos

  @eos_token_id.setter
  def eos_token_id(self, eos) -> None:
    self._eos = eos
    if eos is None:
      self.eos_token_ids = frozenset()
    elif isinstance(eos, int):
      self.eos_token_ids = frozenset([eos])
    else:
      self.eos_token_ids = frozenset(int(t) for t in eos)

  # ------------------------------------------------------------------ requests in
  def add(self, req: Request) -> None:
    n = len(req.prompt)
    if n == 0:
      raise ValueError("a request needs at least one prompt token")
    if n + req.params.max_tokens > self.max_model_len:
      # the reference never checks this and would index past its table (kvcache/memory_pool.py:476-478)
      raise ValueError(f"prompt of {n} tokens plus max_tokens={req.params.max_tokens} exceeds "
                       f"max_model_len={self.max_model_len}")
    why = self.cache.never_fits(n + req.params.max_tokens)
    if why is not None:
      raise ValueError(f"request of up to {n + req.params.max_tokens} tokens can never fit the cache: {why}")
    if not self.enable_chunked_prefill and n + req.params.max_tokens > self.max_num_batched_tokens:
      raise ValueError(f"without chunked prefill a request of up to {n + req.params.max_tokens} tokens must fit the "
                       f"step budget of {self.max_num_batched_tokens}")
    self.waiting.append(req)

  def has_unfinished(self) -> bool:
    return bool(self.waiting or self.running or self.num_unresolved)

  # ------------------------------------------------------------------ one step's plan
  def _preempt(self, req: Request) -> None:
    self.cache.release(req.number)
    self.running.remove(req)
    req.num_computed = 0
    req.num_preemptions += 1
    self.num_preemptions += 1
    self.waiting.appendleft(req)

  def schedule(self) -> Optional[ScheduledStep]:
    if not (self.waiting or self.running):
      return None
    budget = self.max_num_batched_tokens
    cache = self.cache
    room = cache.room()            # free pages per cache group; the plan is booked against this copy
    entries: List[ScheduledEntry] = []
    preempted: List[Request] = []

    def all_fit(reqs) -> bool:
      trial = list(room)
      return all(cache.take(trial, r.number, r.num_tokens) for r in reqs)

    # 1. decodes: one token for every running request whose known tokens are all but one in the cache
    decoding = [r for r in self.running if r.remaining == 1 and r.num_computed > 0]
    while decoding and not all_fit(decoding):
      if self._draining:
        # Finished requests hold pages until their last token is written in, one call from now.  The decodes
        # that need a new page sit this step out (the most recently admitted first) rather than cost a running
        # request its whole cache.
        for r in reversed(list(decoding)):
          if all_fit(decoding):
            break
          if cache.pages_needed(r.number, r.num_tokens) > 0:
            decoding.remove(r)
        break
      victim = self.running[-1]
      self._preempt(victim)
      preempted.append(victim)
      decoding = [r for r in decoding if r is not victim]
      room = cache.room()
    for r in decoding[:budget]:
      if not cache.take(room, r.number, r.num_tokens):
        continue
      entries.append(ScheduledEntry(r, r.num_computed, 1, True))
      budget -= 1
    scheduled = {id(e.request) for e in entries}

    # 2. prompt portions of running requests (a preempted-and-readmitted request included)
    for r in self.running:
      if budget <= 0:
        break
      if id(r) in scheduled or r.remaining <= 0 or (r.remaining == 1 and r.num_computed > 0):
        continue
      n = self._portion(r, budget, room)
      if n <= 0 or not cache.take(room, r.number, r.num_computed + n):
        continue
      entries.append(ScheduledEntry(r, r.num_computed, n, r.num_computed + n == r.num_tokens))
      budget -= n

    # 3. admissions, in arrival order; none while a request had to be preempted in this step
    while self.waiting and budget > 0 and not preempted and len(self.running) < self.max_num_seqs \
        and cache.num_free_slots() > 0:
      r = self.waiting[0]
      # watermark: its whole known sequence must fit, with one spare page for each request already running,
      # so that an admission does not at once force a preemption
      if not cache.fits(room, r.number, r.num_tokens, spare=len(self.running)):
        break
      n = self._portion(r, budget, room)
      if n <= 0 or not cache.take(room, r.number, n):
        break
      self.waiting.popleft()
      cache.admit(r.number)
      self.running.append(r)
      entries.append(ScheduledEntry(r, 0, n, n == r.num_tokens))
      budget -= n

    if not entries:
      if self._draining:
        return None       # finished requests give their pages back as soon as their last token is written in
      if self.running or self.waiting:
        # nothing fits: every running request is stuck on pages and none can be preempted further
        if len(self.running) > 1:
          victim = self.running[-1]
          self._preempt(victim)
          return self.schedule()
        raise RuntimeError("the scheduler cannot make progress: no request fits the cache")
      return None
    return ScheduledStep(entries, preempted)

  def _portion(self, r: Request, budget: int, room) -> int:
    """How many of r's remaining tokens run in this step: bounded by the budget and by the tokens that fit
    the pages r holds plus what `room` still has.  Without chunked prefill it is all of them or none."""
    capacity = self.cache.tokens_that_fit(room, r.number)
    n = min(r.remaining, budget, capacity - r.num_computed)
    if not self.enable_chunked_prefill and n < r.remaining:
      return 0
    return max(n, 0)

  # ------------------------------------------------------------------ results in
  def advance(self, step: ScheduledStep) -> None:
    """The step has been launched: its tokens count as computed, and every entry that samples gets a placeholder
    -(row + 1) for its token, `row` being its place among the sampling entries of the step.  A request that
    reaches max_tokens or the model's length with this token leaves the running list now; its pages stay until
    the token is written in."""
    row = 0
    for e in step.entries:
      r = e.request
      r.num_computed += e.num_tokens
      if not e.samples:
        continue
      e.output_index = len(r.outputs)
      r.append_output(-(row + 1))
      r.pending += 1
      self.num_unresolved += 1
      row += 1
      if r.finish_reason is None:
        if len(r.outputs) >= r.params.max_tokens:
          r.finish_reason = "max_tokens"
        elif r.num_tokens >= self.max_model_len:
          r.finish_reason = "length"
        if r.finished and r in self.running:
          self.running.remove(r)
          self._draining.append(r)

  def resolve(self, step: ScheduledStep, sampled: Dict[int, int]) -> List[Request]:
    """`sampled[request.number]` is the token of every entry of `step` that samples.  Writes the tokens in place
    of their placeholders, ends requests at their end-of-sequence token (placeholders launched after it are
    dropped), and returns the requests that are finished and have no token outstanding; their pages and slots
    are given back here."""
    done = []
    for e in step.entries:
      if not e.samples:
        continue
      r = e.request
      r.pending -= 1
      self.num_unresolved -= 1
      if e.output_index < len(r.outputs):          # else: dropped after an earlier end-of-sequence token
        tok = int(sampled[r.number])
        r.set_output(e.output_index, tok)
        is_eos = not r.params.ignore_eos and tok in self.eos_token_ids
        if is_eos or tok in r.params.stop_token_ids:
          r.finish_reason = "eos" if is_eos else "stop"
          r.truncate_outputs(e.output_index + 1)
          if r in self.running:
            self.running.remove(r)
            self._draining.append(r)
          elif r in self.waiting:                   # preempted meanwhile: it holds nothing
            self.waiting.remove(r)
            self._retired_unadmitted.append(r)
      if r.finished and r.pending == 0:
        if r in self._draining:
          self._draining.remove(r)
          self.cache.release(r.number)
        elif r in self._retired_unadmitted:
          self._retired_unadmitted.remove(r)
        else:
          continue
        self.finished.append(r)
        self.num_finished += 1
        done.append(r)
    return done

  def update(self, step: ScheduledStep, sampled: Dict[int, int]) -> List[Request]:
    """After the step ran: `sampled[request.number]` is the next token of every entry that samples.
    Returns the requests that finished; their pages and slots are given back here."""
    self.advance(step)
    return self.resolve(step, sampled)
