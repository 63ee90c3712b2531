"""The Python entry point, in the manner of the reference's `LLMEngine`
(miniinfer/engine/llm_engine.py:87-141 constructor, :898-1015 generate, :465-557 step, :1309 add_request,
:1271 is_finished, :1301-1306 context manager; examples/minimal_engine.py:60-90).

    with LLMEngine(model="/path/to/folder", max_num_seqs=4, max_model_len=512) as engine:
      outs = engine.generate(prompts, SamplingParams(temperature=0.7, max_tokens=64))
      outs[0]["token_ids"], outs[0]["text"]

Prompts are lists of token ids (always) or strings (when the model folder holds a tokenizer.json).
One loop: schedule, step, sample, update; no processes, no server.  With `enable_overlap` (the default, as in the
reference: config/engine/config.py:8-77, llm_engine.py:559-700) a step is launched before the tokens of the step
before it have been read back: they stay on the device, the new step's embedding reads them there, and the host
catches up while the device works.  What `step()` returns then describes the step before the one it launched.
"""

from __future__ import annotations

import os
import sys
import time
import warnings
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Union

import torch

from ..cache.manager import CacheManager
from ..config import EngineConfig, load_model_config, model_spec_of
from ..kernels import ops
from ..kernels.tuning import tune_products
from ..sampling import Sampler, SamplingParams, request_seed
from ..weights import build_model, fill_random, load_weights
from .runner import ModelRunner, StepEntry
from .scheduler import Request, ScheduledStep, Scheduler

TORCH_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


@dataclass
class StepOutput:
  """What one engine step did (miniinfer/engine/llm_engine.py:62-75)."""
  finished: List[Request] = field(default_factory=list)
  num_prefill_tokens: int = 0
  num_decode_tokens: int = 0
  num_preempted: int = 0


@dataclass
class RequestOutput:
  """One new token of one request, as `stream_generate` yields it (miniinfer/engine/llm_engine.py:49-59)."""
  request_id: str
  delta_text: str
  full_text: str
  token_id: int
  output_token_ids: List[int]
  finished: bool
  finish_reason: Optional[str]


class LLMEngine:
  def __init__(self, model: str, model_config=None, random_weights_seed: Optional[int] = None, **kwargs):
    """model: a folder with config.json and *.safetensors.  With the option `load_format="random"` only its
    config.json is read and the weights are drawn on the device from the option `seed`.  `model_config` (a typed
    configuration) stands in for the folder's config.json; `random_weights_seed` is `load_format="random"` with a
    seed of its own for the weights."""
    kwargs.pop("use_multiprocess", None)   # the reference's examples pass it; there is one process here
    if random_weights_seed is not None:
      kwargs["load_format"] = "random"
    self.config = EngineConfig.from_kwargs(model, **kwargs)
    t_start = time.perf_counter()
    if not torch.cuda.is_available():
      raise RuntimeError("miniinfer_amd needs a GPU: torch.cuda.is_available() is False and there is no CPU path")
    cfg = self.config
    self.dtype = TORCH_DTYPES[cfg.dtype]
    self.device = torch.device(cfg.device)
    torch.cuda.set_device(self.device)
    self.model_config = model_config if model_config is not None else load_model_config(cfg.model_path)
    self.model = build_model(model_spec_of(self.model_config), self.dtype, self.device)
    if cfg.load_format == "random":
      fill_random(self.model, random_weights_seed if random_weights_seed is not None else cfg.seed)
    else:
      load_weights(self.model, cfg.model_path)
    spec = self.model.spec
    self.max_model_len = min(cfg.max_model_len or spec.max_positions, spec.max_positions)
    needs = self.model.cache_needs()
    self.num_pages = cfg.num_pages if cfg.num_pages is not None else self._pages_from_memory(needs)
    self.cache = CacheManager(needs, page_size=cfg.page_size, num_pages=self.num_pages, max_requests=cfg.max_num_seqs,
                              max_model_len=self.max_model_len, dtype=self.dtype, device=self.device,
                              max_step_tokens=cfg.max_num_batched_tokens)
    # Which kernel runs a product of few rows: this engine's own table (another engine in the process has its own).
    # The products are timed after the cache pools exist: where the pools come to lie in memory must not depend on
    # what the timing allocated and gave back (decode attention over 48 requests' pages ran 11% slower in pools
    # allocated after it).
    self.choices = ops.ProductChoices(rule_only=not cfg.timed_kernel_choices)
    if cfg.tune_products and cfg.timed_kernel_choices and self.dtype == torch.bfloat16:
      try:
        with self.choices:
          tune_products(self.model.products())
      except (RuntimeError, torch.cuda.OutOfMemoryError) as e:      # the rule stands in for the measurement
        self.choices.clear()
        torch.cuda.empty_cache()
        warnings.warn(f"timing the product kernels failed ({e}); they are chosen by rule")
    self.runner = ModelRunner(self.model, self.cache, use_graphs=not cfg.enforce_eager, choices=self.choices,
                              compare_captures=cfg.timed_kernel_choices)
    eos = cfg.eos if cfg.eos is not None else self._eos_of_folder(cfg.model_path)
    if eos is None:
      eos = getattr(self.model_config, "eos_token_id", None)
    self.eos_token_id = eos
    self.scheduler = Scheduler(self.cache, max_num_seqs=cfg.max_num_seqs,
                               max_num_batched_tokens=cfg.max_num_batched_tokens, max_model_len=self.max_model_len,
                               enable_chunked_prefill=cfg.enable_chunked_prefill, eos_token_id=eos)
    self.sampler = Sampler(self.device)
    self.tokenizer = self._load_tokenizer(cfg.model_path)
    self._next_number = 0
    self._requests: Dict[str, Request] = {}
    self.num_steps = 0
    # the launched step whose tokens have not been read back yet: (plan, requests that sample, host buffer, event)
    self._pending = None
    self._token_bufs = [torch.zeros(max(1, cfg.max_num_seqs), dtype=torch.int32, pin_memory=True) for _ in range(2)]
    self._token_turn = 0
    torch.cuda.synchronize(self.device)
    self.startup_seconds = time.perf_counter() - t_start     # weights, cache pools, timing of the product kernels
    self.warm_up_seconds = 0.0                                # spent in `warm_up` so far

  # ------------------------------------------------------------------ set-up helpers
  def _pages_from_memory(self, needs) -> int:
    """Pages from the device memory that is free after the weights are loaded, less the share of the device that
    `gpu_memory_utilization` leaves alone and less what the largest step needs for its activations (the reference
    holds back a fifth of the free memory for them, whatever the model: utils/memory_utils.py:85-144; here the
    step's buffers are counted from the model's sizes and the token budget).  Never more pages than
    `max_num_seqs` requests of `max_model_len` tokens can use.  The pools' bytes are the cache manager's own count
    (groups differ in page size, dtype and, with a window, in how many pages they can use at all)."""
    cfg = self.config
    cap = cfg.max_num_seqs * (-(-self.max_model_len // cfg.page_size))

    def pool_bytes(pages: int) -> int:
      return CacheManager.storage_bytes(needs, cfg.page_size, pages, cfg.max_num_seqs, cfg.max_num_batched_tokens,
                                        self.dtype)

    if pool_bytes(cap) == 0:
      return max(1, cap)
    free, total = torch.cuda.mem_get_info(self.device)
    usable = free - int(total * (1.0 - cfg.gpu_memory_utilization)) - self.activation_bytes()
    if pool_bytes(2) > usable:
      raise RuntimeError(f"not enough device memory for a cache: {free >> 20} MiB free, the largest step needs "
                         f"{self.activation_bytes() >> 20} MiB, two pages cost {pool_bytes(2)} bytes")
    lo, hi = 2, cap                      # the most pages whose pools fit: the bytes grow with the pages
    while lo < hi:
      mid = (lo + hi + 1) // 2
      if pool_bytes(mid) <= usable:
        lo = mid
      else:
        hi = mid - 1
    return int(lo)

  def activation_bytes(self) -> int:
    """An upper estimate of the device memory that steps hold beside weights and cache.  One step of the full token
    budget: per token two 32-bit residual rows and, in the activation dtype, the widest rows a block makes (each
    counted twice, since the allocator keeps a freed buffer of one layer while the next layer's is made); while the
    product kernels are timed at start-up, that timing's buffers instead if they are larger.  The 32-bit logits of
    `max_num_seqs` rows with the sampler's scratch.  The captured decode steps: they share one pool for what they
    hold while they run (counted once, for the widest of them) but each keeps its own logits, so one row of logits for
    every row of every (batch, table width) bucket that this engine's limits allow.  And 256 MiB of slack (key-range
    partials of the attention, the k-split products' partial results, the library's workspace)."""
    cfg, spec = self.config, self.model.spec
    esize = 2 if self.dtype == torch.bfloat16 else 4
    widest = spec.hidden_size
    for _, part, ps in self.model.named_params():
      if part is self.model:            # the frame's own tables (embedding, head, positions) are no activations
        continue
      if len(ps.shape) == 2:
        widest = max(widest, ps.shape[0])
    T = cfg.max_num_batched_tokens
    per_token = 2 * 4 * spec.hidden_size + 2 * esize * (2 * widest + 2 * spec.hidden_size)
    step = T * per_token
    if cfg.tune_products and cfg.timed_kernel_choices and self.dtype == torch.bfloat16:
      step = max(step, 640 << 20)       # the timing's flush buffer, operands and partial results
    logits = 3 * 4 * spec.vocab_size * min(cfg.max_num_seqs, 256)
    graphs = 0
    if not cfg.enforce_eager:
      from .runner import graph_bucket_rows
      rows, widths = graph_bucket_rows(cfg.max_num_seqs, self.max_model_len, cfg.page_size)
      graphs = 256 * per_token + rows * widths * 4 * spec.vocab_size
    return int(step + logits + graphs + (256 << 20))

  @staticmethod
  def _eos_of_folder(path: str):
    """`eos_token_id` of the folder's generation_config.json: one id or a list of them; None without the file."""
    gj = os.path.join(path, "generation_config.json") if path and os.path.isdir(path) else None
    if not gj or not os.path.isfile(gj):
      return None
    import json
    with open(gj) as f:
      eos = json.load(f).get("eos_token_id")
    if isinstance(eos, list):
      return [int(t) for t in eos] or None
    return None if eos is None else int(eos)

  @staticmethod
  def _load_tokenizer(path: str):
    tj = os.path.join(path, "tokenizer.json") if path and os.path.isdir(path) else None
    if tj and os.path.isfile(tj):
      try:
        from tokenizers import Tokenizer
        return Tokenizer.from_file(tj)
      except Exception:
        return None
    return None

  # ------------------------------------------------------------------ context manager (llm_engine.py:1301-1306)
  def __enter__(self):
    return self

  def __exit__(self, *exc):
    self.stop()
    return False

  def start(self):
    return self

  def stop(self):
    pass

  # ------------------------------------------------------------------ requests
  def _encode(self, prompt) -> List[int]:
    if isinstance(prompt, str):
      if self.tokenizer is None:
        raise ValueError("a text prompt needs a tokenizer.json in the model folder; pass token ids instead")
      return list(self.tokenizer.encode(prompt).ids)
    return [int(t) for t in prompt]

  def add_request(self, prompt: Union[str, Sequence[int]], sampling_params: Optional[SamplingParams] = None,
                  request_id: Optional[str] = None) -> str:
    """Queues a request and returns its id.  The step that books the request's last token hands the finished
    request out in `StepOutput.finished` (`request_id`, `outputs`, `finish_reason`); the engine keeps no
    reference to it after that (miniinfer/engine/llm_engine.py:1309-1339)."""
    params = sampling_params or SamplingParams()
    ids = self._encode(prompt)
    V = self.model.spec.vocab_size
    if any(t < 0 or t >= V for t in ids):
      raise ValueError(f"prompt holds a token id outside [0, {V})")
    number = self._next_number
    self._next_number += 1
    rid = request_id or f"req-{number}"
    req = Request(number=number, request_id=rid, prompt=ids, params=params,
                  seed=request_seed(self.config.seed, number, params.seed))
    self.scheduler.add(req)
    self._requests[rid] = req
    return rid

  def warm_up(self, max_num_seqs: Optional[int] = None, max_tokens: Optional[int] = None) -> int:
    """Captures the decode graphs ahead of their first use (every batch bucket up to `max_num_seqs`, every table
    width up to `max_tokens` tokens a request; defaults: the engine's limits).  Returns the number of graphs."""
    t0 = time.perf_counter()
    n = self.runner.capture_graphs(max_num_seqs or self.config.max_num_seqs, max_tokens or self.max_model_len)
    torch.cuda.synchronize(self.device)
    self.warm_up_seconds += time.perf_counter() - t0
    return n

  def is_finished(self) -> bool:
    return self._pending is None and not self.scheduler.has_unfinished()

  has_unfinished = property(lambda self: self.scheduler.has_unfinished())

  # ------------------------------------------------------------------ one step
  def _launch(self, plan: ScheduledStep):
    """Runs the plan's batch and samples, all of it queued on the device; the tokens go to the runner's
    `future_tokens` and, by a copy that an event marks, to a pinned host buffer."""
    entries = []
    sampling = []
    for e in plan.entries:
      toks = e.request.tokens[e.start:e.start + e.num_tokens]
      entries.append(StepEntry(req=e.request.number, tokens=toks, want=[e.num_tokens - 1] if e.samples else []))
      if e.samples:
        sampling.append(e.request)
    logits = self.runner.step(entries, allow_future=True)
    host = event = None
    if sampling:
      R = len(sampling)
      dev = self.runner.future_tokens[:R]
      self.sampler.sample_into(logits, [r.params for r in sampling], [r.seed for r in sampling],
                               [len(r.outputs) for r in sampling], dev)
      self._token_turn ^= 1
      host = self._token_bufs[self._token_turn][:R]
      host.copy_(dev, non_blocking=True)
      event = torch.cuda.Event()
      event.record()
    self.scheduler.advance(plan)
    self.num_steps += 1
    return plan, sampling, host, event

  def _resolve(self, pending, out: StepOutput) -> None:
    """Reads a launched step's tokens (waiting for them if need be) and books them."""
    plan, sampling, host, event = pending
    sampled: Dict[int, int] = {}
    if sampling:
      event.synchronize()
      sampled = {r.number: t for r, t in zip(sampling, host.tolist())}
    done = self.scheduler.resolve(plan, sampled)
    for r in done:                      # the step's output hands a finished request out; the engine lets go of it
      self._requests.pop(r.request_id, None)
    out.finished += done
    out.num_prefill_tokens += plan.num_prefill_tokens
    out.num_decode_tokens += plan.num_decode_tokens
    out.num_preempted += len(plan.preempted)

  def step(self) -> StepOutput:
    """schedule -> run the batch -> sample -> update (miniinfer/engine/llm_engine.py:465-557); with
    `enable_overlap`, schedule and launch the next step, then read and book the tokens of the one before
    (llm_engine.py:559-700).  Returns what the booked step did."""
    out = StepOutput()
    if not self.config.enable_overlap:
      plan = self.scheduler.schedule()
      if plan is not None:
        self._resolve(self._launch(plan), out)
      return out
    plan = self.scheduler.schedule()
    launched = self._launch(plan) if plan is not None else None
    if self._pending is not None:
      self._resolve(self._pending, out)
    self._pending = launched
    return out

  # ------------------------------------------------------------------ generate
  def generate(self, prompts, sampling_params: Union[SamplingParams, Sequence[SamplingParams], None] = None,
               use_tqdm: bool = True) -> List[dict]:
    """prompts: a string, a list of strings, a list of token ids, or a list of such lists; sampling_params: one
    for all or one per prompt.  Returns, in the order of the prompts, dicts with "text", "token_ids",
    "request_id" (miniinfer/engine/llm_engine.py:898-1015) and "finish_reason"."""
    if isinstance(prompts, str) or (len(prompts) > 0 and isinstance(prompts[0], int)):
      prompts = [prompts]
    if sampling_params is None:
      sampling_params = SamplingParams()
    if isinstance(sampling_params, SamplingParams):
      sampling_params = [sampling_params] * len(prompts)
    if len(sampling_params) != len(prompts):
      raise ValueError("one SamplingParams for all prompts, or one per prompt")
    rids = [self.add_request(p, sp) for p, sp in zip(prompts, sampling_params)]
    mine = [self._requests[rid] for rid in rids]
    t0 = time.time()
    decoded = 0
    last = t0
    while not self.is_finished():
      so = self.step()
      decoded += so.num_decode_tokens
      if use_tqdm and time.time() - last > 1.0:
        last = time.time()
        print(f"\r[miniinfer_amd] step {self.num_steps}: {decoded / (last - t0):.1f} decoded tok/s", end="",
              file=sys.stderr, flush=True)
    if use_tqdm:
      print(file=sys.stderr)
    results = []
    for rid, r in zip(rids, mine):
      text = self.tokenizer.decode(r.outputs) if self.tokenizer is not None else ""
      results.append({"text": text, "token_ids": list(r.outputs), "request_id": rid, "finish_reason": r.finish_reason})
    return results

  def stream_generate(self, prompts, sampling_params: Union[SamplingParams, Sequence[SamplingParams], None] = None):
    """The same requests, yielded token by token as they are booked: a `RequestOutput` for every new token of
    every request, the last one of a request with `finished` set (miniinfer/engine/llm_engine.py:1341-1400).
    Tokens of one request come in order; requests interleave as the steps produce them."""
    if isinstance(prompts, str) or (len(prompts) > 0 and isinstance(prompts[0], int)):
      prompts = [prompts]
    if sampling_params is None:
      sampling_params = SamplingParams()
    if isinstance(sampling_params, SamplingParams):
      sampling_params = [sampling_params] * len(prompts)
    if len(sampling_params) != len(prompts):
      raise ValueError("one SamplingParams for all prompts, or one per prompt")
    rids = [self.add_request(p, sp) for p, sp in zip(prompts, sampling_params)]
    live = {rid: self._requests[rid] for rid in rids}
    sent = {rid: 0 for rid in rids}
    texts = {rid: "" for rid in rids}
    while live:
      if not self.is_finished():
        self.step()
      for rid in list(live):
        r = live[rid]
        ready = len(r.outputs) - r.pending           # placeholders of tokens still on the device sit at the end
        done = r.finished and r.pending == 0
        for i in range(sent[rid], ready):
          full = self.tokenizer.decode(r.outputs[:i + 1]) if self.tokenizer is not None else ""
          last = done and i == ready - 1
          yield RequestOutput(request_id=rid, delta_text=full[len(texts[rid]):], full_text=full, token_id=r.outputs[i],
                              output_token_ids=list(r.outputs[:i + 1]), finished=last,
                              finish_reason=r.finish_reason if last else None)
          texts[rid] = full
        sent[rid] = ready
        if done:
          del live[rid]
