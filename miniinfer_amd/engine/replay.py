"""Trace replay: feeds given token ids through the model step by step and writes logits.

Nothing is sampled.  The replay drives the same model, step function, cache manager and kernels
that generation uses; it owns no forward pass, cache or loader.  Steps are read as JSON lines:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

For a step in which logits are wanted, `<out>/<step>.f32` holds them as little-endian float32
[wanted, vocab], in the order of the entries and of `want`.  After every step a line
`done <step>` is printed and flushed.

The nearest thing in the reference are its debug scripts that compare decoding from the cache
with recomputing from scratch (tests/debug/test_kv_cache_consistency.py,
tests/debug/test_multi_batch_kv_consistency.py:275-372).
"""

from __future__ import annotations

import json
import os
import sys
from typing import IO, Optional

import numpy as np
import torch

from ..cache.manager import CacheManager
from ..config import normalize_dtype
from ..weights import load_model
from .runner import ModelRunner, StepEntry

TORCH_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


class Replayer:
  def __init__(self, model_dir: str, dtype: str, max_tokens: int, page_size: int = 16, max_requests: int = 16,
               device: str = "cuda:0", choices=None):
    """max_tokens: the tokens the page pools are made for; max_requests: request slots; choices: the runner's table
    of product-kernel choices (default: a new one, every product by rule)."""
    if not torch.cuda.is_available():
      raise RuntimeError("miniinfer_amd needs a GPU: torch.cuda.is_available() is False and there is no CPU path")
    dt = TORCH_DTYPES[normalize_dtype(dtype)]
    self.model, self.config = load_model(model_dir, dt, device)
    if max_tokens <= 0:
      raise ValueError("--max-tokens must be positive")
    num_pages = -(-max_tokens // page_size)
    self.cache = CacheManager(self.model.cache_needs(), page_size=page_size, num_pages=num_pages,
                              max_requests=max_requests, max_model_len=self.model.spec.max_positions,
                              dtype=dt, device=device)
    self.runner = ModelRunner(self.model, self.cache, choices=choices)

  def step(self, record: dict) -> Optional[np.ndarray]:
    entries = []
    for e in record.get("entries", []):
      rid = e["id"]
      if not self.cache.has(rid):
        self.cache.admit(rid)
      entries.append(StepEntry(req=rid, tokens=list(e["tokens"]), want=list(e.get("want", []))))
    out = None
    if entries:
      logits = self.runner.step(entries)
      if logits.shape[0] > 0:
        out = logits.to(torch.float32).cpu().numpy()
    for rid in record.get("end", []):
      if self.cache.has(rid):
        self.cache.release(rid)
    return out


def run(model_dir: str, dtype: str, out_dir: str, max_tokens: int, inp: IO[str] = sys.stdin,
        outp: IO[str] = sys.stdout, page_size: int = 16) -> int:
  os.makedirs(out_dir, exist_ok=True)
  rp = Replayer(model_dir, dtype, max_tokens, page_size=page_size)
  for line in inp:
    line = line.strip()
    if not line:
      continue
    record = json.loads(line)
    step = record["step"]
    logits = rp.step(record)
    if logits is not None:
      logits.astype("<f4").tofile(os.path.join(out_dir, f"{step}.f32"))
    torch.cuda.synchronize()
    print(f"done {step}", file=outp, flush=True)
  return 0
