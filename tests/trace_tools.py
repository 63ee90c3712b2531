"""Builds traces (lists of step records in the format of bin/trace_run) that cut the same requests
in different ways, and gathers the logits a replay returns back into one [len, vocab] array per request."""

import random
from typing import Dict, List

import numpy as np


def whole(requests: Dict[str, List[int]]):
  """Each request alone and whole, in one step."""
  steps = []
  for s, (rid, toks) in enumerate(requests.items()):
    steps.append({"step": s, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}], "end": [rid]})
  return steps


def tail_decoded(requests: Dict[str, List[int]], tail: int = 32):
  """Most of a request in one step, its last `tail` tokens one by one."""
  steps = []
  s = 0
  for rid, toks in requests.items():
    head = max(1, len(toks) - tail)
    steps.append({"step": s, "entries": [{"id": rid, "tokens": toks[:head], "want": list(range(head))}], "end": []})
    s += 1
    for i in range(head, len(toks)):
      steps.append({"step": s, "entries": [{"id": rid, "tokens": toks[i:i + 1], "want": [0]}],
                    "end": [rid] if i == len(toks) - 1 else []})
      s += 1
    if head == len(toks):
      steps[-1]["end"] = [rid]
  return steps


def portions(requests: Dict[str, List[int]], sizes=(2, 3, 7, 2, 16, 5, 33, 2, 9, 64, 1)):
  """Portions of changing size, down to two tokens."""
  steps = []
  s = 0
  for rid, toks in requests.items():
    i, k = 0, 0
    while i < len(toks):
      n = min(sizes[k % len(sizes)], len(toks) - i)
      k += 1
      steps.append({"step": s, "entries": [{"id": rid, "tokens": toks[i:i + n], "want": list(range(n))}],
                    "end": [rid] if i + n == len(toks) else []})
      i += n
      s += 1
  return steps


def mixed(requests: Dict[str, List[int]], max_live: int = 4, seed: int = 0, decode_tail: int = 12,
          max_portion: int = 24):
  """Up to `max_live` live requests: portions of some beside single decoded tokens of others; a request
  may sit a step out; new requests start as others end, so their pages are used again."""
  rng = random.Random(seed)
  waiting = list(requests.items())
  live: Dict[str, int] = {}      # id -> tokens done
  steps = []
  s = 0
  while waiting or live:
    while waiting and len(live) < max_live and (not live or rng.random() < 0.7):
      rid, _ = waiting.pop(0)
      live[rid] = 0
    entries, end = [], []
    for rid in list(live):
      toks = requests[rid]
      done = live[rid]
      if len(live) > 1 and rng.random() < 0.15:
        continue   # sits this step out
      left = len(toks) - done
      if left <= decode_tail:
        n = 1
      else:
        n = min(left - decode_tail, rng.choice([2, 2, 3, 5, 8, 13, max_portion]))
      entries.append({"id": rid, "tokens": toks[done:done + n], "want": list(range(n))})
      live[rid] = done + n
      if live[rid] == len(toks):
        end.append(rid)
        del live[rid]
    if not entries:
      continue
    rng.shuffle(entries)
    steps.append({"step": s, "entries": entries, "end": end})
    s += 1
  return steps


def peak_tokens(steps, requests, granule: int = 64) -> int:
  """The most tokens live requests hold at any time, each request's count rounded up to `granule`."""
  held: Dict[str, int] = {}
  peak = 0
  for st in steps:
    for e in st["entries"]:
      held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
    peak = max(peak, sum(-(-n // granule) * granule for n in held.values()))
    for rid in st["end"]:
      held.pop(rid, None)
  return peak


def gather(steps, outputs, requests, vocab: int) -> Dict[str, np.ndarray]:
  """outputs[i] = array [wanted, vocab] of step i (or None) -> per request [len, vocab], NaN where never asked."""
  res = {rid: np.full((len(t), vocab), np.nan, dtype=np.float32) for rid, t in requests.items()}
  done = {rid: 0 for rid in requests}
  for st, out in zip(steps, outputs):
    r = 0
    for e in st["entries"]:
      for w in e["want"]:
        res[e["id"]][done[e["id"]] + w] = out[r]
        r += 1
    for e in st["entries"]:
      done[e["id"]] += len(e["tokens"])
    assert out is None or r == out.shape[0]
  return res
