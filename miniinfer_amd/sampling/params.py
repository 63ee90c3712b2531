"""Per-request sampling options, with the reference's names, defaults and checks
(miniinfer/utils/sampling_params.py:5-23), plus an optional per-request seed and a list of token ids that end
the request like the end-of-sequence token does."""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional


@dataclass
class SamplingParams:
  temperature: float = 1.0      # 0 = greedy
  max_tokens: int = 1
  ignore_eos: bool = False
  top_k: int = 0                # 0 disables
  top_p: float = 1.0            # 1.0 disables
  seed: Optional[int] = None    # None: derived from the engine's seed and the request's number
  stop_token_ids: List[int] = field(default_factory=list)   # any of these ends the request (reason "stop"); it is
                                # kept as the last output token; `ignore_eos` does not switch these off

  def __post_init__(self):
    if self.temperature < 0:
      raise ValueError("temperature must be >= 0")
    if self.max_tokens <= 0:
      raise ValueError("max_tokens must be > 0")
    if self.top_k is None:
      self.top_k = 0
    if self.top_k < 0:
      raise ValueError("top_k must be >= 0")
    if not (0.0 < float(self.top_p) <= 1.0):
      raise ValueError("top_p must be in (0, 1]")
    self.stop_token_ids = [int(t) for t in (self.stop_token_ids or [])]
    if any(t < 0 for t in self.stop_token_ids):
      raise ValueError("stop_token_ids must be >= 0")
