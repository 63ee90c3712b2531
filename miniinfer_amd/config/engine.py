"""Engine options.

Names and meanings follow the reference's `EngineConfig`
(miniinfer/config/engine/config.py:8-77) and the keyword arguments its examples pass
(`max_num_seqs`, `max_model_len`, `page_size`, `enforce_eager`:
examples/minimal_engine.py:24-73, benchmark/bench_miniinfer.py:16-51).  The reference
drops unknown keyword arguments silently (miniinfer/engine/llm_engine.py:102-104);
here they are errors.
"""

from __future__ import annotations

from dataclasses import dataclass, fields
from typing import Optional

_DTYPES = {"bfloat16": "bfloat16", "bf16": "bfloat16", "float32": "float32", "fp32": "float32"}


def normalize_dtype(dtype) -> str:
  s = str(dtype).replace("torch.", "")
  if s not in _DTYPES:
    raise ValueError(f"dtype {dtype!r} is not supported; use 'bfloat16' or 'float32'")
  return _DTYPES[s]


@dataclass
class EngineConfig:
  model_path: str
  dtype: str = "bfloat16"
  page_size: int = 16
  # cache size: an explicit number of pages per layer group, or a share of device memory
  num_pages: Optional[int] = None
  gpu_memory_utilization: float = 0.9
  max_num_seqs: int = 256
  max_model_len: Optional[int] = None         # clamped to the model's max positions
  max_num_batched_tokens: int = 8192          # token budget of one step (reference: max_extend_len)
  enable_chunked_prefill: bool = True
  enforce_eager: bool = False                 # True: never replay decode steps from HIP graphs
  enable_overlap: bool = True                 # launch a step before the last one's tokens are read back
  tune_products: bool = True                  # time own and library kernels for the model's large products once
  eos: Optional[int] = None                   # None: from generation_config.json, else from config.json
  seed: int = 0
  # "safetensors": the folder's *.safetensors files, by tensor name; "random": only config.json is read and the
  # weights are drawn on the device from `seed` (N(0, initializer_range), norm weights 1 + N(0, 0.1))
  load_format: str = "safetensors"
  # False: products of few rows go where the rule sends them, never where a timing at start-up did, and a captured
  # step is recorded one way only, so that a run's kernels (and with them its bfloat16 roundings) do not depend on
  # timings; implies what `tune_products=False` does
  timed_kernel_choices: bool = True
  device: str = "cuda:0"

  def __post_init__(self):
    self.dtype = normalize_dtype(self.dtype)
    if self.page_size <= 0 or (self.page_size & (self.page_size - 1)) != 0:
      raise ValueError(f"page_size must be a power of two, got {self.page_size}")
    if self.num_pages is not None and self.num_pages <= 0:
      raise ValueError("num_pages must be positive")
    if not (0.0 < self.gpu_memory_utilization <= 1.0):
      raise ValueError("gpu_memory_utilization must be in (0, 1]")
    if self.max_num_seqs <= 0:
      raise ValueError("max_num_seqs must be positive")
    if self.max_num_batched_tokens <= 0:
      raise ValueError("max_num_batched_tokens must be positive")
    if self.max_model_len is not None and self.max_model_len <= 0:
      raise ValueError("max_model_len must be positive")
    if self.load_format not in ("safetensors", "random"):
      raise ValueError(f"load_format must be 'safetensors' or 'random', got {self.load_format!r}")

  # aliases the reference keeps (config.py:63-70)
  @property
  def model(self) -> str:
    return self.model_path

  @classmethod
  def from_kwargs(cls, model: str, **kwargs) -> "EngineConfig":
    aliases = {"max_context_len": "max_model_len", "max_extend_len": "max_num_batched_tokens",
               "memory_ratio": "gpu_memory_utilization"}
    known = {f.name for f in fields(cls)}
    out = {}
    for k, v in kwargs.items():
      k2 = aliases.get(k, k)
      if k2 not in known:
        raise TypeError(f"unknown engine option {k!r}; known options: {sorted(known - {'model_path'})}")
      out[k2] = v
    return cls(model_path=model, **out)
