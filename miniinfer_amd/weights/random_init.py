"""Random weights from a configuration and a seed.

`write_random_model` writes a model folder (config.json, model.safetensors) that the by-name
loader reads like any checkpoint; `fill_random` fills a built model on its device without
touching the disk (for shapes too large to be worth writing, as in measurements).
Matrices are N(0, initializer_range), norm weights 1 + N(0, 0.1).
"""

from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Tuple

import torch

from ..config import model_spec_of
from ..parts import FRAMES, BuildContext, DecoderModel
from .loader import storage_dtype
from .safetensors_io import write_safetensors


def _draw(shape, init: str, std: float, gen: torch.Generator, device) -> torch.Tensor:
  t = torch.randn(shape, generator=gen, dtype=torch.float32, device=device)
  if init == "norm":
    return 1.0 + 0.1 * t
  if init == "normal":
    return std * t
  if init == "zeros":
    return torch.zeros(shape, dtype=torch.float32, device=device)
  raise ValueError(f"unknown init {init!r}")


def random_tensors(config, seed: int, dtype: torch.dtype = torch.bfloat16) -> List[Tuple[str, torch.Tensor]]:
  """(checkpoint name, tensor) for every tensor of the architecture, drawn on the CPU."""
  spec = model_spec_of(config)
  model = FRAMES.build(spec, BuildContext(device=torch.device("cpu"), dtype=dtype))
  gen = torch.Generator(device="cpu")
  gen.manual_seed(seed)
  out = []
  for prefix, part, ps in model.named_params():
    for src in ps.sources:
      name = prefix + src.name
      if name == spec.head_name and not spec.random_writes_head:
        continue
      t = _draw((src.rows,) + tuple(ps.shape[1:]), ps.init, spec.init_std, gen, "cpu")
      out.append((name, t.to(torch.int32 if ps.storage == "int32" else dtype)))
  return out


def write_random_model(config, out_dir: str, seed: int, dtype: torch.dtype = torch.bfloat16) -> str:
  os.makedirs(out_dir, exist_ok=True)
  d = config.to_dict()
  d["torch_dtype"] = str(dtype).replace("torch.", "")
  with open(os.path.join(out_dir, "config.json"), "w") as f:
    json.dump(d, f, indent=2)
  write_safetensors(os.path.join(out_dir, "model.safetensors"), random_tensors(config, seed, dtype))
  return out_dir


def fill_random(model: DecoderModel, seed: int) -> None:
  """Random tensors straight into a built model, drawn on its device."""
  spec, ctx = model.spec, model.ctx
  gen = torch.Generator(device=ctx.device)
  gen.manual_seed(seed)
  for prefix, part, ps in model.named_params():
    if part is model and ps.name == "head" and not spec.random_writes_head:
      continue
    st = storage_dtype(ps.storage, ctx.dtype)
    param = torch.empty(ps.shape, dtype=st, device=ctx.device)
    rows_per_chunk = max(1, (64 << 20) // max(1, math.prod(ps.shape[1:])))
    for r0 in range(0, ps.shape[0], rows_per_chunk):
      r1 = min(ps.shape[0], r0 + rows_per_chunk)
      param[r0:r1].copy_(_draw((r1 - r0,) + tuple(ps.shape[1:]), ps.init, spec.init_std, gen, ctx.device))
    part.set_param(ps.name, param)
  if not spec.random_writes_head:
    model.head = None
  model.finalize()
