"""Weights by tensor name.

The part tree of a model says which tensors it owns and which checkpoint tensors fill them
(q, k, v projections are laid into one fused matrix, gate and up likewise: the fusion of
miniinfer/loader/weight.py:65-98, done while copying instead of with a concatenated temporary).
Tensors are read one at a time from the memory-mapped files and copied straight into their
final device storage, so a checkpoint never exists twice in memory (the reference builds a whole
dict on the device and copies it again into the modules: loader/weight.py:196-206,
models/fused_qwen3.py:81-83).

Every checkpoint tensor must be used and every parameter filled; otherwise ONE error lists the
missing names, the unexpected names and the wrong shapes together.
"""

from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import torch

from ..config import load_model_config, model_spec_of
from ..config.spec import ModelSpec
from ..parts import FRAMES, BuildContext, DecoderModel, ParamSpec, Part
from .safetensors_io import SafetensorsFile, list_safetensors


class WeightsError(RuntimeError):
  def __init__(self, model_dir, missing, unexpected, wrong_shape, other=()):
    self.missing, self.unexpected, self.wrong_shape, self.other = list(missing), list(unexpected), list(wrong_shape), list(other)
    lines = [f"weights in {model_dir!r} do not fit the model:"]
    if self.missing:
      lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
    if self.unexpected:
      lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
    if self.wrong_shape:
      lines.append(f"  wrong shapes ({len(self.wrong_shape)}): " +
                   "; ".join(f"{n}: file has {tuple(got)}, model wants {tuple(want)}" for n, got, want in self.wrong_shape))
    for o in self.other:
      lines.append("  " + o)
    super().__init__("\n".join(lines))


@dataclass
class _Target:
  part: Part
  spec: ParamSpec
  row_offset: int
  shape: Tuple[int, ...]      # shape the checkpoint tensor must have


def storage_dtype(storage: str, compute: torch.dtype) -> torch.dtype:
  if storage == "compute":
    return compute
  if storage == "float32":
    return torch.float32
  if storage == "int32":
    return torch.int32
  raise ValueError(f"unknown storage class {storage!r}")


def expected_tensors(model: DecoderModel) -> Dict[str, _Target]:
  """Checkpoint name -> where it goes."""
  out: Dict[str, _Target] = {}
  for prefix, part, ps in model.named_params():
    off = 0
    for src in ps.sources:
      name = prefix + src.name
      if name in out:
        raise ValueError(f"two parameters claim the checkpoint tensor {name!r}")
      out[name] = _Target(part, ps, off, (src.rows,) + tuple(ps.shape[1:]))
      off += src.rows
    if off != ps.shape[0]:
      raise ValueError(f"parameter {prefix}{ps.name}: sources cover {off} rows of {ps.shape[0]}")
  return out


def build_model(spec: ModelSpec, dtype: torch.dtype, device) -> DecoderModel:
  """The model frame that `spec.kind` names, with its blocks and parts, without tensors."""
  return FRAMES.build(spec, BuildContext(device=torch.device(device), dtype=dtype))


def load_weights(model: DecoderModel, model_dir: str) -> None:
  """Fill a built model from the *.safetensors files of a folder."""
  spec, ctx = model.spec, model.ctx
  files = [SafetensorsFile(p) for p in list_safetensors(model_dir)]
  where: Dict[str, SafetensorsFile] = {}
  duplicate = []
  for f in files:
    for k in f.keys():
      if k in where:
        duplicate.append(f"tensor {k!r} is in two files")
      where[k] = f

  expected = expected_tensors(model)
  # checkpoints may leave the optional prefix ("model.") out: miniinfer/models/fused_qwen3.py:225-226
  opt = spec.optional_name_prefix
  if opt and spec.embedding_name.startswith(opt) and spec.embedding_name not in where \
      and spec.embedding_name[len(opt):] in where:
    expected = {(k[len(opt):] if k.startswith(opt) else k): v for k, v in expected.items()}
    head_name = spec.head_name[len(opt):] if spec.head_name.startswith(opt) else spec.head_name
  else:
    head_name = spec.head_name
  # a head that is absent is the embedding table (miniinfer/layers/embedding.py:41-48)
  alias_head = spec.head_optional and head_name not in where
  if alias_head:
    expected.pop(head_name, None)

  missing = sorted(k for k in expected if k not in where)
  unexpected = sorted(k for k in where if k not in expected)
  wrong = []
  for k, tgt in expected.items():
    if k in where and tuple(where[k].shape(k)) != tuple(tgt.shape):
      wrong.append((k, where[k].shape(k), tgt.shape))
  if missing or unexpected or wrong or duplicate:
    raise WeightsError(model_dir, missing, unexpected, sorted(wrong), duplicate)

  params: Dict[Tuple[int, str], torch.Tensor] = {}
  filled: Dict[Tuple[int, str], int] = {}
  for name in sorted(expected, key=lambda k: (id(where[k]), where[k].header[k]["data_offsets"][0])):
    tgt = expected[name]
    key = (id(tgt.part), tgt.spec.name)
    if key not in params:
      params[key] = torch.empty(tgt.spec.shape, dtype=storage_dtype(tgt.spec.storage, ctx.dtype), device=ctx.device)
      filled[key] = 0
    src = where[name].tensor(name)
    dst = params[key][tgt.row_offset:tgt.row_offset + tgt.shape[0]]
    if dst.dtype == torch.int32 and src.dtype.is_floating_point:
      raise WeightsError(model_dir, [], [], [], [f"tensor {name!r} is {src.dtype}, an integer table is wanted"])
    dst.copy_(src)
    filled[key] += tgt.shape[0]
  for prefix, part, ps in model.named_params():
    key = (id(part), ps.name)
    if key in params:
      if filled[key] != ps.shape[0]:
        raise WeightsError(model_dir, [f"{prefix}{ps.name} (filled {filled[key]} of {ps.shape[0]} rows)"], [], [])
      part.set_param(ps.name, params[key])
  if alias_head:
    model.head = None
  for f in files:
    f.close()
  model.finalize()


def load_model(model_dir: str, dtype: torch.dtype, device) -> Tuple[DecoderModel, object]:
  """config.json + safetensors of a folder -> (model on the device, its typed configuration)."""
  config = load_model_config(model_dir)
  model = build_model(model_spec_of(config), dtype, device)
  load_weights(model, model_dir)
  return model, config
