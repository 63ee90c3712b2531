"""Minimal reader and writer of the safetensors file format.

File = 8-byte little-endian header length, a JSON header {name: {dtype, shape, data_offsets}},
then the raw little-endian tensor data.  The reader memory-maps the file and hands out one
tensor at a time, so a checkpoint far larger than host memory streams to the device tensor by
tensor (the reference reads every tensor into one dict first: miniinfer/loader/weight.py:140-158).
"""

from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, List, Tuple

import numpy as np
import torch

_DTYPES = {
  "F64": (torch.float64, 8), "F32": (torch.float32, 4), "F16": (torch.float16, 2), "BF16": (torch.bfloat16, 2),
  "I64": (torch.int64, 8), "I32": (torch.int32, 4), "I16": (torch.int16, 2), "I8": (torch.int8, 1),
  "U8": (torch.uint8, 1), "BOOL": (torch.bool, 1),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}


class SafetensorsFile:
  def __init__(self, path: str):
    self.path = path
    self._f = open(path, "rb")
    head = self._f.read(8)
    if len(head) != 8:
      raise ValueError(f"{path}: not a safetensors file (shorter than its length field)")
    (n,) = struct.unpack("<Q", head)
    size = os.path.getsize(path)
    if n > size - 8:
      raise ValueError(f"{path}: header length {n} exceeds the file size {size}")
    self.header = json.loads(self._f.read(n).decode("utf-8"))
    self.header.pop("__metadata__", None)
    self._data_start = 8 + n
    self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ) if size > 0 else None
    for name, info in self.header.items():
      if info["dtype"] not in _DTYPES:
        raise ValueError(f"{path}: tensor {name!r} has unsupported dtype {info['dtype']}")
      b, e = info["data_offsets"]
      want = int(np.prod(info["shape"], dtype=np.int64)) * _DTYPES[info["dtype"]][1]
      if e - b != want or self._data_start + e > size:
        raise ValueError(f"{path}: tensor {name!r} has data_offsets {info['data_offsets']} for shape "
                         f"{info['shape']} {info['dtype']}")

  def keys(self) -> List[str]:
    return list(self.header.keys())

  def shape(self, name: str) -> Tuple[int, ...]:
    return tuple(self.header[name]["shape"])

  def dtype(self, name: str) -> torch.dtype:
    return _DTYPES[self.header[name]["dtype"]][0]

  def tensor(self, name: str) -> torch.Tensor:
    """A CPU tensor that views the mapped file (read-only: copy before writing to it)."""
    info = self.header[name]
    dt, _ = _DTYPES[info["dtype"]]
    b, e = info["data_offsets"]
    shape = tuple(info["shape"])
    if e == b:
      return torch.empty(shape, dtype=dt)
    buf = memoryview(self._mm)[self._data_start + b:self._data_start + e]
    import warnings
    with warnings.catch_warnings():
      warnings.simplefilter("ignore")   # torch warns that the buffer is not writable
      return torch.frombuffer(buf, dtype=dt).reshape(shape)

  def close(self):
    # tensors handed out may still view the map; let the garbage collector end it
    self._f.close()


def list_safetensors(model_dir: str) -> List[str]:
  """Every *.safetensors of a folder, sorted (miniinfer/loader/weight.py:109-113)."""
  files = sorted(os.path.join(model_dir, f) for f in os.listdir(model_dir) if f.endswith(".safetensors"))
  if not files:
    raise FileNotFoundError(f"{model_dir!r} holds no *.safetensors file")
  return files


def write_safetensors(path: str, tensors: Iterable[Tuple[str, torch.Tensor]]) -> None:
  tensors = [(k, t.detach().cpu().contiguous()) for k, t in tensors]
  header: Dict[str, dict] = {}
  off = 0
  for k, t in tensors:
    if t.dtype not in _NAMES:
      raise ValueError(f"tensor {k!r}: dtype {t.dtype} cannot be stored")
    n = t.numel() * t.element_size()
    header[k] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [off, off + n]}
    off += n
  blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
  blob += b" " * ((8 - len(blob) % 8) % 8)
  with open(path, "wb") as f:
    f.write(struct.pack("<Q", len(blob)))
    f.write(blob)
    for _, t in tensors:
      if t.numel():
        f.write(t.view(torch.uint8).numpy().tobytes() if t.dim() else t.reshape(1).view(torch.uint8).numpy().tobytes())
