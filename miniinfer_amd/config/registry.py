"""One registry from an architecture's name to its configuration class.

The name is `config.json["architectures"][0]`; `model_type` is a second key to the same
entry.  The reference chooses by an if-chain on `model_type` / `architectures`
(miniinfer/engine/model_runner.py:61-76) and fails later with "Model is not initialized";
here an unknown name fails at once and lists the known ones.

A configuration class has `from_dict(raw) -> config` and `config.build_spec() -> ModelSpec`;
the `ModelSpec` is all the rest of the framework reads.
"""

from __future__ import annotations

import json
import os
from typing import Any, Dict, Optional

from .spec import ModelSpec

_ARCHITECTURES: Dict[str, Any] = {}
_MODEL_TYPES: Dict[str, str] = {}


def register_architecture(name: str, config_cls, model_type: Optional[str] = None) -> None:
  _ARCHITECTURES[name] = config_cls
  if model_type:
    _MODEL_TYPES[model_type] = name


def known_architectures():
  return sorted(_ARCHITECTURES)


def resolve_architecture(raw: Dict[str, Any]):
  archs = raw.get("architectures") or []
  for a in archs:
    if a in _ARCHITECTURES:
      return a, _ARCHITECTURES[a]
  mt = raw.get("model_type")
  if mt in _MODEL_TYPES:
    name = _MODEL_TYPES[mt]
    return name, _ARCHITECTURES[name]
  raise ValueError(f"config.json names architectures={archs!r}, model_type={mt!r}; "
                   f"this engine knows {known_architectures()}")


def read_config_json(model_dir: str) -> Dict[str, Any]:
  path = os.path.join(model_dir, "config.json")
  if not os.path.isfile(path):
    raise FileNotFoundError(f"{model_dir!r} holds no config.json")
  with open(path) as f:
    return json.load(f)


def load_model_config(model_dir: str):
  """config.json of a model folder -> the typed configuration of its architecture."""
  raw = read_config_json(model_dir)
  _, cls = resolve_architecture(raw)
  return cls.from_dict(raw)


def model_spec_of(config) -> ModelSpec:
  return config.build_spec()
