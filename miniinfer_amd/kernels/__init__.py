"""HIP kernels of the engine and their Python face."""

from typing import List

from . import jit

# every shared object of the library: (source name, defines)
# head sizes the MFMA attention is prebuilt for (others are built at a model's first use)
PREBUILT_HEAD_DIMS = (16, 32, 48, 64, 80, 96, 128, 256)
ALL_MODULES = [("elementwise", ()), ("gemm", ()), ("gemm_skinny", ()), ("gemm_skinny", (("SKINNY_NT", 1),)),
               ("attention", ()), ("sampling", ()), ("probes", ())] + \
    [("attention_mfma", (("HEAD_DIM", d),)) for d in PREBUILT_HEAD_DIMS]


def build_all(force: bool = False) -> List[str]:
  """Compile every shared object for gfx950 (all of them again when `force`) and drop built objects of older
  sources from the in-tree build folder."""
  import os
  paths = jit.compile_many(ALL_MODULES, force=force)
  keep = {os.path.abspath(p) for p in paths}
  d = jit.build_dirs()[-2] if len(jit.build_dirs()) > 1 else jit.build_dirs()[0]
  if os.path.isdir(d):
    for fn in os.listdir(d):
      full = os.path.abspath(os.path.join(d, fn))
      if fn.endswith(".so") and full not in keep:
        try:
          os.unlink(full)
        except OSError:
          pass
  return paths


def prepare(dtype, head_dims) -> List[str]:
  """Builds, side by side, the shared objects that a model of this dtype and these head sizes loads and that are not
  built yet; returns what it built.  Each would otherwise be built at its first use, one after the other (a fresh
  checkout's first step: about two minutes; side by side: as long as the slowest, half a minute)."""
  import torch
  jobs = [("elementwise", ()), ("sampling", ()), ("gemm", ()), ("attention", ())]
  if dtype == torch.bfloat16:
    jobs += [("gemm_skinny", ()), ("gemm_skinny", (("SKINNY_NT", 1),))]
    jobs += [("attention_mfma", (("HEAD_DIM", int(d)),)) for d in sorted(set(head_dims)) if d % 16 == 0 and 16 <= d <= 256]
  missing = [j for j in jobs if jit.find_built(j[0], j[1]) is None]
  return jit.compile_many(missing) if missing else []
