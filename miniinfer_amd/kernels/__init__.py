"""HIP kernels of the engine and their Python face."""

from typing import List

from . import jit

# every shared object of the library: (source name, defines)
ALL_MODULES = [("elementwise", ()), ("gemm", ()), ("attention", ()), ("sampling", ())]


def build_all(force: bool = False) -> List[str]:
  """Compile every shared object for gfx950 (all of them again when `force`)."""
  return jit.compile_many(ALL_MODULES, force=force)
