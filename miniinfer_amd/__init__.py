"""miniinfer_amd: a small, whole inference engine for one MI355X (gfx950).

    from miniinfer_amd import LLMEngine, SamplingParams
"""

__version__ = "0.1.0"

from .config import EngineConfig
from .sampling import SamplingParams


def __getattr__(name):
  # the engine pulls in the kernels; keep `import miniinfer_amd` light
  if name in ("LLMEngine", "RequestOutput"):
    from .engine import llm_engine
    return getattr(llm_engine, name)
  raise AttributeError(name)
