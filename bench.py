#!/usr/bin/env python3
"""python bench.py [--gpus 1] [--steps K] [--warmup W] ...: decode and prefill throughput of the engine on one
MI355X (Qwen3-0.6B shape, random weights), as ONE JSON line.  The program itself is `miniinfer_amd/benchmark.py`
(also `python -m miniinfer_amd bench`); its module docstring describes the options and the record."""

import sys

from miniinfer_amd.benchmark import main

if __name__ == "__main__":
  sys.exit(main())
