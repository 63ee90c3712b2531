"""miniinfer_amd: a small, whole inference engine for one MI355X (gfx950)."""

__version__ = "0.1.0"
