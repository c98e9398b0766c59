"""A single-GPU inference engine for AMD MI355X (gfx950)."""

__version__ = "0.1.0"
