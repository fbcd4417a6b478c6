"""zedinfer_amd: a single-GPU inference engine for MI355X (gfx950)."""
__version__ = "0.1.0"
