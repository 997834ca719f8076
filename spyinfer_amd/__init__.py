"""spyinfer_amd: a small, whole inference engine for one AMD MI355X (gfx950)."""
__version__ = "0.1.0"
