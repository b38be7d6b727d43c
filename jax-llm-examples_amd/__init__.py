"""A one-GPU inference engine for Llama 4 on AMD MI355X (gfx950)."""
__version__ = "0.1.0"
