"""machserve_amd: a one-GPU inference engine for the dense Qwen2 decoder on MI355X (gfx950)."""
__version__ = "0.1.0"
