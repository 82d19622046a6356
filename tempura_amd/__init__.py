"""tempura_amd: a small, whole Llama 3 inference engine for one AMD MI355X (gfx950)."""
__version__ = "0.1.0"
