"""fastgen_amd: a small, whole LLM inference engine for one AMD Instinct
MI355X GPU (gfx950), in the manner of facebookresearch/fastgen."""

__version__ = "0.1.0"
