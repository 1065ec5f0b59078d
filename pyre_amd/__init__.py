"""pyre_amd: a small, whole LLM inference engine for one AMD Instinct MI355X (gfx950)."""

__version__ = "0.1.0"
