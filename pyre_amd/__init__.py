"""pyre_amd: a small, whole LLM inference engine for one AMD Instinct MI355X (gfx950)."""

__version__ = "0.1.0"

_API = {"load_model", "Scheduler", "generate", "generate_greedy"}


def __getattr__(name):
    # torch is imported only when the API is used, so that ``import pyre_amd`` stays cheap.
    if name in _API:
        from pyre_amd import api

        return getattr(api, name)
    raise AttributeError(f"module 'pyre_amd' has no attribute {name!r}")
