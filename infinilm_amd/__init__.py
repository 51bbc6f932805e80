"""infinilm_amd: a single-GPU inference engine for MI355X (gfx950)."""
from .sampling import SamplingParams  # noqa: F401


def __getattr__(name):
    if name == "LLM":
        from .llm import LLM
        return LLM
    raise AttributeError(name)


__all__ = ["LLM", "SamplingParams"]
