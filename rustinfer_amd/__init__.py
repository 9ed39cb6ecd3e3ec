"""rustinfer_amd: a small, whole inference engine for MI355X (gfx950)."""
__version__ = "0.1.0"

from .sampling.params import SamplingParams  # noqa: F401


def __getattr__(name):
    if name in ("LLM", "generate", "GenerationResult"):
        from . import llm
        return getattr(llm, name)
    raise AttributeError(name)
