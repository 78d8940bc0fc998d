"""A small, whole inference engine for one MI355X: everything between a request's tokens and
its next token, for the architectures registered in ``sparseengine_amd.models``."""
from . import models  # noqa: F401  (registers the architectures)

__all__ = ["LLM", "SamplingParams", "Config"]


def __getattr__(name):
    if name == "LLM":
        from .engine.llm import LLM
        return LLM
    if name == "SamplingParams":
        from .sampling.params import SamplingParams
        return SamplingParams
    if name == "Config":
        from .config.runtime import Config
        return Config
    raise AttributeError(name)
