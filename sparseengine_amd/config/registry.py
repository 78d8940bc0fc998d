"""The one registry from an architecture's name to its model.

An architecture registers: how its ``config.json`` becomes a typed configuration, how that
becomes a ``ModelSpec`` of parts, which checkpoint tensor fills which parameter, and how random
tensors of its checkpoint are drawn.  Everything else in the framework is architecture-free.
(The reference maps ``model_type`` to a spec and a runtime class name, models/spec.py:103-211,
engine/model_runner.py:150-181.)
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Callable

from .specs import ModelSpec


@dataclass(frozen=True)
class WeightSource:
    """Checkpoint tensor ``name`` fills ``param[index]`` (``index``: ints and slices; () = all)."""
    name: str
    param: str
    index: tuple = ()


@dataclass(frozen=True)
class Architecture:
    name: str                                            # the entry of config.json "architectures"
    model_types: tuple[str, ...]
    parse_config: Callable[[dict], Any]                  # config.json dict -> typed configuration
    build_spec: Callable[[Any], ModelSpec]
    weight_sources: Callable[[Any], list[WeightSource]]
    ignored_tensor: Callable[[str], bool]                # checkpoint tensors that are not loaded
    random_tensor: Callable                              # (config, name, shape, generator, options) -> float32 tensor
    stored_dtype: Callable[[str], str]                   # tensor name -> "bfloat16" | "float32" as a checkpoint stores it
    config_to_dict: Callable[[Any], dict]
    # (ModelSpec, chunk_tokens) -> the model: None builds ``parts.DecoderModel``; an architecture whose two
    # ends differ from it (an embedding multiplier, a scale or cap on the logits) names a subclass here
    model_factory: Callable | None = None

    def make_model(self, spec: ModelSpec, chunk_tokens: int = 16384):
        if self.model_factory is not None:
            return self.model_factory(spec, chunk_tokens=chunk_tokens)
        from ..parts import build_model
        return build_model(spec, chunk_tokens=chunk_tokens)


_ARCHITECTURES: dict[str, Architecture] = {}


def register_architecture(arch: Architecture) -> Architecture:
    _ARCHITECTURES[arch.name] = arch
    return arch


def supported_architectures() -> list[str]:
    return sorted(_ARCHITECTURES)


def resolve_architecture(raw_config: dict) -> Architecture:
    """By ``architectures[0]``, else by ``model_type``."""
    names = raw_config.get("architectures") or []
    for name in names:
        if name in _ARCHITECTURES:
            return _ARCHITECTURES[name]
    model_type = raw_config.get("model_type")
    for arch in _ARCHITECTURES.values():
        if model_type in arch.model_types:
            return arch
    raise NotImplementedError(
        f"architecture {names or model_type!r} is not supported; supported: {supported_architectures()}")


def read_config_json(folder: str) -> dict:
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise FileNotFoundError(f"{folder} has no config.json")
    with open(path) as fh:
        return json.load(fh)
