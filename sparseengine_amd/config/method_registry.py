"""Registry of sparse-attention methods and their prefill policies.

Only the dense method is registered: ``""`` (alias ``"vanilla"``) with the ``all_chunked`` prefill
policy and the paged cache manager.  A method brings three things under its name: the runtime with
its step hooks, its prefill policy and the class of its cache manager, which the model runner builds
in place of the paged one (reference: method_registry.py:19-36,508-525,646-665; the cache-manager
factory by method engine/cache_manager/base.py:537-647; the pass-through runtime
engine/sparse_methods/passthrough.py:11-32).
"""
from __future__ import annotations

from dataclasses import dataclass

PREFILL_POLICY_AUTO = "auto"
METHOD_ALIASES = {"vanilla": "", "none": "", "dense": "", "full": ""}


class MethodRuntime:
    """What a sparse method may do in a step, and the defaults of the dense method.

    One object per engine.  The step function and the attention mixer call it at fixed places:

    ``bind(cache)``                once, with the engine's cache manager;
    ``prepare_step(fb)``           after the step's batch is built, before the first layer;
    ``select(position, meta)``     per cache-keeping schedule position, just before attention: the
                                   view of the request's pages the layer may read (a ``GroupMeta``, or
                                   anything with its fields); the dense method hands back what it gets;
    ``after_attention(position, fb)`` per such position, after its attention has read the cache;
    ``finish_step(fb)``            after the last layer, before logits leave the step;
    ``extra_pages(row, new_tokens)`` pages per group index the method needs for itself on top of
                                   what the cache manager counts for an append (temporary slots);
                                   the scheduler's capacity questions add them.

    (Reference: engine/sparse_methods/base.py:324-500 prepare_step / build_*_selection /
    on_attention_end / finish_step; engine/cache_manager/base.py:1335-1361 the cache-side hooks.)
    """
    name = ""

    def bind(self, cache) -> None:
        self.cache = cache

    def prepare_step(self, fb) -> None:
        pass

    def select(self, position: int, meta):
        return meta

    def after_attention(self, position: int, fb) -> None:
        pass

    def finish_step(self, fb) -> None:
        pass

    def extra_pages(self, row: int | None, new_tokens: int) -> dict[int, int]:
        return {}


class PassThroughMethod(MethodRuntime):
    """The dense method: every hook is the identity (reference engine/sparse_methods/passthrough.py:11-32)."""


@dataclass(frozen=True)
class MethodBinding:
    name: str
    runtime_factory: type
    prefill_policy: str
    cache_manager_cls: type | None = None      # None: cache.manager.CacheManager

    def cache_manager(self) -> type:
        """The class the model runner builds its cache manager from: the method's own (a subclass of
        ``CacheManager``, or anything with its constructor and interface), else the paged one."""
        if self.cache_manager_cls is not None:
            return self.cache_manager_cls
        from ..cache.manager import CacheManager
        return CacheManager


_METHODS: dict[str, MethodBinding] = {}
PREFILL_POLICIES = {"all_chunked"}


def register_method(name: str, runtime_factory, prefill_policy: str, cache_manager_cls: type | None = None) -> None:
    if prefill_policy not in PREFILL_POLICIES:
        raise ValueError(f"unknown prefill policy {prefill_policy!r}; known: {sorted(PREFILL_POLICIES)}")
    if cache_manager_cls is not None and not callable(cache_manager_cls):
        raise TypeError("cache_manager_cls must be a class with the constructor of cache.manager.CacheManager")
    _METHODS[name] = MethodBinding(name, runtime_factory, prefill_policy, cache_manager_cls)


def normalize_sparse_method(name: str | None) -> str:
    key = (name or "").strip().lower()
    key = METHOD_ALIASES.get(key, key)
    if key not in _METHODS:
        shown = sorted({n or "vanilla" for n in _METHODS})
        raise ValueError(f"sparse_method {name!r} is not supported; supported: {shown}")
    return key


def resolve_method(name: str | None) -> MethodBinding:
    return _METHODS[normalize_sparse_method(name)]


def resolve_prefill_schedule_policy(method: str, requested: str = PREFILL_POLICY_AUTO) -> str:
    """The method's own policy; a request for another one is an error."""
    default = resolve_method(method).prefill_policy
    if requested in (None, PREFILL_POLICY_AUTO, default):
        return default
    raise ValueError(f"prefill_schedule_policy {requested!r} does not fit sparse_method "
                     f"{method or 'vanilla'!r}, whose policy is {default!r}")


register_method("", PassThroughMethod, "all_chunked")
