"""Registry of sparse-attention methods and their prefill policies.

Only the dense method is registered: ``""`` (alias ``"vanilla"``) with the ``all_chunked`` prefill
policy.  The hook is kept so that another method could bring its own cache manager and step
hooks later (reference method_registry.py:19-36,508-525,646-665; the pass-through runtime
engine/sparse_methods/passthrough.py:11-32).
"""
from __future__ import annotations

from dataclasses import dataclass

PREFILL_POLICY_AUTO = "auto"
METHOD_ALIASES = {"vanilla": "", "none": "", "dense": "", "full": ""}


class PassThroughMethod:
    """The dense method: every hook is the identity."""
    name = ""

    def select(self, position: int, meta):
        """The keys a layer may read: all of them."""
        return meta

    def after_attention(self, position: int, fb) -> None:
        pass

    def after_step(self, fb) -> None:
        pass


@dataclass(frozen=True)
class MethodBinding:
    name: str
    runtime_factory: type
    prefill_policy: str
    cache_manager: str = "paged"


_METHODS: dict[str, MethodBinding] = {}
PREFILL_POLICIES = {"all_chunked"}


def register_method(name: str, runtime_factory, prefill_policy: str, cache_manager: str = "paged") -> None:
    if prefill_policy not in PREFILL_POLICIES:
        raise ValueError(f"unknown prefill policy {prefill_policy!r}; known: {sorted(PREFILL_POLICIES)}")
    _METHODS[name] = MethodBinding(name, runtime_factory, prefill_policy, cache_manager)


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
