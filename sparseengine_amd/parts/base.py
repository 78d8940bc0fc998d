"""What every part of a layer has in common, and the registries that find a part by the
``kind`` of its spec.

A part is built from its spec alone (no allocation), declares its parameters by local name, is
handed the allocated tensors once (``bind``) and then runs on a ``ForwardBatch``.  It never
learns which model it is in: names of checkpoint tensors, layer counts and the like stay with
the architecture module.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable

import torch


@dataclass(frozen=True)
class ParamDecl:
    """Shape and storage policy of one parameter.

    policy "engine":  the engine's dtype, except that a tensor the checkpoint stores in 32-bit
                      float stays float32;
    policy "float32": always float32 (router tables);
    policy "int32":   integer tables.
    """
    shape: tuple[int, ...]
    policy: str = "engine"


@dataclass(frozen=True)
class PagedKVRequest:
    """A mixer that keeps keys and values of ``window`` (None: all) past tokens in pages of ``page_size``
    tokens (None: the engine's ``kv_page_size``).  Positions whose requests are equal share a pool."""
    kv_heads: int
    head_dim: int
    window: int | None = None
    page_size: int | None = None


@dataclass(frozen=True)
class StateRequest:
    """A mixer that keeps tensors of fixed size per request: name -> (shape, dtype or None for
    the engine's dtype).  They are zeroed when a request is admitted."""
    tensors: tuple[tuple[str, tuple[int, ...], torch.dtype | None], ...]


@dataclass(frozen=True)
class FusedRotation:
    """What a position encoding that is a rotation by a table hands to the mixer's fused kernel (flat QK
    norm, rotation, cache write in one launch): ``table [positions, rotary_dim]`` (cos half, sin half, float32;
    None with ``rotary_dim`` 0: nothing is turned), the number of leading dims of a head that are turned and how
    they pair up ("neox": ``(d, d + rotary_dim / 2)``, "interleaved": ``(2 j, 2 j + 1)``)."""
    table: torch.Tensor | None
    rotary_dim: int
    pairing: str = "neox"


class SlotSum:
    """What a feed-forward hands on when the sum over a token's slots (its chosen experts) is left
    to the reader: ``parts`` holds ``[tokens * slots, hidden]``, a token's slots one after the
    other.  A part that says ``accepts_slot_sum`` takes it in place of ``[tokens, hidden]`` and adds
    the slots up while it reads (a norm does: one kernel and one pass over memory fewer per layer);
    a feed-forward is only asked for it when the part that reads its result accepts it."""

    def __init__(self, parts: torch.Tensor, slots: int):
        self.parts, self.slots = parts, int(slots)

    @property
    def shape(self):
        return (self.parts.shape[0] // self.slots, self.parts.shape[1])


class Part:
    """Base of mixers, feed-forwards, norms, position encodings and blocks."""
    kernel_libraries: tuple[str, ...] = ()

    def param_decls(self) -> dict[str, ParamDecl]:
        return {}

    def bind(self, params: dict[str, torch.Tensor]) -> None:
        self.params = params

    def finalize(self, kernels) -> None:
        """Once, after ``bind``: whatever the part does to its tensors for the kernels that will
        run it (a layout, a table).  The checkpoint's values are not there to be read back afterwards."""

    def children(self) -> dict[str, "Part"]:
        return {}

    def limit_positions(self, positions: int) -> None:
        """Before ``bind``: the engine will never ask for a position at or beyond ``positions``
        (parts with tables by position size them by this; the default hands it to the children)."""
        for child in self.children().values():
            child.limit_positions(positions)

    # flattened views over the tree of parts ---------------------------------------------
    def all_param_decls(self, prefix: str = "") -> dict[str, ParamDecl]:
        out = {prefix + name: decl for name, decl in self.param_decls().items()}
        for child_name, child in self.children().items():
            out.update(child.all_param_decls(f"{prefix}{child_name}."))
        return out

    def bind_all(self, tensors: dict[str, torch.Tensor], prefix: str = "") -> None:
        self.bind({name: tensors[prefix + name] for name in self.param_decls()})
        for child_name, child in self.children().items():
            child.bind_all(tensors, f"{prefix}{child_name}.")

    def finalize_all(self, kernels) -> None:
        self.finalize(kernels)
        for child in self.children().values():
            child.finalize_all(kernels)

    def all_kernel_libraries(self) -> set[str]:
        libs = set(self.kernel_libraries)
        for child in self.children().values():
            libs |= child.all_kernel_libraries()
        return libs


class PartRegistry:
    """kind -> factory(spec, **context).  One instance per family of parts."""

    def __init__(self, family: str, attribute: str = "kind"):
        self.family = family
        self.attribute = attribute      # the field of a spec that names its kind
        self._factories: dict[str, Callable] = {}

    def register(self, kind: str, factory: Callable | None = None):
        def add(f):
            self._factories[kind] = f
            return f
        return add(factory) if factory is not None else add

    def build(self, spec, **context):
        kind = getattr(spec, self.attribute, None)
        if kind not in self._factories:
            raise KeyError(f"no {self.family} registered for kind {kind!r}; known: "
                           f"{sorted(self._factories)}")
        return self._factories[kind](spec, **context)

    def kinds(self) -> list[str]:
        return sorted(self._factories)


MIXERS = PartRegistry("mixer")
FEED_FORWARDS = PartRegistry("feed-forward")
NORMS = PartRegistry("norm")
POSITIONS = PartRegistry("position encoding")
BLOCKS = PartRegistry("block", attribute="block")


@dataclass
class StepScratch:
    """Buffers a part asks for once and reuses every step, sized for the largest step."""
    tensors: dict[str, torch.Tensor] = field(default_factory=dict)
    views: dict[tuple, torch.Tensor] = field(default_factory=dict)     # (purpose, shape, dtype) -> the view handed out

    def get(self, key: str, shape: tuple[int, ...], dtype: torch.dtype, device) -> torch.Tensor:
        t = self.tensors.get(key)
        if t is None or t.dtype != dtype or t.shape[1:] != tuple(shape[1:]) or t.shape[0] < shape[0]:
            t = torch.empty(shape, dtype=dtype, device=device)
            self.tensors[key] = t
            self.views.clear()       # views of the buffer this one replaces must not be handed out again
        return t

    def view(self, key: str, shape: tuple[int, ...], dtype: torch.dtype, device) -> torch.Tensor:
        """The buffer for ``key`` and these trailing sizes, its leading dim cut to ``shape[0]``.  A step
        asks for the same few dozen views layer after layer and step after step; they are kept."""
        at = (key, shape, dtype)
        v = self.views.get(at)
        if v is None:
            shape = tuple(int(s) for s in shape)
            full = self.get(f"{key}{shape[1:]}", shape, dtype, device)
            # one buffer per (purpose, row shape): only the leading dim is ever cut, so views stay dense
            v = full if full.shape[0] == shape[0] else full.narrow(0, 0, shape[0])
            self.views[at] = v
        return v
