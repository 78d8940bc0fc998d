"""A decoder put together from a ``ModelSpec``: embedding, the layers in schedule order, final
norm and output head.  It knows parts and specs only, no architecture.

The step returns logits only for the wanted token places: the final norm and the head run on
those rows alone (the reference keeps the last row of every request, layers/embed_head.py:75-84).
"""
from __future__ import annotations

import torch

from ..config.specs import ModelSpec
from .base import BLOCKS, NORMS, ParamDecl, Part, SlotSum
from .linear import linear, prepare


class Embedding(Part):
    kernel_libraries = ("norm",)

    def __init__(self, vocab_size: int, hidden_size: int):
        self.vocab_size, self.hidden_size = vocab_size, hidden_size

    def param_decls(self):
        return {"weight": ParamDecl((self.vocab_size, self.hidden_size))}


class OutputHead(Part):
    def __init__(self, vocab_size: int, hidden_size: int):
        self.vocab_size, self.hidden_size = vocab_size, hidden_size

    def param_decls(self):
        return {"weight": ParamDecl((self.vocab_size, self.hidden_size))}


class DecoderModel(Part):
    def __init__(self, spec: ModelSpec, chunk_tokens: int = 16384):
        self.spec = spec
        self.embed = Embedding(spec.vocab_size, spec.hidden_size)
        self.layers = [BLOCKS.build(layer, hidden_size=spec.hidden_size, chunk_tokens=chunk_tokens)
                       for layer in spec.layers]
        self.final_norm = NORMS.build(spec.final_norm, hidden_size=spec.hidden_size)
        self.head = None if spec.tie_word_embeddings else OutputHead(spec.vocab_size, spec.hidden_size)
        self._prepared_head = None

    def finalize(self, kernels) -> None:
        self._prepared_head = prepare(kernels, (self.head or self.embed).params["weight"])

    def children(self):
        parts = {"embed": self.embed, "final_norm": self.final_norm}
        parts.update({f"layers.{i}": layer for i, layer in enumerate(self.layers)})
        if self.head is not None:
            parts["head"] = self.head
        return parts

    def cache_requests(self) -> dict[int, object]:
        """schedule position -> what its mixer keeps (positions reading another cache: nothing)."""
        out = {}
        for position, entry in enumerate(self.spec.schedule):
            if entry.cache_from is None:
                request = self.layers[entry.layer].cache_request()
                if request is not None:
                    out[position] = request
        return out

    # The two ends of the model are methods of their own, so that an architecture whose ends differ (an
    # embedding multiplier, a scale or a cap on the logits) brings a subclass that overrides them
    # (``Architecture.model_factory``) and leaves the run of the schedule alone.
    def embed_tokens(self, fb) -> torch.Tensor:
        """``[T, hidden]``: what the first layer reads."""
        x = fb.buffer("model.hidden", (fb.num_tokens, self.spec.hidden_size))
        fb.kernels.embedding(fb.token_ids, self.embed.params["weight"], x)
        return x

    def logits_of(self, fb, last: torch.Tensor) -> torch.Tensor:
        """Logits ``[wanted, vocab]`` (any float type) of the final-normed rows ``last [wanted, hidden]``."""
        weight = (self.head or self.embed).params["weight"]
        return linear(last, weight, out=fb.buffer("model.logits", (last.shape[0], self.spec.vocab_size)),
                      kernels=fb.kernels, prepared=self._prepared_head)

    def forward(self, fb) -> torch.Tensor:
        """float32 logits ``[wanted, vocab]`` of the step."""
        spec = self.spec
        x = self.embed_tokens(fb)
        residual = None
        final = len(spec.schedule) - 1
        for position, entry in enumerate(spec.schedule):
            own = entry.cache_from is None
            layer = self.layers[entry.layer]
            fb.schedule_position = position
            # the sum over a token's expert slots may be left to whoever reads the layer's result:
            # the next layer's first norm, or the final norm
            reader = self.final_norm if position == final else self.layers[spec.schedule[position + 1].layer]
            if getattr(layer, "can_defer_slot_sum", False) and getattr(reader, "accepts_slot_sum", False):
                x, residual = layer.forward(fb, x, residual, position if own else entry.cache_from, own,
                                            defer_slot_sum=True)
            else:
                x, residual = layer.forward(fb, x, residual, position if own else entry.cache_from, own)
            if fb.taps is not None:
                fb.taps.setdefault("layer_out", []).append(_stream_value(x, residual))
        wanted = fb.want_index.numel()
        if wanted == 0:
            return torch.empty(0, spec.vocab_size, dtype=torch.float32, device=fb.device)
        last = fb.buffer("model.wanted", (wanted, spec.hidden_size))
        self.final_norm.forward_rows(fb, x, residual, fb.want_index, last)
        return self.logits_of(fb, last).to(torch.float32, copy=True)      # the caller's own tensor, not the scratch buffer


def _stream_value(x, residual) -> torch.Tensor:
    """The residual stream after a layer, in float, for a tap: ``x + residual``, where ``x`` may still be
    a token's slots waiting to be added up by the next norm (rounded to the storage type first, as that
    norm does)."""
    if isinstance(x, SlotSum):
        tokens, hidden = x.shape
        x = x.parts.view(tokens, x.slots, hidden).float().sum(1).to(x.parts.dtype)
    return x.float() + residual.float()


def build_model(spec: ModelSpec, chunk_tokens: int = 16384) -> DecoderModel:
    return DecoderModel(spec, chunk_tokens)
