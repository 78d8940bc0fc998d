"""Arrangement of a mixer and a feed-forward in one layer.

"prenorm" is the reference's residual wiring (models/minimax_m2.py:381-397, models/qwen3.py:291-325):
the stream is carried as a pair (x, residual); every norm first adds x into the residual and then
norms the sum, so a layer's feed-forward output is added by the *next* norm:

    first layer:  residual = x;            u = norm_in(x)
    later:        residual = x + residual; u = norm_in(residual)
    a = mixer(u); residual = a + residual; m = norm_post(residual); x = feed_forward(m)
"""
from __future__ import annotations

from ..config.specs import LayerSpec
from .base import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, Part


class PreNormBlock(Part):
    def __init__(self, spec: LayerSpec, hidden_size: int, chunk_tokens: int = 16384):
        self.norm_mixer = NORMS.build(spec.norm, hidden_size=hidden_size)
        self.mixer = MIXERS.build(spec.mixer, hidden_size=hidden_size)
        self.norm_ffn = NORMS.build(spec.norm, hidden_size=hidden_size)
        self.ffn = FEED_FORWARDS.build(spec.feed_forward, hidden_size=hidden_size, chunk_tokens=chunk_tokens)

    def children(self):
        return {"norm_mixer": self.norm_mixer, "mixer": self.mixer, "norm_ffn": self.norm_ffn, "ffn": self.ffn}

    def cache_request(self):
        request = getattr(self.mixer, "cache_request", None)
        return request() if request else None

    @property
    def accepts_slot_sum(self) -> bool:
        """Whether ``x`` may come as a ``SlotSum`` (the first norm adds the slots up as it reads)."""
        return bool(getattr(self.norm_mixer, "accepts_slot_sum", False))

    @property
    def can_defer_slot_sum(self) -> bool:
        return bool(getattr(self.ffn, "can_defer_slot_sum", False))

    def forward(self, fb, x, residual, cache_position: int, write_cache: bool, defer_slot_sum: bool = False):
        """``x`` is consumed (normed in place); returns the new pair (x, residual).
        ``defer_slot_sum``: whoever reads the returned ``x`` accepts a ``SlotSum``."""
        if residual is None:
            residual = fb.buffer("block.residual", x.shape)
            residual.copy_(x)
            self.norm_mixer.forward(fb, x)
        else:
            x = self.norm_mixer.forward(fb, x, residual=residual)
        mixed = self.mixer.forward(fb, x, cache_position, write_cache)
        self.norm_ffn.forward(fb, mixed, residual=residual)
        if defer_slot_sum and self.can_defer_slot_sum:
            return self.ffn.forward(fb, mixed, defer_slot_sum=True), residual
        return self.ffn.forward(fb, mixed), residual


BLOCKS.register("prenorm", lambda spec, hidden_size, chunk_tokens=16384: PreNormBlock(spec, hidden_size, chunk_tokens))
