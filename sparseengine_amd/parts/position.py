"""Position encodings.  A position part owns its table and says how a head is rotated; the
attention mixer hands table and sizes to the fused kernel.

Rotary: ``theta_d = base^(-2d/R)`` for ``d in [0, R/2)``, table ``[max_position, R]`` = cos half then
sin half in float32, built on the host exactly as the reference does
(layers/rotary_embedding.py:15-24,217-222); scaled variants follow :26-101.
"""
from __future__ import annotations

import math
import weakref

import torch

from ..config.specs import RotarySpec
from .base import POSITIONS, FusedRotation, Part


def rotary_inverse_frequencies(rotary_dim: int, theta: float, scaling: dict | None):
    """(inv_freq float32 [R/2], factor that multiplies cos and sin)."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim))
    if not scaling:
        return inv_freq, 1.0
    kind = str(scaling.get("rope_type", scaling.get("type", "default"))).lower()
    if kind == "default":
        return inv_freq, 1.0
    factor = float(scaling["factor"])
    if kind == "linear":
        return inv_freq / factor, 1.0
    if kind == "llama3":
        # long wavelengths are slowed by `factor`, short ones kept, the band between blended
        original = float(scaling["original_max_position_embeddings"])
        low, high = float(scaling["low_freq_factor"]), float(scaling["high_freq_factor"])
        wavelength = 2 * math.pi / inv_freq
        slowed = torch.where(wavelength > original / low, inv_freq / factor, inv_freq)
        blend = (original / wavelength - low) / (high - low)
        blended = (1 - blend) * slowed / factor + blend * slowed
        in_band = (wavelength >= original / high) & (wavelength <= original / low)
        return torch.where(in_band, blended, slowed), 1.0
    if kind == "yarn":
        original = float(scaling["original_max_position_embeddings"])
        beta_fast, beta_slow = float(scaling.get("beta_fast", 32.0)), float(scaling.get("beta_slow", 1.0))

        def dim_of_rotations(rotations: float) -> float:
            return rotary_dim * math.log(original / (rotations * 2 * math.pi)) / (2 * math.log(theta))

        low, high = dim_of_rotations(beta_fast), dim_of_rotations(beta_slow)
        if bool(scaling.get("truncate", True)):
            low, high = math.floor(low), math.ceil(high)
        low, high = max(low, 0), min(high, rotary_dim - 1)
        if low == high:
            high += 0.001
        ramp = torch.clamp((torch.arange(rotary_dim // 2, dtype=torch.float32) - low) / (high - low), 0, 1)
        inv = inv_freq / factor * ramp + inv_freq * (1 - ramp)

        def mscale(f: float, multiplier: float = 1.0) -> float:
            return 1.0 if f <= 1.0 else 0.1 * multiplier * math.log(f) + 1.0

        attention = scaling.get("attention_factor")
        if attention is None:
            m, m_all = scaling.get("mscale"), scaling.get("mscale_all_dim")
            attention = mscale(factor, float(m)) / mscale(factor, float(m_all)) if m and m_all else mscale(factor)
        return inv, float(attention)
    raise NotImplementedError(f"rope scaling type {kind!r} is not supported "
                              "(default, linear, llama3, yarn)")


# Tables by (spec, rows, device): layers with the same rotation share one tensor (a 62-layer model
# with 204800 positions would hold 62 copies of the same 52 MB otherwise).  Entries go when the last
# part that uses them goes.
_SHARED_TABLES: "weakref.WeakValueDictionary" = weakref.WeakValueDictionary()


def shared_table(key, build):
    """The table stored under ``key``, built by ``build()`` if nobody holds it yet."""
    table = _SHARED_TABLES.get(key)
    if table is None:
        table = build()
        _SHARED_TABLES[key] = table
    return table


class RotaryPosition(Part):
    """Rotation of the leading ``rotary_dim`` dims of each head; ``pairing`` "neox" turns dims
    ``(d, d + R/2)`` together, "interleaved" dims ``(2 j, 2 j + 1)``; pair ``j`` by ``p * inv_freq[j]``."""
    PAIRINGS = ("neox", "interleaved")

    def __init__(self, spec: RotarySpec, head_dim: int):
        if spec.rotary_dim % 2 or not 0 < spec.rotary_dim <= head_dim:
            raise ValueError(f"rotary_dim must be even and in (0, head_dim={head_dim}], got {spec.rotary_dim}")
        if spec.pairing not in self.PAIRINGS:
            raise NotImplementedError(f"rotary pairing {spec.pairing!r} is not supported ({', '.join(self.PAIRINGS)})")
        if spec.max_position <= 0:
            raise ValueError("a rotary encoding needs max_position > 0")
        self.spec = spec
        self.rotary_dim = spec.rotary_dim
        self.pairing = spec.pairing
        self.rows = spec.max_position
        self.table = None

    def limit_positions(self, positions: int) -> None:
        """No position at or beyond ``positions`` will be asked for: the table need not hold more rows."""
        self.rows = max(1, min(self.spec.max_position, int(positions)))

    def prepare(self, device) -> None:
        spec, rows = self.spec, self.rows

        def build():
            inv_freq, factor = rotary_inverse_frequencies(spec.rotary_dim, spec.theta,
                                                          dict(spec.scaling) if spec.scaling else None)
            angles = torch.arange(rows, dtype=torch.float32)[:, None] * inv_freq[None, :]
            return torch.cat((angles.cos() * factor, angles.sin() * factor), dim=-1).contiguous().to(device)
        self.table = shared_table((spec, rows, str(torch.device(device))), build)

    def fused_rotation(self) -> FusedRotation:
        """A rotation by a table: the mixer's fused kernel applies it between the QK norm and the cache write."""
        return FusedRotation(self.table, self.rotary_dim, self.pairing)


class NoPosition(Part):
    rotary_dim = 0
    pairing = "neox"
    table = None

    def __init__(self, spec=None, head_dim: int = 0):
        pass

    def fused_rotation(self) -> FusedRotation:
        return FusedRotation(None, 0)

    def prepare(self, device) -> None:
        pass

    def limit_positions(self, positions: int) -> None:
        pass


POSITIONS.register("rotary", lambda spec, head_dim: RotaryPosition(spec, head_dim))
POSITIONS.register("none", lambda spec, head_dim: NoPosition(spec, head_dim))
