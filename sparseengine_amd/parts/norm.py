"""RMS normalisation: ``y = z * rsqrt(mean(z^2) + eps) * w`` with the statistic in float.

Reference: layers/layernorm.py:120-159 and kernels/triton/rmsnorm.py:17-66 (the fused form adds
the residual in float, stores the rounded sum as the new residual and norms the unrounded sum).
"""
from __future__ import annotations

from ..config.specs import NormSpec
from .base import NORMS, ParamDecl, Part, SlotSum


class RMSNorm(Part):
    kernel_libraries = ("norm",)

    def __init__(self, spec: NormSpec, hidden_size: int):
        self.eps = float(spec.eps)
        self.hidden_size = int(hidden_size)

    def param_decls(self):
        return {"weight": ParamDecl((self.hidden_size,))}

    accepts_slot_sum = True     # ``x`` may be a ``SlotSum``: the slots are added up as they are read

    def forward(self, fb, x, out=None, residual=None):
        """``out = norm(x (+ residual))``; the residual, if given, becomes ``x + residual``.
        Returns ``out`` (``x`` itself unless ``out`` is given or ``x`` is a ``SlotSum``)."""
        if isinstance(x, SlotSum):
            out = fb.buffer("norm.of_slots", x.shape) if out is None else out
            fb.kernels.rms_norm(x.parts, self.params["weight"], self.eps, out, residual=residual, slots=x.slots)
            return out
        out = x if out is None else out
        fb.kernels.rms_norm(x, self.params["weight"], self.eps, out, residual=residual)
        return out

    def forward_rows(self, fb, x, residual, rows, out):
        """Norm of ``x[rows] (+ residual[rows])`` into ``out``; nothing else is written."""
        if isinstance(x, SlotSum):
            fb.kernels.rms_norm(x.parts, self.params["weight"], self.eps, out, residual=residual, rows=rows,
                                slots=x.slots)
            return out
        fb.kernels.rms_norm(x, self.params["weight"], self.eps, out, residual=residual, rows=rows)
        return out


NORMS.register("rms", lambda spec, hidden_size: RMSNorm(spec, hidden_size))
