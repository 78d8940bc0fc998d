"""Dense projections.  Plain matrix products go to the GPU BLAS library through the tensor
library, as the reference's do (layers/linear.py:174-191); everything fused lives in csrc/."""
from __future__ import annotations

import torch


def linear(x: torch.Tensor, weight: torch.Tensor, out: torch.Tensor | None = None, kernels=None) -> torch.Tensor:
    """``x @ weight.T``.  A weight kept in float32 under a bfloat16 engine is multiplied in
    float32 and the product rounded to the activations' dtype.  ``kernels`` may offer its own
    ``linear`` for shapes the BLAS library serves badly (a few rows against a large matrix)."""
    if weight.dtype == x.dtype:
        if out is None:
            return torch.mm(x, weight.t())
        fast = getattr(kernels, "linear", None)
        if fast is not None:
            return fast(x, weight, out)
        return torch.mm(x, weight.t(), out=out)
    y = torch.mm(x.to(weight.dtype), weight.t())
    if out is None:
        return y.to(x.dtype)
    out.copy_(y)
    return out
