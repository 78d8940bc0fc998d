"""Dense projections.  Plain matrix products go to the GPU BLAS library through the tensor
library, as the reference's do (layers/linear.py:174-191); everything fused lives in csrc/."""
from __future__ import annotations

import torch


def linear(x: torch.Tensor, weight: torch.Tensor, out: torch.Tensor | None = None, kernels=None,
           prepared=None) -> torch.Tensor:
    """``x @ weight.T``.  A weight kept in float32 under a bfloat16 engine is multiplied in
    float32 and the product rounded to the activations' dtype.  ``kernels`` may offer its own
    ``linear`` for shapes the BLAS library serves badly (a few rows against a large matrix);
    ``prepared`` is what its ``prepare_dense_weight`` made of ``weight`` when the model was built
    (``prepare``), if anything."""
    if weight.dtype == x.dtype:
        if out is None:
            return torch.mm(x, weight.t())
        fast = getattr(kernels, "linear", None)
        if fast is not None:
            return fast(x, weight, out) if prepared is None else fast(x, weight, out, prepared=prepared)
        return torch.mm(x, weight.t(), out=out)
    y = torch.mm(x.to(weight.dtype), weight.t())
    if out is None:
        return y.to(x.dtype)
    out.copy_(y)
    return out


def prepare(kernels, weight: torch.Tensor):
    """Once per weight, when the model is built: whatever the kernels object wants to keep beside the
    matrix for its own ``linear`` (a copy in another layout), or None."""
    make = getattr(kernels, "prepare_dense_weight", None)
    return None if make is None else make(weight)
