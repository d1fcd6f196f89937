"""RMSNorm that owns the residual update.

Formula (reference ``src/rmsnorm.py:20-28``): in float32, ``y = x * rsqrt(mean(x^2) + eps) * w``,
one rounding at the store.  The reference adds the residual in the model dtype
before the norm (``src/decoder_layer.py:49,54``); here the residual stream is a
float32 tensor and the add is fused into the norm kernel, so the sum is exact
in 32-bit in both run dtypes.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import DeferredNorm, Norm, Param, register_part, single


class RMSNorm(Norm):
    def __init__(self, prefix: str, hidden_size: int, eps: float) -> None:
        super().__init__(prefix)
        self.hidden_size = int(hidden_size)
        self.eps = float(eps)
        self.weight: Optional[torch.Tensor] = None

    def params(self) -> Dict[str, Param]:
        return {"weight": single("weight", (self.hidden_size,), role="vector", init="one_plus_normal")}

    def deferred_form(self):
        return self.weight, self.eps

    def forward(self, residual, delta, ctx, rows=None):
        if isinstance(delta, DeferredNorm):
            # the product before this norm has added itself to the residual and applied the weight; the rest of the
            # norm is a row scale in whatever multiplies next
            if delta.norm is not self or rows is not None:
                raise ValueError("a DeferredNorm can only go to the norm it was made for, on all rows")
            return delta
        if rows is None:
            return ctx.ops.add_rmsnorm(residual, delta, self.weight, self.eps, ctx.dtype)
        return ctx.ops.add_rmsnorm_rows(residual, delta, rows, self.weight, self.eps, ctx.dtype)


register_part("norm", "rmsnorm", RMSNorm)
