"""Dense gated feed-forward.

Reference ``src/mlp.py:9-15``: one fused product with rows ``[Wgate; Wup]`` (no bias),
``act(gate) * up``, down product (no bias); ``silu(x) = x * sigmoid(x)``.  The
activation and the product ``act(gate) * up`` are computed in float32 with one
rounding at the store; for decode-sized batches they are the epilogue of the
gate/up product itself, which then never writes its ``[T, 2I]`` result.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import FeedForward, Param, fused_rows, register_part, single


class GatedMLP(FeedForward):
    def __init__(self, prefix: str, hidden_size: int, intermediate_size: int, activation: str = "silu") -> None:
        super().__init__(prefix)
        if activation != "silu":
            raise ValueError(f"activation {activation!r} is not implemented (only 'silu')")
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.gate_up_weight: Optional[torch.Tensor] = None
        self.down_weight: Optional[torch.Tensor] = None

    def params(self) -> Dict[str, Param]:
        h, i = self.hidden_size, self.intermediate_size
        return {
            "gate_up_weight": fused_rows(("gate_proj.weight", "up_proj.weight"), ((i, h), (i, h))),
            "down_weight": single("down_proj.weight", (h, i)),
        }

    def prepare_kernels(self, ops) -> None:
        self.prepare_weight(ops, "gate_up_weight", stacked=2)
        self.prepare_weight(ops, "down_weight")

    accepts_sink = True  # its last product may add itself to the residual (ResidualSink)
    accepts_deferred = True  # its first product can read a DeferredNorm

    def forward(self, x, ctx, sink=None):
        ops = ctx.ops
        act = ops.linear_silu_mul(x, self.operand("gate_up_weight"), ctx.dtype)
        return ops.linear(act, self.operand("down_weight"), None, ctx.dtype, partials_ok=True, residual_norm=sink)


register_part("feed_forward", "gated_mlp", GatedMLP)
