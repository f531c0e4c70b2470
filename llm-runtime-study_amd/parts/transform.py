"""Parts of the role "transform": they work in place on float32 rows, the residual stream right after the embedding or
the logits (see parts/base.py)."""

from __future__ import annotations

from ..kernels import ops
from .base import Part, register


class SoftCap(Part):
    """x = cap * tanh(x / cap): keeps every value within (-cap, cap), close to the identity for small ones."""

    graph_safe = True
    plan_safe = True

    def __init__(self, cap: float):
        if not cap > 0:
            raise ValueError(f"cap must be positive, got {cap}")
        self.cap = float(cap)

    def flops(self, tokens, pairs):
        return 0.0

    def forward(self, ctx, x):
        ops.soft_cap(x, self.cap)


register("transform", "soft_cap", SoftCap)
