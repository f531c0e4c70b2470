"""RMSNorm over the last dimension of the float32 residual stream.

Formula (reference mini_llm/nn/norm.py:42-46): y = w * x * rsqrt(mean(x^2) + eps), statistics
in float32.  The kernel rounds once, at the output, to the activation dtype.

`unit_offset`: the checkpoint stores the weight around zero and the norm multiplies by 1 + w; the sum is made
once, in float32, when the weights are bound, so every kernel sees a plain weight.

Besides `forward` (the norm of the stream, for a sublayer to read) a norm can be applied to what a sublayer gives
out: `add_normed(ctx, residual, y)` adds the norm of the float32 rows `y` into the stream, for layer arrangements
that normalise outputs (parts/block.py, OutputNormBlock).
"""

from __future__ import annotations

from ..kernels import ops
from .base import Part, TensorSpec, register
from .linear import LazyNorm


class RMSNorm(Part):
    graph_safe = True  # launches only library kernels on arena buffers
    plan_safe = True
    has_lazy_form = True

    def __init__(self, size: int, eps: float, unit_offset: bool = False):
        if size <= 0:
            raise ValueError(f"size must be positive, got {size}")
        if eps <= 0:
            raise ValueError(f"eps must be positive, got {eps}")
        self.size, self.eps, self.unit_offset = size, eps, unit_offset
        self.weight = None

    def tensors(self):
        return {"weight": TensorSpec((self.size,), role="bias" if self.unit_offset else "norm")}

    def bind(self, weights, dtype):
        self.weight = weights["weight"]
        if self.unit_offset:
            self.weight = (1.0 + self.weight.float()).contiguous()

    rounds_stream = True   # add_normed(..., rounded=buffer) also leaves the updated rows in bfloat16

    def add_normed(self, ctx, residual, y, rounded=None):
        """residual += this norm of the float32 rows y (what a sublayer gave out); rounded: a bfloat16 buffer that
        receives the updated rows as well, for the sublayer that reads the stream next."""
        ops.norm_add(residual, y, self.weight, self.eps, rounded)

    def rms_parameters(self):
        """(weight, eps): says that this norm is w * x * rsqrt(mean(x^2) + eps), so that the matrix
        product before it may begin it (see parts/linear.py)."""
        return self.weight, self.eps

    def forward(self, ctx, h, rows=None, count=None, lazy: bool = False):
        """Normalise rows of h [*, size] (all, or the `count` rows listed in `rows`).

        With `lazy` the work is left to the consumer's matrix product (see parts/linear.py)."""
        n = h.shape[0] if rows is None else count
        pending = LazyNorm(h, self.weight, self.eps, rows, n)
        return pending if lazy else pending.materialize(ctx)


register("norm", "rmsnorm", RMSNorm)


class LayerNorm(Part):
    """y = w * (x - mean) / sqrt(variance + eps) over the last dimension, the variance being the mean of the squared
    deviations; a weight and no bias.  Statistics in float32, one rounding at the output.

    Besides `forward` it serves layer arrangements that normalise the sum of the stream and a sublayer's output
    (parts/block.py, PostNormBlock): `scale_add_normed(ctx, residual, y, alpha)` replaces the stream by the norm of
    alpha * stream + y."""

    graph_safe = True
    plan_safe = True
    rounds_stream = True   # scale_add_normed(..., rounded=buffer) also leaves the new rows in bfloat16

    def __init__(self, size: int, eps: float):
        if size <= 0:
            raise ValueError(f"size must be positive, got {size}")
        if eps <= 0:
            raise ValueError(f"eps must be positive, got {eps}")
        self.size, self.eps = size, eps
        self.weight = None

    def tensors(self):
        return {"weight": TensorSpec((self.size,), role="norm")}

    def bind(self, weights, dtype):
        self.weight = weights["weight"]

    def layer_parameters(self):
        """(weight, eps): says that this norm is w * (x - mean) / sqrt(variance + eps), so that the kernel that makes a
        sublayer's output may apply it to the sum itself (a feed-forward that says `applies_sum_norm`)."""
        return self.weight, self.eps

    def scale_add_normed(self, ctx, residual, y, alpha: float, rounded=None):
        ops.scale_add_layernorm(residual, y, alpha, self.weight, self.eps, rounded)

    def forward(self, ctx, h, rows=None, count=None):
        n = h.shape[0] if rows is None else count
        out = ctx.scratch("norm_out", (n, h.shape[1]), ctx.dtype)
        ops.layernorm(out, h, self.weight, self.eps, rows=rows)
        return out


register("norm", "layernorm", LayerNorm)
