"""What happens to the stream where a repeated stretch of layers begins a pass."""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import StepContext
from .linear import linear
from .registry import register_entry


class Reentry:
    """x <- W [x ; x0] + steps[index] ahead of a layer: x0 is the embedding's output, W [width, 2 width] (the stream's half first),
    `steps` one row a pass. Two products of the rounded rows, W_x x with the pass's row as its bias and W_0 x0 added onto it; the
    sums are 32-bit and land in the stream's own tensor."""

    takes_padding_rows = True
    needs_embedding = True  # the model keeps the embedding's output for `forward`

    def __init__(self, spec, store, dtype: torch.dtype):
        self.dtype, self.width, self.index = dtype, spec.width, int(spec.index)
        d, t = self.width, spec.tensors
        whole = store.fetch(t["weight"], (d, 2 * d), "matrix")
        self.w_stream = store.derived(("columns", t["weight"].name, 0, d), lambda: whole[:, :d].contiguous())
        self.w_embed = store.derived(("columns", t["weight"].name, d, 2 * d), lambda: whole[:, d:].contiguous())
        steps = store.fetch(t["steps"], (int(spec.passes), d), "vector")
        if not 0 <= self.index < int(spec.passes):
            raise ValueError(f"pass {self.index} of {spec.passes}")
        self.step = steps[self.index]

    def forward(self, x: torch.Tensor, embedded: torch.Tensor, ctx: StepContext) -> None:
        """x: the stream, float32 [n, width], rewritten in place; embedded: the embedding's output rounded to the compute dtype."""
        xs = ctx.workspace.get("reentry_stream", tuple(x.shape), self.dtype)
        ops.gather_rows(xs, x)
        linear(xs, self.w_stream, self.step, out=x)
        linear(embedded, self.w_embed, None, residual=x)


register_entry("reentry", Reentry)
