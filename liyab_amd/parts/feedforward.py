"""Feed-forward parts."""

from __future__ import annotations

from typing import Optional

import torch

from .base import StepContext, settled
from .linear import linear, linear_deferred
from .registry import register_ffn


class DenseFFN:
    """The ungated feed-forward: m = act(h . Wup^T + b_up) . Wdown^T + b_down,
    added into the residual (the reference's dense_ffn for FfnKind::Ungated,
    src/core/transformer.cpp:4903-4913; residual :5692). `activation` is
    "gelu_tanh" (:123-130) or "gelu_erf" (:134-142)."""

    # every launch goes through the kernel library and depends on nothing of this object but its
    # tensors and the constants among its attributes: layers of this kind may run from one recorded list
    replayable = True
    # rows behind the step's tokens (token 0 at position 0 of the first request, slot -1) are computed
    # and never read: nothing here writes for them or lets them touch another row
    takes_padding_rows = True

    def __init__(self, spec, store, dtype: torch.dtype):
        self.dtype = dtype
        self.width, self.inner, self.activation = spec.width, spec.inner, spec.activation
        if self.activation not in ("gelu_tanh", "gelu_erf"):
            raise ValueError(f"unknown activation '{self.activation}'")
        t = spec.tensors
        self.up_weight = store.fetch(t["up_weight"], (self.inner, self.width), "matrix")
        self.up_bias = store.fetch(t["up_bias"], (self.inner,), "vector") if "up_bias" in t else None
        self.down_weight = store.fetch(t["down_weight"], (self.width, self.inner), "matrix")
        self.down_bias = store.fetch(t["down_bias"], (self.width,), "vector") if "down_bias" in t else None

    defers = True  # forward(..., defer=True) takes the stream split or whole and may hand it back split

    def forward(self, h, ctx: StepContext, residual: torch.Tensor, defer: bool = False):
        """Adds the feed-forward's output into `residual`. With `defer`, `residual` may be a
        SplitStream, and where the second product runs faster cut over its inner dimension the
        stream with the output added comes back as a SplitStream (None: added in place, to
        the stream's own tensor)."""
        inner = ctx.workspace.get("ffn_inner", (h.shape[0], self.inner), self.dtype)
        linear(h, self.up_weight, self.up_bias, out=inner, activation=self.activation)
        split = linear_deferred(inner, self.down_weight, self.down_bias, ctx, "ffn_parts", residual) if defer else None
        if split is None:
            linear(inner, self.down_weight, self.down_bias, residual=settled(residual))
        return split


register_ffn("dense_ffn", DenseFFN)


class ClampedGLU:
    """down(g * sigmoid(slope * g) * (u + shift)) with g = min(Wg h, limit) and u = clamp(Wu h, -limit, limit): the two
    projections run as one product [gate | up] whose 32-bit sums the activation kernel reads, so that the clamps and the
    gate see unrounded values; the inner rows are rounded once, for the second product."""

    replayable = True
    takes_padding_rows = True

    def __init__(self, spec, store, dtype: torch.dtype):
        self.dtype = dtype
        self.width, self.inner = spec.width, spec.inner
        self.limit, self.slope, self.shift = float(spec.limit), float(spec.slope), float(spec.shift)
        if not self.limit > 0:
            raise ValueError(f"clamped feed-forward: a limit of {self.limit}")
        t = spec.tensors
        self.in_weight = store.fetch_joined([t["gate"], t["up"]], [(self.inner, self.width)] * 2, "matrix", "rows")
        self.down_weight = store.fetch(t["down"], (self.width, self.inner), "matrix")

    def begin(self, h, ctx: StepContext) -> torch.Tensor:
        """The first product, [gate | up] of h in 32 bits: everything of the feed-forward that reads its input. A block whose
        sublayers read one pending norm of the stream runs this before any sublayer adds into the stream."""
        gu = ctx.workspace.get("glu_in", (h.shape[0], 2 * self.inner), torch.float32)
        linear(h, self.in_weight, None, out=gu)
        return gu

    def finish(self, gu: torch.Tensor, ctx: StepContext, residual: Optional[torch.Tensor], out: Optional[torch.Tensor] = None):
        from ..kernels import ops

        inner = ctx.workspace.get("ffn_inner", (gu.shape[0], self.inner), self.dtype)
        ops.glu_clamped(inner, gu, self.limit, self.slope, self.shift)
        if out is not None:
            linear(inner, self.down_weight, None, out=out)
        else:
            linear(inner, self.down_weight, None, residual=settled(residual))
        return None

    def forward(self, h, ctx: StepContext, residual: Optional[torch.Tensor], out: Optional[torch.Tensor] = None):
        """Adds the result into `residual` (float32 [n, width]), or leaves it in `out`."""
        return self.finish(self.begin(h, ctx), ctx, residual, out=out)


register_ffn("clamped_glu", ClampedGLU)


class NormedPowersFFN:
    """down(c1 N(z) + c2 N(z^2) + c3 N(z^3) + c4) with z = up h, powers entry by entry and N(v) = v / sqrt(mean(v^2) + eps) over the
    inner width: the first product leaves its 32-bit sums, one kernel takes the three means of a row and mixes the powers, and the inner
    rows are rounded once, for the second product. The four weights stay on the device."""

    replayable = True
    takes_padding_rows = True

    def __init__(self, spec, store, dtype: torch.dtype):
        self.dtype = dtype
        self.width, self.inner, self.eps = spec.width, spec.inner, float(spec.eps)
        if int(spec.powers) != 3:
            raise ValueError(f"a mix of {spec.powers} powers (3 are taken)")
        t = spec.tensors
        self.up_weight = store.fetch(t["up"], (self.inner, self.width), "matrix")
        self.act = store.fetch(t["act"], (4,), "vector")
        self.down_weight = store.fetch(t["down"], (self.width, self.inner), "matrix")

    def begin(self, h, ctx: StepContext) -> torch.Tensor:
        """The first product in 32 bits: everything of the feed-forward that reads its input."""
        z = ctx.workspace.get("powers_in", (h.shape[0], self.inner), torch.float32)
        linear(h, self.up_weight, None, out=z)
        return z

    def finish(self, z: torch.Tensor, ctx: StepContext, residual: Optional[torch.Tensor], out: Optional[torch.Tensor] = None):
        from ..kernels import ops

        inner = ctx.workspace.get("ffn_inner", (z.shape[0], self.inner), self.dtype)
        ops.normed_powers(inner, z, self.act, self.eps)
        if out is not None:
            linear(inner, self.down_weight, None, out=out)
        else:
            linear(inner, self.down_weight, None, residual=settled(residual))
        return None

    def forward(self, h, ctx: StepContext, residual: Optional[torch.Tensor], out: Optional[torch.Tensor] = None):
        """Adds the result into `residual` (float32 [n, width]), or leaves it in `out`."""
        return self.finish(self.begin(h, ctx), ctx, residual, out=out)


register_ffn("normed_powers_ffn", NormedPowersFFN)
