"""A recurrent block whose state is one number a channel, decayed and fed under real gates."""

from __future__ import annotations

from typing import Optional

import torch

from ..cache.pages import StateSpec
from ..errors import Unsupported
from ..kernels import ops
from .base import StepContext, settled
from .linear import linear
from .registry import register_mixer


class GatedRecurrence:
    """[y | x] = W h + b, one product left in 32 bits; u = conv(x) + bias over the request's own rows in time; in `blocks` equal
    parts of the channels r = sigmoid(Ra u + ba) and i = sigmoid(Ri u + bi); a = exp(-rate * r * softplus(lam));
    S <- a S + sqrt(1 - a^2) i u from S = 0; the output projection of S * gelu_tanh(y). A request's slot holds S [inner] and
    behind it the last taps - 1 rows of x before the convolution (position p at ring place p % (taps - 1)), all 32-bit.
    The two gates of a part are one product a part ([Ra; Ri] stacked, `ops.heads_product`). With bfloat16 matrices it runs on
    the matrix cores, and u enters it as two bfloat16 numbers a value, u = hi + lo, against the matrices twice side by side:
    [W W] [hi; lo] = W u to 16 bits of u, because a decay is multiplied by itself over hundreds of tokens and u rounded to one
    bfloat16 would move it. The gates' sums, the decay, the recurrence and the two branches' meeting are 32-bit; the rows
    the output projection reads are rounded once."""

    replayable = True
    takes_padding_rows = True  # (the convolution writes nothing a request reads for them, the recurrence walks the requests' own rows)

    def __init__(self, spec, store, dtype: torch.dtype):
        self.dtype = dtype
        self.width, self.inner, self.blocks, self.taps, self.rate = spec.width, spec.inner, int(spec.blocks), int(spec.taps), float(spec.rate)
        W, B, d = self.inner, self.blocks, self.width
        if W % B or self.taps < 1:
            raise ValueError(f"gated recurrence: {W} channels in {B} parts, {self.taps} taps")
        if self.taps > ops.CONV_MAX_TAPS:
            raise Unsupported(f"gated recurrence: a convolution of {self.taps} taps is not supported (up to {ops.CONV_MAX_TAPS})")
        t = spec.tensors
        self.in_weight = store.fetch_joined([t["y"], t["x"]], [(W, d)] * 2, "matrix", "rows")
        self.in_bias = store.fetch_joined([t["y_bias"], t["x_bias"]], [(W,)] * 2, "vector", "rows")
        self.conv = store.fetch(t["conv"], (W, self.taps), "vector")
        self.conv_bias = store.fetch(t["conv_bias"], (W,), "vector")
        per = W // B
        gr = store.fetch(t["gate_r"], (B, per, per), "matrix")
        gi = store.fetch(t["gate_i"], (B, per, per), "matrix")
        # both gates of a part as one matrix [2 per, per]; in bfloat16 twice side by side [2 per, 2 per], for u as [hi | lo]
        self.split = dtype == torch.bfloat16
        if self.split:
            self.gates = store.derived(("gates_twice", t["gate_r"].name, t["gate_i"].name), lambda: torch.cat([torch.cat([gr, gr], dim=2), torch.cat([gi, gi], dim=2)], dim=1).contiguous())
        else:
            self.gates = store.derived(("gates_stacked", t["gate_r"].name, t["gate_i"].name), lambda: torch.cat([gr, gi], dim=1).contiguous())
        self.gate_r_bias = store.fetch(t["gate_r_bias"], (B, per), "vector").reshape(W)
        self.gate_i_bias = store.fetch(t["gate_i_bias"], (B, per), "vector").reshape(W)
        self.lam = store.fetch(t["lam"], (W,), "vector")
        self.out_weight = store.fetch(t["out"], (d, W), "matrix")

    def cache_spec(self):
        return None

    def state_spec(self) -> Optional[StateSpec]:
        return StateSpec((self.inner * self.taps,))  # S, then the ring of taps - 1 rows

    can_scale_output = True  # forward(..., out_scale=, add=)

    def forward(self, h, ctx: StepContext, cache, state, residual: Optional[torch.Tensor], writes_cache: bool = True,
                out: Optional[torch.Tensor] = None, proj: Optional[torch.Tensor] = None, out_scale: float = 1.0, add: bool = False):
        """`proj`: the input projection's 32-bit rows (biases added, `in_bias`), when the caller has made them. `out_scale`: a
        factor on the result (taken where the recurrence meets its other branch, before those rows are rounded); `add`: the
        result is added to what `out` holds."""
        if not writes_cache:
            raise Unsupported("gated recurrence: a run that leaves the state as it found it is not supported")
        n, ws, W = h.shape[0], ctx.workspace, self.inner
        if proj is None:
            proj = ws.get("lru_in", (n, 2 * W), torch.float32)
            linear(h, self.in_weight, self.in_bias, out=proj)
        x = proj[:, W:]
        u = ws.get("lru_u", (n, W), torch.float32)
        halves = ws.get("lru_u_halves", (n, 2 * W), torch.bfloat16) if self.split else None
        ops.lru_conv(u, x, self.conv, self.conv_bias, state, W, ctx, blocks=self.blocks, split=halves)
        z = ws.get("lru_gates", (n, 2 * W), torch.float32)
        ops.heads_product(z, halves if self.split else u, self.gates)
        y = ws.get("lru_out", (n, W), self.dtype)
        # (the walk also keeps the step's last rows of x in the slot's ring: the convolution, which reads the ring, has run)
        ops.lru_scan(y, z, u, proj[:, :W], x, self.gate_r_bias, self.gate_i_bias, self.lam, self.rate, state, self.taps, ctx, self.blocks,
                     out_scale=out_scale)
        if out is not None and add:
            linear(y, self.out_weight, None, residual=out)
        elif out is not None:
            linear(y, self.out_weight, None, out=out)
        else:
            linear(y, self.out_weight, None, residual=settled(residual))
        return None


register_mixer("gated_recurrence", GatedRecurrence)
