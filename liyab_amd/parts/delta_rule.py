"""A mixer that carries a matrix of state a head, decays it and takes out of it what the token's key already holds."""

from __future__ import annotations

from typing import Optional

import torch

from ..cache.pages import StateSpec
from ..errors import Unsupported
from ..kernels import ops
from .base import StepContext, settled
from .linear import linear
from .norms import as_tensor
from .registry import register_mixer


def own_state(state, floats: int):
    """A part's stretch of its layer's per-request state: the stretch a block handed over, or, from a block that hands the
    layer's whole state to its mixer, all of it."""
    if isinstance(state, ops.StateSlice):
        return state
    return ops.StateSlice(state, 0, floats)


class DeltaRule:
    """r, k, v = W h a head; a decay w = exp(-decay_scale * sigmoid(W2 tanh(W1 h) + w0)) and a removal rate a = sigmoid(Wa h + ba) a
    head and key channel; with the unit key u = k / sqrt(sum(k^2) + key_eps): S <- diag(w) S - (a * u)(u^T S) + k v^T, both terms
    reading the old S, and o = S^T r; each head's o brought to unit root mean square, times a weight and sigmoid(Wg h), then the
    output projection. The six projections of h run as one product whose 32-bit sums feed the recurrence unrounded; decays, rates,
    unit keys and the state are 32-bit. A request's slot holds the heads' matrices [heads, key, value]."""

    replayable = True
    takes_padding_rows = True  # (the recurrence walks the requests' own rows; rows behind them are computed by the products only)

    def __init__(self, spec, store, dtype: torch.dtype):
        self.dtype = dtype
        self.width, self.n_head, self.head_dim, self.rank, self.eps = spec.width, spec.n_head, spec.head_dim, spec.decay_rank, float(spec.eps)
        self.decay_scale, self.key_eps = float(spec.decay_scale), float(spec.key_eps)
        H, D, d, R = self.n_head, self.head_dim, self.width, self.rank
        if not ops.delta_takes(D):
            raise Unsupported(f"delta rule: heads of {D} are not supported")
        t = spec.tensors
        # [r | k | v | removal | gate | the decay's first, narrow product] of one input
        self.in_weight = store.fetch_joined([t[c] for c in ("r", "k", "v", "a", "g", "w1")], [(H * D, d)] * 5 + [(R, d)], "matrix", "rows")
        self.w2 = store.fetch(t["w2"], (H * D, R), "matrix")
        self.w0 = store.fetch(t["w0"], (H * D,), "vector")
        self.a_bias = store.fetch(t["a_bias"], (H * D,), "vector")
        self.norm = store.fetch(t["norm"], (H * D,), "vector")
        self.out_weight = store.fetch(t["out"], (d, H * D), "matrix")

    def cache_spec(self):
        return None

    def state_spec(self) -> Optional[StateSpec]:
        return StateSpec((self.n_head * self.head_dim * self.head_dim,))

    def forward(self, h, ctx: StepContext, cache, state, residual: Optional[torch.Tensor], writes_cache: bool = True,
                out: Optional[torch.Tensor] = None):
        h = as_tensor(h)
        n, ws, HD, R = h.shape[0], ctx.workspace, self.n_head * self.head_dim, self.rank
        proj = ws.get("delta_in", (n, 5 * HD + R), torch.float32)
        linear(h, self.in_weight, None, out=proj)
        low = ws.get("delta_low", (n, R), self.dtype)
        ops.activate(low, proj[:, 5 * HD:], "tanh")
        wraw = ws.get("delta_decay", (n, HD), torch.float32)
        linear(low, self.w2, None, out=wraw)
        y = ws.get("delta_out", (n, HD), self.dtype)
        ops.delta_rule(y, proj, wraw, self.w0, self.a_bias, self.norm, self.eps, own_state(state, HD * self.head_dim), ctx,
                       n_head=self.n_head, head_dim=self.head_dim, decay_scale=self.decay_scale, key_eps=self.key_eps)
        if out is not None:
            linear(y, self.out_weight, None, out=out)
        else:
            linear(y, self.out_weight, None, residual=settled(residual))
        return None


register_mixer("delta_rule", DeltaRule)
