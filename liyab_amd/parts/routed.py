"""A feed-forward that routes each token to a few of many experts."""

from __future__ import annotations

from typing import Optional

import torch

from ..errors import Unsupported
from ..kernels import ops
from .base import StepContext, settled
from .linear import linear
from .norms import as_tensor
from .registry import register_ffn


class RoutedFFN:
    """z = Wr h + b (32-bit sums, kept in 32 bits); a token takes the `top` experts with the largest z,
    weighted by the softmax over those logits alone; expert e gives Wdown_e (silu(Wgate_e h) * (Wup_e
    h)); the result is the weighted sum. The step's (token, choice) entries are listed by expert in
    tiles, and two grouped products run over the tiles: [gate | up] with the activation, then down
    with the router's weight; an entry's row is added to the others of its token by the reader.
    The spec's options: experts without a gate, Wdown_e act(Wup_e h), with act = the square of the positive part; the choice
    among groups of experts (scores by a softmax over all experts, the best groups only, weights divided by their sum:
    `ops.moe_route(groups=)`); one more expert of the same form that every token takes with weight one, whose result is one
    more row a token for the reader to add."""

    replayable = True
    takes_padding_rows = True  # (they are routed and computed like token 0; nobody reads them)

    def __init__(self, spec, store, dtype: torch.dtype):
        self.dtype = dtype
        self.width, self.inner, self.n_experts, self.top = spec.width, spec.inner, spec.n_experts, spec.top
        self.gated, self.activation = bool(getattr(spec, "gated", True)), spec.activation
        if (self.gated and self.activation != "silu") or (not self.gated and self.activation != "relu2"):
            raise ValueError(f"routed feed-forward: activation '{spec.activation}' of {'gated' if self.gated else 'ungated'} experts is not known")
        self.groups = tuple(int(v) for v in spec.groups) if getattr(spec, "groups", None) is not None else None
        self.shared_inner = int(getattr(spec, "shared_inner", 0) or 0)
        if not 1 <= self.top <= min(self.n_experts, ops.MOE_MAX_TOP):
            raise ValueError(f"routed feed-forward: {self.top} of {self.n_experts} experts a token (at most {ops.MOE_MAX_TOP})")
        t, E, F, d = spec.tensors, self.n_experts, self.inner, self.width
        self.router = store.fetch(t["router"], (E, d), "matrix")
        self.router_bias = store.fetch(t["router_bias"], (E,), "vector") if "router_bias" in t else None
        self.gate = store.fetch_joined([t[("gate", e)] for e in range(E)], [(F, d)] * E, "matrix", "stack") if self.gated else None
        self.up = store.fetch_joined([t[("up", e)] for e in range(E)], [(F, d)] * E, "matrix", "stack")
        self.down = store.fetch_joined([t[("down", e)] for e in range(E)], [(d, F)] * E, "matrix", "stack")
        self.shared_in = self.shared_down = self.joint_in = None
        if self.shared_inner:
            if self.gated:
                raise Unsupported("routed feed-forward: a shared expert beside gated experts is not supported")
            S = self.shared_inner
            names = ([t["shared_gate"]] if self.gated else []) + [t["shared_up"]]
            self.shared_in = store.fetch_joined(names, [(S, d)] * len(names), "matrix", "rows")
            self.shared_down = store.fetch(t["shared_down"], (d, S), "matrix")
            # the router and the shared expert's first product read the same rows: one product [router | shared]
            if self.router_bias is None and self.router.dtype == self.shared_in.dtype:
                rw, sw = self.router, self.shared_in
                self.joint_in = store.derived(("joined_rows", t["router"].name, t["shared_up"].name), lambda: torch.cat([rw, sw], dim=0).contiguous())

    def take_router(self):
        """(weight [experts, width], bias or None): the router's product handed to a caller that runs it as rows
        of a wider product over the same input and passes the logits to `forward(..., router_logits=)`; this
        part then no longer holds the matrix."""
        w, b = self.router, self.router_bias
        self.router = self.router_bias = self.joint_in = None
        return w, b

    rows_a_token = property(lambda self: self.top + (1 if self.shared_inner else 0))  # rows `forward(..., out=)` leaves for each token

    def forward(self, h, ctx: StepContext, residual: Optional[torch.Tensor], out: Optional[torch.Tensor] = None,
                router_logits: Optional[torch.Tensor] = None):
        """Adds the result into `residual`, or, with `out` (float32 [n * rows_a_token, width]), leaves each token's
        `top` weighted expert outputs (and the shared expert's behind them) there in consecutive rows, for a reader that adds them up.
        `router_logits` (float32 [n, experts], rows may be strided): the router's logits where the caller
        has computed them already, beside a product of its own over the same rows (`take_router`)."""
        h = as_tensor(h)
        n, ws, E, top = h.shape[0], ctx.workspace, self.n_experts, self.top
        logits, shared_pre = router_logits, None
        if logits is None and self.joint_in is not None:
            z = ws.get("router_shared", (n, self.joint_in.shape[0]), torch.float32)
            linear(h, self.joint_in, None, out=z)
            logits, shared_pre = z[:, :E], z[:, E:]
        if logits is None:
            logits = ws.get("router_logits", (n, E), torch.float32)
            linear(h, self.router, self.router_bias, out=logits)
        block = ops.moe_block(n * top, E, self.dtype, self.width, self.inner)
        tiles = ops.moe_tiles(n * top, E, block)
        ids = ws.get("routed_ids", (n * top,), torch.int32)
        weights = ws.get("routed_weights", (n * top,), torch.float32)
        rows_list = ws.get("routed_rows", (tiles * block,), torch.int32)
        tile_group = ws.get("routed_tiles", (tiles,), torch.int32)
        ops.moe_route(logits, top, ids, weights, rows_list, tile_group, block=block, groups=self.groups)
        inner = ws.get("routed_inner", (n * top, self.inner), self.dtype)
        if self.gated:
            ops.moe_product(inner, h, self.gate, self.up, rows_list, tile_group, a_div=top, block=block)
        else:
            ops.moe_product(inner, h, self.up, None, rows_list, tile_group, a_div=top, block=block, act=self.activation)
        rows = self.rows_a_token
        y = out if out is not None else ws.get("routed_out", (n * rows, self.width), torch.float32)
        # (the second product's rows are the entries: a_div = 1 for its operand, `top` for where a token's rows lie in y)
        ops.moe_product(y, inner, self.down, None, rows_list, tile_group, row_scale=weights, block=block, out_div=top, out_extra=rows - top)
        if self.shared_inner:
            S = self.shared_inner
            if shared_pre is None:
                shared_pre = ws.get("shared_in", (n, self.shared_in.shape[0]), torch.float32)
                linear(h, self.shared_in, None, out=shared_pre)
            act = ws.get("shared_inner", (n, S), self.dtype)
            ops.activate(act, shared_pre, self.activation)
            # the shared expert's row of each token, behind its `top` rows
            linear(act, self.shared_down, None, out=y.view(n, rows * self.width)[:, top * self.width:])
        if out is None:
            ops.gated_norm_add(settled(residual), y, None, 0.0, n_sum=rows, normalize=False)
        return None


register_ffn("routed_ffn", RoutedFFN)
