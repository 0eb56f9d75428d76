"""Attention over one compressed row a position."""

from __future__ import annotations

from typing import Optional

import torch

from ..cache.pages import KVSpec
from ..cache.storage import LayerCache
from ..errors import Unsupported
from ..kernels import ops
from .attention import AttentionStepPlanner
from .base import StepContext, settled
from .linear import linear
from .norms import as_tensor
from .registry import register_mixer


class LatentAttention:
    """q = Wq h (heads of `head_dim`); c = rmsnorm(Wdown h) * w, `rank` wide: the only thing cached, one row
    a position; per head k_j = Wuk c_j, v_j = Wuv c_j; score_ij = scale * q_i . k_j over the window's
    positions, ordinary softmax; the heads' outputs, side by side, times sigmoid(Wg h) when gated; then
    the output projection. No position enters.

    Keys and values are never made. Since q . (Wuk c) = (Wuk^T q) . c and sum_j p_j (Wuv c_j) = Wuv (sum_j
    p_j c_j), every head's query goes through its Wuk^T first (`rank` wide), attention runs with the
    cached rows as keys and as values of one shared head, which is what the paged attention kernels
    do for grouped queries, and the result goes through the head's Wuv. A step reads each cached row
    once for all heads. Scores, softmax and the norm of c are 32-bit; the three projections of h run as
    one product.

    Options of the spec: `q_rank` > 0, queries through a latent of their own, q = Wuq (rmsnorm(Wdq h) * w) (the
    narrow product is left in 32 bits for its norm); `gate_a_head`, a gate of one logit a head (its matrix's
    rows are repeated over the head's values once, at load, so that the gate stays an epilogue of Wuv's product)."""

    replayable = True
    takes_padding_rows = True  # (slot -1: no row of theirs is cached, and no other row attends to them)
    step_planner = AttentionStepPlanner()  # the same cut of a step's tokens as attention's: ctx.plans["attention"]

    def __init__(self, spec, store, dtype: torch.dtype):
        self.dtype = dtype
        self.width, self.n_head, self.head_dim = spec.width, spec.n_head, spec.head_dim
        self.value_dim, self.rank = spec.value_dim, spec.rank
        self.scale, self.window, self.eps = float(spec.scale), int(spec.window), float(spec.eps)
        self.gated = bool(spec.gated)
        if not ops.attention_takes(self.rank):
            raise Unsupported(f"latent attention: cached rows of {self.rank} are not supported (the attention kernels take up to "
                              f"{ops.ATTENTION_MAX_HEAD_DIM})")
        t = spec.tensors
        H, D, V, R, d = self.n_head, self.head_dim, self.value_dim, self.rank, self.width
        self.q_dim, self.v_dim = H * D, H * V
        self.q_rank = int(getattr(spec, "q_rank", 0) or 0)
        gate_a_head = bool(getattr(spec, "gate_a_head", False))
        if self.q_rank or gate_a_head:
            # [c | gate] of the input; the queries' latent is a product of its own, left in 32 bits for its norm
            self.q_down = store.fetch(t["q_down"], (self.q_rank, d), "matrix") if self.q_rank else None
            self.q_down_norm = store.fetch(t["q_down_norm"], (self.q_rank,), "vector") if self.q_rank and "q_down_norm" in t else None
            self.q_weight = store.fetch(t["q_up"] if self.q_rank else t["q"], (H * D, self.q_rank or d), "matrix")
            down = store.fetch(t["down"], (R, d), "matrix", keep=False)
            parts = [down]
            if self.gated:
                gate = store.fetch(t["gate"], (H if gate_a_head else H * V, d), "matrix", keep=False)
                parts.append(gate.repeat_interleave(V, dim=0) if gate_a_head else gate)
            self.in_weight = store.derived(("latent_in", t["down"].name, t["gate"].name if self.gated else None, V if gate_a_head else 0),
                                           lambda: torch.cat(parts, dim=0).contiguous())
            self.q_dim = 0  # (no queries among the joint product's columns)
        else:
            self.q_weight = None
            srcs, shapes = [t["q"], t["down"]], [(H * D, d), (R, d)]
            if self.gated:
                srcs.append(t["gate"])
                shapes.append((H * V, d))
            self.in_weight = store.fetch_joined(srcs, shapes, "matrix", "rows")  # [q | c | gate] of one input
        self.down_norm = store.fetch(t["down_norm"], (R,), "vector") if "down_norm" in t else None
        up_k = store.fetch(t["up_k"], (H * D, R), "matrix")
        # a head's Wuk^T, [rank, head_dim] with the head's dimensions contiguous: what multiplies its query
        self.up_k_t = store.derived(("heads_transposed", t["up_k"].name, H),
                                    lambda: up_k.view(H, D, R).transpose(1, 2).contiguous())
        self.up_v = store.fetch(t["up_v"], (H * V, R), "matrix").view(H, V, R)
        self.out_weight = store.fetch(t["out"], (d, H * V), "matrix")
        self.out_bias = store.fetch(t["out_bias"], (d,), "vector") if "out_bias" in t else None

    def cache_spec(self) -> Optional[KVSpec]:
        return KVSpec(1, self.rank, self.window, rows=(("c", 1, self.rank),))

    def state_spec(self):
        return None

    def forward(self, h, ctx: StepContext, cache: LayerCache, state, residual: Optional[torch.Tensor],
                writes_cache: bool = True, out: Optional[torch.Tensor] = None):
        """Adds the mixer's result into `residual`, or, with `out` (float32 [n, width]), leaves it there
        for a block that has more to do with it."""
        h = as_tensor(h)
        n, ws, H, R = h.shape[0], ctx.workspace, self.n_head, self.rank
        group = ctx.groups[cache.group]
        rows = cache.rows["c"]
        proj = ws.get("latent_in", (n, self.in_weight.shape[0]), self.dtype)
        linear(h, self.in_weight, None, out=proj)
        if writes_cache:
            ops.latent_store(rows, proj, self.q_dim, self.down_norm, self.eps, group.slots)
        q_c = ws.get("latent_q", (n, H * R), self.dtype)
        if self.q_weight is not None:
            q_in = h
            if self.q_rank:
                low = ws.get("latent_q_low", (n, self.q_rank), torch.float32)
                linear(h, self.q_down, None, out=low)
                q_in = ws.get("latent_q_normed", (n, self.q_rank), self.dtype)
                ops.rmsnorm(q_in, low, self.q_down_norm, self.eps)
            queries = ws.get("latent_queries", (n, H * self.head_dim), self.dtype)
            linear(q_in, self.q_weight, None, out=queries)
        else:
            queries = proj[:, :self.q_dim]
        ops.heads_product(q_c, queries, self.up_k_t)
        att = ws.get("latent_att", (n, H * R), self.dtype)
        splits = ops.attention(att, q_c, rows, rows, group.block_tables, ctx, n_head=H, scale=self.scale, window=self.window)
        assert splits is None
        heads = ws.get("latent_heads", (n, self.v_dim), self.dtype)
        ops.heads_product(heads, att, self.up_v, gate=proj[:, self.q_dim + R:] if self.gated else None)
        if out is not None:
            linear(heads, self.out_weight, self.out_bias, out=out)
        else:
            linear(heads, self.out_weight, self.out_bias, residual=settled(residual))
        return None


register_mixer("latent_attention", LatentAttention)
