"""Attention in two maps a head that share their values."""

from __future__ import annotations

import math
from typing import Optional

import torch

from ..cache.pages import KVSpec, StateSpec
from ..cache.storage import LayerCache
from ..errors import Unsupported
from ..kernels import ops
from .attention import AttentionStepPlanner
from .base import StepContext, settled
from .delta_rule import own_state
from .linear import linear
from .norms import as_tensor
from .registry import register_mixer


class DifferentialAttention:
    """q, k, v = W h + b, one product left in 32 bits; every channel then passes a causal convolution over time (when the spec has
    one; its last taps - 1 inputs are the request's state). A query head holds [map 1 | map 2] and so does a key head; each map is
    an ordinary softmax attention under the window over the same values, and a head's result is a1 - lam * a2, lam = exp(lq1 . lk1) -
    exp(lq2 . lk2) + lam_init (one number a layer, taken once at load), brought to unit root mean square over the head and multiplied
    by `out_scale`; then the output projection.

    The two maps run through the engine's paged attention kernels, once each: the pages hold three planes of one width P (map 1's
    keys, map 2's keys, the values; P the wider of key and value head, a multiple of 8, zeros behind the narrower), and map m's
    queries are a set of heads of their own [n, H * P]."""

    replayable = True
    takes_padding_rows = True  # (slot -1: nothing of theirs is cached, and no other row attends to them)
    step_planner = AttentionStepPlanner()  # the same cut of a step's tokens as attention's: ctx.plans["attention"]

    def __init__(self, spec, store, dtype: torch.dtype):
        self.dtype = dtype
        self.width, self.n_head, self.n_kv_head = spec.width, spec.n_head, spec.n_kv_head
        self.head_dim, self.value_dim = spec.head_dim, spec.value_dim
        H, G, D, V, d = self.n_head, self.n_kv_head, self.head_dim, self.value_dim, self.width
        if H % G:
            raise ValueError(f"{H} query heads are no multiple of {G} key/value heads")
        self.row_dim = -(-max(D, V) // 8) * 8
        if not ops.attention_takes(self.row_dim):
            raise Unsupported(f"differential attention: heads of {max(D, V)} are not supported (the attention kernels take up to {ops.ATTENTION_MAX_HEAD_DIM})")
        self.scale, self.window, self.eps = float(spec.scale), int(spec.window), float(spec.eps)
        self.out_scale, self.taps = float(spec.out_scale), int(spec.conv_taps)
        t = spec.tensors
        self.channels = 2 * H * D + 2 * G * D + G * V
        shapes = [(2 * H * D, d), (2 * G * D, d), (G * V, d)]
        self.in_weight = store.fetch_joined([t[c] for c in "qkv"], shapes, "matrix", "rows")
        self.in_bias = store.fetch_joined([t[c + "_bias"] for c in "qkv"], [(s[0],) for s in shapes], "vector", "rows") if "q_bias" in t else None
        self.conv = None
        if self.taps:
            if not 1 <= self.taps <= ops.SHIFT_MAX_TAPS:
                raise ValueError(f"a convolution of {self.taps} taps (1 to {ops.SHIFT_MAX_TAPS} are taken)")
            joined = store.fetch_joined([t[c + "_conv"] for c in "qkv"], [(s[0], self.taps) for s in shapes], "vector", "rows")
            # [taps, channels]: a tap's channels side by side, as the kernel reads them
            self.conv = store.derived(("taps_major",) + tuple(t[c + "_conv"].name for c in "qkv"), lambda: joined.t().contiguous())
        lam = [store.fetch(t[c], (D,), "vector") for c in ("lq1", "lk1", "lq2", "lk2")]
        self.lam = float(math.exp(float((lam[0].double() * lam[1].double()).sum())) - math.exp(float((lam[2].double() * lam[3].double()).sum()))
                         + float(spec.lam_init))
        self.out_weight = store.fetch(t["out"], (d, H * V), "matrix")

    def cache_spec(self) -> Optional[KVSpec]:
        G, P = self.n_kv_head, self.row_dim
        return KVSpec(G, P, self.window, rows=(("k1", G, P), ("k2", G, P), ("v", G, P)))

    def state_spec(self) -> Optional[StateSpec]:
        return StateSpec(((self.taps - 1) * self.channels,)) if self.taps > 1 else None

    def forward(self, h, ctx: StepContext, cache: LayerCache, state, residual: Optional[torch.Tensor],
                writes_cache: bool = True, out: Optional[torch.Tensor] = None):
        h = as_tensor(h)
        n, ws, H, V, P = h.shape[0], ctx.workspace, self.n_head, self.value_dim, self.row_dim
        if not writes_cache:
            raise Unsupported("differential attention: a run that reads another run's cache is not supported")
        group = ctx.groups[cache.group]
        proj = ws.get("maps_in", (n, self.channels), torch.float32)
        linear(h, self.in_weight, self.in_bias, out=proj)
        ring = own_state(state, (self.taps - 1) * self.channels) if self.taps > 1 else None
        q = ws.get("maps_q", (n, 2, H * P), self.dtype)
        k1, k2, v = cache.rows["k1"], cache.rows["k2"], cache.rows["v"]
        single = ring is not None and ops.single_token_step(ctx)  # (each row then keeps itself in the ring inside the kernel)
        ops.maps_store(proj, q, k1, k2, v, group.slots, self.conv, ring, ctx, n_head=H, n_kv_head=self.n_kv_head, head_dim=self.head_dim,
                       value_dim=V, keep_single=single)
        if ring is not None and not single:
            ops.ring_keep(ring, self.taps - 1, proj, ctx)
        att = ws.get("maps_att", (n, 2, H * P), self.dtype)
        for m, keys in enumerate((k1, k2)):
            splits = ops.attention(att[:, m], q[:, m], keys, v, group.block_tables, ctx, n_head=H, scale=self.scale, window=self.window)
            assert splits is None
        y = ws.get("maps_out", (n, H * V), self.dtype)
        ops.maps_join(y, att[:, 0], att[:, 1], self.lam, self.eps, self.out_scale, n_head=H, value_dim=V)
        if out is not None:
            linear(y, self.out_weight, None, out=out)
        else:
            linear(y, self.out_weight, None, residual=settled(residual))
        return None


register_mixer("differential_attention", DifferentialAttention)
