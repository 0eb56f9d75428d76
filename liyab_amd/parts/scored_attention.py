"""Attention whose queries, keys and scores are worked on between the projection and the softmax."""

from __future__ import annotations

import math
from typing import Optional

import numpy as np
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


def rotary_frequencies(rot) -> np.ndarray:
    """f_i = base^(-2i / dims) for i < dims / 2, the long wavelengths stretched as `rot.scaling` = (factor, low, high,
    original) says: with wavelength l = 2 pi / f, f stays for l < original / high, becomes f / factor for l > original /
    low, and in between is (1 - s) f / factor + s f with s = (original / l - low) / (high - low); or as `rot.ramp` = (factor,
    fast, slow, original) says, by the entry's number (see RotarySpec). float64."""
    f = np.array([float(rot.base) ** (-2.0 * i / rot.dims) for i in range(rot.dims // 2)], dtype=np.float64)
    if rot.scaling is not None:
        factor, low, high, original = (float(v) for v in rot.scaling)
        for i, fi in enumerate(f):
            wavelength = 2.0 * math.pi / fi
            if wavelength < original / high:
                continue
            if wavelength > original / low:
                f[i] = fi / factor
            else:
                s = (original / wavelength - low) / (high - low)
                f[i] = (1.0 - s) * fi / factor + s * fi
    if getattr(rot, "ramp", None) is not None:
        factor, fast, slow, original = (float(v) for v in rot.ramp)

        def at(turns: float) -> float:
            return rot.dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(float(rot.base)))

        lo = max(math.floor(at(fast)), 0)
        hi = min(math.ceil(at(slow)), rot.dims - 1)
        for i, fi in enumerate(f):
            r = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            f[i] = fi / factor * r + fi * (1.0 - r)
    return f


def rotary_magnitude(rot) -> float:
    """What cosine and sine are multiplied by: 1, or ramp_magnitude * ln(factor) + 1 with a ramp."""
    if getattr(rot, "ramp", None) is None:
        return 1.0
    return float(rot.ramp_magnitude) * math.log(float(rot.ramp[0])) + 1.0


def distance_rows(n_rows: int, far: int) -> np.ndarray:
    """The row of a distance-bias table of `n_rows` rows for each distance 0..far: the distance itself below half the rows,
    then half + floor(ln(n / half) / ln(far / half) * (rows - half)), at most the last row (which every distance from `far`
    on takes)."""
    half = n_rows // 2
    out = np.empty(far + 1, dtype=np.int64)
    for n in range(far + 1):
        if n < half:
            out[n] = n
        else:
            out[n] = min(n_rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (n_rows - half))))
    return out


class ScoredAttention:
    """q, k (and v, unless the values are the keys as projected) are one product of the mixer's input, left in 32 bits; one
    kernel then norms, turns and scales the heads as the spec says and writes queries to a buffer and keys and values to
    their pages (keys `head_dim` wide, values `value_dim`: two planes of the cache with widths of their own); the attention
    kernel applies the soft cap and the bias by distance to the scores, and the gate to its result; then the output
    projection. The bias by distance is looked up in a table a distance [distance_bias + 1, heads] made once from the learned
    rows, so that no kernel computes a logarithm a key."""

    replayable = True
    takes_padding_rows = True  # (slot -1: nothing of theirs is cached, and no other row attends to them)
    step_planner = AttentionStepPlanner()  # the same cut of a step's tokens as attention's: ctx.plans["attention"]

    def __init__(self, spec, store, dtype: torch.dtype):
        self.dtype = dtype
        self.width, self.n_head, self.n_kv_head = spec.width, spec.n_head, spec.n_kv_head
        self.head_dim, self.value_dim = spec.head_dim, spec.value_dim
        if self.n_head % self.n_kv_head:
            raise ValueError(f"{self.n_head} query heads are no multiple of {self.n_kv_head} key/value heads")
        if spec.values_are_keys and self.value_dim != self.head_dim:
            raise ValueError(f"values that are the keys are as wide as the keys ({self.head_dim}), not {self.value_dim}")
        if self.head_dim > 512 or self.value_dim > 256:
            raise Unsupported(f"scored attention: keys of {self.head_dim} / values of {self.value_dim} are not supported (up to 512 / 256)")
        self.scale, self.eps, self.window, self.softcap = float(spec.scale), float(spec.eps), int(spec.window), float(spec.softcap or 0.0)
        self.values_are_keys, self.gated = bool(spec.values_are_keys), bool(spec.gated)
        H, G, D, V, d = self.n_head, self.n_kv_head, self.head_dim, self.value_dim, self.width
        t = spec.tensors
        srcs, shapes = [t["q"], t["k"]], [(H * D, d), (G * D, d)]
        self.q_off, self.k_off = 0, H * D
        at = H * D + G * D
        self.v_off = self.k_off
        if not self.values_are_keys:
            srcs.append(t["v"])
            shapes.append((G * V, d))
            self.v_off, at = at, at + G * V
        self.gate_off = at
        if self.gated:
            srcs.append(t["gate"])
            shapes.append((H * V, d))
            at += H * V
        self.in_weight = store.fetch_joined(srcs, shapes, "matrix", "rows")
        # biases on the projections of queries, keys and values: one vector over the joint product's columns, zeros for the gate's
        self.in_bias = None
        if getattr(spec, "biased", False):
            names = [t["q_bias"], t["k_bias"]] + ([] if self.values_are_keys else [t["v_bias"]])
            bias = store.fetch_joined(names, [(r[0],) for r in shapes[:len(names)]], "vector", "rows")
            if self.gated:
                bias = store.derived(("bias_zeros_behind", tuple(b.name for b in names), H * V),
                                     lambda: torch.cat([bias, torch.zeros(H * V, dtype=torch.float32, device=bias.device)]).contiguous())
            self.in_bias = bias
        self.sinks = store.fetch(t["sink"], (H,), "vector") if getattr(spec, "sink", False) else None
        # values shared between layers of a step: the first such layer keeps its values as projected, the later ones mix theirs
        # with those at a learned rate (one float, read on the device); both find the rows under one name in the step's workspace
        self.value_mix = getattr(spec, "value_mix", "") or ""
        if self.value_mix not in ("", "first", "later") or (self.value_mix and self.values_are_keys):
            raise ValueError(f"scored attention: value_mix '{self.value_mix}'")
        self.v_lam = store.fetch(t["vmix"], (), "vector").reshape(1) if self.value_mix else None
        self.out_weight = store.fetch(t["out"], (d, H * V), "matrix")
        # Keys and values of different widths: both planes of the pages as wide as the wider (a multiple of 8), zeros behind the
        # narrower heads, which is what the engine's paged attention kernels take; zeros in keys and queries add nothing to a
        # score, zeros in values give zeros in the result, and the output projection gets zero columns for them.
        self.row_dim = 0
        if D != V and not self.gated and max(D, V) <= ops.ATTENTION_MAX_HEAD_DIM:
            P = self.row_dim = -(-max(D, V) // 8) * 8
            w = self.out_weight
            self.out_weight = store.derived(("padded_heads", t["out"].name, P), lambda: torch.nn.functional.pad(w.view(d, H, V), (0, P - V)).reshape(d, H * P).contiguous())
        self.q_norm = store.fetch(t["q_norm"], (D,), "vector") if spec.qk_norm else None
        self.k_norm = store.fetch(t["k_norm"], (D,), "vector") if spec.qk_norm else None
        self.rot_dims, self.freqs, self.rot_halves, self.rot_mag = 0, None, False, 1.0
        if spec.rotary is not None:
            rot = spec.rotary
            if rot.dims % 2 or not 0 < rot.dims <= D:
                raise ValueError(f"rotary encoding over {rot.dims} of {D} entries")
            self.rot_dims = int(rot.dims)
            self.rot_halves, self.rot_mag = bool(getattr(rot, "halves", False)), rotary_magnitude(rot)
            self.freqs = store.derived(("rotary", rot.dims, rot.base, rot.scaling, getattr(rot, "ramp", None)),
                                       lambda: torch.from_numpy(rotary_frequencies(rot).astype(np.float64)).to(self.out_weight.device))
        self.temp_coef, self.temp_every = (float(spec.q_temp[0]), int(spec.q_temp[1])) if spec.q_temp else (0.0, 0)
        self.bias_table = None
        if spec.distance_bias:
            rel = store.fetch(t["rel"], (spec.bias_rows, H), "vector")
            far, rows = int(spec.distance_bias), int(spec.bias_rows)
            if rows < 2 or far <= rows // 2:
                raise ValueError(f"a bias by distance of {rows} rows up to distance {far}")
            self.bias_table = store.derived(("distance_bias", t["rel"].name, far),
                                            lambda: rel[torch.from_numpy(distance_rows(rows, far)).to(rel.device)].contiguous())

    def _shared_values(self, ws, n: int) -> dict:
        if not self.value_mix:
            return {}
        rows = ws.get("first_values", (n * self.n_kv_head * self.value_dim,), torch.float32)
        return {"v_keep": rows} if self.value_mix == "first" else {"v_first": rows, "v_lam": self.v_lam}

    def cache_spec(self) -> Optional[KVSpec]:
        return KVSpec(self.n_kv_head, self.head_dim, self.window,
                      rows=(("k", self.n_kv_head, self.row_dim or self.head_dim), ("v", self.n_kv_head, self.row_dim or self.value_dim)))

    def state_spec(self):
        return None

    @property
    def can_scale_output(self) -> bool:
        """Whether forward(..., out_scale=, add=) is taken: the factor rides on the gate's pass over the heads' rows."""
        return self.gated and (self.head_dim == self.value_dim or bool(self.row_dim))

    def forward(self, h, ctx: StepContext, cache: LayerCache, state, residual: Optional[torch.Tensor],
                writes_cache: bool = True, out: Optional[torch.Tensor] = None, proj: Optional[torch.Tensor] = None,
                out_scale: float = 1.0, add: bool = False):
        """Adds the mixer's result into `residual`, or, with `out` (float32 [n, width]), leaves it there. `proj`: the input
        projection's 32-bit rows (biases added, `in_bias`), when the caller has made them (as columns of a wider product)."""
        n, ws, H, D, V = h.shape[0], ctx.workspace, self.n_head, self.head_dim, self.value_dim
        group = ctx.groups[cache.group]
        if proj is None:
            proj = ws.get("scored_in", (n, self.in_weight.shape[0]), torch.float32)
            linear(h, self.in_weight, self.in_bias, out=proj)
        P = self.row_dim
        q = ws.get("scored_q", (n, H * (P or D)), self.dtype)
        if not writes_cache:
            raise Unsupported("scored attention: a run that reads another run's cache is not supported")
        ops.qk_prepare(proj, q, cache.k, cache.v, group.slots, ctx.positions, q_off=self.q_off, k_off=self.k_off, v_off=self.v_off,
                       n_head=H, q_norm=self.q_norm, k_norm=self.k_norm, eps=self.eps, freqs=self.freqs, rot_dims=self.rot_dims,
                       temp_coef=self.temp_coef, temp_every=self.temp_every, head_dim=D, value_dim=V, rot_halves=self.rot_halves,
                       rot_mag=self.rot_mag, **self._shared_values(ws, n))
        att = ws.get("scored_att", (n, H * (P or V)), self.dtype)
        gate = proj[:, self.gate_off:self.gate_off + H * V] if self.gated else None
        if D == V or P:
            # keys and values of one width: the paged attention kernels of the engine (tiles of a prompt's queries on the matrix
            # cores, single tokens in splits, the 32-bit form), which cap and bias the scores when asked to
            splits = ops.attention(att, q, cache.k, cache.v, group.block_tables, ctx, n_head=H, scale=self.scale, window=self.window,
                                   softcap=self.softcap, bias_table=self.bias_table, sinks=self.sinks)
            assert splits is None
            if gate is not None:
                ops.gate_rows(att, gate, out_scale)
            elif out_scale != 1.0:
                raise Unsupported("scored attention: a factor on the result needs the gate's pass (can_scale_output)")
        else:
            if out_scale != 1.0:
                raise Unsupported("scored attention: a factor on the result needs the gate's pass (can_scale_output)")
            ops.attention_scored(att, q, cache.k, cache.v, group.block_tables, ctx, n_head=H, scale=self.scale, softcap=self.softcap,
                                 window=self.window, bias_table=self.bias_table, gate=gate, sinks=self.sinks)
        if out is not None and add:
            linear(att, self.out_weight, None, residual=out)
        elif out is not None:
            linear(att, self.out_weight, None, out=out)
        else:
            linear(att, self.out_weight, None, residual=settled(residual))
        return None


register_mixer("scored_attention", ScoredAttention)
