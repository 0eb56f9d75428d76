"""Two mixers that read the same input, their results joined."""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from .base import StepContext, settled
from .linear import linear
from .norms import as_tensor
from .registry import build_part, register_mixer


class SideBySide:
    """result = weight * (left(h) / rms(left(h)) * w_left + right(h) / rms(right(h)) * w_right), the root mean squares over
    the model's width; or, for a spec that is not `normed`, left_weight * left(h) + right_weight * right(h). The two mixers are parts of the mixer registry that can leave their result to the caller
    (`forward(..., out=)`); at most one of them keeps rows in the pages and at most one keeps state, and this part passes
    the layer's cache and slot on to the one that does."""

    replayable = True

    @property
    def takes_padding_rows(self) -> bool:
        return bool(getattr(self.left, "takes_padding_rows", False)) and bool(getattr(self.right, "takes_padding_rows", False))

    def __init__(self, spec, store, dtype: torch.dtype):
        self.dtype = dtype
        self.width, self.eps, self.weight = spec.width, float(spec.eps), float(spec.weight)
        self.left = build_part("mixer", spec.left, store, dtype)
        self.right = build_part("mixer", spec.right, store, dtype)
        for part in (self.left, self.right):
            if "out" not in part.forward.__code__.co_varnames:
                raise ValueError("mixers side by side must be able to leave their result to the caller (forward(..., out=))")
        if self.left.cache_spec() is not None and self.right.cache_spec() is not None:
            raise ValueError("mixers side by side: only one of them may keep rows in the pages")
        if self.left.state_spec() is not None and self.right.state_spec() is not None:
            raise ValueError("mixers side by side: only one of them may keep state")
        t = spec.tensors
        self.normed = bool(getattr(spec, "normed", True))
        self.left_weight, self.right_weight = float(getattr(spec, "left_weight", 1.0)), float(getattr(spec, "right_weight", 1.0))
        self.left_out = store.fetch(t["left_out"], (self.width,), "vector") if self.normed else None
        self.right_out = store.fetch(t["right_out"], (self.width,), "vector") if self.normed else None
        # both read the same rows: where both have one input projection and take its rows from the caller (`in_weight`,
        # forward(..., proj=)), the two run as one product [left | right]
        self.joint_weight = self.joint_bias = None
        if all(isinstance(getattr(p, "in_weight", None), torch.Tensor) and "proj" in p.forward.__code__.co_varnames for p in (self.left, self.right)) \
                and self.left.in_weight.dtype == self.right.in_weight.dtype:
            lw, rw = self.left.in_weight, self.right.in_weight
            self.joint_weight = store.derived(("joined_rows", id(lw), id(rw)), lambda: torch.cat([lw, rw], dim=0).contiguous())
            self.left_cols = lw.shape[0]
            lb, rb = getattr(self.left, "in_bias", None), getattr(self.right, "in_bias", None)
            if lb is not None or rb is not None:
                zeros = lambda rows: torch.zeros(rows, dtype=torch.float32, device=lw.device)  # noqa: E731
                self.joint_bias = store.derived(("joined_bias", id(lw), id(rw)), lambda: torch.cat(
                    [lb if lb is not None else zeros(lw.shape[0]), rb if rb is not None else zeros(rw.shape[0])]).contiguous())
        planners = [p for p in (getattr(self.left, "step_planner", None), getattr(self.right, "step_planner", None)) if p is not None]
        if len(planners) > 1:
            raise ValueError("mixers side by side: only one of them may plan a step")
        if planners:
            self.step_planner = planners[0]

    def cache_spec(self):
        return self.left.cache_spec() or self.right.cache_spec()

    def state_spec(self):
        return self.left.state_spec() or self.right.state_spec()

    def forward(self, h, ctx: StepContext, cache, state, residual: Optional[torch.Tensor], writes_cache: bool = True,
                out: Optional[torch.Tensor] = None):
        n, ws = h.shape[0], ctx.workspace
        if not self.normed and all(getattr(p, "can_scale_output", False) for p in (self.left, self.right)):
            # constant weights on results that are not normed: each mixer takes its factor where it rounds its rows for its last
            # product, the first writes the sum's place and the second adds to it
            y = out if out is not None else ws.get("side_left", (n, self.width), torch.float32)
            proj_l = proj_r = None
            if self.joint_weight is not None:
                proj = ws.get("side_in", (n, self.joint_weight.shape[0]), torch.float32)
                linear(h, self.joint_weight, self.joint_bias, out=proj)
                proj_l, proj_r = proj[:, :self.left_cols], proj[:, self.left_cols:]
            self.left.forward(h, ctx, cache, state, None, writes_cache=writes_cache, out=y, proj=proj_l, out_scale=self.left_weight)
            self.right.forward(h, ctx, cache, state, None, writes_cache=writes_cache, out=y, proj=proj_r, out_scale=self.right_weight, add=True)
            if out is None:
                ops.add_into_(settled(residual), y)
            return None
        a = ws.get("side_left", (n, self.width), torch.float32)
        b = ws.get("side_right", (n, self.width), torch.float32)
        if self.joint_weight is not None:
            proj = ws.get("side_in", (n, self.joint_weight.shape[0]), torch.float32)
            linear(h, self.joint_weight, self.joint_bias, out=proj)
            self.left.forward(h, ctx, cache, state, None, writes_cache=writes_cache, out=a, proj=proj[:, :self.left_cols])
            self.right.forward(h, ctx, cache, state, None, writes_cache=writes_cache, out=b, proj=proj[:, self.left_cols:])
        else:
            self.left.forward(h, ctx, cache, state, None, writes_cache=writes_cache, out=a)
            self.right.forward(h, ctx, cache, state, None, writes_cache=writes_cache, out=b)
        if not self.normed:
            if out is not None:
                ops.weighted_sum(out, a, b, self.left_weight, self.right_weight)
            else:
                ops.weighted_sum(a, a, b, self.left_weight, self.right_weight)
                ops.add_into_(settled(residual), a)
        elif out is not None:
            ops.fill_(out, 0)
            ops.mean_norm_add(out, a, b, self.left_out, self.right_out, self.eps, self.weight)
        else:
            ops.mean_norm_add(settled(residual), a, b, self.left_out, self.right_out, self.eps, self.weight)
        return None


register_mixer("side_by_side", SideBySide)
