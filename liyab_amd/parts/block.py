"""How a layer's parts are arranged."""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import SplitStream, StepContext, settled
from .linear import linear
from .norms import as_tensor
from .registry import register_block


class PreNormBlock:
    """x += mixer(norm_mixer(x)); x += ffn(norm_ffn(x)): the reference's
    run_block for a sequential pre-norm layer (src/core/transformer.cpp:5514-5726:
    norm :5565-5577, mixer, residual :5647, norm :5663-5666, ffn, residual :5692)."""

    # every launch goes through the kernel library and depends on nothing of this object but its
    # tensors and the constants among its attributes: layers of this kind may run from one recorded list
    replayable = True
    # rows behind the step's tokens (token 0 at position 0 of the first request, slot -1) are computed
    # and never read: nothing here writes for them or lets them touch another row
    takes_padding_rows = True

    def __init__(self, spec, mixer, ffn, norm_mixer, norm_ffn):
        self.mixer, self.ffn, self.norm_mixer, self.norm_ffn = mixer, ffn, norm_mixer, norm_ffn
        # phases are named after the parts' kinds (the reference's: attention, dense_ffn, ...)
        self.mixer_phase = getattr(getattr(spec, "mixer", None), "kind", "mixer")
        self.ffn_phase = getattr(getattr(spec, "ffn", None), "kind", "ffn")

    takes_pending = True  # forward(..., pending=) takes the stream split and may return it split

    def forward(self, x: torch.Tensor, ctx: StepContext, cache, state, writes_cache: bool = True, pending=None):
        """x: the residual stream's own tensor. `pending`: the stream as a SplitStream when the
        previous layer left it split (x is then stale). Returns the stream as a SplitStream if
        this layer leaves it split, else None (x holds it)."""
        stream = pending if pending is not None else x
        if ctx.phases is not None:
            ctx.phases.mark(self.mixer_phase)
        h, stream = self._normed(self.norm_mixer, stream, ctx)
        if getattr(self.mixer, "defers", False):
            stream = self.mixer.forward(h, ctx, cache, state, stream, writes_cache=writes_cache, defer=True) or x
        else:
            self.mixer.forward(h, ctx, cache, state, settled(stream), writes_cache=writes_cache)
            stream = x
        if self.ffn is not None:
            if ctx.phases is not None:
                ctx.phases.mark(self.ffn_phase)
            h, stream = self._normed(self.norm_ffn, stream, ctx)
            if getattr(self.ffn, "defers", False):
                stream = self.ffn.forward(h, ctx, stream, defer=True) or x
            else:
                self.ffn.forward(h, ctx, settled(stream))
                stream = x
        return stream if isinstance(stream, SplitStream) else None

    @staticmethod
    def _normed(norm, stream, ctx):
        """The norm of the stream and the stream as it is afterwards (settled if the norm cannot
        read it split). The norm's output is left pending when the norm allows it, so that the
        next product may fold it in (parts that need the rows call `as_tensor`)."""
        rows = stream
        if isinstance(stream, SplitStream):
            takes = getattr(norm, "takes_planes", None)
            if takes is not None and takes(stream.planes):
                rows = stream.planes
            else:
                rows = stream = stream.settle()
        return (norm.lazy(rows, ctx) if hasattr(norm, "lazy") else norm.forward(rows, ctx)), stream


register_block("pre_norm", PreNormBlock)


class ParallelBlock:
    """h = norm(x); x += mixer(h) + ffn(h): one norm, and both sublayers read its output. Each sublayer adds its result into
    the 32-bit stream from its last product's epilogue; h is a buffer of its own, so the second sublayer still reads the
    norm of the stream as the layer found it."""

    replayable = True
    takes_padding_rows = True
    takes_pending = False

    def __init__(self, spec, mixer, ffn, norm_mixer, norm_ffn):
        if norm_ffn is not None:
            raise ValueError("a parallel block has one norm (norm_mixer)")
        self.mixer, self.ffn, self.norm_mixer, self.norm_ffn = mixer, ffn, norm_mixer, None
        self.mixer_phase = getattr(getattr(spec, "mixer", None), "kind", "mixer")
        self.ffn_phase = getattr(getattr(spec, "ffn", None), "kind", "ffn")

    def forward(self, x: torch.Tensor, ctx: StepContext, cache, state, writes_cache: bool = True):
        if ctx.phases is not None:
            ctx.phases.mark(self.mixer_phase)
        # The norm is left pending where it can be: in steps of few rows the products that read it apply it to their own operand
        # (one launch less), and a part that needs the rows themselves computes them once (`as_tensor`). A pending norm reads
        # the stream when a product runs, so everything that reads h runs before anything adds into the stream: a feed-forward
        # that can be run in two halves (`begin` / `finish`) makes its first product ahead of the mixer; any other gets the rows.
        norm, ffn = self.norm_mixer, self.ffn
        h = norm.lazy(x, ctx, name="block_in") if hasattr(norm, "lazy") else norm.forward(x, ctx, name="block_in")
        begun = None
        if ffn is not None:
            if hasattr(ffn, "begin"):
                begun = ffn.begin(h, ctx)
            else:
                h = as_tensor(h)
        self.mixer.forward(h, ctx, cache, state, x, writes_cache=writes_cache)
        if ffn is not None:
            if ctx.phases is not None:
                ctx.phases.mark(self.ffn_phase)
            if begun is not None:
                ffn.finish(begun, ctx, x)
            else:
                ffn.forward(h, ctx, x)
        return None


register_block("parallel", ParallelBlock)


class PostNormGatedBlock:
    """x += norm_mixer(g1 * mixer(conv(x))); x += norm_ffn(g2 * ffn(x)): the sublayers read the stream
    itself, and the norms stand on their results. g = sigmoid(W x + b) from the stream as the sublayer
    gets it (before the convolution); `conv`: what the mixer reads is x + a short causal convolution of
    x over time, whose last inputs are the layer's per-request state. Gates and the convolution are
    optional, the feed-forward too. The sum into the stream, the norms and the gates are 32-bit; the
    sublayers and the gates' products read x rounded to the compute dtype.

    Kernels a sublayer beside its own: the convolution (which also rounds x), the gate's product, and
    one update of the rows (sum of the sublayer's rows a token, gate, norm, addition, the rounded rows
    for the next sublayer, and the rows the next step's convolution needs)."""

    replayable = True
    takes_padding_rows = True
    takes_pending = False  # the stream is whole when this block gets it and when it leaves it

    def __init__(self, spec, mixer, ffn, norm_mixer, norm_ffn, input_conv=None, gate_mixer=None, gate_ffn=None):
        self.mixer, self.ffn, self.norm_mixer, self.norm_ffn = mixer, ffn, norm_mixer, norm_ffn
        self.conv, self.gate_mixer, self.gate_ffn = input_conv, gate_mixer, gate_ffn if ffn is not None else None
        self.dtype = mixer.dtype
        self.mixer_phase = getattr(getattr(spec, "mixer", None), "kind", "mixer")
        self.ffn_phase = getattr(getattr(spec, "ffn", None), "kind", "ffn")
        for part, what in ((mixer, "mixer"), (ffn, "feed-forward")):
            if part is not None and "out" not in part.forward.__code__.co_varnames:
                raise ValueError(f"a post-norm block needs a {what} that can leave its result to the block (forward(..., out=))")
        for norm in (norm_mixer, norm_ffn if ffn is not None else norm_mixer):
            if not getattr(norm, "root_mean_square", False):
                raise ValueError("a post-norm block's row update applies a root-mean-square norm (kind 'rmsnorm')")
        if mixer.state_spec() is not None and self.conv is not None and self.conv.state_spec() is not None:
            raise ValueError("a mixer with state of its own under an input convolution: one state a layer")
        # The feed-forward's gate and its router read the same rows: one product [gate | router] instead of two
        # (a launch less a layer). The joint matrix is made once for the two matrices it is made of, so that
        # layers sharing their tensors share it, and the parts give theirs up.
        self.joint_weight = self.joint_bias = None
        if self.gate_ffn is not None and hasattr(ffn, "take_router") and ffn.router is not None and ffn.router.dtype == self.gate_ffn.weight.dtype:
            gw, gb = self.gate_ffn.weight, self.gate_ffn.bias
            rw, rb = ffn.take_router()
            hit = getattr(gw, "_joint_rows", None)  # (layers that share their tensors get the same tensor objects from the store)
            if hit is None or hit[2] is not rw:
                bias = None
                if gb is not None or rb is not None:
                    bias = torch.cat([gb if gb is not None else torch.zeros(gw.shape[0], dtype=torch.float32, device=gw.device),
                                      rb if rb is not None else torch.zeros(rw.shape[0], dtype=torch.float32, device=gw.device)])
                hit = gw._joint_rows = (torch.cat([gw, rw], dim=0).contiguous(), bias, rw)
            self.joint_weight, self.joint_bias = hit[0], hit[1]
            self.gate_ffn.weight = self.gate_ffn.bias = None

    def state_spec(self):
        return (self.conv.state_spec() if self.conv is not None else None) or self.mixer.state_spec()

    def forward(self, x: torch.Tensor, ctx: StepContext, cache, state, writes_cache: bool = True):
        ws, n, d = ctx.workspace, x.shape[0], x.shape[1]
        if ctx.phases is not None:
            ctx.phases.mark(self.mixer_phase)
        xh = ws.get("stream_cast", (n, d), self.dtype)
        conv_state = state if self.conv is not None and self.conv.state_spec() is not None else None
        if self.conv is not None:
            h = self.conv.forward(x, ctx, conv_state, cast_out=xh)
        else:
            ops.gather_rows(xh, x)
            h = xh
        gate = self.gate_mixer.forward(xh, ctx, "gate_logits") if self.gate_mixer is not None else None
        y = ws.get("sublayer_out", (n, d), torch.float32)
        self.mixer.forward(h, ctx, cache, None if conv_state is not None else state, None, writes_cache=writes_cache, out=y)
        keep = (conv_state, ctx) if conv_state is not None and writes_cache else None
        ops.gated_norm_add(x, y, self.norm_mixer.weight, self.norm_mixer.eps, gate=gate, cast_out=xh if self.ffn is not None else None,
                           keep=keep)
        if self.ffn is not None:
            if ctx.phases is not None:
                ctx.phases.mark(self.ffn_phase)
            k = int(getattr(self.ffn, "rows_a_token", 1))
            y = ws.get("sublayer_rows", (n * k, d), torch.float32) if k > 1 else y
            if self.joint_weight is not None:
                z = ws.get("gate_router_logits", (n, self.joint_weight.shape[0]), torch.float32)
                linear(xh, self.joint_weight, self.joint_bias, out=z)
                gate = z[:, :d]
                self.ffn.forward(xh, ctx, None, out=y, router_logits=z[:, d:])
            else:
                gate = self.gate_ffn.forward(xh, ctx, "gate_logits") if self.gate_ffn is not None else None
                self.ffn.forward(xh, ctx, None, out=y)
            ops.gated_norm_add(x, y, self.norm_ffn.weight, self.norm_ffn.eps, n_sum=k, gate=gate)
        return None


register_block("post_norm_gated", PostNormGatedBlock)


class SandwichBlock:
    """x += post_norm_mixer(mixer(norm_mixer(x))); x += post_norm_ffn(ffn(norm_ffn(x))): a norm before each sublayer and a
    root-mean-square norm behind it. The sublayers leave their 32-bit results to the block (`forward(..., out=)`; a
    feed-forward may leave several rows a token, `rows_a_token`), and one kernel a sublayer takes the sum of a token's rows, its
    root mean square, the weight and the addition into the 32-bit stream. The feed-forward is optional."""

    replayable = True
    takes_padding_rows = True
    takes_pending = False

    def chain_norm(self, following) -> bool:
        """Called once, when the model is built, for a block that runs right before `following` in every pass: this block's last
        update of the rows then also takes `following`'s first norm of them, and `following` reads those rows instead of taking its
        norm itself. True if the two were chained (both sandwich blocks whose first norms are weighted root-mean-square norms)."""
        norm = getattr(following, "norm_mixer", None)
        if not isinstance(following, SandwichBlock) or not getattr(norm, "root_mean_square", False) or norm.weight is None or norm.dtype != self.norm_mixer.dtype:
            return False
        self.next_weight, self.next_eps = norm.weight, float(norm.eps)
        following.input_normed = True
        return True

    def __init__(self, spec, mixer, ffn, norm_mixer, norm_ffn, post_norm_mixer=None, post_norm_ffn=None):
        self.next_weight, self.next_eps, self.input_normed = None, 0.0, False
        self.mixer, self.ffn, self.norm_mixer, self.norm_ffn = mixer, ffn, norm_mixer, norm_ffn if ffn is not None else None
        self.post_norm_mixer, self.post_norm_ffn = post_norm_mixer, post_norm_ffn if ffn is not None else None
        self.mixer_phase = getattr(getattr(spec, "mixer", None), "kind", "mixer")
        self.ffn_phase = getattr(getattr(spec, "ffn", None), "kind", "ffn")
        for part, what in ((mixer, "mixer"), (ffn, "feed-forward")):
            if part is not None and "out" not in part.forward.__code__.co_varnames:
                raise ValueError(f"a sandwich block needs a {what} that can leave its result to the block (forward(..., out=))")
        for norm in (post_norm_mixer, post_norm_ffn if ffn is not None else post_norm_mixer):
            if norm is None or not getattr(norm, "root_mean_square", False):
                raise ValueError("a sandwich block's row update applies a root-mean-square norm behind each sublayer (kind 'rmsnorm')")
        if norm_mixer is None or (ffn is not None and norm_ffn is None):
            raise ValueError("a sandwich block has a norm before each sublayer")

    def forward(self, x: torch.Tensor, ctx: StepContext, cache, state, writes_cache: bool = True):
        ws, n, d = ctx.workspace, x.shape[0], x.shape[1]
        if ctx.phases is not None:
            ctx.phases.mark(self.mixer_phase)
        # (the block before may have left this block's first norm of the rows where this block's own norm would put it)
        h = ws.get("block_in", (n, d), self.norm_mixer.dtype) if self.input_normed else self.norm_mixer.forward(x, ctx, name="block_in")
        y = ws.get("sublayer_out", (n, d), torch.float32)
        self.mixer.forward(h, ctx, cache, state, None, writes_cache=writes_cache, out=y)
        # the update of the rows also takes the next norm of the new rows, where that is a root-mean-square norm too: the feed-forward's
        # own, or, behind the layer's last sublayer, the next layer's first
        chained = (self.next_weight, self.next_eps) if self.next_weight is not None else None
        fused = self.ffn is not None and getattr(self.norm_ffn, "root_mean_square", False) and self.norm_ffn.weight is not None
        if fused:
            h = ws.get("block_in", (n, d), self.norm_ffn.dtype)
            ops.gated_norm_add(x, y, self.post_norm_mixer.weight, self.post_norm_mixer.eps, cast_out=h, next_norm=(self.norm_ffn.weight, self.norm_ffn.eps))
        elif self.ffn is None and chained is not None:
            ops.gated_norm_add(x, y, self.post_norm_mixer.weight, self.post_norm_mixer.eps, cast_out=ws.get("block_in", (n, d), self.norm_mixer.dtype), next_norm=chained)
        else:
            ops.gated_norm_add(x, y, self.post_norm_mixer.weight, self.post_norm_mixer.eps)
        if self.ffn is not None:
            if ctx.phases is not None:
                ctx.phases.mark(self.ffn_phase)
            if not fused:
                h = self.norm_ffn.forward(x, ctx, name="block_in")
            k = int(getattr(self.ffn, "rows_a_token", 1))
            y = ws.get("sublayer_rows", (n * k, d), torch.float32) if k > 1 else y
            self.ffn.forward(h, ctx, None, out=y)
            if chained is not None:
                ops.gated_norm_add(x, y, self.post_norm_ffn.weight, self.post_norm_ffn.eps, n_sum=k, cast_out=ws.get("block_in", (n, d), self.norm_mixer.dtype),
                                   next_norm=chained)
            else:
                ops.gated_norm_add(x, y, self.post_norm_ffn.weight, self.post_norm_ffn.eps, n_sum=k)
        return None


register_block("sandwich", SandwichBlock)


class ParallelPairBlock:
    """x += mixer(c1(norm_mixer(x))) + ffn(c2(norm_ffn(x))): two root-mean-square norms of the same stream (they share the root
    mean square, so one pass over a row gives both), each followed by a short causal convolution over time of its own, h <- h +
    conv(h), whose last taps - 1 inputs (the normalised rows, 32-bit) are the layer's per-request state. The convolutions and the
    feed-forward are optional. Each sublayer adds its result into the 32-bit stream from its last product's epilogue; what they read
    is a buffer of its own, so both see the stream as the layer found it.

    A slot of the layer's state holds the convolutions' ring first ((taps - 1) places of [sublayers, width] floats, position p at
    place p % (taps - 1)) and the mixer's own state behind it; the mixer gets its stretch as a `StateSlice`."""

    replayable = True
    takes_padding_rows = True
    takes_pending = False

    def __init__(self, spec, mixer, ffn, norm_mixer, norm_ffn, input_conv=None, ffn_conv=None):
        self.mixer, self.ffn, self.norm_mixer, self.norm_ffn = mixer, ffn, norm_mixer, norm_ffn if ffn is not None else None
        self.conv, self.ffn_conv = input_conv, ffn_conv if ffn is not None else None
        self.dtype = mixer.dtype
        self.mixer_phase = getattr(getattr(spec, "mixer", None), "kind", "mixer")
        self.ffn_phase = getattr(getattr(spec, "ffn", None), "kind", "ffn")
        norms = [norm_mixer] + ([norm_ffn] if ffn is not None else [])
        for norm in norms:
            if norm is None or not getattr(norm, "root_mean_square", False) or norm.weight is None:
                raise ValueError("a parallel pair's sublayers each read a weighted root-mean-square norm (kind 'rmsnorm')")
        if len({float(n.eps) for n in norms}) != 1:
            raise ValueError("a parallel pair's norms share their root mean square: one epsilon")
        if ffn is not None and not (hasattr(ffn, "begin") and hasattr(ffn, "finish")):
            raise ValueError("a parallel pair needs a feed-forward in two halves (begin / finish)")
        self.eps, self.width = float(norm_mixer.eps), norm_mixer.width
        self.n_sub = len(norms)
        self.norm_weights = torch.stack([n.weight for n in norms]).contiguous()
        convs = [input_conv] + ([self.ffn_conv] if ffn is not None else [])
        self.taps = max((int(c.taps) for c in convs if c is not None), default=0)
        self.conv_weights = None
        if self.taps:
            if any(c is not None and int(c.taps) != self.taps for c in convs):
                raise ValueError("a parallel pair's convolutions have one number of taps")
            zero = torch.zeros((self.width, self.taps), dtype=torch.float32, device=self.norm_weights.device)
            # [sublayers, taps, width]: a tap's channels side by side, as the kernel reads them
            self.conv_weights = torch.stack([c.weight if c is not None else zero for c in convs]).transpose(1, 2).contiguous()
        self.ring_floats = max(self.taps - 1, 0) * self.n_sub * self.width
        own = mixer.state_spec()
        if own is not None and (len(own.shape) != 1 or own.dtype != "float32"):
            raise ValueError("a parallel pair keeps its mixer's state behind its own in one flat 32-bit vector a slot")
        self.mixer_floats = int(own.shape[0]) if own is not None else 0

    def state_spec(self):
        from ..cache.pages import StateSpec

        total = self.ring_floats + self.mixer_floats
        return StateSpec((total,)) if total else None

    def forward(self, x: torch.Tensor, ctx: StepContext, cache, state, writes_cache: bool = True):
        ws, n, d, S = ctx.workspace, x.shape[0], x.shape[1], self.n_sub
        if ctx.phases is not None:
            ctx.phases.mark(self.mixer_phase)
        ring = ops.StateSlice(state, 0, self.ring_floats) if self.ring_floats else None
        h = ws.get("pair_in", (S, n, d), self.dtype)
        # (a step of single tokens: each row takes its place in the ring inside the kernel that reads the ring)
        single = ring is not None and writes_cache and ops.single_token_step(ctx)
        kept = ws.get("pair_normed", (n, S * d), torch.float32) if ring is not None and writes_cache and not single else None
        ops.norm_shift(h, x, self.norm_weights, 0.0, self.eps, self.conv_weights, ring, ctx, hbuf=kept, keep_single=single)
        # everything that reads the ring has run: the step's last rows take their places in it
        if kept is not None:
            ops.ring_keep(ring, self.taps - 1, kept, ctx)
        begun = self.ffn.begin(h[1], ctx) if self.ffn is not None else None
        mixer_state = ops.StateSlice(state, self.ring_floats, self.mixer_floats) if self.mixer_floats else None
        self.mixer.forward(h[0], ctx, cache, mixer_state, x, writes_cache=writes_cache)
        if self.ffn is not None:
            if ctx.phases is not None:
                ctx.phases.mark(self.ffn_phase)
            self.ffn.finish(begun, ctx, x)
        return None


register_block("parallel_pair", ParallelPairBlock)
