"""Dopilorn's typed configuration, read from its own config.json keys.

A decoder of parallel layers with two norms: the mixer and the feed-forward each read a root-mean-square norm of their own
(weights stored around zero) of the same stream, each through a short convolution over time, and their results are added to
the stream together. A stretch of the layers may run several times over with the same tensors, the stream re-entering it
through a product with the embedding's output beside it. No position enters anywhere. config.json:

    architecture   "Dopilorn"
    vocab, width
    norm.eps       the epsilon of every root-mean-square norm
    canon.taps     the taps of the two input convolutions of a layer (no `canon`: none)
    logit_softcap  optional: logits <- cap * tanh(logits / cap)
    loop           optional {start, stop, times}: layers start .. stop - 1 run `times` times in a row; every pass has its own
                   cache and state, and begins with x <- loop.in [x ; embedding output] + loop.step[pass]
    max_positions  optional: the longest context (nothing in the design bounds it; default 32,768)
    layers[i]      type, mixer {...}, mlp (null, or {kind "dense", ff})
      type "general_delta":    mixer {heads, dim}; the decay's rank is the shape of mix.w1
      type "attention":        mixer {heads, kv_heads, dim, vdim, scale, diff, conv (taps; optional), mask.size (optional)}
      type "latent_attention": mixer {heads, dim, vdim, kv_rank, q_rank, scale}

Tensors: embed, loop.in, loop.step, final.norm, head; layer i's start with "l<i>.": norm1, norm2, canon1, canon2,
mlp.{up, down, act}, and
  general_delta:    mix.{r, k, v, a, a.b, g, w1, w2, w0, norm, o}
  attention:        mix.{q, k, v}(.b, .conv), mix.{lq1, lk1, lq2, lk2, o}
  latent_attention: mix.{dq, dq.norm, uq, dkv, dkv.norm, uk, uv, g, o}
Matrices are stored [out, in].
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, Optional, Tuple

from ..errors import InvalidModel, Unsupported
from .plan import (
    CausalConvSpec,
    DeltaRuleSpec,
    DifferentialAttentionSpec,
    HeadSpec,
    Init,
    LatentAttentionSpec,
    LayerSpec,
    ModelPlan,
    NormedPowersFFNSpec,
    NormSpec,
    OrderEntry,
    ReentrySpec,
    TensorSource,
    TokenEmbeddingSpec,
)
from .registry import register_architecture

_LIMIT = 1 << 24
DEFAULT_MAX_POSITIONS = 1 << 15
DEFAULT_DECAY_RANK = 16


def _int(raw, key: str, what: str, least: int = 1) -> int:
    v = raw.get(key) if isinstance(raw, dict) else None
    if isinstance(v, bool) or not isinstance(v, int) or v < least or v > _LIMIT:
        raise InvalidModel(f"missing or invalid {what}")
    return v


def _number(raw, key: str, what: str, positive: bool = True) -> float:
    v = raw.get(key) if isinstance(raw, dict) else None
    if isinstance(v, bool) or not isinstance(v, (int, float)) or not math.isfinite(v) or (positive and v <= 0):
        raise InvalidModel(f"missing or invalid {what}")
    return float(v)


@dataclass(frozen=True)
class DopilornDelta:
    n_head: int
    head_dim: int
    decay_rank: int


@dataclass(frozen=True)
class DopilornAttention:
    n_head: int
    n_kv_head: int
    head_dim: int
    value_dim: int
    scale: float
    diff: float
    taps: int  # 0: q, k and v go to attention as projected
    window: int  # 0: every earlier position


@dataclass(frozen=True)
class DopilornLatent:
    n_head: int
    head_dim: int
    value_dim: int
    kv_rank: int
    q_rank: int
    scale: float


@dataclass(frozen=True)
class DopilornLayer:
    kind: str  # "general_delta" | "attention" | "latent_attention"
    mixer: Any
    ff: int  # 0: no feed-forward


@dataclass(frozen=True)
class DopilornLoop:
    start: int
    stop: int
    times: int


KINDS = ("attention", "general_delta", "latent_attention")


@dataclass(frozen=True)
class DopilornConfig:
    vocab: int
    width: int
    eps: float
    taps: int  # 0: no input convolutions
    softcap: float  # 0: none
    loop: Optional[DopilornLoop]
    max_positions: int
    layers: Tuple[DopilornLayer, ...]

    architecture = "Dopilorn"

    @classmethod
    def from_json(cls, raw: dict, shapes: Optional[dict] = None) -> "DopilornConfig":
        """`shapes`: tensor name -> shape, for the one size that only a tensor's shape gives (the rank of a decay); without it
        config.json's optional key `decay_rank` is read."""
        vocab, width = _int(raw, "vocab", "vocab"), _int(raw, "width", "width")
        eps = _number(raw.get("norm"), "eps", "norm.eps")
        taps = _int(raw.get("canon"), "taps", "canon.taps") if raw.get("canon") is not None else 0
        softcap = _number(raw, "logit_softcap", "logit_softcap") if raw.get("logit_softcap") is not None else 0.0
        max_positions = _int(raw, "max_positions", "max_positions") if raw.get("max_positions") is not None else DEFAULT_MAX_POSITIONS
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise InvalidModel("missing or invalid layers")
        layers = []
        for i, entry in enumerate(listed):
            if not isinstance(entry, dict):
                raise InvalidModel(f"invalid layers[{i}]")
            kind, m, where = entry.get("type"), entry.get("mixer"), f"layers[{i}].mixer"
            if kind not in KINDS:
                raise Unsupported(f"layers[{i}].type '{kind}' is not supported (supported: {', '.join(KINDS)})")
            if not isinstance(m, dict):
                raise InvalidModel(f"missing or invalid {where}")
            H, D = _int(m, "heads", where + ".heads"), _int(m, "dim", where + ".dim")
            if kind == "general_delta":
                rank = m.get("decay_rank")
                name = f"l{i}.mix.w1"
                if shapes is not None and name in shapes and len(shapes[name]) == 2:
                    rank = int(shapes[name][0])
                mixer = DopilornDelta(n_head=H, head_dim=D, decay_rank=rank if isinstance(rank, int) and not isinstance(rank, bool) and rank > 0 else DEFAULT_DECAY_RANK)
            elif kind == "attention":
                G = _int(m, "kv_heads", where + ".kv_heads") if m.get("kv_heads") is not None else H
                if H % G:
                    raise InvalidModel(f"invalid {where}: {H} heads are no multiple of {G} kv_heads")
                mask = m.get("mask")
                window = _int(mask, "size", where + ".mask.size") if mask is not None and (not isinstance(mask, dict) or mask.get("size") is not None) else 0
                mixer = DopilornAttention(
                    n_head=H, n_kv_head=G, head_dim=D, value_dim=_int(m, "vdim", where + ".vdim") if m.get("vdim") is not None else D,
                    scale=_number(m, "scale", where + ".scale"), diff=_number(m, "diff", where + ".diff", positive=False),
                    taps=_int(m, "conv", where + ".conv") if m.get("conv") is not None else 0, window=window)
            else:
                mixer = DopilornLatent(n_head=H, head_dim=D, value_dim=_int(m, "vdim", where + ".vdim") if m.get("vdim") is not None else D,
                                       kv_rank=_int(m, "kv_rank", where + ".kv_rank"), q_rank=_int(m, "q_rank", where + ".q_rank"),
                                       scale=_number(m, "scale", where + ".scale"))
            mlp = entry.get("mlp")
            ff = 0
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") != "dense":
                    raise Unsupported(f"layers[{i}].mlp.kind '{mlp.get('kind') if isinstance(mlp, dict) else mlp}' is not supported (supported: dense)")
                ff = _int(mlp, "ff", f"layers[{i}].mlp.ff")
            layers.append(DopilornLayer(kind=kind, mixer=mixer, ff=ff))
        loop = None
        if raw.get("loop") is not None:
            lp = raw["loop"]
            loop = DopilornLoop(start=_int(lp, "start", "loop.start", 0), stop=_int(lp, "stop", "loop.stop", 0), times=_int(lp, "times", "loop.times", 0))
            if not loop.start <= loop.stop <= len(layers):
                raise InvalidModel(f"invalid loop: layers {loop.start} to {loop.stop} of {len(layers)}")
        return cls(vocab=vocab, width=width, eps=eps, taps=taps, softcap=softcap, loop=loop, max_positions=max_positions, layers=tuple(layers))

    def to_json(self) -> dict:
        layers = []
        for layer in self.layers:
            m = layer.mixer
            if layer.kind == "general_delta":
                mixer = {"heads": m.n_head, "dim": m.head_dim, "decay_rank": m.decay_rank}
            elif layer.kind == "attention":
                mixer = {"heads": m.n_head, "kv_heads": m.n_kv_head, "dim": m.head_dim, "vdim": m.value_dim, "scale": m.scale, "diff": m.diff}
                if m.taps:
                    mixer["conv"] = m.taps
                if m.window:
                    mixer["mask"] = {"size": m.window}
            else:
                mixer = {"heads": m.n_head, "dim": m.head_dim, "vdim": m.value_dim, "kv_rank": m.kv_rank, "q_rank": m.q_rank, "scale": m.scale}
            layers.append({"type": layer.kind, "mixer": mixer, "mlp": {"kind": "dense", "ff": layer.ff} if layer.ff else None})
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
               "max_positions": self.max_positions, "layers": layers}
        if self.taps:
            out["canon"] = {"taps": self.taps}
        if self.softcap:
            out["logit_softcap"] = self.softcap
        if self.loop is not None:
            out["loop"] = {"start": self.loop.start, "stop": self.loop.stop, "times": self.loop.times}
        return out

    def runs(self):
        """[(layer, pass that begins here or None)] in the order the layers run."""
        n, loop = len(self.layers), self.loop
        if loop is None:
            return [(i, None) for i in range(n)]
        out = [(i, None) for i in range(loop.start)]
        for t in range(loop.times):
            out += [(i, t if i == loop.start else None) for i in range(loop.start, loop.stop)]
        return out + [(i, None) for i in range(loop.stop, n)]

    def plan(self) -> ModelPlan:
        d, V = self.width, self.vocab
        wide = Init(1.0 / math.sqrt(d))

        def norm(name: str) -> NormSpec:
            return NormSpec(kind="rmsnorm", width=d, eps=self.eps, weight_offset=1.0, tensors={"weight": TensorSource(name, init=Init(0.1))})

        def conv(name: str):
            return CausalConvSpec(kind="causal_conv", width=d, taps=self.taps, tensors={"weight": TensorSource(name, init=Init(0.3))}) if self.taps else None

        # A layer that runs several times is listed once a run, with the same tensor names (the weights' store hands every
        # run the same device tensors) and a cache and state of its own.
        layers = []
        for i, begins in self.runs():
            layer, p = self.layers[i], f"l{i}"
            m = layer.mixer
            if layer.kind == "general_delta":
                H, D, R = m.n_head, m.head_dim, m.decay_rank
                mixer = DeltaRuleSpec(kind="delta_rule", width=d, n_head=H, head_dim=D, decay_rank=R, eps=self.eps, tensors={
                    **{c: TensorSource(f"{p}.mix.{c}", init=wide) for c in ("r", "k", "v", "a", "g", "w1")},
                    "a_bias": TensorSource(p + ".mix.a.b", init=Init(0.5)),
                    "w2": TensorSource(p + ".mix.w2", init=Init(1.0 / math.sqrt(R))), "w0": TensorSource(p + ".mix.w0", init=Init(1.0, -1.0)),
                    "norm": TensorSource(p + ".mix.norm", init=Init(0.1, 1.0)), "out": TensorSource(p + ".mix.o", init=Init(1.0 / math.sqrt(H * D)))})
            elif layer.kind == "attention":
                H, G, D, Vd = m.n_head, m.n_kv_head, m.head_dim, m.value_dim
                tensors = {"out": TensorSource(p + ".mix.o", init=Init(1.0 / math.sqrt(H * Vd)))}
                for c in "qkv":
                    tensors[c] = TensorSource(f"{p}.mix.{c}", init=wide)
                    tensors[c + "_bias"] = TensorSource(f"{p}.mix.{c}.b", init=Init(0.2))
                    if m.taps:
                        tensors[c + "_conv"] = TensorSource(f"{p}.mix.{c}.conv", init=Init(0.5))
                for c in ("lq1", "lk1", "lq2", "lk2"):
                    tensors[c] = TensorSource(f"{p}.mix.{c}", init=Init(0.1))
                mixer = DifferentialAttentionSpec(kind="differential_attention", width=d, n_head=H, n_kv_head=G, head_dim=D, value_dim=Vd, scale=m.scale,
                                                  window=m.window, lam_init=m.diff, out_scale=1.0 - m.diff, eps=self.eps, conv_taps=m.taps, tensors=tensors)
            else:
                H, D, Vd, R, Q = m.n_head, m.head_dim, m.value_dim, m.kv_rank, m.q_rank
                mixer = LatentAttentionSpec(
                    kind="latent_attention", width=d, n_head=H, head_dim=D, value_dim=Vd, rank=R, scale=m.scale, window=0, eps=self.eps,
                    gated=True, gate_a_head=True, q_rank=Q, tensors={
                        "q_down": TensorSource(p + ".mix.dq", init=wide), "q_down_norm": TensorSource(p + ".mix.dq.norm", init=Init(0.1, 1.0)),
                        "q_up": TensorSource(p + ".mix.uq", init=Init(1.0 / math.sqrt(Q))),
                        "down": TensorSource(p + ".mix.dkv", init=wide), "down_norm": TensorSource(p + ".mix.dkv.norm", init=Init(0.1, 1.0)),
                        "up_k": TensorSource(p + ".mix.uk", init=Init(1.0 / math.sqrt(R))), "up_v": TensorSource(p + ".mix.uv", init=Init(1.0 / math.sqrt(R))),
                        "gate": TensorSource(p + ".mix.g", init=wide), "out": TensorSource(p + ".mix.o", init=Init(1.0 / math.sqrt(H * Vd)))})
            ffn = None
            if layer.ff:
                ffn = NormedPowersFFNSpec(kind="normed_powers_ffn", width=d, inner=layer.ff, eps=self.eps, powers=3, tensors={
                    "up": TensorSource(p + ".mlp.up", init=wide), "act": TensorSource(p + ".mlp.act", init=Init(0.5, 0.3)),
                    "down": TensorSource(p + ".mlp.down", init=Init(1.0 / math.sqrt(layer.ff)))})
            entry = None
            if begins is not None:
                entry = ReentrySpec(kind="reentry", width=d, index=begins, passes=self.loop.times, tensors={
                    "weight": TensorSource("loop.in", init=Init(1.0 / math.sqrt(2 * d))), "steps": TensorSource("loop.step", init=Init(0.3))})
            layers.append(LayerSpec(mixer=mixer, ffn=ffn, norm_mixer=norm(p + ".norm1"), norm_ffn=norm(p + ".norm2") if ffn is not None else None,
                                    arrangement="parallel_pair", input_conv=conv(p + ".canon1"), ffn_conv=conv(p + ".canon2") if ffn is not None else None,
                                    entry=entry))
        ignorable = []
        for i, layer in enumerate(self.layers):  # a layer without a feed-forward may still hold the norm and convolution nobody reads
            if not layer.ff:
                ignorable += [f"l{i}.norm2", f"l{i}.canon2"]
        if not any(begins is not None for _, begins in self.runs()):
            ignorable += ["loop.in", "loop.step"]
        return ModelPlan(
            architecture=self.architecture, width=d, vocab_size=V, max_positions=self.max_positions,
            embedding=TokenEmbeddingSpec(kind="token_embedding", vocab_size=V, width=d, scale=1.0, tensors={"table": TensorSource("embed", init=Init(1.0))}),
            residual_position=None,
            layers=layers,
            order=[OrderEntry(layer=i) for i in range(len(layers))],
            final_norm=norm("final.norm"),
            head=HeadSpec(kind="lm_head", width=d, vocab_size=V, logit_scale=1.0, softcap=self.softcap, tensors={"weight": TensorSource("head", init=wide)}),
            ignorable=tuple(ignorable), name_prefixes=("",), eos_token_id=None,
        )


register_architecture("Dopilorn", DopilornConfig)
