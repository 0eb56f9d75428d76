"""Larulorn's typed configuration, read from its own config.json keys.

A decoder whose layers have a root-mean-square norm before and behind each sublayer: x <- x + n1b(mixer(n1(x))), then
x <- x + n2b(ff(n2(x))). No position table: positions enter inside the mixers. A layer's mixer is one of two kinds, its
feed-forward one of two or none. config.json:

    architecture     "Larulorn"
    vocab, width
    norm.eps         the epsilon of every norm
    logit_scale      the factor on the logits
    max_positions    optional: the longest context (nothing in the design bounds it; default 32,768)
    layers[i]        type, mixer {...}, mlp (null, {kind "dense", ff, limit} or {kind "moe", expert {ff}, router {experts, top,
                     groups {count, keep} (optional)}, shared {ff} (optional)})
      type "attention": mixer {heads, kv_heads, dim, vdim, scale, rot {dims, base, scaling {factor, original, fast, slow} (optional)}
                     (optional), v_mix (optional)}: biases on q, k and v, a sink a head in the softmax, values mixed with those of
                     the first layer that says v_mix
      type "parallel":  mixer {left {heads, kv_heads, dim, vdim, scale, rot {...} (optional)}, right {width, blocks, conv},
                     left_scale, right_scale}: gated attention beside a recurrent block with a gated linear recurrence

Tensors: embed, final.norm, head; layer i's start with "l<i>.": norm1, norm1b, norm2, norm2b, and
  attention: mix.{q, q.b, k, k.b, v, v.b, sink, o} and mix.vmix where values are mixed
  parallel:  mix.left.{q, k, v, g, o}, mix.right.{y, y.b, x, x.b, conv, conv.b, ra, ra.b, ri, ri.b, lam, o}
  dense:     mlp.{gate, up, down};  moe: mlp.router, mlp.e<k>.{up, down}, mlp.shared.{up, down}
Matrices are stored [out, in]; the recurrence's gates [blocks, out, in].
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, Optional, Tuple

from ..errors import InvalidModel, Unsupported
from .plan import (
    ClampedGLUSpec,
    GatedRecurrenceSpec,
    HeadSpec,
    Init,
    LayerSpec,
    ModelPlan,
    NormSpec,
    OrderEntry,
    RotarySpec,
    RoutedFFNSpec,
    ScoredAttentionSpec,
    SideBySideSpec,
    TensorSource,
    TokenEmbeddingSpec,
)
from .registry import register_architecture

_LIMIT = 1 << 24
DEFAULT_MAX_POSITIONS = 1 << 15
# what the design fixes
RECURRENCE_RATE = 8.0  # log a = -8 r softplus(lam)
GLU_SLOPE, GLU_SHIFT = 1.702, 1.0  # g * sigmoid(1.702 g) * (u + 1)
RAMP_MAGNITUDE = 0.1  # cosine and sine times 0.1 ln(factor) + 1


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
class LarulornAttention:
    n_head: int
    n_kv_head: int
    head_dim: int
    value_dim: int
    scale: float
    rot_dims: int  # 0: no rotary encoding
    rot_base: float
    rot_ramp: Optional[Tuple[float, float, float, float]]  # factor, fast, slow, original
    v_mix: bool = False


@dataclass(frozen=True)
class LarulornRecurrence:
    inner: int
    blocks: int
    taps: int


@dataclass(frozen=True)
class LarulornParallel:
    left: LarulornAttention
    right: LarulornRecurrence
    left_scale: float
    right_scale: float


@dataclass(frozen=True)
class LarulornMLP:
    kind: str  # "dense" | "moe"
    ff: int  # dense: the inner width; moe: an expert's
    limit: float = 0.0  # dense
    experts: int = 0
    top: int = 0
    groups: int = 1
    keep: int = 1
    shared_ff: int = 0  # 0: no shared expert


@dataclass(frozen=True)
class LarulornLayer:
    kind: str  # "attention" | "parallel"
    mixer: Any  # LarulornAttention | LarulornParallel
    mlp: Optional[LarulornMLP]


def _attention(m, where: str, mixes: bool) -> LarulornAttention:
    if not isinstance(m, dict):
        raise InvalidModel(f"missing or invalid {where}")
    H, G = _int(m, "heads", where + ".heads"), _int(m, "kv_heads", where + ".kv_heads")
    if H % G:
        raise InvalidModel(f"invalid {where}: {H} heads are no multiple of {G} kv_heads")
    D = _int(m, "dim", where + ".dim")
    rot = m.get("rot")
    dims, base, ramp = 0, 0.0, None
    if rot is not None:
        dims, base = _int(rot, "dims", where + ".rot.dims"), _number(rot, "base", where + ".rot.base")
        if dims % 2 or dims > D:
            raise InvalidModel(f"invalid {where}.rot: {dims} turned entries of heads of {D}")
        sc = rot.get("scaling") if isinstance(rot, dict) else None
        if sc is not None:
            ramp = tuple(_number(sc, k, f"{where}.rot.scaling.{k}") for k in ("factor", "fast", "slow", "original"))
            if base == 1.0:
                raise InvalidModel(f"invalid {where}.rot: a ramp over the entries needs a base other than one")
    v_mix = m.get("v_mix", False)
    if not isinstance(v_mix, bool) or (v_mix and not mixes):
        raise InvalidModel(f"invalid {where}.v_mix")
    return LarulornAttention(n_head=H, n_kv_head=G, head_dim=D, value_dim=_int(m, "vdim", where + ".vdim"), scale=_number(m, "scale", where + ".scale"),
                             rot_dims=dims, rot_base=base, rot_ramp=ramp, v_mix=v_mix)


def _mlp(raw, where: str) -> Optional[LarulornMLP]:
    if raw is None:
        return None
    kind = raw.get("kind") if isinstance(raw, dict) else None
    if kind == "dense":
        return LarulornMLP(kind="dense", ff=_int(raw, "ff", where + ".ff"), limit=_number(raw, "limit", where + ".limit"))
    if kind == "moe":
        r = raw.get("router")
        E, top = _int(r, "experts", where + ".router.experts"), _int(r, "top", where + ".router.top")
        g = r.get("groups") if isinstance(r, dict) else None
        count, keep = (_int(g, "count", where + ".router.groups.count"), _int(g, "keep", where + ".router.groups.keep")) if g is not None else (1, 1)
        if E % count or keep > count or top > keep * (E // count):
            raise InvalidModel(f"invalid {where}.router: {top} of {E} experts in {keep} of {count} groups")
        shared = raw.get("shared")
        return LarulornMLP(kind="moe", ff=_int(raw.get("expert"), "ff", where + ".expert.ff"), experts=E, top=top, groups=count, keep=keep,
                           shared_ff=_int(shared, "ff", where + ".shared.ff") if shared is not None else 0)
    raise Unsupported(f"{where}.kind '{kind}' is not supported (supported: dense, moe)")


@dataclass(frozen=True)
class LarulornConfig:
    vocab: int
    width: int
    eps: float
    logit_scale: float
    max_positions: int
    layers: Tuple[LarulornLayer, ...]

    architecture = "Larulorn"

    @classmethod
    def from_json(cls, raw: dict) -> "LarulornConfig":
        vocab, width = _int(raw, "vocab", "vocab"), _int(raw, "width", "width")
        eps = _number(raw.get("norm"), "eps", "norm.eps")
        logit_scale = _number(raw, "logit_scale", "logit_scale") if raw.get("logit_scale") is not None else 1.0
        max_positions = _int(raw, "max_positions", "max_positions") if raw.get("max_positions") is not None else DEFAULT_MAX_POSITIONS
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise InvalidModel("missing or invalid layers")
        layers = []
        for i, entry in enumerate(listed):
            if not isinstance(entry, dict):
                raise InvalidModel(f"invalid layers[{i}]")
            kind, m, where = entry.get("type"), entry.get("mixer"), f"layers[{i}].mixer"
            if not isinstance(m, dict):
                raise InvalidModel(f"missing or invalid {where}")
            if kind == "attention":
                mixer = _attention(m, where, mixes=True)
            elif kind == "parallel":
                r = m.get("right")
                right = LarulornRecurrence(inner=_int(r, "width", where + ".right.width"), blocks=_int(r, "blocks", where + ".right.blocks"),
                                           taps=_int(r, "conv", where + ".right.conv"))
                if right.inner % right.blocks:
                    raise InvalidModel(f"invalid {where}.right: {right.inner} channels are no multiple of {right.blocks} blocks")
                mixer = LarulornParallel(left=_attention(m.get("left"), where + ".left", mixes=False), right=right,
                                         left_scale=_number(m, "left_scale", where + ".left_scale", positive=False),
                                         right_scale=_number(m, "right_scale", where + ".right_scale", positive=False))
            else:
                raise Unsupported(f"layers[{i}].type '{kind}' is not supported (supported: attention, parallel)")
            layers.append(LarulornLayer(kind=kind, mixer=mixer, mlp=_mlp(entry.get("mlp"), f"layers[{i}].mlp")))
        shared = {(layer.mixer.n_kv_head, layer.mixer.value_dim) for layer in layers if layer.kind == "attention" and layer.mixer.v_mix}
        if len(shared) > 1:
            raise InvalidModel("invalid layers: the layers that mix values do not have values of one shape")
        return cls(vocab=vocab, width=width, eps=eps, logit_scale=logit_scale, max_positions=max_positions, layers=tuple(layers))

    @staticmethod
    def _attention_json(a: LarulornAttention) -> dict:
        out = {"heads": a.n_head, "kv_heads": a.n_kv_head, "dim": a.head_dim, "vdim": a.value_dim, "scale": a.scale}
        if a.rot_dims:
            out["rot"] = {"dims": a.rot_dims, "base": a.rot_base}
            if a.rot_ramp is not None:
                out["rot"]["scaling"] = dict(zip(("factor", "fast", "slow", "original"), a.rot_ramp))
        return out

    def to_json(self) -> dict:
        layers = []
        for layer in self.layers:
            m = layer.mixer
            if layer.kind == "attention":
                mixer = self._attention_json(m)
                if m.v_mix:
                    mixer["v_mix"] = True
            else:
                mixer = {"left": self._attention_json(m.left), "right": {"width": m.right.inner, "blocks": m.right.blocks, "conv": m.right.taps},
                         "left_scale": m.left_scale, "right_scale": m.right_scale}
            f, mlp = layer.mlp, None
            if f is not None and f.kind == "dense":
                mlp = {"kind": "dense", "ff": f.ff, "limit": f.limit}
            elif f is not None:
                mlp = {"kind": "moe", "expert": {"ff": f.ff}, "router": {"experts": f.experts, "top": f.top, "groups": {"count": f.groups, "keep": f.keep}}}
                if f.shared_ff:
                    mlp["shared"] = {"ff": f.shared_ff}
            layers.append({"type": layer.kind, "mixer": mixer, "mlp": mlp})
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
                "logit_scale": self.logit_scale, "max_positions": self.max_positions, "layers": layers}

    def plan(self) -> ModelPlan:
        d, V = self.width, self.vocab
        wide = Init(1.0 / math.sqrt(d))

        def norm(name: str) -> NormSpec:
            return NormSpec(kind="rmsnorm", width=d, eps=self.eps, tensors={"weight": TensorSource(name, init=Init(0.1, 1.0))})

        layers = []
        first_mix = next((i for i, layer in enumerate(self.layers) if layer.kind == "attention" and layer.mixer.v_mix), None)
        for i, layer in enumerate(self.layers):
            p = f"l{i}"
            m = layer.mixer
            if layer.kind == "attention":
                mixer = self._attention_spec(p + ".mix", m, wide, plain=False, value_mix=("first" if i == first_mix else "later") if m.v_mix else "")
            else:
                left = self._attention_spec(p + ".mix.left", m.left, wide, plain=True, value_mix="")
                W, B, r = m.right.inner, m.right.blocks, p + ".mix.right"
                per = W // B
                right = GatedRecurrenceSpec(kind="gated_recurrence", width=d, inner=W, blocks=B, taps=m.right.taps, rate=RECURRENCE_RATE, tensors={
                    "y": TensorSource(r + ".y", init=wide), "y_bias": TensorSource(r + ".y.b", init=Init(0.1)),
                    "x": TensorSource(r + ".x", init=wide), "x_bias": TensorSource(r + ".x.b", init=Init(0.1)),
                    "conv": TensorSource(r + ".conv", init=Init(0.4)), "conv_bias": TensorSource(r + ".conv.b", init=Init(0.1)),
                    "gate_r": TensorSource(r + ".ra", init=Init(1.0 / math.sqrt(per))), "gate_r_bias": TensorSource(r + ".ra.b", init=Init(0.5)),
                    "gate_i": TensorSource(r + ".ri", init=Init(1.0 / math.sqrt(per))), "gate_i_bias": TensorSource(r + ".ri.b", init=Init(0.5)),
                    "lam": TensorSource(r + ".lam", init=Init(1.0, -2.0)), "out": TensorSource(r + ".o", init=Init(1.0 / math.sqrt(W)))})
                mixer = SideBySideSpec(kind="side_by_side", width=d, left=left, right=right, eps=self.eps, normed=False,
                                       left_weight=m.left_scale, right_weight=m.right_scale)
            f, ffn = layer.mlp, None
            if f is not None and f.kind == "dense":
                ffn = ClampedGLUSpec(kind="clamped_glu", width=d, inner=f.ff, limit=f.limit, slope=GLU_SLOPE, shift=GLU_SHIFT, tensors={
                    "gate": TensorSource(p + ".mlp.gate", init=wide), "up": TensorSource(p + ".mlp.up", init=wide),
                    "down": TensorSource(p + ".mlp.down", init=Init(1.0 / math.sqrt(f.ff)))})
            elif f is not None:
                tensors = {"router": TensorSource(p + ".mlp.router", init=Init(4.0 / math.sqrt(d)))}
                for e in range(f.experts):
                    tensors[("up", e)] = TensorSource(f"{p}.mlp.e{e}.up", init=wide)
                    tensors[("down", e)] = TensorSource(f"{p}.mlp.e{e}.down", init=Init(1.0 / math.sqrt(f.ff)))
                if f.shared_ff:
                    tensors["shared_up"] = TensorSource(p + ".mlp.shared.up", init=wide)
                    tensors["shared_down"] = TensorSource(p + ".mlp.shared.down", init=Init(1.0 / math.sqrt(f.shared_ff)))
                ffn = RoutedFFNSpec(kind="routed_ffn", width=d, inner=f.ff, n_experts=f.experts, top=f.top, activation="relu2", gated=False,
                                    groups=(f.groups, f.keep), shared_inner=f.shared_ff, tensors=tensors)
            layers.append(LayerSpec(mixer=mixer, ffn=ffn, norm_mixer=norm(p + ".norm1"), norm_ffn=norm(p + ".norm2") if ffn is not None else None,
                                    arrangement="sandwich", post_norm_mixer=norm(p + ".norm1b"),
                                    post_norm_ffn=norm(p + ".norm2b") if ffn is not None else None))
        return ModelPlan(
            architecture=self.architecture, width=d, vocab_size=V, max_positions=self.max_positions,
            embedding=TokenEmbeddingSpec(kind="token_embedding", vocab_size=V, width=d, scale=1.0, tensors={"table": TensorSource("embed", init=Init(1.0))}),
            residual_position=None,
            layers=layers,
            order=[OrderEntry(layer=i) for i in range(len(layers))],
            final_norm=norm("final.norm"),
            head=HeadSpec(kind="lm_head", width=d, vocab_size=V, logit_scale=self.logit_scale, tensors={"weight": TensorSource("head", init=wide)}),
            # (a layer without a feed-forward may still carry its norms, and one that mixes no values its rate)
            ignorable=("l*.norm2", "l*.norm2b", "l*.mix.vmix"), name_prefixes=("",), eos_token_id=None,
        )

    def _attention_spec(self, p: str, m: LarulornAttention, wide: Init, plain: bool, value_mix: str) -> ScoredAttentionSpec:
        """`plain`: the attention beside the recurrence (no biases, no sink, an output gate); otherwise the layer's own."""
        H, G, D, Vd = m.n_head, m.n_kv_head, m.head_dim, m.value_dim
        tensors = {"q": TensorSource(p + ".q", init=wide), "k": TensorSource(p + ".k", init=wide), "v": TensorSource(p + ".v", init=wide),
                   "out": TensorSource(p + ".o", init=Init(1.0 / math.sqrt(H * Vd)))}
        if plain:
            tensors["gate"] = TensorSource(p + ".g", init=wide)
        else:
            tensors.update({"q_bias": TensorSource(p + ".q.b", init=Init(0.1)), "k_bias": TensorSource(p + ".k.b", init=Init(0.1)),
                            "v_bias": TensorSource(p + ".v.b", init=Init(0.1)), "sink": TensorSource(p + ".sink", init=Init(1.0))})
            if value_mix:
                tensors["vmix"] = TensorSource(p + ".vmix", init=Init(0.1, 0.4))
        rotary = RotarySpec(dims=m.rot_dims, base=m.rot_base, halves=True, ramp=m.rot_ramp, ramp_magnitude=RAMP_MAGNITUDE) if m.rot_dims else None
        return ScoredAttentionSpec(kind="scored_attention", width=self.width, n_head=H, n_kv_head=G, head_dim=D, value_dim=Vd, scale=m.scale, eps=self.eps,
                                   rotary=rotary, gated=plain, biased=not plain, sink=not plain, value_mix=value_mix, tensors=tensors)


register_architecture("Larulorn", LarulornConfig)
