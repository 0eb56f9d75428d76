"""The model plan: what an architecture's configuration turns into.

A plan is plain data. It lists the parts of each layer (mixer, feed-forward,
norms, position encoding) with their sizes and constants, the tensors each
part reads, and the order in which layers run. The engine builds parts from
a plan through the part registries and never looks at the architecture's
name again. The reference does the same with `ModelConfig` + one `BlockPlan`
per block (`src/compat/architecture.h:282-380, 452-630`): per-block mixer
kind, feed-forward kind, head counts, width and attention scale.

Every spec class carries a `kind` string; a registry maps the kind to the
part's class (`liyab_amd.parts.registry`). New kinds need no change here:
any dataclass with a `kind` attribute can stand in a `LayerSpec`.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Optional, Sequence


@dataclass(frozen=True)
class Init:
    """How the random-weights mode draws a tensor: N(mean, std)."""

    std: float
    mean: float = 0.0


@dataclass(frozen=True)
class TensorSource:
    """Where a part's tensor lives in the weights file.

    `layout` says how a matrix is stored: "out_in" = row per output feature
    (the reference's and this engine's working layout: `y = x . W^T`,
    `include/liyab/backend.h:35`), "in_out" = row per input feature (GPT-2's
    four projection matrices). The loader brings every matrix to "out_in".
    `init` is the distribution the random-weights mode draws the tensor from
    (None: N(0, 0.02)).
    """

    name: str
    layout: str = "out_in"
    required: bool = True
    init: Optional[Init] = None


@dataclass(frozen=True)
class NormSpec:
    kind: str  # "layernorm" | "rmsnorm" (weight only) | "dyt" (tanh(alpha x) * weight + bias: tensors weight, bias, alpha)
    width: int
    eps: float
    tensors: dict = field(default_factory=dict)  # "weight", "bias"
    # what is added to the stored weight before it multiplies (a weight stored around zero: 1.0); "rmsnorm" takes it
    weight_offset: float = 0.0


@dataclass(frozen=True)
class TokenEmbeddingSpec:
    kind: str  # "token_embedding"
    vocab_size: int
    width: int
    scale: float
    tensors: dict = field(default_factory=dict)  # "table"


@dataclass(frozen=True)
class PositionSpec:
    """A position encoding. `where` = "residual" (added to the embeddings, as learned
    positions are: the model's `residual_position`) or "mixer" (applied to queries and keys
    inside a mixer: that mixer's `position` field; the part then has `rotate(q, k, ctx)`)."""

    kind: str  # "learned_positions" | "none"
    where: str
    max_positions: int
    width: int
    tensors: dict = field(default_factory=dict)  # "table"


@dataclass(frozen=True)
class AttentionSpec:
    kind: str  # "attention"
    width: int
    n_head: int
    n_kv_head: int
    head_dim: int
    scale: float  # multiplies q.k before the softmax
    window: int  # 0 = every earlier position
    tensors: dict = field(default_factory=dict)  # qkv_weight, qkv_bias, out_weight, out_bias
    # a position encoding that acts on queries and keys (a spec with a `kind` of the position
    # registry and where = "mixer"), applied after the projection and before keys go to the cache
    position: Any = None


@dataclass(frozen=True)
class DenseFFNSpec:
    kind: str  # "dense_ffn"
    width: int
    inner: int
    activation: str  # "gelu_tanh" | "gelu_erf"
    tensors: dict = field(default_factory=dict)  # up_weight, up_bias, down_weight, down_bias


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Attention over one compressed row a position: the row c (`rank` wide, normalised) is what the cache
    keeps, and each head's keys (`head_dim` wide) and values (`value_dim` wide) are linear in it. No
    position enters the scores. `window` as in AttentionSpec; `gated`: the heads' outputs are
    multiplied by the sigmoid of a projection of the mixer's input before the output projection
    (`gate_a_head`: that projection has one row a head, whose sigmoid multiplies the head's whole
    output). `q_rank` > 0: queries go through a latent of their own, q = Wuq (rmsnorm(Wdq h) * w)."""

    kind: str  # "latent_attention"
    width: int
    n_head: int
    head_dim: int
    value_dim: int
    rank: int
    scale: float
    window: int  # 0 = every earlier position
    eps: float  # of the compressed row's norm
    gated: bool = True
    tensors: dict = field(default_factory=dict)  # q (or q_down, q_down_norm, q_up), down, down_norm, up_k, up_v, gate, out
    q_rank: int = 0
    gate_a_head: bool = False


@dataclass(frozen=True)
class RoutedFFNSpec:
    """A mixture of gated feed-forward units: each token takes the `top` experts with the largest router
    logits, weighted by the softmax over those logits alone. Expert: down(act(gate h) * (up h)).
    `gated` False: an expert is down(act(up h)) (activation "relu2": the square of the positive part).
    `groups` = (count, keep): scores are the softmax over all experts; the experts form `count` equal groups of
    neighbours, a group's score is its largest, and only experts of the `keep` best groups can be chosen; the
    weights are the chosen scores divided by their sum. `shared_inner` > 0: one more expert of the same form
    and that inner width runs for every token with weight one (tensors shared_up, shared_down, and shared_gate
    if gated)."""

    kind: str  # "routed_ffn"
    width: int
    inner: int
    n_experts: int
    top: int
    activation: str  # "silu" | "relu2"
    tensors: dict = field(default_factory=dict)  # router, router_bias, and per expert e: ("gate", e), ("up", e), ("down", e)
    gated: bool = True
    groups: Optional[tuple] = None  # (count, keep)
    shared_inner: int = 0


@dataclass(frozen=True)
class CausalConvSpec:
    """A causal convolution over time on each channel of what a sublayer reads: h <- h + conv(h),
    `taps` inputs back; the last taps - 1 inputs are part of a request's state."""

    kind: str  # "causal_conv"
    width: int
    taps: int
    tensors: dict = field(default_factory=dict)  # "weight" [width, taps]


@dataclass(frozen=True)
class GateSpec:
    """A gate on a sublayer's result: result * sigmoid(W h + b), h the sublayer's input."""

    kind: str  # "sigmoid_gate"
    width: int
    tensors: dict = field(default_factory=dict)  # "weight" [width, width], "bias"


@dataclass(frozen=True)
class RotarySpec:
    """Pairs (2i, 2i + 1) of the first `dims` entries of a head turned by position * f_i, f_i = base^(-2i / dims);
    `scaling` (factor, low, high, original) stretches the long wavelengths: f stays where the wavelength is under
    original / high, becomes f / factor where it is over original / low, and is blended in between.
    `halves`: the pairs are (i, i + dims / 2) instead. `ramp` (factor, fast, slow, original): the other way of stretching, by the
    entry's number: with at(t) = dims ln(original / (2 pi t)) / (2 ln base), lo = max(floor(at(fast)), 0), hi = min(ceil(at(slow)),
    dims - 1) and r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), f_i becomes f_i / factor * r_i + f_i (1 - r_i), and cosine and
    sine are multiplied by `ramp_magnitude` * ln(factor) + 1."""

    dims: int
    base: float
    scaling: Optional[tuple] = None  # (factor, low, high, original)
    halves: bool = False
    ramp: Optional[tuple] = None  # (factor, fast, slow, original)
    ramp_magnitude: float = 0.1


@dataclass(frozen=True)
class ScoredAttentionSpec:
    """Attention over paged keys and values whose queries, keys and scores are worked on: keys `head_dim` wide, values
    `value_dim`; each of these optional: a root-mean-square norm of every query and key head (`qk_norm`, weights shared by
    the heads), a rotary encoding (`rotary`), a factor on the query that grows with the position's logarithm (`q_temp` =
    (coef, every): 1 + coef * ln(floor((p + 1) / every) + 1)), a soft cap on the scores (`softcap`: cap * tanh(score / cap)),
    a learned bias by distance (`distance_bias` = the distance from which the table's last row holds; the table's rows:
    the distance itself below half of them, then logarithmic steps), values that are the keys as projected
    (`values_are_keys`), a sigmoid gate on the heads' results from a projection of the mixer's input (`gated`), biases on
    the three projections (`biased`), a learned logit a head that joins the softmax's denominator with no key and no value
    (`sink`), values shared between layers (`value_mix`: "first" = this layer's values, as projected, are kept for the later
    layers of the same step; "later" = v <- (1 - lam) v + lam v_first with the learned scalar `vmix`, and the mixed values are
    what is cached)."""

    kind: str  # "scored_attention"
    width: int
    n_head: int
    n_kv_head: int
    head_dim: int
    value_dim: int
    scale: float
    eps: float
    window: int = 0
    softcap: float = 0.0
    qk_norm: bool = False
    rotary: Optional[RotarySpec] = None
    q_temp: Optional[tuple] = None  # (coef, every)
    distance_bias: int = 0  # 0: none
    bias_rows: int = 0
    values_are_keys: bool = False
    gated: bool = False
    tensors: dict = field(default_factory=dict)  # q, k, v, gate, out, q_norm, k_norm, rel, q_bias, k_bias, v_bias, sink, vmix
    biased: bool = False
    sink: bool = False
    value_mix: str = ""  # "" | "first" | "later"


@dataclass(frozen=True)
class WKVSpec:
    """A mixer that carries a matrix of state a head: five learned mixes of a token's input with the one before it feed
    receptance, key, value, gate and a low-rank decay (`decay_rank` wide); o = (S + diag(u) k v^T)^T r, S <- diag(w) S + k v^T;
    each head's result brought to unit root mean square, times a weight and silu(gate), then the output projection."""

    kind: str  # "wkv"
    width: int
    n_head: int
    head_dim: int
    decay_rank: int
    eps: float
    tensors: dict = field(default_factory=dict)  # mu_r, mu_k, mu_v, mu_g, mu_w, r, k, v, g, w1, w2, w0, u, norm, out


@dataclass(frozen=True)
class StateSpaceSpec:
    """A selective state-space mixer: one projection gives [z | x | B | C | dt]; x, B and C pass a short causal convolution
    (`taps`) with a bias and silu; per head S <- exp(-exp(A_log) dt) S + dt B x^T with dt = softplus(dt + dt_bias), y = S^T C +
    D x; y * silu(z) is brought to unit root mean square in `norm_groups` equal parts, times a weight, then the output
    projection. Heads share B and C in `n_groups` groups."""

    kind: str  # "state_space"
    width: int
    n_head: int
    head_dim: int
    n_state: int
    n_groups: int
    taps: int
    norm_groups: int
    eps: float
    tensors: dict = field(default_factory=dict)  # in, conv, conv_bias, dt_bias, A_log, D, norm, out


@dataclass(frozen=True)
class SideBySideSpec:
    """Two mixers that read the same input; the result is `weight` times the sum of their results, each brought to unit
    root mean square over the model's width first and multiplied by a weight of its own. Without `normed`: the results as
    they are, left_weight * left + right_weight * right, and no tensors."""

    kind: str  # "side_by_side"
    width: int
    left: Any
    right: Any
    eps: float
    weight: float = 0.5
    tensors: dict = field(default_factory=dict)  # left_out, right_out
    normed: bool = True
    left_weight: float = 1.0
    right_weight: float = 1.0


@dataclass(frozen=True)
class GatedRecurrenceSpec:
    """A recurrent block with a linear recurrence a channel under real gates: two branches `inner` wide, y = gelu_tanh(Wy h + by)
    and u = conv(Wx h + bx) (a causal convolution of `taps` taps a channel with a bias, no activation; its last taps - 1 inputs are
    part of a request's state); u in `blocks` equal parts, in each r = sigmoid(Ra u + ba) and i = sigmoid(Ri u + bi) with square
    matrices; a = exp(-rate * r * softplus(lam)); S <- a S + sqrt(1 - a^2) i u from S = 0; the output projection of S * y."""

    kind: str  # "gated_recurrence"
    width: int
    inner: int
    blocks: int
    taps: int
    rate: float = 8.0
    tensors: dict = field(default_factory=dict)  # y, y_bias, x, x_bias, conv, conv_bias, gate_r, gate_r_bias, gate_i, gate_i_bias, lam, out


@dataclass(frozen=True)
class ClampedGLUSpec:
    """A gated feed-forward whose halves are clamped before they meet: g = min(Wg h, limit), u = clamp(Wu h, -limit, limit),
    down(g * sigmoid(slope * g) * (u + shift))."""

    kind: str  # "clamped_glu"
    width: int
    inner: int
    limit: float
    slope: float = 1.702
    shift: float = 1.0
    tensors: dict = field(default_factory=dict)  # gate, up, down


@dataclass(frozen=True)
class DeltaRuleSpec:
    """A mixer that carries a matrix of state a head and both decays it and takes out of it what its key already holds: with
    the unit key u = k / sqrt(sum(k^2) + key_eps), a decay w = exp(-decay_scale * sigmoid(W2 tanh(W1 h) + w0)) and a removal
    rate a = sigmoid(Wa h + ba) a head and key channel, S <- diag(w) S - (a * u)(u^T S) + k v^T (both terms read the old S),
    o = S^T r; each head's o brought to unit root mean square, times a weight and sigmoid(Wg h), then the output projection."""

    kind: str  # "delta_rule"
    width: int
    n_head: int
    head_dim: int
    decay_rank: int
    eps: float
    decay_scale: float = 0.6065306597126334  # exp(-1/2)
    key_eps: float = 1e-6
    tensors: dict = field(default_factory=dict)  # r, k, v, a, a_bias, g, w1, w2, w0, norm, out


@dataclass(frozen=True)
class DifferentialAttentionSpec:
    """Attention in two maps a head that share their values: queries and keys hold [map 1 | map 2] a head, each map an
    ordinary softmax attention under the window, and a head's result is o = a1 - lam * a2 with lam = exp(lq1 . lk1) -
    exp(lq2 . lk2) + lam_init, brought to unit root mean square over the head (no weight) and multiplied by `out_scale`.
    `conv_taps` > 0: every channel of the projected q, k and v passes a causal convolution over time first, whose last
    taps - 1 inputs are part of a request's state."""

    kind: str  # "differential_attention"
    width: int
    n_head: int
    n_kv_head: int
    head_dim: int
    value_dim: int
    scale: float
    window: int  # 0 = every earlier position
    lam_init: float
    out_scale: float
    eps: float
    conv_taps: int = 0
    tensors: dict = field(default_factory=dict)  # q, q_bias, k, k_bias, v, v_bias, q_conv, k_conv, v_conv, lq1, lk1, lq2, lk2, out


@dataclass(frozen=True)
class NormedPowersFFNSpec:
    """A feed-forward whose activation is a learned mix of the first `len(act)` - 1 powers of its input, each brought to unit root
    mean square over the inner width: down(c_1 N(z) + c_2 N(z^2) + ... + c_last), z = up h, powers entry by entry."""

    kind: str  # "normed_powers_ffn"
    width: int
    inner: int
    eps: float
    powers: int = 3
    tensors: dict = field(default_factory=dict)  # up, act [powers + 1], down


@dataclass(frozen=True)
class ReentrySpec:
    """What happens to the stream ahead of a layer at which a repeated stretch of layers begins a pass: x <- W [x ; x0] + steps[index],
    x0 being the embedding's output, W [width, 2 width] and `steps` one row a pass."""

    kind: str  # "reentry"
    width: int
    index: int
    passes: int
    tensors: dict = field(default_factory=dict)  # weight, steps


@dataclass(frozen=True)
class LayerSpec:
    """One block: which parts it has and how they are arranged.

    arrangement "pre_norm": x += mixer(norm_mixer(x)); x += ffn(norm_ffn(x)).
    arrangement "parallel": h = norm_mixer(x); x += mixer(h) + ffn(h): one norm, both sublayers read its output.
    arrangement "post_norm_gated": x += norm_mixer(gate_mixer * mixer(conv(x))); x += norm_ffn(gate_ffn *
    ffn(x)): the sublayers read the stream itself, the norms stand on their results; `input_conv`
    (what the mixer reads is first convolved over time) and the gates are optional.
    arrangement "parallel_pair": x += mixer(c1(norm_mixer(x))) + ffn(c2(norm_ffn(x))): two norms of the same x, each
    followed by a convolution over time of its own (`input_conv`, `ffn_conv`: h <- h + conv(h); optional).
    arrangement "sandwich": x += post_norm_mixer(mixer(norm_mixer(x))); x += post_norm_ffn(ffn(norm_ffn(x))): a norm before and
    a norm behind each sublayer.
    `entry`: what is done to the stream before the layer runs (a spec of the entry registry), or None.
    """

    mixer: Any
    ffn: Any
    norm_mixer: Any
    norm_ffn: Any
    arrangement: str = "pre_norm"
    input_conv: Any = None
    gate_mixer: Any = None
    gate_ffn: Any = None
    ffn_conv: Any = None
    entry: Any = None
    post_norm_mixer: Any = None
    post_norm_ffn: Any = None


@dataclass(frozen=True)
class OrderEntry:
    """One entry of the run order. `layer` indexes `ModelPlan.layers`;
    `cache_of` names the layer whose cache this run reads and writes
    (itself unless another layer's cache is shared)."""

    layer: int
    cache_of: Optional[int] = None
    writes_cache: bool = True

    @property
    def cache_layer(self) -> int:
        return self.layer if self.cache_of is None else self.cache_of


@dataclass(frozen=True)
class HeadSpec:
    kind: str  # "lm_head"
    width: int
    vocab_size: int
    logit_scale: float
    tensors: dict = field(default_factory=dict)  # "weight" (may name the embedding table), "bias"
    softcap: float = 0.0  # > 0: logits <- softcap * tanh(logits / softcap), last of all


@dataclass(frozen=True)
class ModelPlan:
    architecture: str
    width: int
    vocab_size: int
    max_positions: int
    embedding: TokenEmbeddingSpec
    residual_position: Optional[PositionSpec]
    layers: Sequence[LayerSpec]
    order: Sequence[OrderEntry]
    final_norm: Any
    head: HeadSpec
    # tensor-name patterns (fnmatch) that a file may hold and the engine ignores
    ignorable: Sequence[str] = ()
    # prefixes that may stand before every tensor name in a file
    name_prefixes: Sequence[str] = ("",)
    eos_token_id: Optional[int] = None
