"""A plain, slow Larulorn: whole sequences, no cache, no carried state, float64, one function a mechanism.

It shares no code with `liyab_amd`: it takes a dict of numpy tensors by their file names and config.json
as a dict, and computes with numpy from the design's equations. In this file's notation (x: the residual
stream, rows = tokens; p: a row's position; unit(v) = v / sqrt(mean(v^2) + eps); s: the logistic function):

  x_0     = embed[token]
  layer:    x <- x + unit(mixer(unit(x) w1)) w1b
            x <- x + unit(ff(unit(x) w2)) w2b                          (a layer may have no feed-forward)
  logits  = logit_scale * head (unit(x) w_f)

  mixer "attention": q, k, v = W h + b a head; the first rot.dims entries of q and k turned in pairs (i, i + dims / 2) by
      p f_i (the slow f_i divided by `factor` along a ramp, cosine and sine times 0.1 ln(factor) + 1); in layers that mix
      values, but the first of them, v <- (1 - lam) v + lam v_first; weights exp(scale q.k) over j <= i, divided by their sum
      plus exp(sink) of the head; Wo.
  mixer "parallel":  left_scale * left(h) + right_scale * right(h)
      left:  q, k, v = W h; the same turn without the ramp; ordinary causal softmax; heads times s(Wg h); Wo.
      right: y = gelu(Wy h + by); u = conv(Wx h + bx) + bc over time; in `blocks` parts r = s(Ra u + ba), i = s(Ri u + bi);
             a = exp(-8 r softplus(lam)); S <- a S + sqrt(1 - a^2) i u from S = 0; Wo (S y).
  feed-forward "dense": g = min(Wg h, L), u = clip(Wu h, -L, L), Wd (g s(1.702 g) (u + 1))
  feed-forward "moe":   z = Wr h, s = softmax(z); experts in groups.count groups of neighbours, a group's score its largest
      s, the best groups.keep groups stay; of their experts the `top` largest s, weights s / (sum + 1e-20);
      sum of weight * Wd relu(Wu h)^2, plus a shared expert of the same form for every token.
"""

from __future__ import annotations

import math

import numpy as np


def round_to_bf16(a):
    """float -> the nearest bfloat16 (ties to even), as float64."""
    f = np.ascontiguousarray(a, dtype=np.float32)
    bits = f.view(np.uint32).astype(np.uint64)
    bits = (bits + 0x7FFF + ((bits >> 16) & 1)) & 0xFFFF0000
    return bits.astype(np.uint32).view(np.float32).astype(np.float64).reshape(np.shape(a))


def logistic(z):
    return 1.0 / (1.0 + np.exp(-z))


def softplus(z):
    return np.logaddexp(0.0, z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def unit(v, eps):
    """v / sqrt(mean(v^2) + eps) over the last axis."""
    return v / np.sqrt((v * v).mean(axis=-1, keepdims=True) + eps)


def turn_frequencies(rot):
    """(f [dims / 2], factor on cosine and sine): f_i = base^(-2i / dims), the slow ones divided along a ramp."""
    dims, base = rot["dims"], rot["base"]
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, orig = sc["factor"], sc["original"]

    def at(turns):
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(at(sc["fast"])), 0)
    hi = min(math.ceil(at(sc["slow"])), dims - 1)
    ramp = np.clip((np.arange(dims // 2) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def turn_halves(v, positions, rot):
    """v [n, heads, dim]: pairs (i, i + dims / 2) of the first rot.dims entries turned by position * f_i."""
    f, mag = turn_frequencies(rot)
    half = rot["dims"] // 2
    a = positions[:, None] * f[None, :]
    c, s = (np.cos(a) * mag)[:, None, :], (np.sin(a) * mag)[:, None, :]
    out = v.copy()
    lo, hi = v[..., :half], v[..., half:2 * half]
    out[..., :half] = lo * c - hi * s
    out[..., half:2 * half] = hi * c + lo * s
    return out


def causal_weights(scores, sink=None):
    """scores [n, n]: row i over columns j <= i; with `sink`, exp(sink) joins every row's denominator."""
    n = scores.shape[0]
    seen = np.arange(n)[None, :] <= np.arange(n)[:, None]
    s = np.where(seen, scores, -np.inf)
    top = s.max(axis=-1, keepdims=True)
    if sink is not None:
        top = np.maximum(top, sink)
    p = np.exp(s - top)
    total = p.sum(axis=-1, keepdims=True)
    if sink is not None:
        total = total + np.exp(sink - top)
    return p / total


def heads_attend(q, k, v, scale, sinks=None):
    """q [n, H, D], k [n, G, D], v [n, G, V] -> [n, H * V]."""
    n, H, G = q.shape[0], q.shape[1], k.shape[1]
    out = np.zeros((n, H, v.shape[-1]))
    for hd in range(H):
        g = hd // (H // G)
        w = causal_weights((q[:, hd] @ k[:, g].T) * scale, None if sinks is None else float(sinks[hd]))
        out[:, hd] = w @ v[:, g]
    return out.reshape(n, -1)


def sink_attention(h, t, prefix, m, positions, first_values):
    """`first_values`: a one-entry list holding the values of the first layer that mixes them (None before it has run)."""
    n = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ t[prefix + "q"].T + t[prefix + "q.b"]).reshape(n, H, D)
    k = (h @ t[prefix + "k"].T + t[prefix + "k.b"]).reshape(n, G, D)
    v = (h @ t[prefix + "v"].T + t[prefix + "v.b"]).reshape(n, G, V)
    if m.get("rot"):
        q, k = turn_halves(q, positions, m["rot"]), turn_halves(k, positions, m["rot"])
    if m.get("v_mix"):
        if first_values[0] is None:
            first_values[0] = v
        else:
            lam = float(t[prefix + "vmix"])
            v = (1.0 - lam) * v + lam * first_values[0]
    return heads_attend(q, k, v, m["scale"], t[prefix + "sink"]) @ t[prefix + "o"].T


def gated_attention(h, t, prefix, m, positions):
    n = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ t[prefix + "q"].T).reshape(n, H, D)
    k = (h @ t[prefix + "k"].T).reshape(n, G, D)
    v = (h @ t[prefix + "v"].T).reshape(n, G, V)
    if m.get("rot"):
        q, k = turn_halves(q, positions, m["rot"]), turn_halves(k, positions, m["rot"])
    return (heads_attend(q, k, v, m["scale"]) * logistic(h @ t[prefix + "g"].T)) @ t[prefix + "o"].T


def short_convolution(x, w, bias):
    """x [n, channels], w [channels, taps] (last column: the current row), zeros before the first row."""
    n, taps = x.shape[0], w.shape[1]
    padded = np.concatenate([np.zeros((taps - 1, x.shape[1])), x])
    out = np.zeros_like(x) + bias
    for j in range(taps):
        out += w[:, j] * padded[j:j + n]
    return out


def gated_recurrence(h, t, prefix, m):
    n, W, B = h.shape[0], m["width"], m["blocks"]
    y = gelu_tanh(h @ t[prefix + "y"].T + t[prefix + "y.b"])
    u = short_convolution(h @ t[prefix + "x"].T + t[prefix + "x.b"], t[prefix + "conv"], t[prefix + "conv.b"])
    ub = u.reshape(n, B, W // B)
    r = logistic(np.einsum("boi,nbi->nbo", t[prefix + "ra"], ub) + t[prefix + "ra.b"]).reshape(n, W)
    gate = logistic(np.einsum("boi,nbi->nbo", t[prefix + "ri"], ub) + t[prefix + "ri.b"]).reshape(n, W)
    a = np.exp(-8.0 * r * softplus(t[prefix + "lam"]))
    S = np.zeros(W)
    out = np.zeros((n, W))
    for i in range(n):
        S = a[i] * S + np.sqrt(1.0 - a[i] ** 2) * gate[i] * u[i]
        out[i] = S
    return (out * y) @ t[prefix + "o"].T


def parallel_mixer(h, t, prefix, m, positions):
    return m["left_scale"] * gated_attention(h, t, prefix + "left.", m["left"], positions) \
        + m["right_scale"] * gated_recurrence(h, t, prefix + "right.", m["right"])


def dense_feed_forward(h, t, prefix, m):
    L = m["limit"]
    g = np.minimum(h @ t[prefix + "gate"].T, L)
    u = np.clip(h @ t[prefix + "up"].T, -L, L)
    return (g * logistic(1.702 * g) * (u + 1.0)) @ t[prefix + "down"].T


def squared_relu_expert(h, t, prefix):
    return np.maximum(h @ t[prefix + "up"].T, 0.0) ** 2 @ t[prefix + "down"].T


def route(z, top, groups, keep):
    """z [n, E] router logits -> (chosen [n, top], weights [n, top])."""
    n, E = z.shape
    s = np.exp(z - z.max(axis=-1, keepdims=True))
    s = s / s.sum(axis=-1, keepdims=True)
    per = E // groups
    chosen, weights = np.zeros((n, top), dtype=np.int64), np.zeros((n, top))
    for i in range(n):
        best = np.argsort(-s[i].reshape(groups, per).max(axis=-1), kind="stable")[:keep]
        allowed = np.full(E, -1.0)
        for g in best:
            allowed[g * per:(g + 1) * per] = s[i, g * per:(g + 1) * per]
        chosen[i] = np.argsort(-allowed, kind="stable")[:top]
        picked = s[i, chosen[i]]
        weights[i] = picked / (picked.sum() + 1e-20)
    return chosen, weights


def routed_feed_forward(h, t, prefix, m, router_input=None):
    r = m["router"]
    E, top = r["experts"], r["top"]
    groups = r.get("groups") or {"count": 1, "keep": 1}
    z = (h if router_input is None else router_input) @ t[prefix + "router"].T
    chosen, weights = route(z, top, groups["count"], groups["keep"])
    out = np.zeros((h.shape[0], t[prefix + "e0.down"].shape[0]))
    for i in range(h.shape[0]):
        for e, w in zip(chosen[i], weights[i]):
            out[i] += w * squared_relu_expert(h[i:i + 1], t, f"{prefix}e{e}.")[0]
    if m.get("shared") is not None:
        out += squared_relu_expert(h, t, prefix + "shared.")
    return out


def forward(config, t, tokens, streams=None):
    """float64 logits [n, vocab] of a whole sequence; `streams` (a list) gets the stream after every layer."""
    tokens = np.asarray(tokens)
    positions = np.arange(len(tokens), dtype=np.float64)
    eps = config["norm"]["eps"]
    x = t["embed"][tokens].astype(np.float64)
    first_values = [None]
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        h = unit(x, eps) * t[p + "norm1"]
        if layer["type"] == "attention":
            y = sink_attention(h, t, p + "mix.", layer["mixer"], positions, first_values)
        elif layer["type"] == "parallel":
            y = parallel_mixer(h, t, p + "mix.", layer["mixer"], positions)
        else:
            raise ValueError(layer["type"])
        x = x + unit(y, eps) * t[p + "norm1b"]
        mlp = layer.get("mlp")
        if mlp is not None:
            h = unit(x, eps) * t[p + "norm2"]
            y = dense_feed_forward(h, t, p + "mlp.", mlp) if mlp["kind"] == "dense" else routed_feed_forward(h, t, p + "mlp.", mlp)
            x = x + unit(y, eps) * t[p + "norm2b"]
        if streams is not None:
            streams.append(x.copy())
    return (unit(x, eps) * t["final.norm"]) @ t["head"].T * config["logit_scale"]
