"""A plain, slow Dopilorn: whole sequences, no cache, no carried state, float64, one function a mechanism.

It shares no code with `liyab_amd`: it takes a dict of numpy tensors by their file names and config.json
as a dict, and computes with numpy from the design's equations. In this file's notation (x: the residual
stream, rows = tokens; unit(v) = v / sqrt(mean(v^2) + eps); s: the logistic function):

  x0      = embed[token]
  run:      the layers in their order; a stretch [start, stop) of them runs `times` times over with the same tensors.
            Ahead of every pass t of the stretch: x <- Win [x ; x0] + step[t]
  layer:    hm = shift(unit(x) (1 + n1), canon1), hf = shift(unit(x) (1 + n2), canon2)
            x <- x + mixer(hm) + feed_forward(hf)
            shift(h, c)_t = h_t + sum_j c[:, j] h_(t - taps + 1 + j)          (rows before the first are zero)
  logits  = cap tanh((head (unit(x) (1 + nf))) / cap)

  feed-forward:  z = Wup h;  Wdown (a unit(z) + b unit(z^2) + c unit(z^3) + e)       (powers entry by entry)

  mixer "general_delta":  r, k, v = W h a head; decay d = exp(-exp(-1/2) s(W2 tanh(W1 h) + w0)); rate a = s(Wa h + ba);
      u = k / sqrt(sum(k^2) + 1e-6); state S [key, value], from zero:  S <- diag(d) S - (a u)(u^T S) + k v^T  (both read
      the old S);  o = S^T r;  Wo (unit(o) a head * weight * s(Wg h))
  mixer "attention":  q, k, v = W h + b, then each channel through a causal convolution over time (y_t = sum_j c[:, j] u_(t - taps
      + 1 + j)); a query head holds two maps [q1 | q2], a key head [k1 | k2]; both maps attend over the same values under
      a window of `size` positions with an ordinary softmax;  o = a1 - lam a2,  lam = exp(lq1 . lk1) - exp(lq2 . lk2) + diff;
      Wo (unit(o) a head * (1 - diff))
  mixer "latent_attention":  q = Wuq (unit(Wdq h) nq);  c = unit(Wdkv h) nc;  k = Wuk c, v = Wuv c a head;
      causal softmax of scale q.k;  a head's result times s(Wg h)_head;  Wo
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


def unit(v, eps):
    """v / sqrt(mean(v^2) + eps) over the last axis."""
    return v / np.sqrt((v * v).mean(axis=-1, keepdims=True) + eps)


def offset_norm(x, w, eps):
    """unit(x) * (1 + w): the weight is stored around zero."""
    return unit(x, eps) * (1.0 + w)


def time_conv(u, c):
    """y_t = sum_j c[:, j] * u_(t - taps + 1 + j) on each channel, rows before the first being zero. u [n, channels], c [channels, taps]."""
    n, taps = u.shape[0], c.shape[1]
    y = np.zeros_like(u)
    for j in range(taps):
        back = taps - 1 - j
        if back < n:
            y[back:] += u[:n - back] * c[:, j]
    return y


def poly_norm(z, act, eps):
    a, b, c, e = (float(v) for v in act)
    return a * unit(z, eps) + b * unit(z * z, eps) + c * unit(z * z * z, eps) + e


def feed_forward(h, t, prefix, eps):
    return poly_norm(h @ t[prefix + "up"].T, t[prefix + "act"], eps) @ t[prefix + "down"].T


def windowed_softmax(scores, window):
    """scores [n, n]: row i over columns j with 0 <= i - j < window (window 0: every j <= i)."""
    n = scores.shape[0]
    dist = np.arange(n)[:, None] - np.arange(n)[None, :]
    seen = (dist >= 0) & ((dist < window) if window else True)
    s = np.where(seen, scores, -np.inf)
    p = np.exp(s - s.max(axis=-1, keepdims=True))
    return p / p.sum(axis=-1, keepdims=True)


def general_delta(h, t, p, m, eps):
    H, D = m["heads"], m["dim"]
    n = h.shape[0]
    r = (h @ t[p + "r"].T).reshape(n, H, D)
    k = (h @ t[p + "k"].T).reshape(n, H, D)
    v = (h @ t[p + "v"].T).reshape(n, H, D)
    decay = np.exp(-math.exp(-0.5) * logistic(np.tanh(h @ t[p + "w1"].T) @ t[p + "w2"].T + t[p + "w0"])).reshape(n, H, D)
    rate = logistic(h @ t[p + "a"].T + t[p + "a.b"]).reshape(n, H, D)
    u = k / np.sqrt((k * k).sum(axis=-1, keepdims=True) + 1e-6)
    o = np.zeros((n, H, D))
    for head in range(H):
        S = np.zeros((D, D))
        for i in range(n):
            seen = u[i, head] @ S  # [value]
            S = decay[i, head][:, None] * S - np.outer(rate[i, head] * u[i, head], seen) + np.outer(k[i, head], v[i, head])
            o[i, head] = r[i, head] @ S
    o = unit(o, eps).reshape(n, H * D) * t[p + "norm"] * logistic(h @ t[p + "g"].T)
    return o @ t[p + "o"].T


def differential_attention(h, t, p, m, eps):
    H, D = m["heads"], m["dim"]
    G, V = m.get("kv_heads", H), m.get("vdim", D)
    window = (m.get("mask") or {}).get("size", 0)
    diff = float(m["diff"])
    n = h.shape[0]
    q = h @ t[p + "q"].T + t[p + "q.b"]
    k = h @ t[p + "k"].T + t[p + "k.b"]
    v = h @ t[p + "v"].T + t[p + "v.b"]
    if p + "q.conv" in t:
        q, k, v = time_conv(q, t[p + "q.conv"]), time_conv(k, t[p + "k.conv"]), time_conv(v, t[p + "v.conv"])
    q, k, v = q.reshape(n, H, 2, D), k.reshape(n, G, 2, D), v.reshape(n, G, V)
    lam = math.exp(float(t[p + "lq1"] @ t[p + "lk1"])) - math.exp(float(t[p + "lq2"] @ t[p + "lk2"])) + diff
    out = np.zeros((n, H, V))
    for head in range(H):
        g = head // (H // G)
        maps = [windowed_softmax(q[:, head, i] @ k[:, g, i].T * m["scale"], window) @ v[:, g] for i in range(2)]
        out[:, head] = unit(maps[0] - lam * maps[1], eps) * (1.0 - diff)
    return out.reshape(n, H * V) @ t[p + "o"].T


def latent_attention(h, t, p, m, eps):
    H, D, V = m["heads"], m["dim"], m["vdim"]
    n = h.shape[0]
    q = ((unit(h @ t[p + "dq"].T, eps) * t[p + "dq.norm"]) @ t[p + "uq"].T).reshape(n, H, D)
    c = unit(h @ t[p + "dkv"].T, eps) * t[p + "dkv.norm"]
    k = (c @ t[p + "uk"].T).reshape(n, H, D)
    v = (c @ t[p + "uv"].T).reshape(n, H, V)
    gate = logistic(h @ t[p + "g"].T)  # [n, H]
    out = np.zeros((n, H, V))
    for head in range(H):
        out[:, head] = windowed_softmax(q[:, head] @ k[:, head].T * m["scale"], 0) @ v[:, head] * gate[:, head:head + 1]
    return out.reshape(n, H * V) @ t[p + "o"].T


MIXERS = {"general_delta": general_delta, "attention": differential_attention, "latent_attention": latent_attention}


def run_order(cfg):
    """[(layer, pass or None)]: a layer's number, and which pass of the looped stretch begins with this run."""
    L = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop or loop["times"] < 1 or loop["stop"] <= loop["start"]:
        return [(i, None) for i in range(L)]
    out = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        out += [(i, t if i == loop["start"] else None) for i in range(loop["start"], loop["stop"])]
    return out + [(i, None) for i in range(loop["stop"], L)]


def layer(x, t, i, entry, cfg):
    eps = cfg["norm"]["eps"]
    p = f"l{i}."
    hm = offset_norm(x, t[p + "norm1"], eps)
    if cfg.get("canon"):
        hm = hm + time_conv(hm, t[p + "canon1"])
    y = MIXERS[entry["type"]](hm, t, p + "mix.", entry["mixer"], eps)
    if entry.get("mlp") is not None:
        hf = offset_norm(x, t[p + "norm2"], eps)
        if cfg.get("canon"):
            hf = hf + time_conv(hf, t[p + "canon2"])
        y = y + feed_forward(hf, t, p + "mlp.", eps)
    return x + y


def forward(tokens, t, cfg, streams=None):
    """Logits [n, vocab] of one sequence; `streams`, a list, gets the stream after every layer run."""
    x0 = t["embed"][np.asarray(tokens)]
    x = x0
    for i, begins in run_order(cfg):
        if begins is not None:
            x = np.concatenate([x, x0], axis=-1) @ t["loop.in"].T + t["loop.step"][begins]
        x = layer(x, t, i, cfg["layers"][i], cfg)
        if streams is not None:
            streams.append(x)
    logits = offset_norm(x, t["final.norm"], cfg["norm"]["eps"]) @ t["head"].T
    cap = cfg.get("logit_softcap")
    return cap * np.tanh(logits / cap) if cap else logits
