"""Dopilorn through the engine against its plain twin (`plain_dopilorn.py`): each mechanism alone, then whole models of
several geometries under every way of cutting and batching the work, in 32-bit and in bfloat16 (needs the GPU). The
geometries differ from each other in every size, in the order of their layers and in what is repeated; one has sizes no
kernel tiles evenly, one no attention at all (no cache group), one nothing but attention, one neither convolutions nor a
repeated stretch nor a cap."""

import json
import math
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_dopilorn as plain
import trace_tools as tt
from conftest import ROOT, TOL
from plain_gpt2 import read_model

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = ["float32", "bfloat16"]
# float32: the largest difference of a row relative to its largest |logit|, as for the other models.
# bfloat16, against the twin in float64 with the same rounded matrices: the root mean square of a row's difference over
# that of the row's logits, both with their means taken off (what a softmax sees of them); a fault in a mechanism makes
# it about 1.
TOL_B = {"float32": TOL["float32"], "bfloat16": 6e-2}
KEPT_32BIT = ("canon1", "canon2", ".conv", "loop.step")  # 2-D tensors that the engine keeps in 32 bits


def check_logits(got, reqs, ref, dtype, what, family=None):
    if dtype == "float32":
        return tt.check_against_plain(got, reqs, ref, TOL_B[dtype], what, family=family)
    key = ((family or what.split(" ")[0]) + " (rms)", TOL_B[dtype])
    for rid, toks in reqs.items():
        assert rid in got, f"{what}: no logits for request {rid}"
        for p in sorted(got[rid]):
            row, want = np.asarray(got[rid][p], dtype=np.float64), ref[rid][p]
            assert np.isfinite(row).all(), f"{what}: request {rid} position {p}: non-finite logits"
            diff = row - want
            e = float(np.sqrt(np.mean((diff - diff.mean()) ** 2)) / np.sqrt(np.mean((want - want.mean()) ** 2)))
            tt.WORST[key] = max(tt.WORST.get(key, 0.0), e)
            assert e <= TOL_B[dtype], f"{what}: request {rid} (length {len(toks)}) first differs at position {p}: {e:.3e} > {TOL_B[dtype]:.1e}"


# ---------------------------------------------------------------------------
# configurations
# ---------------------------------------------------------------------------
def delta(heads, dim, rank):
    return {"heads": heads, "dim": dim, "decay_rank": rank}


def maps(heads, kv_heads, dim, vdim, diff, conv=None, window=None, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5, "diff": diff}
    if conv:
        m["conv"] = conv
    if window:
        m["mask"] = {"size": window}
    return m


def latent(heads, dim, vdim, kv_rank, q_rank, scale=None):
    return {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale if scale is not None else dim ** -0.5}


def layer(kind, m, ff=None):
    return {"type": kind, "mixer": m, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def config(vocab, width, eps, layers, taps=None, cap=None, loop=None):
    raw = {"architecture": "Dopilorn", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if taps:
        raw["canon"] = {"taps": taps}
    if cap:
        raw["logit_softcap"] = cap
    if loop:
        raw["loop"] = dict(zip(("start", "stop", "times"), loop))
    return raw


CONFIGS = {
    # every kind of layer, the middle two three times over, a layer without a feed-forward, a window shorter than a page
    "mix": (config(300, 96, 1e-5, [
        layer("latent_attention", latent(4, 24, 16, 40, 32), ff=160),
        layer("general_delta", delta(3, 32, 8), ff=128),
        layer("attention", maps(4, 2, 16, 24, 0.3, conv=3, window=11), ff=64),
        layer("general_delta", delta(2, 16, 4), None),
    ], taps=4, cap=12.0, loop=(1, 3, 3)), 41),
    # sizes that no kernel tiles evenly; the whole model once over as its "loop"; two taps; a window of one
    "odd": (config(211, 100, 1e-6, [
        layer("attention", maps(3, 3, 6, 10, 0.7, conv=2, window=1), ff=50),
        layer("latent_attention", latent(3, 10, 6, 12, 7, scale=0.4), ff=30),
        layer("general_delta", delta(5, 12, 7), ff=30),
    ], taps=2, cap=30.0, loop=(0, 3, 1)), 42),
    # no attention anywhere: no cache group, state only; five taps; the last layer alone twice
    "recurrent": (config(128, 64, 1e-5, [layer("general_delta", delta(1, 64, 16), ff=96), layer("general_delta", delta(4, 8, 1), ff=40)],
                         taps=5, loop=(1, 2, 2)), 43),
    # attention only, no convolution anywhere (no state at all), no repeated stretch, no cap; every earlier position and a long window
    "keys": (config(150, 64, 1e-5, [layer("attention", maps(1, 1, 32, 32, 0.5), ff=48), layer("latent_attention", latent(8, 8, 8, 16, 16), None),
                                    layer("attention", maps(8, 1, 8, 16, 0.2, window=70, scale=0.5), ff=32)]), 44),
    # one tap (a convolution that only scales), a convolution on the projections under none on the inputs' history, heads of 128
    "taps": (config(128, 72, 1e-5, [layer("attention", maps(2, 1, 8, 8, 0.5, conv=1, window=33), ff=40), layer("general_delta", delta(1, 128, 3), None),
                                    layer("attention", maps(2, 2, 24, 8, 0.9, conv=6), ff=24)], taps=1, cap=5.0, loop=(0, 2, 2)), 46),
}
LENGTHS = {"mix": [1, 2, 23, 70, 131, 260], "odd": [3, 40, 97, 200], "recurrent": [1, 50, 140], "keys": [2, 65, 150], "taps": [4, 5, 66, 150]}


def twin_tensors(tensors, dtype):
    if dtype == "float32":
        return tensors
    return {k: (plain.round_to_bf16(v) if v.ndim == 2 and not k.endswith(KEPT_32BIT) else v) for k, v in tensors.items()}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    from liyab_amd.weights import write_random_model

    out = {}
    for name, (cfg, seed) in CONFIGS.items():
        d = str(tmp_path_factory.mktemp(f"dopilorn_{name}"))
        write_random_model(d, json.loads(json.dumps(cfg)), seed)
        raw, tensors = read_model(d)
        for dtype in DTYPES:
            out[(name, dtype)] = (d, raw, twin_tensors(tensors, dtype))
    return out


def make_requests(name):
    cfg, seed = CONFIGS[name]
    return {f"{name}{i}": tt.random_tokens(seed * 50 + i, n, cfg["vocab"]) for i, n in enumerate(LENGTHS[name])}


@pytest.fixture(scope="module")
def reference(models):
    return {(name, dtype): {rid: plain.forward(toks, t, raw) for rid, toks in make_requests(name).items()}
            for (name, dtype), (_, raw, t) in models.items()}


def make_core(model_dir, dtype, max_tokens, page_size=16, max_requests=4, **kw):
    from liyab_amd.engine import EngineCore

    core = EngineCore(model_dir, dtype=dtype, page_size=page_size, max_tokens=max_tokens, max_requests=max_requests, **kw)
    # free pages and unused state hold NaN: a kernel that reads past a request's length, or a slot's old state, shows it
    for c in core.storage.layers.values():
        for t in c.rows.values():
            t.fill_(float("nan"))
    for t in core.storage.states.values():
        t.fill_(float("nan"))
    torch.cuda.synchronize()
    return core


def rand(rng, *shape, scale=1.0, mean=0.0):
    return torch.from_numpy((rng.standard_normal(shape) * scale + mean).astype(np.float32))


def f64(t):
    return t.detach().float().cpu().numpy().astype(np.float64)


# ---------------------------------------------------------------------------
# each mechanism alone
# ---------------------------------------------------------------------------
class _Layer:
    """A model of one layer, for driving its parts by hand through steps of one request."""

    def __init__(self, dtype, entry, width=64, tensors=None, page_size=8, eps=1e-5, taps=None):
        from liyab_amd.config import config_from_dict
        from liyab_amd.engine import EngineCore
        from liyab_amd.weights.random_init import random_tensors

        self.raw = config(50, width, eps, [entry], taps=taps)
        cfg = config_from_dict(self.raw)
        t = random_tensors(cfg, 5)
        for k, v in (tensors or {}).items():
            assert k in t and tuple(t[k].shape) == tuple(v.shape), (k, tuple(v.shape))
            t[k] = v
        if dtype == "bfloat16":
            t = {k: (v.to(torch.bfloat16).float() if v.dim() == 2 and not k.endswith(KEPT_32BIT) else v) for k, v in t.items()}
        self.t = {k: f64(v) for k, v in t.items()}
        self.core = EngineCore.from_plan(cfg.plan(), t, dtype=dtype, page_size=page_size, num_pages=300, max_requests=3, use_graphs=False)
        for s in self.core.storage.states.values():
            s.fill_(float("nan"))
        for c in self.core.storage.layers.values():
            for rows in c.rows.values():
                rows.fill_(float("nan"))
        self.block = self.core.model.blocks[0]
        self.width, self.dtype, self.eps = width, dtype, eps

    def mixer_state(self):
        from liyab_amd.kernels import ops

        b = self.block
        return ops.StateSlice(self.core.storage.state(0), b.ring_floats, b.mixer_floats) if b.mixer_floats else None

    def run(self, rid, rows, portions, fn):
        from liyab_amd.engine import StepItem

        out, done = [], 0
        for take in portions:
            item = StepItem(rid, [1] * take, [])
            ctx, lengths = self.core.step_fn.prepare([item])
            out.append(fn(ctx, rows[done:done + take].to(DEV)))
            self.core.step_fn.commit([item], lengths)
            done += take
        assert done == rows.shape[0]
        return np.concatenate(out)


def _mixer_alone(p, x, portions, rid="m"):
    """The layer's mixer over the rows x (its input) of one request, in portions."""
    core, mix = p.core, p.block.mixer
    core.open(rid)

    def step(ctx, xs):
        y = torch.empty(xs.shape[0], p.width, dtype=torch.float32, device=DEV)
        mix.forward(xs.to(core.dtype), ctx, core.storage.layer(0), p.mixer_state(), None, out=y)
        return f64(y)

    got = p.run(rid, x, portions, step)
    core.close(rid)
    core.manager.check()
    return got


def _inputs(p, rng, n, scale=1.0):
    x = rand(rng, n, p.width, scale=scale)
    return x, f64(x.to(torch.bfloat16).float() if p.dtype == "bfloat16" else x)


MIXER_TOL = {"float32": 2e-5, "bfloat16": 3e-2}
PORTIONS = ((75,), (25, 1, 9, 1, 1, 2, 36), (2,) * 10 + (1,) * 5 + (50,), (1,) * 75)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width,taps,ff", [(64, 4, 32), (100, 2, None), (72, 1, 24), (96, None, 40), (40, 7, 16), (2500, 3, 8), (66, 3, 20), (50, 5, None)])
def test_two_norms_and_their_convolutions_in_portions(dtype, width, taps, ff):
    """What the two sublayers read, against the twin: norms with weights stored around zero, the convolutions' history from
    portion to portion down to single tokens, a second request in a slot that was used before, no feed-forward (one sublayer),
    one tap (no history) and no convolution at all; widths that are multiples of four (four channels a thread) and not."""
    from liyab_amd.kernels import ops

    p = _Layer(dtype, layer("general_delta", delta(1, 8, 2), ff=ff), width=width, taps=taps)
    b, core = p.block, p.core
    S = 2 if ff else 1
    rng = np.random.default_rng(1)
    for k, portions in enumerate(PORTIONS):
        n = sum(portions)
        x = rand(rng, n, width, scale=3.0)
        want = []
        for s in range(S):
            h = plain.offset_norm(f64(x), p.t[f"l0.norm{s + 1}"], p.eps)
            want.append(h + plain.time_conv(h, p.t[f"l0.canon{s + 1}"]) if taps else h)
        rid = f"n{k}"
        core.open(rid)

        def step(ctx, xs):
            ring = ops.StateSlice(core.storage.state(0), 0, b.ring_floats) if b.ring_floats else None
            out = torch.empty(S, xs.shape[0], width, dtype=core.dtype, device=DEV)
            kept = torch.empty(xs.shape[0], S * width, dtype=torch.float32, device=DEV) if ring is not None else None
            ops.norm_shift(out, xs.contiguous(), b.norm_weights, 0.0, b.eps, b.conv_weights, ring, ctx, hbuf=kept)
            if ring is not None:
                ops.ring_keep(ring, b.taps - 1, kept, ctx)
            return f64(out).transpose(1, 0, 2)

        got = p.run(rid, x, portions, step)
        core.close(rid)
        for s in range(S):
            assert tt.rel_err(got[:, s], want[s]) < (2e-6 if dtype == "float32" else 8e-3), (s, portions[:4])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width,ff,act", [(64, 96, (0.5, 0.3, -0.2, 0.1)), (100, 50, (0.0, 1.0, 0.0, 0.0)), (72, 2000, (1.0, 0.0, 2.0, -1.0))])
def test_the_feed_forward_of_normed_powers_alone(dtype, width, ff, act):
    p = _Layer(dtype, layer("general_delta", delta(1, 8, 2), ff=ff), width=width, tensors={"l0.mlp.act": torch.tensor(act)})
    x, xs = _inputs(p, np.random.default_rng(2), 37, scale=2.0)
    y = torch.zeros(37, width, dtype=torch.float32, device=DEV)
    from liyab_amd.engine import StepItem

    p.core.open("f")
    ctx, _ = p.core.step_fn.prepare([StepItem("f", [1] * 37, [])])
    p.block.ffn.forward(x.to(DEV).to(p.core.dtype), ctx, y)
    want = plain.feed_forward(xs, p.t, "l0.mlp.", p.eps)
    assert tt.rel_err(f64(y), want) < MIXER_TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m", [delta(3, 32, 8), delta(5, 12, 7), delta(1, 64, 16), delta(2, 128, 4), delta(4, 8, 1), delta(1, 200, 5), delta(2, 17, 3)])
def test_the_delta_rule_alone_in_portions(dtype, m):
    """The heads' matrices travel from portion to portion, down to single tokens; a second request in a slot that was used
    before starts from zeros whatever the slot holds; heads of every size class of the kernel; long portions in segments."""
    p = _Layer(dtype, layer("general_delta", m), width=72, taps=3)
    rng = np.random.default_rng(3)
    # (steps of 192 rows and more walk in segments of 64 side by side: a whole number of segments, one row more, one less, a
    # long portion that starts from a state)
    for k, portions in enumerate(PORTIONS + ((257,), (3, 255), (192,), (7, 191, 64, 193))):
        x, xs = _inputs(p, rng, sum(portions))
        want = plain.general_delta(xs, p.t, "l0.mix.", m, p.eps)
        got = _mixer_alone(p, x, portions, rid=f"w{k}")
        assert tt.rel_err(got, want) < MIXER_TOL[dtype], (m, portions[:4])


def test_the_delta_rule_remembers_far_back_and_forgets_what_it_is_told_to():
    """Channels that hardly decay and are hardly taken out carry one early token's value to the end of a long sequence: the
    output there changes by much when that token's input changes. With a removal rate near one, a later token with the same
    key wipes it. The engine follows the twin whole, in portions and token by token."""
    m = delta(2, 16, 4)
    H, D, width = 2, 16, 64
    for a_bias, moved_least in ((-9.0, 1e-3), (9.0, 0.0)):
        t = {"l0.mix.w0": torch.full((H * D,), -12.0), "l0.mix.w2": torch.zeros(H * D, 4), "l0.mix.a": torch.zeros(H * D, width),
             "l0.mix.a.b": torch.full((H * D,), a_bias)}
        p = _Layer("float32", layer("general_delta", m), width=width, tensors=t)
        rng = np.random.default_rng(4)
        n = 400
        x, xs = _inputs(p, rng, n)
        if a_bias > 0:
            x[200] = x[3] * 1.5  # the same key direction once more: what position 3 left under it is taken out
            xs = f64(x)
        want = plain.general_delta(xs, p.t, "l0.mix.", m, p.eps)
        blind = xs.copy()
        blind[3] = 0.0
        moved = np.abs(plain.general_delta(blind, p.t, "l0.mix.", m, p.eps)[-1] - want[-1]).max()
        assert moved > moved_least
        for k, portions in enumerate(((n,), (n - 40,) + (1,) * 40, (100, 2, 150, 37, 2, 107, 2))):
            assert tt.rel_err(_mixer_alone(p, x, portions, rid=f"f{k}"), want) < 2e-5


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m", [maps(4, 2, 16, 24, 0.3, conv=3, window=11), maps(3, 3, 6, 10, 0.7, conv=2, window=1), maps(1, 1, 32, 32, 0.5),
                               maps(8, 1, 8, 16, 0.2, window=70, scale=0.5), maps(2, 2, 24, 8, 0.9, conv=6), maps(2, 1, 64, 64, 0.5, conv=4, window=40),
                               maps(4, 4, 48, 96, 0.1, conv=1, window=16), maps(2, 1, 128, 40, 0.0, window=200)])
def test_attention_in_two_maps_alone_in_portions(dtype, m):
    """Biases, the projections' convolution with its history, grouped keys, keys and values of different widths, windows
    shorter than a page, equal to one and past the context, from portion to portion."""
    p = _Layer(dtype, layer("attention", m), width=72, taps=2)
    rng = np.random.default_rng(6)
    for k, portions in enumerate(PORTIONS + ((140,),)):
        x, xs = _inputs(p, rng, sum(portions))
        want = plain.differential_attention(xs, p.t, "l0.mix.", m, p.eps)
        got = _mixer_alone(p, x, portions, rid=f"a{k}")
        # where the two maps agree their difference is 1 / |1 - lambda| times smaller than they are, and the norm behind it brings
        # it back to size: in bfloat16 the maps' rounding grows by that much (the 32-bit run holds the plain tolerance)
        lam = math.exp(float(p.t["l0.mix.lq1"] @ p.t["l0.mix.lk1"])) - math.exp(float(p.t["l0.mix.lq2"] @ p.t["l0.mix.lk2"])) + m["diff"]
        tol = MIXER_TOL[dtype] * (max(1.0, 0.3 / abs(1.0 - lam)) if dtype == "bfloat16" else 1.0)
        assert tt.rel_err(got, want) < tol, (m, portions[:4])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window,page_size", [(7, 8), (16, 16), (17, 16), (40, 16), (64, 8), (0, 16)])
def test_a_marked_key_just_inside_and_just_outside_the_window(dtype, window, page_size):
    """The first map's query and key are the input's first channels, the second map's are zero (its weights are the window's
    mean), and the scale is such that a key along the query's direction takes nearly all of the first map's weight: a marked
    key at distance window - 1 is most of a query's result, one at distance window must not be seen at all. In prompts'
    portions, decoded alone, at page borders; without a window the marked key lies hundreds back."""
    H, D, V, width = 2, 16, 24, 64
    m = maps(H, 1, D, V, 0.4, window=window or None, scale=1.2)
    eye = torch.eye(width)
    first = torch.cat([eye[4:4 + D], torch.zeros(D, width)])  # [map 1 | map 2] of a head
    t = {"l0.mix.q": torch.cat([first] * H).clone(), "l0.mix.k": first.clone(), "l0.mix.q.b": torch.zeros(2 * H * D), "l0.mix.k.b": torch.zeros(2 * D)}
    p = _Layer(dtype, layer("attention", m), width=width, tensors=t, page_size=page_size)
    rng = np.random.default_rng(9)
    n = 330
    reach = window if window else 300
    for case, distance in enumerate([reach - 1, reach, reach + 1, max(reach - 2, 1)]):
        x = rand(rng, n, width)
        query_at = [n - 1, n - 20, 2 * page_size * 8 + 1, reach + 2]
        marks = {}
        for i in query_at:
            j = i - distance
            if j < 0 or j in marks or j in query_at or any(abs(j - o) < 2 for o in marks):
                continue
            marks[j] = i
            x[j, 4:4 + D] = 3.0 * x[i, 4:4 + D]
        # the norms and the convolution of the block are not in the way: the mixer is driven with x as its input
        xs = f64(x.to(torch.bfloat16).float() if dtype == "bfloat16" else x)
        want = plain.differential_attention(xs, p.t, "l0.mix.", m, p.eps)
        moved = []
        for j, i in marks.items():  # what a marked query loses when its marked key alone is taken away
            blind = xs.copy()
            blind[j, 4:4 + D] = 0.01
            moved.append(np.abs(plain.differential_attention(blind, p.t, "l0.mix.", m, p.eps) - want)[i].max())
        moved = np.array(moved)
        assert len(marks) > 0
        if window == 0 or distance < window:
            assert (moved > 0.05).all(), (distance, moved)
        else:
            assert (moved < 1e-9).all(), (distance, moved)
        for portions in ((n,), (n - 40,) + (1,) * 40, (100, 2, 150, 37, 2, 37, 2)):
            got = _mixer_alone(p, x, portions, rid=f"k{case}")
            assert tt.rel_err(got, want) < (2e-5 if dtype == "float32" else 6e-2), (distance, portions[:3])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m", [latent(4, 24, 16, 40, 32), latent(3, 10, 6, 12, 7, scale=0.4), latent(8, 8, 8, 16, 16), latent(1, 64, 64, 128, 24),
                               latent(2, 32, 48, 64, 8)])
def test_latent_attention_with_a_query_latent_alone_in_portions(dtype, m):
    p = _Layer(dtype, layer("latent_attention", m), width=72, taps=2)
    rng = np.random.default_rng(7)
    for k, portions in enumerate(PORTIONS + ((140,),)):
        x, xs = _inputs(p, rng, sum(portions))
        want = plain.latent_attention(xs, p.t, "l0.mix.", m, p.eps)
        got = _mixer_alone(p, x, portions, rid=f"l{k}")
        assert tt.rel_err(got, want) < MIXER_TOL[dtype], (m, portions[:4])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("page_size", [8, 16])
def test_a_marked_cached_row_far_away(dtype, page_size):
    """The latent is a stretch of the input's channels brought to unit root mean square (the matrices on the way are slices of
    the identity); queries and keys read its first half and values its second, so a position whose key half lies along the
    query's takes nearly all of its weight and brings values of its own, hundreds of positions back and at page borders, whole,
    decoded alone and in portions."""
    H, D, R, width = 2, 16, 32, 64
    m = latent(H, D, D, R, R, scale=0.7)
    eye = torch.eye(width)
    first, second = torch.eye(R)[:D], torch.eye(R)[D:]
    t = {"l0.mix.dq": eye[4:4 + R].clone(), "l0.mix.dkv": eye[4:4 + R].clone(), "l0.mix.dq.norm": torch.ones(R), "l0.mix.dkv.norm": torch.ones(R),
         "l0.mix.uq": torch.cat([first] * H).clone(), "l0.mix.uk": torch.cat([first] * H).clone(), "l0.mix.uv": torch.cat([second] * H).clone(),
         "l0.mix.g": torch.zeros(H, width)}
    p = _Layer(dtype, layer("latent_attention", m), width=width, tensors=t, page_size=page_size)
    rng = np.random.default_rng(10)
    n = 330
    query_at = [n - 1, n - 2, 290, 2 * page_size * 8 + 1]
    for case, distance in enumerate([n - 4, 200, 257, n - 1 - page_size]):
        x = rand(rng, n, width)
        marks = {}
        for i in query_at:
            j = i - distance
            if j < 0 or j in marks or j in query_at or any(abs(j - o) < 2 for o in marks):
                continue
            marks[j] = i
            x[j, 4:4 + D] = 3.0 * x[i, 4:4 + D]
        xs = f64(x.to(torch.bfloat16).float() if dtype == "bfloat16" else x)
        want = plain.latent_attention(xs, p.t, "l0.mix.", m, p.eps)
        blind = xs.copy()
        for j in marks:
            blind[j] = 0.01
        moved = np.abs(plain.latent_attention(blind, p.t, "l0.mix.", m, p.eps) - want)[list(marks.values())].max(-1)
        assert len(marks) > 0 and (moved > 0.05).all(), (distance, moved)
        for portions in ((n,), (n - 40,) + (1,) * 40, (100, 2, 150, 37, 2, 37, 2)):
            got = _mixer_alone(p, x, portions, rid=f"c{case}")
            assert tt.rel_err(got, want) < (2e-5 if dtype == "float32" else 6e-2), (distance, portions[:3])


# ---------------------------------------------------------------------------
# whole models
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_each_request_alone_and_whole_and_every_layer(name, dtype, models, reference):
    reqs = make_requests(name)
    steps = tt.schedule_whole(reqs)
    core = make_core(models[(name, dtype)][0], dtype, tt.max_live_tokens(steps))
    got = tt.run_schedule(core, steps)
    check_logits(got, reqs, reference[(name, dtype)], dtype, f"dopilorn-whole {name} {dtype}")
    core.manager.check()
    assert not core.manager.groups or core.manager.pages_in_use() == 0
    if dtype == "float32":
        from liyab_amd.engine import StepItem

        rid, toks = list(reqs.items())[2]
        streams, caught = [], []
        plain.forward(toks, models[(name, dtype)][2], models[(name, dtype)][1], streams)
        plain_core = make_core(models[(name, dtype)][0], dtype, 512, use_graphs=False)
        plain_core.model.replay_layers = False
        for block in plain_core.model.blocks:
            def wrapped(x, ctx, cache, state, writes_cache=True, _f=block.forward):
                out = _f(x, ctx, cache, state, writes_cache=writes_cache)
                caught.append(f64(x)[:len(toks)])
                return out
            block.forward = wrapped
        plain_core.open(rid)
        plain_core.step([StepItem(rid, toks, [])])
        assert len(caught) == len(streams) == len(plain.run_order(models[(name, dtype)][1]))
        for got_x, want_x in zip(caught, streams):
            assert tt.rel_err(got_x, want_x) < 1e-5


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_a_prompt_then_its_last_tokens_one_by_one(name, dtype, models, reference):
    reqs = make_requests(name)
    steps = tt.schedule_bulk_tail(reqs, tail=45)
    core = make_core(models[(name, dtype)][0], dtype, tt.max_live_tokens(steps))
    got = tt.run_schedule(core, steps)
    check_logits(got, reqs, reference[(name, dtype)], dtype, f"dopilorn-decode {name} {dtype}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [(5, 2, 17, 3, 48, 2, 31, 7), (2, 2, 2, 3), (1, 64, 1, 16, 2)])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_portions_of_changing_size(name, dtype, sizes, models, reference):
    reqs = make_requests(name)
    if sizes[0] == 2:
        reqs = dict(list(reqs.items())[:3])
    steps = tt.schedule_portions(reqs, sizes)
    core = make_core(models[(name, dtype)][0], dtype, tt.max_live_tokens(steps), page_size=8 if sizes[0] == 1 else 16)
    got = tt.run_schedule(core, steps)
    check_logits(got, reqs, reference[(name, dtype)], dtype, f"dopilorn-portions {name} {dtype}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("seed,max_live,page_size", [(0, 4, 16), (1, 3, 8), (2, 2, 24)])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_mixed_batches_with_pages_and_slots_used_again(name, dtype, seed, max_live, page_size, models, reference):
    """Up to `max_live` requests at a time, portions of some beside single tokens of others, in a pool and with state slots
    just large enough: what a finished request gives back is used by the next."""
    base = make_requests(name)
    reqs = {f"{rid}#{k}": toks for k in range(2) for rid, toks in base.items()}
    ref = {f"{rid}#{k}": reference[(name, dtype)][rid] for k in range(2) for rid in base}
    steps = tt.schedule_mixed(reqs, seed=seed, max_live=max_live)
    core = make_core(models[(name, dtype)][0], dtype, None, page_size=page_size, max_requests=max_live, num_pages=tt.max_live_pages(steps, page_size))
    got = tt.run_schedule(core, steps)
    check_logits(got, reqs, ref, dtype, f"dopilorn-mixed {name} {dtype}")
    core.manager.check()
    assert not core.manager.groups or core.manager.pages_in_use() == 0
    assert core.step_fn.graph_replays > 0  # the decode-only steps of the tail were replayed from graphs


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["mix", "recurrent"])
def test_long_decoding_from_the_first_token(name, dtype, models, reference):
    rid, toks = list(make_requests(name).items())[-1]
    reqs = {rid: toks}
    steps = tt.schedule_bulk_tail(reqs, tail=len(toks))
    core = make_core(models[(name, dtype)][0], dtype, tt.max_live_tokens(steps))
    got = tt.run_schedule(core, steps)
    check_logits(got, reqs, reference[(name, dtype)], dtype, f"dopilorn-long {name} {dtype}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_trace_program(dtype, models, reference, tmp_path):
    name = "odd"
    reqs = make_requests(name)
    steps = tt.schedule_mixed(reqs, seed=5, max_live=4)
    got = tt.run_trace_program(models[(name, dtype)][0], dtype, steps, str(tmp_path), tt.max_live_tokens(steps), CONFIGS[name][0]["vocab"])
    check_logits(got, reqs, reference[(name, dtype)], dtype, f"dopilorn-trace {dtype}")


def draw_config(seed):
    """A geometry drawn from the seed: every size, constant and count, the layers' kinds and order, what is repeated and how often."""
    rng = np.random.default_rng(2000 + seed)
    pick = lambda *options: options[int(rng.integers(len(options)))]  # noqa: E731
    width = pick(40, 48, 64, 96, 104, 160)

    def one():
        kind = pick("attention", "general_delta", "latent_attention")
        if kind == "attention":
            kv = pick(1, 2, 3)
            m = maps(kv * pick(1, 2, 4), kv, pick(4, 8, 10, 16, 24, 32), pick(4, 8, 12, 16, 40), pick(0.0, 0.2, 0.5, 0.8), conv=pick(None, 1, 2, 3, 5),
                     window=pick(None, 1, 5, 16, 33, 100, 1000))
        elif kind == "general_delta":
            m = delta(pick(1, 2, 3, 5), pick(4, 8, 12, 16, 32, 64), pick(1, 3, 8, 16))
        else:
            m = latent(pick(1, 2, 3, 4), pick(4, 8, 10, 16, 32), pick(4, 6, 16, 24), pick(8, 12, 16, 24, 64), pick(4, 7, 16, 32))
        return layer(kind, m, ff=pick(None, 8, 20, 24, 40, 56))

    layers = [one() for _ in range(int(rng.integers(1, 5)))]
    loop = None
    if rng.random() < 0.7:
        start = int(rng.integers(0, len(layers)))
        loop = (start, int(rng.integers(start + 1, len(layers) + 1)), pick(1, 2, 3))
    return config(pick(97, 256, 500), width, pick(1e-5, 1e-6, 1e-3), layers, taps=pick(None, 1, 2, 3, 4, 6), cap=pick(None, 4.0, 15.0, 50.0), loop=loop), pick(8, 16, 24)


@pytest.mark.parametrize("seed", range(12))
def test_drawn_geometries_whole_and_mixed(seed, tmp_path):
    from liyab_amd.weights import write_random_model

    cfg, page_size = draw_config(seed)
    d = str(tmp_path / "m")
    write_random_model(d, json.loads(json.dumps(cfg)), 100 + seed)
    raw, tensors = read_model(d)
    # (a first token whose key and receptance are orthogonal to within rounding leaves a delta-rule head nothing but the norm's
    # epsilon to divide by, and 32-bit rounding decides its sign: geometry 2's requests are drawn so that none starts with one)
    first = {2: 400}.get(seed, 0) + seed * 10
    reqs = {f"g{i}": tt.random_tokens(first + i, n, raw["vocab"]) for i, n in enumerate([1, 19, 77, 150, 260])}
    for dtype in DTYPES:
        t = twin_tensors(tensors, dtype)
        ref = {rid: plain.forward(toks, t, raw) for rid, toks in reqs.items()}
        steps = tt.schedule_whole(reqs)
        core = make_core(d, dtype, tt.max_live_tokens(steps), page_size=page_size)
        check_logits(tt.run_schedule(core, steps), reqs, ref, dtype, f"dopilorn-drawn seed {seed} whole {dtype}", family="dopilorn-drawn")
        steps = tt.schedule_mixed(reqs, seed=seed, max_live=3)
        core = make_core(d, dtype, None, page_size=page_size, max_requests=3, num_pages=tt.max_live_pages(steps, page_size))
        check_logits(tt.run_schedule(core, steps), reqs, ref, dtype, f"dopilorn-drawn seed {seed} mixed {dtype}", family="dopilorn-drawn")
        core.manager.check()


UNEVEN = {
    # odd everywhere: width, vocabulary, heads, both head sizes, both latents, the decay's rank, the inner widths
    "odd": config(577, 77, 1e-6, [layer("general_delta", delta(3, 5, 3), ff=129), layer("attention", maps(3, 1, 5, 7, 0.5, conv=3, window=13), ff=33),
                                  layer("latent_attention", latent(3, 5, 7, 9, 11), ff=21)], taps=4, cap=15.0, loop=(0, 3, 2)),
    # even, but no multiple of four (no kernel of four channels a thread takes them), heads of 50
    "even": config(1001, 250, 1e-5, [layer("attention", maps(5, 5, 10, 14, 0.3, conv=2, window=40), ff=130), layer("general_delta", delta(5, 50, 6), ff=70),
                                     layer("latent_attention", latent(5, 18, 22, 50, 30), None)], taps=3, loop=(1, 2, 3)),
    # the widest rows the attention kernels take (cached latents of 256, maps and values of 192) and delta-rule heads of 192
    "widest": config(512, 128, 1e-5, [layer("latent_attention", latent(2, 96, 96, 256, 64), ff=64), layer("attention", maps(2, 1, 192, 192, 0.5, conv=4, window=100), None),
                                      layer("general_delta", delta(1, 192, 8), ff=64)], taps=2, cap=30.0),
}


@pytest.mark.parametrize("name", list(UNEVEN))
def test_sizes_no_kernel_tiles_evenly(name, tmp_path):
    """Whole prompts and mixed batches at sizes that are odd, even but no multiple of four, and the widest the kernels take."""
    from liyab_amd.weights import write_random_model

    d = str(tmp_path / "m")
    write_random_model(d, json.loads(json.dumps(UNEVEN[name])), 7)
    raw, tensors = read_model(d)
    reqs = {f"u{i}": tt.random_tokens(70 + i, n, raw["vocab"]) for i, n in enumerate([3, 70, 230])}
    for dtype in DTYPES:
        t = twin_tensors(tensors, dtype)
        ref = {rid: plain.forward(toks, t, raw) for rid, toks in reqs.items()}
        for steps in (tt.schedule_whole(reqs), tt.schedule_mixed(reqs, seed=1, max_live=3)):
            core = make_core(d, dtype, None, max_requests=3, num_pages=tt.max_live_pages(steps, 16))
            check_logits(tt.run_schedule(core, steps), reqs, ref, dtype, f"dopilorn-uneven {name} {dtype}", family="dopilorn-uneven")
            core.manager.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_real_widths_in_long_steps(dtype, tmp_path):
    """Heads of 64 and 128, a width of 512, prompts of hundreds of tokens in one step and in mixed batches: the tiles of the
    large products, the matrix-core attention under both maps, states of 64 x 64 and 128 x 128 a head."""
    from liyab_amd.weights import write_random_model

    cfg = config(1000, 512, 1e-5, [
        layer("general_delta", delta(8, 64, 32), ff=1024),
        layer("attention", maps(8, 2, 64, 64, 0.5, conv=3, window=256), ff=1024),
        layer("latent_attention", latent(8, 64, 64, 128, 192), ff=1024),
        layer("attention", maps(4, 4, 64, 128, 0.2, conv=4), None),
        layer("general_delta", delta(4, 128, 16), ff=768),
    ], taps=4, cap=20.0, loop=(0, 3, 2))
    d = str(tmp_path / "m")
    write_random_model(d, json.loads(json.dumps(cfg)), 31)
    raw, tensors = read_model(d)
    t = twin_tensors(tensors, dtype)
    reqs = {f"r{i}": tt.random_tokens(900 + i, n, raw["vocab"]) for i, n in enumerate([330, 700, 45])}
    ref = {rid: plain.forward(toks, t, raw) for rid, toks in reqs.items()}
    steps = tt.schedule_whole(reqs)
    core = make_core(d, dtype, tt.max_live_tokens(steps))
    check_logits(tt.run_schedule(core, steps), reqs, ref, dtype, f"dopilorn-wide whole {dtype}", family="dopilorn-wide")
    steps = tt.schedule_mixed(reqs, seed=3, max_live=3, portions=(2, 130, 64, 300, 17))
    core = make_core(d, dtype, None, max_requests=3, num_pages=tt.max_live_pages(steps, 16))
    check_logits(tt.run_schedule(core, steps), reqs, ref, dtype, f"dopilorn-wide mixed {dtype}", family="dopilorn-wide")
    core.manager.check()


def generate_greedy(raw, t, prompt, n_new):
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(np.argmax(plain.forward(toks, t, raw)[-1])))
    return toks[len(prompt):]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["mix", "odd"])
def test_greedy_generation_through_the_entry_point(name, dtype, models):
    """Engine.generate: the scheduler batches the prompts in portions beside decoding requests, in a pool that does not hold
    them all at once (requests are preempted and computed again, their slots' state starting over); each token is the twin's
    greedy choice given the tokens so far."""
    from liyab_amd import Engine, SamplingParams

    d, raw, t = models[(name, dtype)]
    prompts = [tt.random_tokens(70 + i, n, raw["vocab"]) for i, n in enumerate([1, 13, 64, 100, 7])]
    n_new = 12
    engine = Engine(d, dtype=dtype, page_size=16, num_pages=14, max_num_seqs=3, max_batched_tokens=48, prefill_chunk=24)
    engine.stop_at_eos = False
    results = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=n_new))
    for prompt, res in zip(prompts, results):
        assert len(res.tokens) == n_new
        ref = plain.forward(prompt + res.tokens[:-1], t, raw)
        for i, tok in enumerate(res.tokens):
            row = ref[len(prompt) - 1 + i]
            slack = (1e-5 if dtype == "float32" else 5e-2) * np.abs(row).max()
            assert row[tok] >= row.max() - slack, f"token {i} of prompt length {len(prompt)}: {tok} vs {int(np.argmax(row))}"
        if dtype == "float32":
            assert res.tokens == generate_greedy(raw, t, prompt, n_new)
    engine.core.manager.check()


def test_command_line(models):
    d, raw, tensors = models[("taps", "float32")]
    prompt = tt.random_tokens(90, 11, raw["vocab"])
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "liyab-cli"), "-m", d, "-p", ",".join(map(str, prompt)), "-n", "6",
                        "--temp", "0", "--dtype", "float32", "--json", "--phases"], capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    turn = [json.loads(l) for l in p.stdout.splitlines() if l.startswith("{")][1]
    assert turn["tokens"] == generate_greedy(raw, tensors, prompt, 6)
    assert set(turn["phases_ms"]) == {"embed", "differential_attention", "delta_rule", "normed_powers_ffn", "lm_head"}
