"""Larulorn through the engine against its plain twin (`plain_larulorn.py`): each mechanism alone, then whole models of
several geometries under every way of cutting and batching the work, in 32-bit and in bfloat16 (needs the GPU). The
geometries differ from each other in every size and in the order of their layers; one has sizes no kernel tiles evenly,
one no attention layer of its own, one nothing but attention, one the values that other geometries happen to share (one
group of experts, one expert a token, weights of one on both mixers, keys and values of different widths under a gate)."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_larulorn as plain
import trace_tools as tt
from conftest import ROOT, TOL
from plain_gpt2 import read_model

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = ["float32", "bfloat16"]
# float32: the largest difference of a row relative to its largest |logit|, as for the other models.
# bfloat16, against the twin in float64 with the same rounded matrices: the root mean square of a row's difference over
# that of the row's logits, both with their means taken off; a fault in a mechanism makes it about 1.
# The five geometries and the wide model show 0.01 to 0.03. Among the drawn geometries a row here and there reaches 0.13 (the
# row's 99th percentile stays below 0.04): every sublayer's result passes a norm before it joins the stream, which brings each
# rounding back to the stream's own size, layer after layer, and a drawn scale may leave a softmax closely contested.
TOL_B = {"float32": TOL["float32"], "bfloat16": 6e-2}
TOL_DRAWN = 2e-1
KEPT_32BIT = (".conv", ".ra.b", ".ri.b")  # 2-D tensors that the engine keeps in 32 bits
ROUNDED_3D = (".ra", ".ri")  # the recurrence's gates, a matrix a part


def check_logits(got, reqs, ref, dtype, what, family=None, tol=None):
    if dtype == "float32":
        return tt.check_against_plain(got, reqs, ref, TOL_B[dtype], what, family=family)
    tol = tol or TOL_B[dtype]
    key = ((family or what.split(" ")[0]) + " (rms)", tol)
    for rid, toks in reqs.items():
        assert rid in got, f"{what}: no logits for request {rid}"
        for p in sorted(got[rid]):
            row, want = np.asarray(got[rid][p], dtype=np.float64), ref[rid][p]
            assert np.isfinite(row).all(), f"{what}: request {rid} position {p}: non-finite logits"
            diff = row - want
            e = float(np.sqrt(np.mean((diff - diff.mean()) ** 2)) / np.sqrt(np.mean((want - want.mean()) ** 2)))
            tt.WORST[key] = max(tt.WORST.get(key, 0.0), e)
            assert e <= tol, f"{what}: request {rid} (length {len(toks)}) first differs at position {p}: {e:.3e} > {tol:.1e}"


# ---------------------------------------------------------------------------
# configurations
# ---------------------------------------------------------------------------
def att(heads, kv_heads, dim, vdim, rot=None, v_mix=False, scale=None):
    """rot = (dims, base) or (dims, base, (factor, original, fast, slow))."""
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5}
    if rot:
        m["rot"] = {"dims": rot[0], "base": rot[1]}
        if len(rot) > 2:
            m["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), rot[2]))
    if v_mix:
        m["v_mix"] = True
    return m


def par(left, width, blocks, conv, left_scale=0.7, right_scale=1.2):
    return {"left": left, "right": {"width": width, "blocks": blocks, "conv": conv}, "left_scale": left_scale, "right_scale": right_scale}


def dense(ff, limit=1.0):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(ff, experts, top, groups=None, shared=None):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if groups:
        m["router"]["groups"] = {"count": groups[0], "keep": groups[1]}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def layer(kind, m, mlp=None):
    return {"type": kind, "mixer": m, "mlp": mlp}


def config(vocab, width, eps, layers, logit_scale=1.0):
    return {"architecture": "Larulorn", "vocab": vocab, "width": width, "norm": {"eps": eps}, "logit_scale": logit_scale, "layers": layers}


CONFIGS = {
    # every kind of layer and feed-forward; values mixed in three layers with one between them that keeps its own; grouped keys; a ramp
    "mix": (config(300, 96, 1e-5, [
        layer("attention", att(4, 2, 24, 16, rot=(12, 10000.0, (4.0, 64, 8.0, 1.0)), v_mix=True), moe(24, 8, 2, groups=(4, 2), shared=40)),
        layer("parallel", par(att(4, 2, 16, 16, rot=(8, 500.0)), 48, 3, 4), dense(160, 0.8)),
        layer("attention", att(2, 2, 16, 16, rot=(16, 10000.0)), moe(16, 6, 3)),
        layer("attention", att(6, 2, 8, 16, rot=(4, 100.0, (2.0, 32, 4.0, 0.5)), v_mix=True), dense(64, 2.0)),
        layer("attention", att(2, 2, 32, 16, v_mix=True), None),
    ], logit_scale=0.7), 51),
    # sizes that no kernel tiles evenly; two taps; three groups of which two stay
    "odd": (config(211, 100, 1e-6, [
        layer("attention", att(3, 3, 10, 6, rot=(6, 777.0)), moe(13, 6, 3, groups=(3, 2), shared=7)),
        layer("parallel", par(att(3, 1, 6, 6, rot=(2, 50.0), scale=0.3), 51, 3, 2, left_scale=-0.5, right_scale=0.9), dense(30, 0.5)),
        layer("attention", att(5, 1, 6, 10, rot=(6, 30.0, (8.0, 40, 3.0, 0.25))), dense(50, 1.5)),
    ], logit_scale=1.5), 52),
    # no attention layer of its own; one tap (no history), one part, five taps; a layer without a feed-forward
    "recurrent": (config(128, 64, 1e-5, [
        layer("parallel", par(att(1, 1, 32, 32, rot=(32, 10000.0)), 64, 1, 1), moe(32, 4, 1, shared=16)),
        layer("parallel", par(att(4, 4, 8, 8), 40, 5, 5), None),
        layer("parallel", par(att(2, 1, 16, 16, rot=(8, 1000.0, (3.0, 16, 2.0, 1.0))), 96, 2, 3), dense(40)),
    ]), 53),
    # attention only (no state at all), one layer alone mixes values (so nothing is mixed), heads of 64 and 128
    "keys": (config(150, 64, 1e-5, [layer("attention", att(1, 1, 64, 64, rot=(64, 10000.0)), dense(48)), layer("attention", att(2, 1, 128, 8, rot=(32, 5000.0), v_mix=True), None),
                                    layer("attention", att(8, 4, 8, 8, rot=(8, 20.0)), moe(8, 4, 4, groups=(2, 2)))], logit_scale=0.25), 54),
    # what other geometries share or make one: one group, one expert a token, weights of one, keys wider than values under a gate
    "ones": (config(128, 72, 1e-5, [layer("parallel", par(att(2, 1, 24, 8, rot=(24, 100.0)), 72, 1, 2, left_scale=1.0, right_scale=1.0), moe(20, 1, 1, groups=(1, 1))),
                                    layer("attention", att(2, 2, 8, 8, v_mix=True), moe(12, 5, 1, shared=12)),
                                    layer("attention", att(4, 2, 4, 8, rot=(2, 2.0), v_mix=True), dense(24, 100.0))]), 56),
}
LENGTHS = {"mix": [1, 2, 23, 70, 131, 260], "odd": [3, 40, 97, 200], "recurrent": [1, 50, 140], "keys": [2, 65, 150], "ones": [4, 5, 66, 150]}


def weigh_all(cfg):
    """The same model with routers that weigh every expert: in bfloat16 a rounding ahead of a router whose candidates lie a
    rounding apart takes another expert than the twin, and the row then differs by far more than any rounding. The choice
    itself is compared in 32-bit throughout, and in bfloat16 where the router is run alone."""
    cfg = json.loads(json.dumps(cfg))
    for entry in cfg["layers"]:
        mlp = entry["mlp"]
        if mlp is not None and mlp["kind"] == "moe":
            mlp["router"]["top"] = mlp["router"]["experts"]
            if "groups" in mlp["router"]:
                mlp["router"]["groups"]["keep"] = mlp["router"]["groups"]["count"]
    return cfg


def twin_tensors(tensors, dtype):
    if dtype == "float32":
        return tensors
    return {k: (plain.round_to_bf16(v) if (v.ndim == 2 and not k.endswith(KEPT_32BIT)) or k.endswith(ROUNDED_3D) else v) for k, v in tensors.items()}


def write_model(folder, cfg, seed, dtype):
    """A folder with random weights for `cfg` (in bfloat16 runs: its routers weigh every expert; the tensors are the same)."""
    from liyab_amd.weights import write_random_model

    write_random_model(folder, json.loads(json.dumps(cfg if dtype == "float32" else weigh_all(cfg))), seed)
    raw, tensors = read_model(folder)
    return raw, twin_tensors(tensors, dtype)


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, (cfg, seed) in CONFIGS.items():
        for dtype in DTYPES:
            d = str(tmp_path_factory.mktemp(f"larulorn_{name}_{dtype}"))
            out[(name, dtype)] = (d,) + write_model(d, cfg, seed, dtype)
    return out


def make_requests(name):
    cfg, seed = CONFIGS[name]
    return {f"{name}{i}": tt.random_tokens(seed * 50 + i, n, cfg["vocab"]) for i, n in enumerate(LENGTHS[name])}


@pytest.fixture(scope="module")
def reference(models):
    return {(name, dtype): {rid: plain.forward(raw, t, toks) for rid, toks in make_requests(name).items()}
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

    def __init__(self, dtype, entry, width=64, tensors=None, page_size=8, eps=1e-5):
        from liyab_amd.config import config_from_dict
        from liyab_amd.engine import EngineCore
        from liyab_amd.weights.random_init import random_tensors

        self.raw = config(50, width, eps, [entry])
        cfg = config_from_dict(self.raw)
        t = random_tensors(cfg, 5)
        for k, v in (tensors or {}).items():
            assert k in t and tuple(t[k].shape) == tuple(v.shape), (k, tuple(v.shape))
            t[k] = v
        if dtype == "bfloat16":
            t = {k: (v.to(torch.bfloat16).float() if (v.dim() == 2 and not k.endswith(KEPT_32BIT)) or k.endswith(ROUNDED_3D) else v) for k, v in t.items()}
        self.t = {k: f64(v) for k, v in t.items()}
        self.core = EngineCore.from_plan(cfg.plan(), t, dtype=dtype, page_size=page_size, num_pages=300, max_requests=3, use_graphs=False)
        for s in self.core.storage.states.values():
            s.fill_(float("nan"))
        for c in self.core.storage.layers.values():
            for rows in c.rows.values():
                rows.fill_(float("nan"))
        self.block = self.core.model.blocks[0]
        self.width, self.dtype, self.eps, self.entry = width, dtype, eps, entry

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


def _mixer_alone(p, x, portions, rid="m", part=None):
    """A mixer of the layer (its whole mixer, or one side of a pair) over the rows x of one request, in portions."""
    core, mix = p.core, part if part is not None else p.block.mixer
    core.open(rid)

    def step(ctx, xs):
        y = torch.empty(xs.shape[0], p.width, dtype=torch.float32, device=DEV)
        mix.forward(xs.to(core.dtype), ctx, core.storage.layer(0), core.storage.state(0), None, out=y)
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


def test_turning_frequencies_and_their_ramp():
    """The table of frequencies the kernels read against the twin's, with and without a ramp, and the factor on cosine and sine."""
    from liyab_amd.config.plan import RotarySpec
    from liyab_amd.parts.scored_attention import rotary_frequencies, rotary_magnitude

    for dims, base, ramp in ((64, 10000.0, None), (12, 10000.0, (4.0, 8.0, 1.0, 64)), (6, 30.0, (8.0, 3.0, 0.25, 40)), (32, 5e5, (2.0, 32.0, 1.0, 4096)), (4, 100.0, (2.0, 4.0, 0.5, 32))):
        rot = {"dims": dims, "base": base}
        if ramp:
            rot["scaling"] = {"factor": ramp[0], "fast": ramp[1], "slow": ramp[2], "original": ramp[3]}
        want, mag = plain.turn_frequencies(rot)
        spec = RotarySpec(dims=dims, base=base, halves=True, ramp=ramp)
        assert np.allclose(rotary_frequencies(spec), want, rtol=1e-12, atol=0)
        assert abs(rotary_magnitude(spec) - mag) < 1e-12
        if ramp:
            assert mag > 1.0 and (want <= np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)]) + 1e-15).all()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m", [att(4, 2, 24, 16, rot=(12, 10000.0, (4.0, 64, 8.0, 1.0))), att(3, 3, 10, 6, rot=(6, 777.0)), att(2, 1, 128, 48, rot=(32, 20000.0, (3.0, 1024, 16.0, 2.0))),
                               att(8, 4, 8, 8, rot=(8, 20.0)), att(1, 1, 64, 64), att(5, 1, 6, 10, rot=(2, 3.0))])
def test_attention_with_biases_and_a_sink_alone_in_portions(dtype, m):
    """Keys and values of their own widths, grouped keys, turned halves with and without the ramp, biases and the sink, from
    portion to portion down to single tokens; a second request finds pages that were used before."""
    p = _Layer(dtype, layer("attention", m), width=72)
    rng = np.random.default_rng(3)
    for k, portions in enumerate(PORTIONS):
        x, xs = _inputs(p, rng, sum(portions))
        want = plain.sink_attention(xs, p.t, "l0.mix.", m, np.arange(len(xs), dtype=np.float64), [None])
        got = _mixer_alone(p, x, portions, rid=f"a{k}")
        assert tt.rel_err(got, want) < MIXER_TOL[dtype], (m, portions[:4])


def _marked(width, n, j, rng, gain=6.0):
    """Rows of which the last and row j are large in channel 0 and small elsewhere: with a query and key weight that
    takes channel 0 to an entry the turning leaves alone, row j gets most of the last row's weight. Row j is large in
    channel 1 too, which only its value reads: a value unlike the last row's own."""
    x = rand(rng, n, width, scale=0.3)
    x[:, 0] *= 0.1
    x[j, 0] = gain
    x[j, 1] = 1.5 * gain
    x[n - 1, 0] = gain
    return x


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("page_size", [8, 16])
def test_a_marked_key_far_back_at_page_borders_and_at_the_start_beside_a_sink(dtype, page_size):
    """One earlier position holds most of the last query's weight, next to a sink of about its size: the result changes by
    much when that position's row is taken away, and by much when the sink is; the engine finds both, with the position
    hundreds back, on either side of a page's border, at the very start, in a prompt and decoded token by token."""
    H, G, D, V, width, n = 2, 1, 16, 8, 48, 420
    m = att(H, G, D, V, rot=(8, 10000.0), scale=1.0)
    q = torch.zeros(H * D, width)
    kk = torch.zeros(G * D, width)
    for h in range(H):
        q[h * D + 12, 0] = 1.0  # entry 12 lies behind the turned ones
    kk[12, 0] = 1.0
    zeros = {"l0.mix.q.b": torch.zeros(H * D), "l0.mix.k.b": torch.zeros(G * D)}
    for case, j in enumerate((3, 0, 2 * page_size - 1, 2 * page_size, n - 2 * page_size - 1, n - 2)):
        rng = np.random.default_rng(10 + case)
        sink = torch.full((H,), 35.0)  # the marked score is 36; every other is below 4
        p = _Layer(dtype, layer("attention", m), width=width, tensors={"l0.mix.q": q, "l0.mix.k": kk, "l0.mix.sink": sink, **zeros}, page_size=page_size)
        x = _marked(width, n, j, rng)
        xs = f64(x.to(torch.bfloat16).float() if dtype == "bfloat16" else x)
        pos = np.arange(n, dtype=np.float64)
        want = plain.sink_attention(xs, p.t, "l0.mix.", m, pos, [None])
        blind = xs.copy()
        blind[j] = 0.0
        no_sink = dict(p.t)
        no_sink["l0.mix.sink"] = np.full(H, -50.0)
        scale_of = np.abs(want[-1]).max()
        assert np.abs(plain.sink_attention(blind, p.t, "l0.mix.", m, pos, [None])[-1] - want[-1]).max() > 0.3 * scale_of
        assert np.abs(plain.sink_attention(xs, no_sink, "l0.mix.", m, pos, [None])[-1] - want[-1]).max() > 0.1 * scale_of
        for k, portions in enumerate(((n,), (n - 40,) + (1,) * 40, (100, 2, 150, 37, 2, n - 291))):
            got = _mixer_alone(p, x, portions, rid=f"k{case}_{k}")
            assert tt.rel_err(got, want) < (2e-5 if dtype == "float32" else 6e-2), (j, portions[:3])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m", [att(4, 2, 16, 16, rot=(8, 500.0)), att(3, 1, 6, 6, rot=(2, 50.0), scale=0.3), att(2, 1, 24, 8, rot=(24, 100.0)), att(1, 1, 64, 64, rot=(64, 1e4)), att(2, 2, 8, 12)])
def test_gated_attention_alone_in_portions(dtype, m):
    """The attention beside the recurrence: no biases, no sink, an output gate; keys and values of one width (the engine's
    paged kernels) and of two (the plain kernel)."""
    p = _Layer(dtype, layer("parallel", par(m, 16, 1, 1)), width=72)
    rng = np.random.default_rng(4)
    for k, portions in enumerate(PORTIONS):
        x, xs = _inputs(p, rng, sum(portions))
        want = plain.gated_attention(xs, p.t, "l0.mix.left.", m, np.arange(len(xs), dtype=np.float64))
        got = _mixer_alone(p, x, portions, rid=f"g{k}", part=p.block.mixer.left)
        assert tt.rel_err(got, want) < MIXER_TOL[dtype], (m, portions[:4])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width,blocks,taps", [(48, 3, 4), (51, 3, 2), (64, 1, 1), (40, 5, 5), (176, 2, 4), (300, 2, 3), (8, 8, 7)])
def test_the_gated_recurrence_alone_in_portions(dtype, width, blocks, taps):
    """The state and the convolution's last inputs travel from portion to portion, down to single tokens; a second request in a
    slot that was used before starts from zeros whatever the slot holds; one tap keeps no inputs, one part is one matrix."""
    m = par(att(1, 1, 8, 8), width, blocks, taps)
    p = _Layer(dtype, layer("parallel", m), width=72)
    rng = np.random.default_rng(5)
    for k, portions in enumerate(PORTIONS + ((260,), (3, 255, 2))):
        x, xs = _inputs(p, rng, sum(portions))
        want = plain.gated_recurrence(xs, p.t, "l0.mix.right.", m["right"])
        got = _mixer_alone(p, x, portions, rid=f"r{k}", part=p.block.mixer.right)
        assert tt.rel_err(got, want) < MIXER_TOL[dtype], (width, blocks, taps, portions[:4])


def test_the_recurrence_carries_a_token_far():
    """Channels that hardly decay carry one early token to the end of a long sequence: the output there changes by much
    when that token's input changes. The engine follows the twin whole, in portions and token by token."""
    W, width, n = 32, 64, 400
    m = par(att(1, 1, 8, 8), W, 2, 3)
    p = _Layer("float32", layer("parallel", m), width=width, tensors={"l0.mix.right.lam": torch.full((W,), -7.6)})
    rng = np.random.default_rng(6)
    x, xs = _inputs(p, rng, n)
    x[3] *= 30.0
    xs = f64(x)
    want = plain.gated_recurrence(xs, p.t, "l0.mix.right.", m["right"])
    blind = xs.copy()
    blind[3] = 0.0
    moved = np.abs(plain.gated_recurrence(blind, p.t, "l0.mix.right.", m["right"])[-1] - want[-1]).max()
    assert moved > 0.05 * np.abs(want[-1]).max()
    for k, portions in enumerate(((n,), (n - 40,) + (1,) * 40, (100, 2, 150, 37, 2, 107, 2))):
        assert tt.rel_err(_mixer_alone(p, x, portions, rid=f"f{k}", part=p.block.mixer.right), want) < 2e-5


@pytest.mark.parametrize("dtype", DTYPES)
def test_two_mixers_side_by_side_with_their_weights(dtype):
    m = par(att(4, 2, 16, 16, rot=(8, 500.0)), 48, 3, 4, left_scale=-0.6, right_scale=1.7)
    p = _Layer(dtype, layer("parallel", m), width=72)
    rng = np.random.default_rng(7)
    for k, portions in enumerate(PORTIONS[:3]):
        x, xs = _inputs(p, rng, sum(portions))
        want = plain.parallel_mixer(xs, p.t, "l0.mix.", m, np.arange(len(xs), dtype=np.float64))
        assert tt.rel_err(_mixer_alone(p, x, portions, rid=f"s{k}"), want) < MIXER_TOL[dtype]


def _ffn_alone(p, x):
    from liyab_amd.engine import StepItem

    n = x.shape[0]
    ffn = p.block.ffn
    k = int(getattr(ffn, "rows_a_token", 1))
    y = torch.zeros(n * k, p.width, dtype=torch.float32, device=DEV)
    p.core.open("f")
    ctx, _ = p.core.step_fn.prepare([StepItem("f", [1] * n, [])])
    ffn.forward(x.to(DEV).to(p.core.dtype), ctx, None, out=y)
    p.core.close("f")
    return f64(y).reshape(n, k, p.width)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("ff,limit", [(96, 1.0), (50, 0.05), (200, 100.0)])
def test_the_clamped_feed_forward_alone(dtype, ff, limit):
    """Limits that clamp some, most and no entries."""
    p = _Layer(dtype, layer("attention", att(1, 1, 8, 8), dense(ff, limit)), width=72)
    x, xs = _inputs(p, np.random.default_rng(8), 37, scale=2.0)
    want = plain.dense_feed_forward(xs, p.t, "l0.mlp.", {"limit": limit})
    assert tt.rel_err(_ffn_alone(p, x)[:, 0], want) < MIXER_TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m", [moe(24, 8, 2, groups=(4, 2), shared=40), moe(13, 6, 3, groups=(3, 2), shared=7), moe(16, 6, 3), moe(20, 1, 1, groups=(1, 1)), moe(8, 4, 4, groups=(2, 2)),
                               moe(12, 12, 5, groups=(6, 3), shared=3), moe(48, 16, 5, groups=(4, 2), shared=80)])
def test_experts_chosen_among_groups_alone(dtype, m):
    """Who is chosen, with which weight, and the experts' sum with the shared expert's row, for few rows (the small tiles) and
    many; the twin's router reads the same rounded rows, so the choice is compared in bfloat16 too."""
    from liyab_amd.kernels import ops

    p = _Layer(dtype, layer("attention", att(1, 1, 8, 8), m), width=72)
    r = m["router"]
    g = r.get("groups") or {"count": 1, "keep": 1}
    for n in (1, 9, 300):
        x, xs = _inputs(p, np.random.default_rng(9 + n), n, scale=1.5)
        want = plain.routed_feed_forward(xs, p.t, "l0.mlp.", m)
        got = _ffn_alone(p, x)
        assert got.shape[1] == r["top"] + (1 if "shared" in m else 0)
        assert tt.rel_err(got.sum(axis=1), want) < MIXER_TOL[dtype], (m, n)
        # the choice itself
        z = torch.from_numpy(xs @ p.t["l0.mlp.router"].T).float().to(DEV).contiguous()
        E, top = r["experts"], r["top"]
        block = ops.GROUPED_ROWS
        tiles = ops.moe_tiles(n * top, E, block)
        ids = torch.empty(n * top, dtype=torch.int32, device=DEV)
        w = torch.empty(n * top, dtype=torch.float32, device=DEV)
        ops.moe_route(z, top, ids, w, torch.empty(tiles * block, dtype=torch.int32, device=DEV), torch.empty(tiles, dtype=torch.int32, device=DEV),
                      block=block, groups=(g["count"], g["keep"]))
        chosen, weights = plain.route(f64(z), top, g["count"], g["keep"])
        assert (ids.cpu().numpy().reshape(n, top) == chosen).all()
        assert np.abs(f64(w).reshape(n, top) - weights).max() < 1e-5
        per = E // g["count"]
        assert all(len({int(e) // per for e in row}) <= g["keep"] for row in chosen)


def test_groups_keep_a_better_expert_out():
    """The largest logit lies in one group, the next three in another that is not kept: the choice stays inside the kept group."""
    from liyab_amd.kernels import ops

    z = torch.tensor([[0.0, 5.0, 0.1, 0.2, 4.0, 4.5, 4.8, 0.3], [3.0, 2.9, 2.8, 2.7, 0.0, 0.0, 0.0, 3.1]], device=DEV)
    ids = torch.empty(4, dtype=torch.int32, device=DEV)
    w = torch.empty(4, dtype=torch.float32, device=DEV)
    tiles = ops.moe_tiles(4, 8, ops.GROUPED_ROWS)
    ops.moe_route(z, 2, ids, w, torch.empty(tiles * 64, dtype=torch.int32, device=DEV), torch.empty(tiles, dtype=torch.int32, device=DEV), groups=(2, 1))
    assert ids.cpu().tolist() == [1, 3, 7, 4]
    chosen, weights = plain.route(f64(z), 2, 2, 1)
    assert chosen.tolist() == [[1, 3], [7, 4]] and np.abs(f64(w).reshape(2, 2) - weights).max() < 1e-6
    assert abs(float(w[0] + w[1]) - 1.0) < 1e-6


@pytest.mark.parametrize("dtype", DTYPES)
def test_values_of_the_first_layer_reach_the_later_ones(dtype, tmp_path):
    """Three attention layers that mix values at rates near one: what the later layers cache is nearly the first layer's
    values, so a fault in whose values are kept, or at which rate, shows in full; whole, in portions and token by token."""
    cfg = config(90, 48, 1e-5, [layer("attention", att(2, 1, 8, 8, rot=(4, 100.0), v_mix=True)), layer("attention", att(4, 1, 16, 8, v_mix=True), dense(32)),
                                layer("attention", att(2, 2, 8, 8)), layer("attention", att(1, 1, 8, 8, rot=(8, 10.0), v_mix=True))])
    from liyab_amd.weights import write_random_model

    d = str(tmp_path / "m")
    write_random_model(d, json.loads(json.dumps(cfg)), 3)
    raw, tensors = read_model(d)
    tensors["l1.mix.vmix"] = np.array(0.9)
    tensors["l3.mix.vmix"] = np.array(-0.8)
    tensors["l0.mix.vmix"] = np.array(123.0)  # the first layer's rate is read by nobody
    from safetensors.numpy import save_file

    save_file({k: v.astype(np.float32) for k, v in tensors.items()}, os.path.join(d, "model.safetensors"))
    t = twin_tensors(tensors, dtype)
    reqs = {f"v{i}": tt.random_tokens(30 + i, n, 90) for i, n in enumerate([1, 40, 90])}
    ref = {rid: plain.forward(raw, t, toks) for rid, toks in reqs.items()}
    same = dict(t)
    same["l1.mix.vmix"] = np.array(0.0)
    assert np.abs(plain.forward(raw, same, reqs["v1"]) - ref["v1"]).max() > 0.05 * np.abs(ref["v1"]).max()
    for steps in (tt.schedule_whole(reqs), tt.schedule_bulk_tail(reqs, tail=20), tt.schedule_portions(reqs, (2, 5, 1, 9)), tt.schedule_mixed(reqs, seed=2, max_live=3)):
        core = make_core(d, dtype, None, max_requests=3, num_pages=tt.max_live_pages(steps, 16))
        check_logits(tt.run_schedule(core, steps), reqs, ref, dtype, f"larulorn-values {dtype}", family="larulorn-values")


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
    check_logits(got, reqs, reference[(name, dtype)], dtype, f"larulorn-whole {name} {dtype}")
    core.manager.check()
    assert not core.manager.groups or core.manager.pages_in_use() == 0
    if dtype == "float32":
        from liyab_amd.engine import StepItem

        rid, toks = list(reqs.items())[2]
        streams, caught = [], []
        plain.forward(models[(name, dtype)][1], models[(name, dtype)][2], toks, streams)
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
        assert len(caught) == len(streams) == len(models[(name, dtype)][1]["layers"])
        for got_x, want_x in zip(caught, streams):
            assert tt.rel_err(got_x, want_x) < 1e-5


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_a_prompt_then_its_last_tokens_one_by_one(name, dtype, models, reference):
    reqs = make_requests(name)
    steps = tt.schedule_bulk_tail(reqs, tail=45)
    core = make_core(models[(name, dtype)][0], dtype, tt.max_live_tokens(steps))
    got = tt.run_schedule(core, steps)
    check_logits(got, reqs, reference[(name, dtype)], dtype, f"larulorn-decode {name} {dtype}")


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
    check_logits(got, reqs, reference[(name, dtype)], dtype, f"larulorn-portions {name} {dtype}")


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
    check_logits(got, reqs, ref, dtype, f"larulorn-mixed {name} {dtype}")
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
    check_logits(got, reqs, reference[(name, dtype)], dtype, f"larulorn-long {name} {dtype}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_trace_program(dtype, models, reference, tmp_path):
    name = "odd"
    reqs = make_requests(name)
    steps = tt.schedule_mixed(reqs, seed=5, max_live=4)
    got = tt.run_trace_program(models[(name, dtype)][0], dtype, steps, str(tmp_path), tt.max_live_tokens(steps), CONFIGS[name][0]["vocab"])
    check_logits(got, reqs, reference[(name, dtype)], dtype, f"larulorn-trace {dtype}")


def draw_config(seed):
    """A geometry drawn from the seed: every size, constant and count, the layers' kinds and order, which layers mix values."""
    rng = np.random.default_rng(3000 + seed)
    pick = lambda *options: options[int(rng.integers(len(options)))]  # noqa: E731
    width = pick(40, 48, 64, 96, 104, 160)
    shared_values = (pick(1, 2), pick(4, 8, 12, 16))  # key/value heads and the values' width of every layer that mixes values

    def rot(dim):
        if rng.random() < 0.2:
            return None
        dims = 2 * int(rng.integers(1, dim // 2 + 1))
        base = pick(10.0, 500.0, 10000.0, 5e5)
        return (dims, base, (pick(1.5, 2.0, 8.0), pick(16, 64, 1024), pick(4.0, 32.0), pick(0.25, 1.0))) if rng.random() < 0.5 else (dims, base)

    def attention(own):
        v_mix = own and rng.random() < 0.6
        kv, vdim = shared_values if v_mix else (pick(1, 2, 3), pick(4, 8, 12, 16, 40))
        dim = pick(4, 8, 10, 16, 24, 32) if own else pick(vdim, vdim, 8, 16)
        # (a score's 32-bit rounding enters its weight as it is, not relative to it: scores of wide heads under a scale of one
        # reach 30 and more, and the comparison then measures their rounding; such heads draw a smaller scale)
        return att(kv * pick(1, 2, 4), kv, dim, vdim, rot=rot(dim), v_mix=v_mix, scale=pick(None, 0.3, 1.0 if dim <= 8 else 0.4))

    def feed_forward():
        kind = pick(None, "dense", "moe", "moe")
        if kind == "dense":
            return dense(pick(8, 20, 24, 40, 56), pick(0.3, 1.0, 7.0))
        if kind == "moe":
            count = pick(1, 2, 3)
            per = pick(1, 2, 4)
            keep = int(rng.integers(1, count + 1))
            return moe(pick(8, 12, 24), count * per, int(rng.integers(1, keep * per + 1)), groups=pick(None, (count, keep)) if count == keep == 1 else (count, keep), shared=pick(None, 8, 20))
        return None

    def one():
        if rng.random() < 0.6:
            return layer("attention", attention(True), feed_forward())
        blocks = pick(1, 2, 3, 4)
        return layer("parallel", par(attention(False), blocks * pick(4, 8, 13, 20), blocks, pick(1, 2, 3, 4, 6), left_scale=pick(1.0, 0.7, -0.4), right_scale=pick(1.0, 1.3, 0.3)), feed_forward())

    layers = [one() for _ in range(int(rng.integers(1, 6)))]
    return config(pick(97, 256, 500), width, pick(1e-5, 1e-6, 1e-3), layers, logit_scale=pick(1.0, 0.4, 2.0)), pick(8, 16, 24)


@pytest.mark.parametrize("seed", range(12))
def test_drawn_geometries_whole_and_mixed(seed, tmp_path):
    cfg, page_size = draw_config(seed)
    reqs = {f"g{i}": tt.random_tokens(seed * 10 + i, n, cfg["vocab"]) for i, n in enumerate([1, 19, 77, 150, 260])}
    for dtype in DTYPES:
        d = str(tmp_path / f"m_{dtype}")
        raw, t = write_model(d, cfg, 100 + seed, dtype)
        ref = {rid: plain.forward(raw, t, toks) for rid, toks in reqs.items()}
        steps = tt.schedule_whole(reqs)
        core = make_core(d, dtype, tt.max_live_tokens(steps), page_size=page_size)
        check_logits(tt.run_schedule(core, steps), reqs, ref, dtype, f"larulorn-drawn seed {seed} whole {dtype}", family="larulorn-drawn", tol=TOL_DRAWN)
        steps = tt.schedule_mixed(reqs, seed=seed, max_live=3)
        core = make_core(d, dtype, None, page_size=page_size, max_requests=3, num_pages=tt.max_live_pages(steps, page_size))
        check_logits(tt.run_schedule(core, steps), reqs, ref, dtype, f"larulorn-drawn seed {seed} mixed {dtype}", family="larulorn-drawn", tol=TOL_DRAWN)
        core.manager.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_real_widths_in_long_steps(dtype, tmp_path):
    """Heads of 64 and 128, a width of 512, a recurrence of 768 channels in parts of 256, prompts of hundreds of tokens in one
    step and in mixed batches: the tiles of the large products, the matrix-core attention with a sink, the experts' large tiles."""
    cfg = config(1000, 512, 1e-5, [
        layer("attention", att(8, 2, 64, 64, rot=(32, 10000.0, (4.0, 256, 16.0, 1.0)), v_mix=True), moe(128, 16, 4, groups=(4, 2), shared=256)),
        layer("parallel", par(att(4, 2, 64, 64, rot=(64, 10000.0)), 768, 3, 4), dense(1024)),
        layer("attention", att(4, 2, 128, 64, rot=(64, 5e5), v_mix=True), dense(768, 0.5)),
        layer("parallel", par(att(8, 8, 32, 32, rot=(16, 100.0)), 512, 1, 4, left_scale=1.0, right_scale=0.5), moe(64, 8, 2)),
    ], logit_scale=0.6)
    d = str(tmp_path / "m")
    raw, t = write_model(d, cfg, 31, dtype)
    reqs = {f"r{i}": tt.random_tokens(900 + i, n, raw["vocab"]) for i, n in enumerate([330, 700, 45])}
    ref = {rid: plain.forward(raw, t, toks) for rid, toks in reqs.items()}
    steps = tt.schedule_whole(reqs)
    core = make_core(d, dtype, tt.max_live_tokens(steps))
    check_logits(tt.run_schedule(core, steps), reqs, ref, dtype, f"larulorn-wide whole {dtype}", family="larulorn-wide")
    steps = tt.schedule_mixed(reqs, seed=3, max_live=3, portions=(2, 130, 64, 300, 17))
    core = make_core(d, dtype, None, max_requests=3, num_pages=tt.max_live_pages(steps, 16))
    check_logits(tt.run_schedule(core, steps), reqs, ref, dtype, f"larulorn-wide mixed {dtype}", family="larulorn-wide")
    core.manager.check()


def generate_greedy(raw, t, prompt, n_new):
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(np.argmax(plain.forward(raw, t, toks)[-1])))
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
        ref = plain.forward(raw, t, prompt + res.tokens[:-1])
        for i, tok in enumerate(res.tokens):
            row = ref[len(prompt) - 1 + i]
            slack = (1e-5 if dtype == "float32" else 5e-2) * np.abs(row).max()
            assert row[tok] >= row.max() - slack, f"token {i} of prompt length {len(prompt)}: {tok} vs {int(np.argmax(row))}"
        if dtype == "float32":
            assert res.tokens == generate_greedy(raw, t, prompt, n_new)
    engine.core.manager.check()


def test_command_line(models):
    d, raw, tensors = models[("mix", "float32")]
    prompt = tt.random_tokens(90, 11, raw["vocab"])
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "liyab-cli"), "-m", d, "-p", ",".join(map(str, prompt)), "-n", "6",
                        "--temp", "0", "--dtype", "float32", "--json", "--phases"], capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    turn = [json.loads(l) for l in p.stdout.splitlines() if l.startswith("{")][1]
    assert turn["tokens"] == generate_greedy(raw, tensors, prompt, 6)
    assert set(turn["phases_ms"]) == {"embed", "scored_attention", "side_by_side", "routed_ffn", "clamped_glu", "lm_head"}
