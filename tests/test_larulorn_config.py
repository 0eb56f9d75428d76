"""Larulorn's configuration, plan and random-weights mode, and the twin's own small checks (no GPU)."""

import json

import numpy as np
import pytest

import plain_larulorn as plain
from liyab_amd.config import config_from_dict
from liyab_amd.config.larulorn import LarulornConfig
from liyab_amd.errors import InvalidModel, Unsupported

RAW = {
    "architecture": "Larulorn", "vocab": 97, "width": 40, "norm": {"eps": 1e-5}, "logit_scale": 0.75,
    "layers": [
        {"type": "attention", "mixer": {"heads": 4, "kv_heads": 2, "dim": 6, "vdim": 10, "scale": 0.3, "v_mix": True,
                                        "rot": {"dims": 4, "base": 100.0, "scaling": {"factor": 4.0, "original": 32, "fast": 4.0, "slow": 0.5}}},
         "mlp": {"kind": "moe", "expert": {"ff": 12}, "router": {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 2}}, "shared": {"ff": 20}}},
        {"type": "parallel", "mixer": {"left": {"heads": 2, "kv_heads": 1, "dim": 8, "vdim": 8, "scale": 0.35, "rot": {"dims": 8, "base": 50.0}},
                                       "right": {"width": 24, "blocks": 3, "conv": 3}, "left_scale": 0.6, "right_scale": 1.3},
         "mlp": {"kind": "dense", "ff": 30, "limit": 0.7}},
        {"type": "attention", "mixer": {"heads": 2, "kv_heads": 2, "dim": 8, "vdim": 10, "scale": 0.2, "v_mix": True}, "mlp": None},
        {"type": "attention", "mixer": {"heads": 1, "kv_heads": 1, "dim": 16, "vdim": 4, "scale": 0.25}, "mlp": {"kind": "moe", "expert": {"ff": 8}, "router": {"experts": 3, "top": 1}}},
    ],
}


def fresh():
    return json.loads(json.dumps(RAW))


def test_the_registry_finds_it_and_the_keys_come_back():
    cfg = config_from_dict(fresh())
    assert isinstance(cfg, LarulornConfig)
    assert config_from_dict(cfg.to_json()) == cfg
    a, p = cfg.layers[0].mixer, cfg.layers[1].mixer
    assert (a.n_head, a.n_kv_head, a.head_dim, a.value_dim, a.rot_dims, a.rot_ramp, a.v_mix) == (4, 2, 6, 10, 4, (4.0, 4.0, 0.5, 32.0), True)
    assert (p.right.inner, p.right.blocks, p.right.taps, p.left_scale, p.right_scale, p.left.rot_ramp) == (24, 3, 3, 0.6, 1.3, None)
    m = cfg.layers[0].mlp
    assert (m.kind, m.ff, m.experts, m.top, m.groups, m.keep, m.shared_ff) == ("moe", 12, 6, 2, 3, 2, 20)
    assert (cfg.layers[3].mlp.groups, cfg.layers[3].mlp.keep, cfg.layers[3].mlp.shared_ff) == (1, 1, 0)  # (nothing says otherwise)
    assert cfg.logit_scale == 0.75 and cfg.layers[2].mlp is None


def test_the_plan_names_the_tensors_and_who_keeps_the_values():
    plan = config_from_dict(fresh()).plan()
    assert [spec.arrangement for spec in plan.layers] == ["sandwich"] * 4
    mixes = [getattr(spec.mixer, "value_mix", None) for spec in plan.layers]
    assert mixes == ["first", None, "later", ""]
    first, pair, later, own = (spec.mixer for spec in plan.layers)
    assert first.sink and first.biased and not first.gated and first.rotary.halves and first.rotary.ramp == (4.0, 4.0, 0.5, 32.0)
    assert pair.left.gated and not pair.left.sink and not pair.left.biased and pair.left.rotary.ramp is None and not pair.normed
    assert (pair.left_weight, pair.right_weight, pair.right.rate, pair.right.taps) == (0.6, 1.3, 8.0, 3)
    assert later.tensors["vmix"].name == "l2.mix.vmix" and own.rotary is None and "vmix" not in own.tensors
    assert plan.layers[0].post_norm_ffn.tensors["weight"].name == "l0.norm2b" and plan.layers[2].norm_ffn is None and plan.layers[2].post_norm_ffn is None
    ffn = plan.layers[0].ffn
    assert (ffn.groups, ffn.shared_inner, ffn.gated, ffn.activation, ffn.tensors[("down", 5)].name) == ((3, 2), 20, False, "relu2", "l0.mlp.e5.down")
    assert plan.head.logit_scale == 0.75 and plan.final_norm.tensors["weight"].name == "final.norm"
    glu = plan.layers[1].ffn
    assert (glu.limit, glu.slope, glu.shift) == (0.7, 1.702, 1.0)


@pytest.mark.parametrize("change,error", [
    (lambda r: r.pop("vocab"), InvalidModel),
    (lambda r: r["norm"].pop("eps"), InvalidModel),
    (lambda r: r["layers"][0].update(type="convolution"), Unsupported),
    (lambda r: r["layers"][0]["mixer"].update(kv_heads=3), InvalidModel),
    (lambda r: r["layers"][0]["mixer"]["rot"].update(dims=5), InvalidModel),
    (lambda r: r["layers"][0]["mixer"]["rot"].update(dims=8), InvalidModel),
    (lambda r: r["layers"][1]["mixer"]["right"].update(blocks=5), InvalidModel),
    (lambda r: r["layers"][1]["mixer"].pop("left_scale"), InvalidModel),
    (lambda r: r["layers"][1]["mixer"]["left"].update(v_mix=True), InvalidModel),
    (lambda r: r["layers"][2]["mixer"].update(vdim=12), InvalidModel),  # (values of another shape than the first layer's cannot be mixed with them)
    (lambda r: r["layers"][0]["mlp"]["router"].update(top=5), InvalidModel),
    (lambda r: r["layers"][0]["mlp"]["router"]["groups"].update(count=4), InvalidModel),
    (lambda r: r["layers"][1]["mlp"].update(kind="gated"), Unsupported),
    (lambda r: r["layers"][1]["mlp"].pop("limit"), InvalidModel),
])
def test_what_is_wrong_is_refused(change, error):
    raw = fresh()
    change(raw)
    with pytest.raises(error):
        config_from_dict(raw)


def test_random_weights_fit_the_twin(tmp_path):
    """The random-weights mode draws every tensor the twin reads; the twin runs on them, and a change of any constant of the
    configuration changes its logits."""
    from liyab_amd.weights import write_random_model
    from plain_gpt2 import read_model

    d = write_random_model(str(tmp_path / "m"), fresh(), 3)
    raw, t = read_model(d)
    assert {"embed", "head", "final.norm", "l0.mix.q.b", "l0.mix.sink", "l0.mix.vmix", "l2.mix.vmix", "l0.mlp.e5.up", "l0.mlp.shared.down", "l0.mlp.router",
            "l1.mix.left.g", "l1.mix.right.ra.b", "l1.mix.right.conv.b", "l1.mix.right.lam", "l1.norm2b", "l3.mlp.e2.down"} <= set(t)
    assert "l2.norm2" not in t and "l3.mix.vmix" not in t and "l3.mlp.shared.up" not in t
    assert t["l1.mix.right.ra"].shape == (3, 8, 8) and t["l1.mix.right.conv"].shape == (24, 3) and t["l0.mix.vmix"].shape == ()
    toks = [5, 17, 3, 9, 11, 60, 2, 4, 8, 1, 96, 33]
    streams = []
    base = plain.forward(raw, t, toks, streams)
    assert base.shape == (len(toks), 97) and np.isfinite(base).all() and len(streams) == 4
    for change in (lambda r: r["layers"][0]["mixer"]["rot"]["scaling"].update(factor=2.0), lambda r: r["layers"][0]["mixer"]["rot"]["scaling"].update(slow=2.0),
                   lambda r: r["layers"][1]["mixer"].update(right_scale=1.0), lambda r: r["layers"][0]["mlp"]["router"]["groups"].update(keep=1),
                   lambda r: r["layers"][1]["mlp"].update(limit=0.2), lambda r: r["layers"][2]["mixer"].update(v_mix=False),
                   lambda r: r.update(logit_scale=1.0), lambda r: r["norm"].update(eps=1e-2), lambda r: r["layers"][3]["mixer"].update(scale=0.5)):
        other = json.loads(json.dumps(raw))
        change(other)
        assert np.abs(plain.forward(other, t, toks) - base).max() > 1e-6


def test_the_twins_parts_on_cases_worked_by_hand():
    # a ramp: entries below `lo` keep their frequency, entries from `hi` on are divided by the factor
    f, mag = plain.turn_frequencies({"dims": 8, "base": 16.0, "scaling": {"factor": 4.0, "original": 8, "fast": 1.0, "slow": 0.25}})
    plain_f = np.array([16.0 ** (-2.0 * i / 8) for i in range(4)])
    at = lambda turns: 8 * np.log(8 / (2 * np.pi * turns)) / (2 * np.log(16.0))  # noqa: E731
    lo, hi = max(np.floor(at(1.0)), 0), min(np.ceil(at(0.25)), 7)
    ramp = np.clip((np.arange(4) - lo) / max(hi - lo, 0.001), 0, 1)
    assert np.allclose(f, plain_f / 4.0 * ramp + plain_f * (1 - ramp)) and abs(mag - (0.1 * np.log(4.0) + 1)) < 1e-15
    # a turn keeps a pair's length (times the factor) and leaves what lies behind the turned entries alone
    v = np.arange(1.0, 13.0).reshape(1, 1, 12)
    out = plain.turn_halves(v, np.array([3.0]), {"dims": 8, "base": 10.0})
    assert np.allclose(out[..., 8:], v[..., 8:]) and np.allclose(out[0, 0, 0] ** 2 + out[0, 0, 4] ** 2, 1.0 + 25.0)
    # a sink takes its share of the weight: one key with score 0 beside a sink of 0 weighs one half
    assert np.allclose(plain.causal_weights(np.zeros((1, 1)), sink=0.0), 0.5) and np.allclose(plain.causal_weights(np.zeros((2, 2)))[1], 0.5)
    # the recurrence from a zero state: the first output is sqrt(1 - a^2) i u, with no special case
    t = {"p.y": np.zeros((2, 3)), "p.y.b": np.ones(2), "p.x": np.eye(2, 3), "p.x.b": np.zeros(2), "p.conv": np.array([[0.0, 1.0], [0.5, 1.0]]), "p.conv.b": np.zeros(2),
         "p.ra": np.zeros((1, 2, 2)), "p.ra.b": np.zeros((1, 2)), "p.ri": np.zeros((1, 2, 2)), "p.ri.b": np.zeros((1, 2)), "p.lam": np.zeros(2), "p.o": np.eye(2)}
    h = np.array([[1.0, 2.0, 0.0], [0.0, 1.0, 0.0]])
    out = plain.gated_recurrence(h, t, "p.", {"width": 2, "blocks": 1, "conv": 2})
    a = np.exp(-8.0 * 0.5 * np.log(2.0))
    g = plain.gelu_tanh(np.ones(2))
    first = np.sqrt(1 - a * a) * 0.5 * np.array([1.0, 2.0])
    assert np.allclose(out[0], first * g)
    assert np.allclose(out[1], (a * first + np.sqrt(1 - a * a) * 0.5 * np.array([0.0, 1.0 + 0.5 * 2.0])) * g)
    # groups: the best expert's group is kept, a better expert outside it is not chosen
    chosen, weights = plain.route(np.array([[0.0, 5.0, 0.1, 0.2, 4.0, 4.5, 4.8, 0.3]]), 2, 2, 1)
    assert chosen.tolist() == [[1, 3]] and abs(weights.sum() - 1.0) < 1e-12 and weights[0, 0] > 0.99
