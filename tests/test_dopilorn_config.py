"""Dopilorn's configuration, plan and random-weights mode (no GPU)."""

import json

import numpy as np
import pytest

import plain_dopilorn as plain
from liyab_amd.config import config_from_dict
from liyab_amd.config.dopilorn import DopilornConfig
from liyab_amd.errors import InvalidModel, Unsupported

RAW = {
    "architecture": "Dopilorn", "vocab": 97, "width": 40, "norm": {"eps": 1e-5}, "canon": {"taps": 3}, "logit_softcap": 9.0,
    "loop": {"start": 1, "stop": 3, "times": 2},
    "layers": [
        {"type": "general_delta", "mixer": {"heads": 2, "dim": 12, "decay_rank": 5}, "mlp": {"kind": "dense", "ff": 24}},
        {"type": "attention", "mixer": {"heads": 4, "kv_heads": 2, "dim": 6, "vdim": 10, "scale": 0.3, "diff": 0.4, "conv": 2, "mask": {"size": 7}}, "mlp": None},
        {"type": "latent_attention", "mixer": {"heads": 3, "dim": 8, "vdim": 6, "kv_rank": 12, "q_rank": 10, "scale": 0.2}, "mlp": {"kind": "dense", "ff": 30}},
        {"type": "general_delta", "mixer": {"heads": 1, "dim": 16}, "mlp": None},
    ],
}


def fresh():
    return json.loads(json.dumps(RAW))


def test_the_registry_finds_it_and_the_keys_come_back():
    cfg = config_from_dict(fresh())
    assert isinstance(cfg, DopilornConfig)
    again = config_from_dict(cfg.to_json())
    assert again == cfg
    assert cfg.layers[3].mixer.decay_rank == 16  # (nothing says otherwise: the default)
    assert cfg.layers[1].mixer.window == 7 and cfg.layers[1].mixer.taps == 2 and cfg.taps == 3 and cfg.softcap == 9.0


def test_the_decays_rank_is_the_shape_of_its_tensor():
    cfg = config_from_dict(fresh(), shapes={"l0.mix.w1": (7, 40), "l3.mix.w1": (3, 40)})
    assert cfg.layers[0].mixer.decay_rank == 7 and cfg.layers[3].mixer.decay_rank == 3


def test_the_run_order_follows_the_twin():
    for loop in (None, {"start": 1, "stop": 3, "times": 2}, {"start": 0, "stop": 4, "times": 3}, {"start": 3, "stop": 4, "times": 1},
                 {"start": 2, "stop": 2, "times": 5}, {"start": 0, "stop": 1, "times": 4}):
        raw = fresh()
        if loop is None:
            del raw["loop"]
        else:
            raw["loop"] = loop
        cfg = config_from_dict(raw)
        assert cfg.runs() == plain.run_order(raw)
        plan = cfg.plan()
        assert len(plan.layers) == len(cfg.runs()) == len(plan.order)
        for spec, (i, begins) in zip(plan.layers, cfg.runs()):
            assert spec.norm_mixer.tensors["weight"].name == f"l{i}.norm1"
            assert (spec.entry is None) == (begins is None)
            if begins is not None:
                assert spec.entry.index == begins and spec.entry.passes == loop["times"]
            assert (spec.ffn is None) == (raw["layers"][i]["mlp"] is None) and (spec.ffn_conv is None) == (spec.ffn is None)


def test_what_is_optional_may_be_absent():
    raw = fresh()
    del raw["canon"], raw["logit_softcap"], raw["loop"]
    del raw["layers"][1]["mixer"]["mask"], raw["layers"][1]["mixer"]["conv"], raw["layers"][1]["mixer"]["kv_heads"], raw["layers"][1]["mixer"]["vdim"]
    cfg = config_from_dict(raw)
    att = cfg.layers[1].mixer
    assert (cfg.taps, cfg.softcap, cfg.loop) == (0, 0.0, None)
    assert (att.window, att.taps, att.n_kv_head, att.value_dim) == (0, 0, 4, 6)
    plan = cfg.plan()
    assert plan.head.softcap == 0.0 and all(spec.input_conv is None and spec.entry is None for spec in plan.layers)
    assert "loop.in" in plan.ignorable


@pytest.mark.parametrize("change,error", [
    (lambda r: r.pop("vocab"), InvalidModel),
    (lambda r: r["norm"].pop("eps"), InvalidModel),
    (lambda r: r["layers"][0].update(type="convolution"), Unsupported),
    (lambda r: r["layers"][1]["mixer"].update(kv_heads=3), InvalidModel),
    (lambda r: r["layers"][2]["mixer"].pop("kv_rank"), InvalidModel),
    (lambda r: r["layers"][0].update(mlp={"kind": "moe"}), Unsupported),
    (lambda r: r["loop"].update(stop=9), InvalidModel),
    (lambda r: r["canon"].update(taps=0), InvalidModel),
])
def test_what_is_wrong_is_refused(change, error):
    raw = fresh()
    change(raw)
    with pytest.raises(error):
        config_from_dict(raw)


def test_random_weights_fit_the_twin(tmp_path):
    """The random-weights mode draws every tensor the twin reads, a looped layer's once; the twin runs on them, and a change of any
    constant of the design changes its logits."""
    from liyab_amd.weights import write_random_model
    from plain_gpt2 import read_model

    d = write_random_model(str(tmp_path / "m"), fresh(), 3)
    raw, t = read_model(d)
    assert {"loop.in", "loop.step", "l1.mix.q.conv", "l1.mix.lk2", "l2.mix.dq.norm", "l0.mix.a.b", "l0.canon2", "l3.mix.w0"} <= set(t)
    assert "l1.norm2" not in t and "l3.canon2" not in t and t["l0.mix.w1"].shape == (5, 40) and t["loop.step"].shape == (2, 40)
    toks = [5, 17, 3, 9, 11, 60, 2, 4, 8, 1, 96, 33]
    base = plain.forward(toks, t, raw)
    assert base.shape == (len(toks), 97) and np.isfinite(base).all() and np.abs(base).max() <= 9.0
    for change in (lambda r: r["layers"][1]["mixer"].update(diff=0.1), lambda r: r["layers"][1]["mixer"]["mask"].update(size=6),
                   lambda r: r["loop"].update(times=1), lambda r: r.update(logit_softcap=5.0), lambda r: r["norm"].update(eps=1e-2)):
        other = json.loads(json.dumps(raw))
        change(other)
        assert np.abs(plain.forward(toks, t, other) - base).max() > 1e-6
