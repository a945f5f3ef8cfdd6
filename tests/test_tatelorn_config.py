"""The Tatelorn configuration, its model spec and the plain implementation, without a GPU."""
import copy

import numpy as np
import pytest

from plain import tatelorn_plain as T


def att(heads, kv_heads, dim, vdim, scale, softcap, v_mix, mlp):
    return {"type": "attention", "mlp": mlp,
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "softcap": softcap,
                      "v_mix": v_mix}}


def moe(experts, top, ff, limit, shared=None):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit},
            "shared": None if shared is None else {"ff": shared[0], "limit": shared[1]}}


CFG = {
    "architecture": "Tatelorn", "vocab": 50, "width": 24, "max_positions": 40, "logit_scale": 0.5,
    "embedding": {"scale": 3.0}, "norm": {"eps": 1e-5},
    "layers": [
        att(2, 1, 6, 10, 0.3, 7.0, False, moe(3, 1, 8, 2.0)),
        att(4, 2, 4, 6, 0.2, 4.0, True, {"kind": "dense", "ff": 40}),
        att(2, 2, 8, 6, 0.25, 30.0, True, None),
        att(6, 2, 4, 6, 0.5, 9.0, True, moe(5, 3, 12, 1.0, shared=(20, 0.75))),
    ],
}


def random_weights(cfg, seed=0, spread=0.3):
    """Weights by the file's names for a config.json dict, drawn here (not by the package)."""
    rng = np.random.default_rng(seed)
    d = cfg["width"]
    w = {"embed": rng.normal(0, spread, (cfg["vocab"], d)), "pos": rng.normal(0, spread, (cfg["max_positions"], d)),
         "embed.norm": rng.normal(0, 0.1, d), "final.norm": rng.normal(0, 0.1, d)}
    for i, layer in enumerate(cfg["layers"]):
        p, m, f = f"l{i}.", layer["mixer"], layer["mlp"]
        w[p + "norm1"] = rng.normal(0, 0.1, d)
        w[p + "mix.q"] = rng.normal(0, spread, (m["heads"] * m["dim"], d))
        w[p + "mix.k"] = rng.normal(0, spread, (m["kv_heads"] * m["dim"], d))
        w[p + "mix.v"] = rng.normal(0, spread, (m["kv_heads"] * m["vdim"], d))
        w[p + "mix.o"] = rng.normal(0, spread, (d, m["heads"] * m["vdim"]))
        w[p + "mix.q.norm"], w[p + "mix.k.norm"] = rng.normal(1, 0.1, m["dim"]), rng.normal(1, 0.1, m["dim"])
        if m.get("v_mix"):
            w[p + "mix.vmix"] = np.asarray(rng.uniform(0.2, 0.8))
        if f is None:
            continue
        w[p + "norm2"] = rng.normal(0, 0.1, d)
        if f["kind"] == "dense":
            sets = [(p + "mlp.", f["ff"])]
        else:
            sets = [(f"{p}mlp.e{e}.", f["expert"]["ff"]) for e in range(f["router"]["experts"])]
            w[p + "mlp.router"] = rng.normal(0, 1.0, (f["router"]["experts"], d))
            if f.get("shared"):
                sets.append((p + "mlp.shared.", f["shared"]["ff"]))
                w[p + "mlp.shared.sg"] = rng.normal(0, spread, (1, d))
        for q, ff in sets:
            w[q + "gate"], w[q + "up"], w[q + "down"] = (rng.normal(0, spread, (ff, d)), rng.normal(0, spread, (ff, d)),
                                                       rng.normal(0, spread, (d, ff)))
    return w


def test_configuration_round_trip_and_spec():
    from sonicboom_amd.config import architecture_of
    arch = architecture_of(CFG)
    cfg = arch.config_class.from_dict(CFG)
    assert cfg.to_dict() == CFG
    assert cfg.layers[3].mlp.shared_ff == 20 and cfg.layers[0].mlp.shared_ff == 0 and cfg.layers[2].mlp is None
    spec = arch.build_spec(cfg)
    shapes = {t.name: t.shape for t in spec.all_tensors()}
    assert set(shapes) == set(random_weights(CFG)), "the spec names the tensors of the file, no more and no fewer"
    for name, a in random_weights(CFG).items():
        assert shapes[name] == a.shape, name
    assert shapes["l1.mix.vmix"] == () and "l0.mix.vmix" not in shapes and "l2.norm2" not in shapes
    assert shapes["l0.mix.o"] == (24, 20) and shapes["l3.mlp.shared.sg"] == (1, 24) and shapes["pos"] == (40, 24)
    # every layer keeps keys and values of its own; the first mixing layer hands its values on
    assert [(e.cache, e.writes_cache) for e in spec.order] == [(i, True) for i in range(4)]
    mix = [b.parts["mixer"].params["value_mix"] for b in spec.blocks]
    assert mix == [None, "first", "mix", "mix"]
    m0 = spec.blocks[0].parts["mixer"].params
    assert (m0["v_dim"], m0["softcap"], m0["sink"], m0["qk_norm"], m0["scale"]) == (10, 7.0, True, True, 0.3)
    assert spec.blocks[0].kind == "outnorm" and spec.blocks[0].parts["mixer_norm"].params["offset"] == 1.0
    assert spec.head.params["scale"] == 0.5 and spec.embedding.params["scale"] == 3.0 and spec.max_positions == 40
    assert spec.blocks[1].parts["ffn"].params["activation"] == "relu"
    assert spec.blocks[3].parts["ffn"].params["alpha"] == 1.702


@pytest.mark.parametrize("edit, message", [
    (lambda c: c["layers"][0]["mixer"].pop("heads"), "layers[0].mixer.heads"),
    (lambda c: c["layers"][1].update(type="lstm"), "unknown layer type"),
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=3), "not a multiple"),
    (lambda c: c["layers"][2]["mixer"].update(vdim=8), "differ from those of layer 1"),
    (lambda c: c["layers"][3]["mlp"]["router"].update(top=6), "router"),
    (lambda c: c["layers"][3]["mlp"]["expert"].pop("limit"), "layers[3].mlp.expert.limit"),
    (lambda c: c["layers"][3]["mlp"].update(kind="sparse"), "unknown feed-forward"),
    (lambda c: c.pop("norm"), "norm"),
    (lambda c: c.pop("max_positions"), "max_positions"),
])
def test_configuration_errors_name_the_key(edit, message):
    from sonicboom_amd.config import ConfigError, architecture_of
    bad = copy.deepcopy(CFG)
    edit(bad)
    with pytest.raises(ConfigError, match=message.replace("[", r"\[").replace("]", r"\]")):
        architecture_of(bad).config_class.from_dict(bad)


def test_the_plain_implementation_is_causal_and_counts_positions():
    w = random_weights(CFG, seed=3)
    tokens = [int(t) for t in np.random.default_rng(1).integers(0, 50, size=17)]
    whole = T.forward(CFG, w, tokens)
    assert np.allclose(whole[:9], T.forward(CFG, w, tokens[:9]), atol=1e-12), "a prefix's logits do not change"
    # the learned positions count: the same token at another place gives another row
    assert not np.allclose(T.start(CFG, w, [5, 5])[0], T.start(CFG, w, [5, 5])[1])


def test_the_sink_takes_weight_and_the_cap_bounds_scores():
    s = np.array([[0.0, -np.inf], [50.0, 50.0]])
    p = T.sink_softmax(s, np.array([[True, False], [True, True]]))
    assert np.allclose(p[0], [0.5, 0.0]) and np.allclose(p[1].sum(), 1.0 - 1.0 / (1.0 + 2.0 * np.exp(50.0)))
    q, k = np.array([[100.0, 0.0]]), np.array([[1.0, 0.0], [-1.0, 0.0], [0.001, 0.0]])
    c = T.capped_scores(q, k, 1.0, 5.0)
    assert np.all(np.abs(c) <= 5.0) and abs(c[0, 0] - 5.0) < 1e-9 and abs(c[0, 2] - 5.0 * np.tanh(0.02)) < 1e-12


def test_routing_takes_the_largest_and_norms_over_the_chosen():
    z = np.array([[0.1, 2.0, 2.0, -1.0], [3.0, 0.0, 1.0, 1.0]])
    chosen, weight = T.route(z, 2)
    assert chosen.tolist() == [[1, 2], [0, 2]], "ties go to the lower number"
    assert np.allclose(weight[0], [0.5, 0.5]) and np.allclose(weight[1], np.exp([3.0, 1.0]) / np.exp([3.0, 1.0]).sum())


def test_value_mixing_takes_the_first_mixing_layers_values():
    w = random_weights(CFG, seed=4)
    x = np.random.default_rng(2).normal(size=(5, 24))
    v1, first = T.attention_values(CFG["layers"][1]["mixer"], w, "l1.mix.", x, None)
    assert first is v1, "the first mixing layer keeps its own values and hands them on"
    v2, still = T.attention_values(CFG["layers"][2]["mixer"], w, "l2.mix.", x, first)
    lam = float(w["l2.mix.vmix"])
    assert still is first and np.allclose(v2, (1 - lam) * T.linear(x, w["l2.mix.v"]) + lam * first)
    v0, none = T.attention_values(CFG["layers"][0]["mixer"], w, "l0.mix.", x, None)
    assert none is None and np.allclose(v0, T.linear(x, w["l0.mix.v"])), "a layer that does not mix is left alone"
