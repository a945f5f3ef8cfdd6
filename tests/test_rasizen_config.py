"""The Rasizen configuration, its model spec and the plain implementation, without a GPU."""
import copy
import json

import numpy as np
import pytest

from plain import rasizen_plain as R

CFG = {
    "architecture": "Rasizen", "vocab": 50, "width": 24, "residual_mult": 0.5, "norm": {"eps": 1e-5, "groups": 3},
    "layers": [
        {"type": "latent_attention", "mlp": {"kind": "dense", "ff": 40},
         "mixer": {"heads": 2, "dim": 6, "rot_dim": 4, "vdim": 10, "kv_rank": 12, "scale": 0.3,
                   "mask": {"size": 5}, "rot": {"base": 100.0, "dims": 2}}},
        {"type": "mingru", "mixer": {"width": 20}, "mlp": None},
        {"type": "latent_attention", "mlp": None,
         "mixer": {"heads": 3, "dim": 4, "rot_dim": 4, "vdim": 6, "kv_rank": 12, "scale": 0.2, "kv_from": 0,
                   "mask": {"size": 9}, "rot": {"base": 100.0, "dims": 2}}},
    ],
}


def test_configuration_round_trip_and_spec():
    from sonicboom_amd.config import architecture_of
    arch = architecture_of(CFG)
    cfg = arch.config_class.from_dict(CFG)
    assert cfg.to_dict() == CFG
    assert cfg.layers[2].mixer.kv_from == 0 and cfg.layers[0].mixer.rot_dims == 2 and cfg.norm_groups == 3
    spec = arch.build_spec(cfg)
    shapes = {t.name: t.shape for t in spec.all_tensors()}
    assert shapes["embed"] == (50, 24) and shapes["final.norm"] == (24,)
    assert shapes["l0.mix.q"] == (2 * 10, 24) and shapes["l0.mix.dkv"] == (16, 24) and shapes["l0.mix.dkv.norm"] == (12,)
    assert shapes["l0.mix.uk"] == (12, 12) and shapes["l0.mix.uv"] == (20, 12) and shapes["l0.mix.g"] == (20, 24)
    assert shapes["l0.mlp.up"] == (40, 24) and shapes["l0.mlp.act"] == (2,) and "l0.norm2" in shapes
    assert shapes["l1.mix.z"] == (20, 24) and shapes["l1.mix.x.b"] == (20,) and shapes["l1.mix.o"] == (24, 20)
    assert "l1.norm2" not in shapes and "l2.mix.dkv" not in shapes and "l2.mlp.up" not in shapes
    # the reader names the writer's cache and does not write it; the recurrence keeps no rows
    assert [(e.cache, e.writes_cache) for e in spec.order] == [(0, True), (None, True), (0, False)]
    assert spec.blocks[0].parts["mixer"].params["out_scale"] == 0.5
    assert spec.blocks[0].parts["mixer_norm"].params["groups"] == 3


@pytest.mark.parametrize("edit, message", [
    (lambda c: c["layers"][0]["mixer"].pop("heads"), "layers[0].mixer.heads"),
    (lambda c: c["layers"][1].update(type="lstm"), "unknown layer type"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=1), "kv_from"),
    (lambda c: c["layers"][2]["mixer"].update(kv_rank=8), "differ from those of layer 0"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=3), "rot.dims"),
    (lambda c: c["norm"].update(groups=5), "groups"),
    (lambda c: c.pop("norm"), "norm"),
    (lambda c: c["layers"][0]["mlp"].update(kind="moe"), "unknown feed-forward"),
])
def test_configuration_errors_name_the_key(edit, message):
    from sonicboom_amd.config import ConfigError, architecture_of
    bad = copy.deepcopy(CFG)
    edit(bad)
    with pytest.raises(ConfigError, match=message.replace("[", r"\[").replace("]", r"\]")):
        architecture_of(bad).config_class.from_dict(bad)


def test_unknown_architecture_is_refused():
    from sonicboom_amd.config import ConfigError, architecture_of
    with pytest.raises(ConfigError, match="unknown architecture"):
        architecture_of({"architecture": "Nothing"})


def test_a_shared_cache_keeps_what_its_widest_reader_sees():
    """The writer's window is 5, the reader's 9: the cache entry must hold 9 (and everything, if a
    reader has no window)."""
    from sonicboom_amd.parts import RowsSpec

    def entry_window(windows):
        need = None
        for w in windows:
            key = RowsSpec((16,), w).key()
            need = key if need is None else key[:2] + (0 if 0 in (need[2], key[2]) else max(need[2], key[2]),)
        return need[2]
    assert entry_window([5, 9]) == 9 and entry_window([9, 5]) == 9 and entry_window([5, 0]) == 0


def random_weights(cfg, seed=0, scale=0.4):
    from sonicboom_amd.config import architecture_of
    arch = architecture_of(cfg)
    spec = arch.build_spec(arch.config_class.from_dict(cfg))
    rng = np.random.default_rng(seed)
    return {t.name: rng.normal(t.init[0], scale, size=t.shape) for t in spec.all_tensors()}


def test_plain_prefix_property_and_window():
    """The plain implementation itself: logits of a prefix do not change when tokens follow, and a
    token outside every window does not reach a position's logits through attention alone."""
    w = random_weights(CFG)
    tokens = list(np.random.default_rng(1).integers(0, 50, size=30))
    full = R.forward(CFG, w, tokens)
    assert np.allclose(R.forward(CFG, w, tokens[:17]), full[:17], atol=1e-12)
    # attention-only model: change token 0; positions whose every window excludes it keep their logits
    att = copy.deepcopy(CFG)
    att["layers"] = [att["layers"][0], att["layers"][2]]
    att["layers"][1]["mixer"]["kv_from"] = 0
    wa = random_weights(att, 2)
    other = [int((tokens[0] + 1) % 50)] + tokens[1:]
    a, b = R.forward(att, wa, tokens), R.forward(att, wa, other)
    # layer 0 carries token 0 four positions on; the reader takes its keys and values from layer 0's own
    # rows, which come from the embedding alone, so it reaches eight positions back and no further
    reach = max(5 - 1, 9 - 1)
    assert np.allclose(a[reach + 1:], b[reach + 1:], atol=1e-12) and not np.allclose(a[reach], b[reach], atol=1e-9)


def test_plain_mechanisms():
    x = np.random.default_rng(3).normal(size=(4, 12))
    y = R.grouped_rms_norm(x, None, 0.0, 3)
    assert np.allclose((y.reshape(4, 3, 4) ** 2).mean(-1), 1.0)
    r = R.rotate_pairs(x, [0, 1, 2, 3], 4, 10.0)
    assert np.allclose(r[0], x[0]) and np.allclose(r[:, 4:], x[:, 4:])
    assert np.allclose(r[1, 0] ** 2 + r[1, 1] ** 2, x[1, 0] ** 2 + x[1, 1] ** 2)
    assert np.allclose(r[2, 2], x[2, 2] * np.cos(2 * 10 ** -0.5) - x[2, 3] * np.sin(2 * 10 ** -0.5))
    z = np.array([-2.0, 0.0, 3.0])
    assert np.allclose(R.xielu(z, 0.0, 0.0), [(0.5 + np.log(2)) * (np.exp(-2) - 1 + 2) - 1, 0.0, np.log(2) * 9 + 1.5])
    g = np.full((3, 2), 0.25)
    s = R.mingru_scan(g, np.ones((3, 2)))
    assert np.allclose(s[:, 0], [0.25, 0.4375, 0.578125])
