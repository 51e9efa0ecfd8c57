"""The Sidirax design on the host: its configuration and what it becomes (parts, tensor names, cache units,
state), and the plain implementation's mechanisms against direct sums."""
import copy
import math

import numpy as np
import pytest

import braidinfer_amd as B
import plain_sidirax as P
from braidinfer_amd.config import config_from_dict, config_from_folder, spec_of
from braidinfer_amd.engine.model import DecoderModel
from braidinfer_amd.errors import ConfigError


def small():
    rot = {"dims": 4, "base": 100.0, "scaling": {"factor": 2.0, "original": 32, "fast": 8.0, "slow": 1.0}}
    att = {"heads": 2, "dim": 8, "rot_dim": 4, "vdim": 6, "q_rank": 10, "kv_rank": 12, "scale": 0.3, "rot": rot}
    return {"architecture": "Sidirax", "vocab": 40, "width": 24, "norm": {"eps": 1e-5}, "layers": [
        {"type": "wkv", "mixer": {"heads": 2, "dim": 6, "decay_rank": 3}, "mlp": {"kind": "dense", "ff": 20, "limit": 2.0}},
        {"type": "latent_attention", "mixer": copy.deepcopy(att), "mlp": {"kind": "moe", "expert": {"ff": 8}, "router": {"experts": 3, "top": 2}}},
        {"type": "latent_attention", "mixer": dict(copy.deepcopy(att), kv_from=1, heads=3), "mlp": None}]}


def test_configuration_round_trip_and_registry():
    d = small()
    cfg = config_from_dict(d)
    assert isinstance(cfg, B.SidiraxConfig) and cfg.to_dict() == d
    assert config_from_dict(dict(d, architectures=["Sidirax"], architecture=None)).to_dict() == d
    assert "Sidirax" in B.registered_architectures()
    assert B.any_preset("sidirax-tiny").width == 96


@pytest.mark.parametrize("change,what", [
    (lambda d: d["layers"][2]["mixer"].__setitem__("kv_from", 2), "earlier layer"),
    (lambda d: d["layers"][2]["mixer"].__setitem__("kv_from", 0), "keeps no rows"),
    (lambda d: d["layers"][2]["mixer"].__setitem__("kv_rank", 16), "differ"),
    (lambda d: d["layers"][1]["mixer"]["rot"].__setitem__("dims", 6), "rot.dims"),
    (lambda d: d["layers"][1]["mlp"]["router"].__setitem__("top", 4), "chooses"),
    (lambda d: d["layers"][0]["mlp"].__setitem__("kind", "other"), "kind"),
    (lambda d: d["layers"][0].__setitem__("type", "attention"), "type"),
    (lambda d: d["layers"][0]["mlp"].pop("limit"), "limit"),
])
def test_configurations_that_are_refused(change, what):
    d = small()
    change(d)
    with pytest.raises(ConfigError, match=what):
        config_from_dict(d)


def test_parts_units_state_and_tensor_names():
    cfg = config_from_dict(small())
    spec = spec_of(cfg)
    assert [l.block for l in spec.layers] == ["parallel_residual"] * 3
    assert [(e.cache, e.writes_cache) for e in spec.schedule] == [(0, True), (1, True), (1, False)]
    model = DecoderModel(spec)
    needs = model.cache_needs()
    assert list(needs) == [1] and needs[1].kv_heads == 1 and needs[1].head_dim == 16 and needs[1].val_dim == 12
    states = model.state_needs()
    assert list(states) == [("entry", 0)] and states[("entry", 0)].shape[0] >= 2 * 6 * 6 + 24
    names = {s.name: tuple(s.shape) for s in model.weight_specs()}
    assert names["embed"] == (40, 24) and names["final.norm"] == (24,) and "head.weight" not in names
    assert names["l0.mix.w1"] == (3, 24) and names["l0.mix.w2"] == (12, 3) and names["l0.mix.u"] == (2, 6) and names["l0.mix.mu.w"] == (24,)
    assert names["l0.mlp.gate.b"] == (20,) and names["l0.mlp.down.b"] == (24,)
    assert names["l1.mix.dkv"] == (16, 24) and names["l1.mix.dkv.norm"] == (12,) and names["l1.mix.uq"] == (24, 10)
    assert names["l1.mix.uk"] == (16, 12) and names["l1.mix.uv"] == (12, 12) and names["l1.mix.sink"] == (2,)
    assert names["l1.mlp.e2.down"] == (24, 8) and names["l1.mlp.router"] == (3, 24) and names["l1.mlp.router.b"] == (3,)
    assert "l2.mix.dkv" not in names and "l2.mix.dkv.norm" not in names and names["l2.mix.uk"] == (24, 12)
    assert not any(n.startswith("l2.mlp") for n in names)
    assert list(spec.positions) == ["rope4@100.0/2.0,32.0,8.0,1.0"] and spec.positions["rope4@100.0/2.0,32.0,8.0,1.0"].params["pairing"] == "adjacent"


def test_a_size_that_only_a_tensor_gives(tmp_path):
    d = small()
    w = P.random_weights(d, seed=1)
    del d["layers"][0]["mixer"]["decay_rank"]
    with pytest.raises(ConfigError, match="decay_rank"):
        spec_of(config_from_dict(d))
    P.write_folder(str(tmp_path), d, w)
    cfg = config_from_folder(str(tmp_path))
    assert cfg.layers[0]["mixer"]["decay_rank"] == 3 and not cfg.missing_tensor_sizes()
    assert {s.name for s in DecoderModel(spec_of(cfg)).weight_specs()} == set(w)
    del w["l0.mix.w1"]
    P.write_folder(str(tmp_path), d, w)
    with pytest.raises(ConfigError, match="l0.mix.w1"):
        config_from_folder(str(tmp_path))


# ---------------------------------------------------- the plain mechanisms, directly -----
def test_plain_recurrence_is_the_sum_over_earlier_tokens():
    rng = np.random.default_rng(0)
    T, H, d = 9, 2, 3
    r, k, v = (rng.standard_normal((T, H, d)) for _ in range(3))
    decay = rng.uniform(0.2, 0.9, (T, H, d))
    u = rng.standard_normal((H, d))
    o, S = P.decayed_outer_recurrence(r, k, v, decay, u)
    for t in range(T):
        for h in range(H):
            want = (r[t, h] * u[h] * k[t, h]).sum() * v[t, h]
            for j in range(t):
                w = np.prod(decay[j + 1:t, h], axis=0)            # the decays of the tokens between j and t
                want = want + (r[t, h] * w * k[j, h]).sum() * v[j, h]
            assert np.allclose(o[t, h], want)
    o2, S2 = P.decayed_outer_recurrence(r[5:], k[5:], v[5:], decay[5:], u, state=P.decayed_outer_recurrence(r[:5], k[:5], v[:5], decay[:5], u)[1])
    assert np.allclose(o2, o[5:]) and np.allclose(S2, S)


def test_plain_attention_sink_and_mask():
    rng = np.random.default_rng(1)
    T, H = 6, 2
    q, k, v = rng.standard_normal((T, H, 4)), rng.standard_normal((T, H, 4)), rng.standard_normal((T, H, 3))
    sink = np.array([0.7, -1.0])
    o = P.sink_softmax_attention(q, k, v, 0.5, sink)
    for i in range(T):
        for h in range(H):
            e = np.exp(k[:i + 1, h] @ q[i, h] * 0.5)
            assert np.allclose(o[i, h], (e[:, None] * v[:i + 1, h]).sum(axis=0) / (e.sum() + math.exp(sink[h])))
    far = P.sink_softmax_attention(q, k, v, 0.5, np.array([-1e9, -1e9]))
    assert np.allclose(far, P.sink_softmax_attention(q, k, v, 0.5, None))
    assert np.allclose(far[0], v[0])                            # the first token sees itself alone


def test_plain_rotation_and_scaled_frequencies():
    f, mag = P.scaled_frequencies(8, 100.0, None)
    assert np.allclose(f, 100.0 ** (-np.arange(4) / 4.0)) and mag == 1.0
    sc = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}
    g, mag = P.scaled_frequencies(8, 100.0, sc)
    assert abs(mag - (0.1 * math.log(4.0) + 1.0)) < 1e-15
    assert np.isclose(g[0], f[0]) and np.isclose(g[-1], f[-1] / 4.0) and np.all(np.diff(g / f) <= 1e-12)
    x = np.random.default_rng(2).standard_normal((5, 3, 10))
    y = P.rotate_pairs(x, np.arange(5), g, mag)
    assert np.array_equal(y[..., 8:], x[..., 8:]) and np.allclose(y[0], np.concatenate([x[0, :, :8] * mag, x[0, :, 8:]], axis=-1))
    n = np.hypot(y[..., 0:8:2], y[..., 1:8:2])
    assert np.allclose(n, mag * np.hypot(x[..., 0:8:2], x[..., 1:8:2]))
    # a relative rotation: the product of a rotated query and key depends on the distance only
    a, b = x[:1, :1, :8], x[1:2, :1, :8]
    dots = [float((P.rotate_pairs(a, [p + 3], g)[0, 0] * P.rotate_pairs(b, [p], g)[0, 0]).sum()) for p in (0, 11, 40)]
    assert np.allclose(dots, dots[0])


def test_plain_experts_and_gated_unit():
    rng = np.random.default_rng(3)
    W, F, E = 6, 4, 3
    h = rng.standard_normal((5, W))
    w = {"router": rng.standard_normal((E, W)), "router.b": rng.standard_normal(E)}
    for e in range(E):
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = rng.standard_normal((F, W)), rng.standard_normal((F, W)), rng.standard_normal((W, F))
    every = P.routed_ff(h, w, "", E, E)
    z = h @ w["router"].T + w["router.b"]
    p = np.exp(z) / np.exp(z).sum(axis=1, keepdims=True)
    want = sum(p[:, e:e + 1] * ((P.silu(h @ w[f"e{e}.gate"].T) * (h @ w[f"e{e}.up"].T)) @ w[f"e{e}.down"].T) for e in range(E))
    assert np.allclose(every, want)
    one = P.routed_ff(h, w, "", E, 1)
    for t in range(5):
        e = int(np.argmax(z[t]))
        assert np.allclose(one[t], (P.silu(h[t] @ w[f"e{e}.gate"].T) * (h[t] @ w[f"e{e}.up"].T)) @ w[f"e{e}.down"].T)
    d = {"gate": rng.standard_normal((F, W)) * 3, "gate.b": rng.standard_normal(F), "up": rng.standard_normal((F, W)) * 3,
         "up.b": rng.standard_normal(F), "down": np.eye(W, F), "down.b": np.arange(W, dtype=float)}
    y = P.clamped_glu_ff(h, d, "", 1.5) - d["down.b"]
    assert np.all(y[:, :F] <= 1.5 * 2.5 + 1e-12) and np.all(y[:, F:] == 0)
    big = P.clamped_glu_ff(h, d, "", 1e9) - d["down.b"]
    g, u = h @ d["gate"].T + d["gate.b"], h @ d["up"].T + d["up.b"]
    assert np.allclose(big[:, :F], g * P.sigmoid(1.702 * g) * (u + 1))
