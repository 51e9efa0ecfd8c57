"""Host-side pieces of the Kesitar design: its configuration and part list, the cache units that keep one
row per block of tokens, the rule of which token rows stay, and the plain implementation against itself."""
import copy

import numpy as np
import pytest

import plain_kesitar as P
import braidinfer_amd as B
from braidinfer_amd.cache import CacheNeed, SequenceCache, StateNeed
from braidinfer_amd.config import config_from_dict, spec_of
from braidinfer_amd.engine.model import DecoderModel
from braidinfer_amd.errors import CacheError, ConfigError
from braidinfer_amd.parts.pooled_attention import window_and_open_block


def small():
    return copy.deepcopy(B.any_preset("kesitar-tiny").to_dict())


def test_config_round_trip_and_registry():
    d = small()
    cfg = config_from_dict(d)
    assert isinstance(cfg, B.KesitarConfig) and cfg.to_dict() == d
    assert config_from_dict(dict(d, architectures=["Kesitar"], architecture=None)).to_dict() == d
    spec = spec_of(cfg)
    assert [l.mixer.kind for l in spec.layers] == ["pooled_window_attention", "hgrn2", "hgrn2", "pooled_window_attention"]
    assert [l.mixer.params.get("value_mix") for l in spec.layers] == ["source", None, None, "mix"]
    assert all(l.block == "sandwich_residual" for l in spec.layers)


@pytest.mark.parametrize("change", [
    lambda d: d["layers"][0].update(type="conv"),
    lambda d: d["layers"][0]["mixer"].update(kv_heads=4),
    lambda d: d["layers"][0]["mixer"]["mask"].update(size=0),
    lambda d: d["layers"][0]["mixer"]["rot"].update(dims=7),
    lambda d: d["layers"][0]["mixer"]["rot"].update(dims=64),
    lambda d: d["layers"][1]["mlp"].update(kind="experts"),
    lambda d: d["layers"][3]["mixer"].update(vdim=8),
    lambda d: d.pop("vocab"),
    lambda d: d["norm"].pop("eps"),
])
def test_config_refuses(change):
    d = small()
    change(d)
    with pytest.raises(ConfigError):
        config_from_dict(d)


def test_tensor_names_and_units():
    cfg = B.any_preset("kesitar-tiny")
    model = DecoderModel(spec_of(cfg))
    names = [s.name for s in model.weight_specs()]
    assert names[0] == "embed" and names[-1] == "final.norm"
    assert names[1:5] == ["l0.norm1", "l0.norm2", "l0.norm1b", "l0.norm2b"]
    assert [n for n in names if n.startswith("l0.mix.")] == ["l0.mix." + x for x in
                                                             ("q", "q.b", "k", "k.b", "v", "v.b", "q.norm", "k.norm", "vmix", "o")]
    assert [n for n in names if n.startswith("l1.mix.")] == ["l1.mix." + x for x in ("q", "f", "f.b", "lower", "v", "norm", "o")]
    needs = model.cache_needs()
    assert sorted(needs) == [0, 3, 4, 7] and needs[4].tokens_per_row == 4 and needs[0].live_from is needs[3].live_from
    assert sorted(model.state_needs()) == [("entry", 1), ("entry", 2)]


def test_which_token_rows_stay():
    f = window_and_open_block(10, 4)
    assert f is window_and_open_block(10, 4)
    for L in range(0, 200):
        first = f(L)
        assert first <= max(0, L - 9)                      # the next query's window
        assert first <= (L // 4) * 4                       # the open block has yet to be pooled
        assert first == max(0, min(L - 9, (L // 4) * 4))
    assert window_and_open_block(3, 0)(50) == 48


def test_cache_rows_per_block():
    tok = CacheNeed(kv_heads=1, head_dim=8, value_dim=4, live_from=window_and_open_block(70, 5))
    blk = CacheNeed(kv_heads=1, head_dim=8, value_dim=4, tokens_per_row=5)
    c = SequenceCache({0: tok, 1: blk}, {("entry", 2): StateNeed((2, 3))}, max_tokens=1024, dtype=None)
    g_tok, g_blk = c.unit_group(0), c.unit_group(1)
    s = c.alloc_slot()
    c.reserve([s], [319])
    c.commit([s], [319])
    assert len(g_blk.pages[s]) == 1 and sum(p >= 0 for p in g_tok.pages[s]) == 2      # 63 rows; tokens 250.. live
    c.reserve([s], [1])
    c.commit([s], [1])
    assert len(g_blk.pages[s]) == 1                        # 64 rows fill the page
    c.reserve([s], [5])
    c.commit([s], [5])
    assert len(g_blk.pages[s]) == 2
    held = [g.pool.held_count for g in c.groups]
    c.free_slot(s)
    assert [g.pool.held_count for g in c.groups] == [0, 0] and held[1] == 2
    with pytest.raises(CacheError):
        SequenceCache({0: CacheNeed(kv_heads=1, head_dim=8, window=4, tokens_per_row=2)}, {}, max_tokens=64, dtype=None)


def test_plain_attention_against_a_direct_sum():
    """The plain implementation's attention, written once more without blocks gathered beforehand."""
    rng = np.random.default_rng(0)
    T, size, pool = 40, 6, 4
    q, k, v = rng.standard_normal((T, 2, 5)), rng.standard_normal((T, 1, 5)), rng.standard_normal((T, 1, 3))
    got = P.pooled_window_attention(q, k, v, 0.5, size, pool)
    for i in (0, 5, 6, 9, 10, 13, 39):
        for h in range(2):
            num, den = np.zeros(3), 1.0
            for j in range(max(0, i - size + 1), i + 1):
                p = np.exp(0.5 * q[i, h] @ k[j, 0])
                num, den = num + p * v[j, 0], den + p
            b = 0
            while b * pool + pool - 1 <= i - size:
                p = np.exp(0.5 * q[i, h] @ k[b * pool:(b + 1) * pool, 0].mean(axis=0))
                num, den = num + p * v[b * pool:(b + 1) * pool, 0].mean(axis=0), den + p
                b += 1
            assert np.allclose(got[i, h], num / den)


def test_plain_recurrence_is_a_decayed_sum():
    rng = np.random.default_rng(1)
    T = 9
    q, f, v = rng.standard_normal((T, 1, 3)), rng.uniform(0.1, 0.9, (T, 1, 3)), rng.standard_normal((T, 1, 2))
    o, _ = P.gated_recurrence(q, f, v)
    t = T - 1
    want = np.zeros(2)
    for s in range(t + 1):
        decay = np.prod(f[s + 1:t + 1, 0], axis=0)
        want += ((decay * (1 - f[s, 0]) * q[t, 0])[:, None] * v[s, 0][None, :]).sum(axis=0)
    assert np.allclose(o[t, 0], want)
