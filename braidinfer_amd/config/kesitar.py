"""Typed configuration of the `Kesitar` design and its translation into parts.

A Kesitar model is a stack of layers, each with one mixer (`"attention"`: grouped-query
attention over a sliding window with pooled blocks, a sink in the softmax, query/key norms,
partial rotary positions and value mixing across layers; or `"hgrn2"`: a gated linear
recurrence) and an optional dense gated feed-forward, every half between two layer norms:
x += norm_b(half(norm_a(x))).  The embedding is scaled on the way in; the output head is the
embedding table itself with a scale of its own.  The reference has no such model; its
configuration is one flat struct (crates/braidinfer-runtime/src/config.rs:75-115), this one keeps
the nesting of the design's config.json:

    {"architecture": "Kesitar", "vocab": V, "width": W, "norm": {"eps": e},
     "embedding": {"scale": s}, "logit_scale": s,
     "layers": [{"type": "attention",
                 "mixer": {"heads", "kv_heads", "dim", "vdim", "scale", "v_mix",
                           "mask": {"size", "pool"}, "rot": {"dims", "base"}},
                 "mlp": {"kind": "dense", "ff": F} | null},
                {"type": "hgrn2", "mixer": {"heads", "dim", "vdim"}, "mlp": ...}, ...]}

Tensor names: `embed`, `final.norm`, and under `l<i>.`: `norm1`, `norm1b`, `norm2`, `norm2b`,
`mix.*`, `mlp.gate|up|down`.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Tuple

from ..errors import ConfigError
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

ARCHITECTURE = "Kesitar"
MIXERS = ("attention", "hgrn2")
# a sequence is as long as the cache lets it be: rotary angles are defined for every position
MAX_POSITIONS = 1 << 24


def _num(d, key, where, kind=(int, float), default=None, required=True):
    v = d.get(key) if isinstance(d, dict) else None
    if v is None:
        if required:
            raise ConfigError(f"config.json: {where} has no '{key}'")
        return default
    if isinstance(v, bool) or not isinstance(v, kind):
        raise ConfigError(f"config.json: {where}.{key} must be a number, found {v!r}")
    return v


def _pos_int(d, key, where, required=True, default=None):
    v = _num(d, key, where, kind=int, required=required, default=default)
    if v is not None and v <= 0:
        raise ConfigError(f"config.json: {where}.{key} must be positive, found {v}")
    return v


@dataclass(frozen=True)
class KesitarConfig:
    vocab: int
    width: int
    norm_eps: float
    embedding_scale: float
    logit_scale: float
    layers: Tuple[Dict[str, Any], ...]        # as in config.json, checked

    architecture = ARCHITECTURE

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "KesitarConfig":
        layers = d.get("layers")
        if not isinstance(layers, (list, tuple)) or not layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        cfg = cls(vocab=_pos_int(d, "vocab", "the model"), width=_pos_int(d, "width", "the model"),
                  norm_eps=float(_num(d.get("norm"), "eps", "norm")),
                  embedding_scale=float(_num(d.get("embedding"), "scale", "embedding", required=False, default=1.0)),
                  logit_scale=float(_num(d, "logit_scale", "the model", required=False, default=1.0)),
                  layers=tuple(copy.deepcopy(l) for l in layers))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.norm_eps < 0:
            raise ConfigError(f"config.json: norm.eps must not be negative, found {self.norm_eps}")
        mixed_width = None
        for i, l in enumerate(self.layers):
            where = f"layers[{i}]"
            if not isinstance(l, dict) or l.get("type") not in MIXERS:
                raise ConfigError(f"config.json: {where}.type must be one of {MIXERS}, found {l.get('type') if isinstance(l, dict) else l!r}")
            m = l.get("mixer")
            if not isinstance(m, dict):
                raise ConfigError(f"config.json: {where} has no 'mixer'")
            heads = _pos_int(m, "heads", where + ".mixer")
            _pos_int(m, "dim", where + ".mixer")
            vdim = _pos_int(m, "vdim", where + ".mixer")
            if l["type"] == "attention":
                kv = _pos_int(m, "kv_heads", where + ".mixer", required=False, default=heads)
                if heads % kv:
                    raise ConfigError(f"config.json: {where}.mixer: {heads} heads are not a multiple of {kv} kv heads")
                _num(m, "scale", where + ".mixer", required=False)
                mask = m.get("mask")
                _pos_int(mask, "size", where + ".mixer.mask")
                pool = _num(mask, "pool", where + ".mixer.mask", kind=int, required=False, default=0)
                if pool < 0:
                    raise ConfigError(f"config.json: {where}.mixer.mask.pool must not be negative, found {pool}")
                rot = m.get("rot")
                if rot is not None:
                    dims = _pos_int(rot, "dims", where + ".mixer.rot")
                    if dims % 2 or dims > m["dim"]:
                        raise ConfigError(f"config.json: {where}.mixer.rot.dims must be even and at most dim, found {dims}")
                    if float(_num(rot, "base", where + ".mixer.rot")) <= 0:
                        raise ConfigError(f"config.json: {where}.mixer.rot.base must be positive")
                if m.get("v_mix"):
                    if mixed_width not in (None, kv * vdim):
                        raise ConfigError(f"config.json: {where}.mixer mixes values of width {kv * vdim} with the first "
                                          f"such layer's of width {mixed_width}")
                    mixed_width = kv * vdim
            mlp = l.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"config.json: {where}.mlp.kind must be 'dense', found {mlp!r}")
                _pos_int(mlp, "ff", where + ".mlp")

    def to_dict(self) -> Dict[str, Any]:
        return {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
                "embedding": {"scale": self.embedding_scale}, "logit_scale": self.logit_scale,
                "layers": [copy.deepcopy(l) for l in self.layers]}


def _rope_name(dims: int, base: float) -> str:
    return f"rope{dims}@{base!r}"


def build_spec(cfg: KesitarConfig) -> ModelSpec:
    """Kesitar as parts: `sandwich_residual` layers of `layernorm` norms around a
    `pooled_window_attention` or `hgrn2` mixer and a `swiglu` feed-forward."""
    W = cfg.width

    def norm(tensor=""):
        return PartSpec("layernorm", {"size": W, "eps": cfg.norm_eps, "tensor": tensor})

    layers: List[LayerSpec] = []
    schedule: List[ScheduleEntry] = []
    positions: Dict[str, PartSpec] = {}
    n = len(cfg.layers)
    mix_source_seen = False
    for i, l in enumerate(cfg.layers):
        m = l["mixer"]
        more_caches: Dict[str, int] = {}
        if l["type"] == "attention":
            rot = m.get("rot")
            position = None
            if rot is not None:
                position = _rope_name(rot["dims"], float(rot["base"]))
                positions[position] = PartSpec("rope", {"rotary_dim": rot["dims"], "theta": float(rot["base"]), "pairing": "half"})
            value_mix = None
            if m.get("v_mix"):
                value_mix = "mix" if mix_source_seen else "source"
                mix_source_seen = True
            pool = int(m["mask"].get("pool") or 0)
            mixer = PartSpec("pooled_window_attention", {
                "hidden_size": W, "num_heads": m["heads"], "num_kv_heads": m.get("kv_heads", m["heads"]),
                "key_dim": m["dim"], "value_dim": m["vdim"], "window": m["mask"]["size"], "pool": pool,
                "scale": m.get("scale"), "sink": True, "bias": True, "qk_norm_eps": cfg.norm_eps,
                "position": position, "value_mix": value_mix,
                "names": {"q": "q", "k": "k", "v": "v", "o": "o", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b",
                          "q_norm": "q.norm", "k_norm": "k.norm", "value_mix": "vmix"}})
            if pool:
                more_caches["pooled"] = n + i          # units 0..n-1 are the layers' own, n..2n-1 their pooled rows
        else:
            mixer = PartSpec("hgrn2", {
                "hidden_size": W, "num_heads": m["heads"], "key_dim": m["dim"], "value_dim": m["vdim"],
                "norm_eps": cfg.norm_eps,
                "names": {"q": "q", "f": "f", "f_bias": "f.b", "v": "v", "lower": "lower", "norm": "norm", "o": "o"}})
        norms = {"mixer": norm(), "mixer_out": norm()}
        names = {"norm.mixer": "norm1"}
        ffn = None
        if l.get("mlp") is not None:
            ffn = PartSpec("swiglu", {"hidden_size": W, "intermediate_size": l["mlp"]["ff"],
                                      "names": {"gate": "gate", "up": "up", "down": "down"}})
            norms.update({"feed_forward": norm(), "feed_forward_out": norm()})
            names["norm.feed_forward"] = "norm2"
        # the order of the model's name table: norm1, norm2, norm1b, norm2b, mix.*, mlp.*
        names["norm.mixer_out"] = "norm1b"
        if ffn is not None:
            names["norm.feed_forward_out"] = "norm2b"
        names["mixer"] = "mix."
        if ffn is not None:
            names["feed_forward"] = "mlp."
        layers.append(LayerSpec(prefix=f"l{i}.", mixer=mixer, feed_forward=ffn, norms=norms, block="sandwich_residual",
                                names=names))
        schedule.append(ScheduleEntry(layer=i, cache=i, more_caches=more_caches))
    return ModelSpec(
        architecture=ARCHITECTURE, hidden_size=W, vocab_size=cfg.vocab,
        embedding=PartSpec("embedding", {"vocab_size": cfg.vocab, "hidden_size": W, "scale": cfg.embedding_scale, "tensor": ""}),
        layers=layers, schedule=schedule, final_norm=norm(),
        lm_head=PartSpec("lm_head", {"vocab_size": cfg.vocab, "hidden_size": W, "tied_to": "embed", "scale": cfg.logit_scale}),
        positions=positions, max_position_embeddings=MAX_POSITIONS,
        embedding_prefix="embed", final_norm_prefix="final.norm", lm_head_prefix="head.",
        stop_token_ids=[], bos_token_id=None)


def _attention(heads, kv_heads, dim, vdim, size, pool, rot_dims, base=10000.0, v_mix=True):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                                           "scale": dim ** -0.5, "v_mix": v_mix, "mask": {"size": size, "pool": pool},
                                           "rot": {"dims": rot_dims, "base": base}}}


def _hgrn2(heads, dim, vdim):
    return {"type": "hgrn2", "mixer": {"heads": heads, "dim": dim, "vdim": vdim}}


def _stack(pattern: str, attention, recurrent, ff: int) -> List[Dict[str, Any]]:
    out = []
    for ch in pattern:
        l = copy.deepcopy(attention if ch == "a" else recurrent)
        l["mlp"] = {"kind": "dense", "ff": ff}
        out.append(l)
    return out


# Shapes without a model folder: two tiny ones for tests and tools, and two of the size of a real
# model's layers (one attention layer in four, as in the hybrid stacks this design resembles).
PRESETS: Dict[str, Dict[str, Any]] = {
    "kesitar-tiny": dict(vocab=384, width=96, norm={"eps": 1e-5}, embedding={"scale": 0.7}, logit_scale=1.5,
                         layers=_stack("arra", _attention(6, 3, 32, 16, 9, 4, 16), _hgrn2(3, 16, 32), 160)),
    "kesitar-1b": dict(vocab=32768, width=2048, norm={"eps": 1e-6}, embedding={"scale": 1.0}, logit_scale=1.0,
                       layers=_stack("arrr" * 4, _attention(16, 4, 128, 128, 1024, 16, 64), _hgrn2(16, 128, 128), 5632)),
    "kesitar-7b": dict(vocab=32768, width=4096, norm={"eps": 1e-6}, embedding={"scale": 1.0}, logit_scale=1.0,
                       layers=_stack("arrr" * 8, _attention(32, 8, 128, 128, 2048, 32, 64), _hgrn2(32, 128, 128), 14336)),
}


def preset(name: str, **overrides) -> KesitarConfig:
    if name not in PRESETS:
        raise ConfigError(f"unknown preset {name!r}; known: {sorted(PRESETS)}")
    d = dict(copy.deepcopy(PRESETS[name]), architecture=ARCHITECTURE)
    d.update(overrides)
    return KesitarConfig.from_dict(d)
