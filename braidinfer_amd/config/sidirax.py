"""Typed configuration of the `Sidirax` design and its translation into parts.

A Sidirax model is a stack of parallel layers, x += mixer(n) + feed_forward(n) with one RMS norm n = norm(x) a
layer.  The mixer is `"latent_attention"` (queries and keys/values through narrow normed latents, a rotated key
part shared by the heads, interleaved rotary pairs with scaled frequencies, a learnt sink score per head; a layer
may read the rows another layer keeps, `kv_from`) or `"wkv"` (a linear recurrence with token-dependent decay and
inputs mixed with the token before).  The feed-forward is a dense clamped gated unit with biases, a set of routed
experts, or absent.  The output head is the embedding table.  The reference has no such model; its configuration
is one flat struct (crates/braidinfer-runtime/src/config.rs:75-115), this one keeps the nesting of the design's
config.json:

    {"architecture": "Sidirax", "vocab": V, "width": W, "norm": {"eps": e},
     "layers": [{"type": "latent_attention",
                 "mixer": {"heads", "dim", "rot_dim", "vdim", "q_rank", "kv_rank", "scale", "kv_from"?,
                           "rot": {"dims", "base", "scaling": {"factor", "original", "fast", "slow"}?}},
                 "mlp": {"kind": "dense", "ff": F, "limit": L}
                      | {"kind": "moe", "expert": {"ff": F}, "router": {"experts": E, "top": k}} | null},
                {"type": "wkv", "mixer": {"heads", "dim", "decay_rank"?}, "mlp": ...}, ...]}

`decay_rank` (the inner width of a wkv layer's decay projection) may be left out of config.json: it is then read
from the shape of the layer's `mix.w1` tensor when the configuration comes from a model folder.

Tensor names: `embed`, `final.norm`, and under `l<i>.`: `norm1`, `mix.*`, `mlp.*` (`mlp.e<j>.gate|up|down`,
`mlp.router`, `mlp.router.b` for routed experts).
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, replace
from typing import Any, Callable, Dict, List, Optional, Tuple

from ..errors import ConfigError
from .kesitar import MAX_POSITIONS, _num, _pos_int
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

ARCHITECTURE = "Sidirax"
MIXERS = ("latent_attention", "wkv")
GLU_ALPHA = 1.702          # the design's constant in g * sigmoid(alpha g)


@dataclass(frozen=True)
class SidiraxConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: Tuple[Dict[str, Any], ...]        # as in config.json, checked

    architecture = ARCHITECTURE

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "SidiraxConfig":
        layers = d.get("layers")
        if not isinstance(layers, (list, tuple)) or not layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        cfg = cls(vocab=_pos_int(d, "vocab", "the model"), width=_pos_int(d, "width", "the model"),
                  norm_eps=float(_num(d.get("norm"), "eps", "norm")), layers=tuple(copy.deepcopy(l) for l in layers))
        cfg.validate()
        return cfg

    # ---- sizes that only the tensors give -------------------------------------------------
    def missing_tensor_sizes(self) -> List[str]:
        """Names of the tensors whose shapes complete this configuration (`with_tensor_shapes`)."""
        return [f"l{i}.mix.w1" for i, l in enumerate(self.layers) if l["type"] == "wkv" and l["mixer"].get("decay_rank") is None]

    def with_tensor_shapes(self, shape_of: Callable[[str], Optional[Tuple[int, ...]]]) -> "SidiraxConfig":
        """The configuration with every size config.json left to the tensors filled in; `shape_of(name)` is a
        tensor's shape or None."""
        layers = [copy.deepcopy(l) for l in self.layers]
        for name in self.missing_tensor_sizes():
            i = int(name[1:name.index(".")])
            shape = shape_of(name)
            if shape is None or len(shape) != 2 or shape[1] != self.width or shape[0] <= 0:
                raise ConfigError(f"config.json: layers[{i}].mixer has no 'decay_rank' and the tensor {name} "
                                  f"({'absent' if shape is None else tuple(shape)}) does not give one")
            layers[i]["mixer"]["decay_rank"] = int(shape[0])
        return replace(self, layers=tuple(layers))

    def validate(self) -> None:
        if self.norm_eps < 0:
            raise ConfigError(f"config.json: norm.eps must not be negative, found {self.norm_eps}")
        for i, l in enumerate(self.layers):
            where = f"layers[{i}]"
            if not isinstance(l, dict) or l.get("type") not in MIXERS:
                raise ConfigError(f"config.json: {where}.type must be one of {MIXERS}, found {l.get('type') if isinstance(l, dict) else l!r}")
            m = l.get("mixer")
            if not isinstance(m, dict):
                raise ConfigError(f"config.json: {where} has no 'mixer'")
            _pos_int(m, "heads", where + ".mixer")
            _pos_int(m, "dim", where + ".mixer")
            if l["type"] == "wkv":
                _pos_int(m, "decay_rank", where + ".mixer", required=False)
            else:
                for key in ("vdim", "q_rank", "kv_rank"):
                    _pos_int(m, key, where + ".mixer")
                rot_dim = _num(m, "rot_dim", where + ".mixer", kind=int)
                if rot_dim < 0:
                    raise ConfigError(f"config.json: {where}.mixer.rot_dim must not be negative, found {rot_dim}")
                _num(m, "scale", where + ".mixer")
                rot = m.get("rot")
                if rot_dim and not isinstance(rot, dict):
                    raise ConfigError(f"config.json: {where}.mixer has a rotated part and no 'rot'")
                if isinstance(rot, dict):
                    dims = _pos_int(rot, "dims", where + ".mixer.rot")
                    if dims % 2 or dims > rot_dim:
                        raise ConfigError(f"config.json: {where}.mixer.rot.dims must be even and at most rot_dim, found {dims}")
                    if float(_num(rot, "base", where + ".mixer.rot")) <= 1.0:
                        raise ConfigError(f"config.json: {where}.mixer.rot.base must be above 1")
                    sc = rot.get("scaling")
                    if sc is not None:
                        for key in ("factor", "original", "fast", "slow"):
                            if float(_num(sc, key, where + ".mixer.rot.scaling")) <= 0:
                                raise ConfigError(f"config.json: {where}.mixer.rot.scaling.{key} must be positive")
                src = m.get("kv_from")
                if src is not None:
                    if isinstance(src, bool) or not isinstance(src, int) or not 0 <= src < i:
                        raise ConfigError(f"config.json: {where}.mixer.kv_from must name an earlier layer, found {src!r}")
                    other = self.layers[src]
                    om = other.get("mixer", {}) if isinstance(other, dict) else {}
                    if other.get("type") != "latent_attention" or om.get("kv_from") is not None:
                        raise ConfigError(f"config.json: {where}.mixer.kv_from names layer {src}, which keeps no rows of its own")
                    if any(om.get(k) != m.get(k) for k in ("kv_rank", "rot_dim", "rot")):
                        raise ConfigError(f"config.json: {where}.mixer reads the rows of layer {src}, whose kv_rank, rot_dim "
                                          "or rot differ")
            mlp = l.get("mlp")
            if mlp is None:
                continue
            if not isinstance(mlp, dict) or mlp.get("kind") not in ("dense", "moe"):
                raise ConfigError(f"config.json: {where}.mlp.kind must be 'dense' or 'moe', found {mlp!r}")
            if mlp["kind"] == "dense":
                _pos_int(mlp, "ff", where + ".mlp")
                if float(_num(mlp, "limit", where + ".mlp")) <= 0:
                    raise ConfigError(f"config.json: {where}.mlp.limit must be positive")
            else:
                _pos_int(mlp.get("expert"), "ff", where + ".mlp.expert")
                n = _pos_int(mlp.get("router"), "experts", where + ".mlp.router")
                top = _pos_int(mlp.get("router"), "top", where + ".mlp.router")
                if top > n:
                    raise ConfigError(f"config.json: {where}.mlp.router chooses {top} of {n} experts")

    def to_dict(self) -> Dict[str, Any]:
        return {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
                "layers": [copy.deepcopy(l) for l in self.layers]}


def _rope_name(rot: Dict[str, Any]) -> str:
    sc = rot.get("scaling")
    tail = "" if sc is None else "/" + ",".join(repr(float(sc[k])) for k in ("factor", "original", "fast", "slow"))
    return f"rope{rot['dims']}@{float(rot['base'])!r}{tail}"


def build_spec(cfg: SidiraxConfig) -> ModelSpec:
    """Sidirax as parts: `parallel_residual` layers of one `rmsnorm`, a `latent_attention` or `wkv` mixer and a
    `clamped_glu` or `routed_experts` feed-forward; one rotary encoding per (dims, base, scaling); layer i's rows in
    cache unit i, which a layer with `kv_from` reads instead of writing one of its own."""
    W = cfg.width
    missing = cfg.missing_tensor_sizes()
    if missing:
        raise ConfigError(f"the configuration leaves sizes to the tensors {missing}; read it from a model folder or give "
                          "'decay_rank'")

    def norm():
        return PartSpec("rmsnorm", {"size": W, "eps": cfg.norm_eps, "tensor": ""})

    layers: List[LayerSpec] = []
    schedule: List[ScheduleEntry] = []
    positions: Dict[str, PartSpec] = {}
    for i, l in enumerate(cfg.layers):
        m = l["mixer"]
        unit, writes = i, True
        if l["type"] == "latent_attention":
            rot, position = m.get("rot"), None
            if rot is not None and m["rot_dim"]:
                position = _rope_name(rot)
                params = {"rotary_dim": rot["dims"], "theta": float(rot["base"]), "pairing": "adjacent"}
                if rot.get("scaling") is not None:
                    params["scaling"] = {k: float(rot["scaling"][k]) for k in ("factor", "original", "fast", "slow")}
                positions[position] = PartSpec("rope", params)
            src = m.get("kv_from")
            if src is not None:
                unit, writes = src, False
            mixer = PartSpec("latent_attention", {
                "hidden_size": W, "num_heads": m["heads"], "head_dim": m["dim"], "rot_dim": m["rot_dim"], "value_dim": m["vdim"],
                "q_rank": m["q_rank"], "kv_rank": m["kv_rank"], "scale": float(m["scale"]), "norm_eps": cfg.norm_eps,
                "position": position, "sink": True, "own_rows": src is None})
        else:
            mixer = PartSpec("wkv", {"hidden_size": W, "num_heads": m["heads"], "head_dim": m["dim"],
                                     "decay_rank": m["decay_rank"], "norm_eps": cfg.norm_eps})
        mlp, ffn = l.get("mlp"), None
        if mlp is not None and mlp["kind"] == "dense":
            ffn = PartSpec("clamped_glu", {"hidden_size": W, "intermediate_size": mlp["ff"], "limit": float(mlp["limit"]),
                                           "alpha": GLU_ALPHA})
        elif mlp is not None:
            ffn = PartSpec("routed_experts", {"hidden_size": W, "intermediate_size": mlp["expert"]["ff"],
                                              "num_experts": mlp["router"]["experts"], "top": mlp["router"]["top"]})
        names = {"norm.mixer": "norm1", "mixer": "mix."}
        if ffn is not None:
            names["feed_forward"] = "mlp."
        layers.append(LayerSpec(prefix=f"l{i}.", mixer=mixer, feed_forward=ffn, norms={"mixer": norm()},
                                block="parallel_residual", names=names))
        schedule.append(ScheduleEntry(layer=i, cache=unit, writes_cache=writes))
    return ModelSpec(
        architecture=ARCHITECTURE, hidden_size=W, vocab_size=cfg.vocab,
        embedding=PartSpec("embedding", {"vocab_size": cfg.vocab, "hidden_size": W, "scale": 1.0, "tensor": ""}),
        layers=layers, schedule=schedule, final_norm=norm(),
        lm_head=PartSpec("lm_head", {"vocab_size": cfg.vocab, "hidden_size": W, "tied_to": "embed", "scale": 1.0}),
        positions=positions, max_position_embeddings=MAX_POSITIONS,
        embedding_prefix="embed", final_norm_prefix="final.norm", lm_head_prefix="head.",
        stop_token_ids=[], bos_token_id=None)


def _latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, base=10000.0, scaling=None, kv_from=None):
    rot = {"dims": rot_dim, "base": base}
    if scaling is not None:
        rot["scaling"] = dict(scaling)
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
         "scale": (dim + rot_dim) ** -0.5, "rot": rot}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m}


def _wkv(heads, dim, decay_rank):
    return {"type": "wkv", "mixer": {"heads": heads, "dim": dim, "decay_rank": decay_rank}}


def _dense(ff, limit=7.0):
    return {"kind": "dense", "ff": ff, "limit": limit}


def _moe(ff, experts, top):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def _with(layer, mlp):
    return dict(copy.deepcopy(layer), mlp=mlp)


_YARN = {"factor": 8.0, "original": 4096, "fast": 32.0, "slow": 1.0}
# Shapes without a model folder: a tiny one for tests and tools, and two of the size of a real model's layers
# (attention layers between recurrent ones, the second attention layer reading the first one's rows; a dense
# feed-forward first, routed experts after it, of which a token's share equals the dense layer's inner width).
PRESETS: Dict[str, Dict[str, Any]] = {
    "sidirax-tiny": dict(vocab=320, width=96, norm={"eps": 1e-5}, layers=[
        _with(_latent(3, 24, 8, 16, 40, 24, scaling={"factor": 4.0, "original": 64, "fast": 16.0, "slow": 1.0}), _dense(136, 3.0)),
        _with(_wkv(2, 24, 8), _moe(48, 6, 2)),
        _with(_latent(3, 24, 8, 16, 40, 24, scaling={"factor": 4.0, "original": 64, "fast": 16.0, "slow": 1.0}, kv_from=0), _moe(48, 6, 2)),
        _with(_wkv(2, 24, 8), None)]),
    "sidirax-1b": dict(vocab=32768, width=2048, norm={"eps": 1e-6}, layers=[
        _with(_latent(16, 64, 32, 64, 768, 160, scaling=_YARN), _dense(5632)),
        _with(_wkv(32, 64, 64), _moe(1408, 16, 4)),
        _with(_wkv(32, 64, 64), _moe(1408, 16, 4)),
        _with(_wkv(32, 64, 64), _moe(1408, 16, 4)),
        _with(_latent(16, 64, 32, 64, 768, 160, scaling=_YARN, kv_from=0), _moe(1408, 16, 4)),
        _with(_wkv(32, 64, 64), _moe(1408, 16, 4)),
        _with(_wkv(32, 64, 64), _moe(1408, 16, 4)),
        _with(_wkv(32, 64, 64), _moe(1408, 16, 4))]),
    "sidirax-7b": dict(vocab=32768, width=4096, norm={"eps": 1e-6}, layers=[
        _with(_latent(32, 64, 32, 64, 1536, 224, scaling=_YARN), _dense(14336)),
        _with(_wkv(64, 64, 64), _moe(1792, 32, 8)),
        _with(_wkv(64, 64, 64), _moe(1792, 32, 8)),
        _with(_wkv(64, 64, 64), _moe(1792, 32, 8)),
        _with(_latent(32, 64, 32, 64, 1536, 224, scaling=_YARN, kv_from=0), _moe(1792, 32, 8)),
        _with(_wkv(64, 64, 64), _moe(1792, 32, 8)),
        _with(_wkv(64, 64, 64), _moe(1792, 32, 8)),
        _with(_wkv(64, 64, 64), _moe(1792, 32, 8))]),
}


def preset(name: str, **overrides) -> SidiraxConfig:
    if name not in PRESETS:
        raise ConfigError(f"unknown preset {name!r}; known: {sorted(PRESETS)}")
    d = dict(copy.deepcopy(PRESETS[name]), architecture=ARCHITECTURE)
    d.update(overrides)
    return SidiraxConfig.from_dict(d)
