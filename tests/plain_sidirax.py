"""A plain, slow implementation of the Sidirax design in NumPy float64, one function per
mechanism, written from the design's equations.  It shares no code with the library: the
tests hold the engine against it.

Notation: a sequence's tokens are rows; positions count from 0.  `cfg` is the model's
configuration as a dict (the keys of its config.json), `w` maps tensor names to float arrays.
"""
from __future__ import annotations

import json
import math
import os
import struct

import numpy as np


# ------------------------------------------------------------------ mechanisms ------
def rms_norm(x, weight, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis, times `weight` (None: no weight)."""
    ms = (x * x).mean(axis=-1, keepdims=True)
    y = x / np.sqrt(ms + eps)
    return y if weight is None else y * weight


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def scaled_frequencies(dims, base, scaling):
    """(frequency of each of the dims / 2 pairs, the factor on cos and sin).  Without `scaling`:
    base^(-2i / dims) and 1.  With {factor, original, fast, slow}: pairs that turn more than `fast` times
    over `original` positions keep their frequency, pairs that turn fewer than `slow` times have it divided
    by `factor`, a linear ramp over the pair index between the two; cos and sin grow by 0.1 ln(factor) + 1."""
    i = np.arange(dims // 2, dtype=np.float64)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def pair_of(turns):          # the (real-valued) pair index whose wavelength makes `turns` turns over `original`
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(pair_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(pair_of(float(scaling["slow"]))), dims - 1)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_pairs(x, positions, freqs, magnitude=1.0):
    """Rotary positions on the first 2 len(freqs) elements of the last axis of x [T, ..., d]: elements 2i and
    2i + 1 are a pair turned by the angle position * freqs[i]; cos and sin times `magnitude`."""
    out = np.array(x, dtype=np.float64, copy=True)
    n = 2 * len(freqs)
    ang = np.asarray(positions, dtype=np.float64)[:, None] * freqs[None, :]
    shape = (x.shape[0],) + (1,) * (x.ndim - 2) + (len(freqs),)
    c, s = (np.cos(ang) * magnitude).reshape(shape), (np.sin(ang) * magnitude).reshape(shape)
    u, v = x[..., 0:n:2], x[..., 1:n:2]
    out[..., 0:n:2] = u * c - v * s
    out[..., 1:n:2] = v * c + u * s
    return out


def sink_softmax_attention(q, k, v, scale, sink):
    """Causal attention of one sequence from position 0: q [T, H, d], k [T, H, d], v [T, H, e]; the softmax's
    denominator also holds exp(sink[h]) (None: no sink), which has no value.  Returns [T, H, e]."""
    T, H, _ = q.shape
    out = np.zeros((T, H, v.shape[2]))
    for i in range(T):
        for h in range(H):
            s = k[:i + 1, h] @ q[i, h] * scale
            m = s.max() if sink is None else max(s.max(), sink[h])
            p = np.exp(s - m)
            den = p.sum() + (0.0 if sink is None else math.exp(sink[h] - m))
            out[i, h] = (p / den) @ v[:i + 1, h]
    return out


def latent_rows(h, w, p, m, eps, positions):
    """What a latent-attention layer keeps per token: the normed latent [T, kv_rank] and the shared rotated key
    part [T, rot_dim] (after rotation)."""
    r = m["kv_rank"]
    dkv = h @ w[p + "dkv"].T
    c = rms_norm(dkv[:, :r], w[p + "dkv.norm"], eps)
    freqs, mag = scaled_frequencies(m["rot"]["dims"], float(m["rot"]["base"]), m["rot"].get("scaling"))
    return c, rotate_pairs(dkv[:, r:], positions, freqs, mag)


def latent_attention_mixer(h, w, p, m, eps, kept=None):
    """Latent attention over one sequence from position 0.  `kept`: (latent, rotated key part) of the layer whose
    rows this one reads, None when it makes its own.  Returns (output [T, width], the rows it used)."""
    T = h.shape[0]
    H, d, dr, e = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    positions = np.arange(T)
    if kept is None:
        kept = latent_rows(h, w, p, m, eps, positions)
    c, k_rot = kept
    cq = rms_norm(h @ w[p + "dq"].T, w[p + "dq.norm"], eps)
    q = (cq @ w[p + "uq"].T).reshape(T, H, d + dr)
    freqs, mag = scaled_frequencies(m["rot"]["dims"], float(m["rot"]["base"]), m["rot"].get("scaling"))
    q = np.concatenate([q[..., :d], rotate_pairs(q[..., d:], positions, freqs, mag)], axis=-1)
    k = np.concatenate([(c @ w[p + "uk"].T).reshape(T, H, d), np.repeat(k_rot[:, None, :], H, axis=1)], axis=-1)
    v = (c @ w[p + "uv"].T).reshape(T, H, e)
    o = sink_softmax_attention(q, k, v, float(m["scale"]), w.get(p + "sink"))
    return o.reshape(T, H * e) @ w[p + "o"].T, kept


def shifted_mix(h, mu, first=None):
    """h + (h' - h) * mu with h' the row before (zeros, or `first`, before the first row)."""
    prev = np.concatenate([np.zeros((1, h.shape[1])) if first is None else first[None, :], h[:-1]], axis=0)
    return h + (prev - h) * mu


def decayed_outer_recurrence(r, k, v, decay, bonus, state=None):
    """Per head: o_t = (S_(t-1) + diag(bonus) k_t v_t^T)^T r_t, then S_t = diag(decay_t) S_(t-1) + k_t v_t^T.
    r, k, decay [T, H, d], v [T, H, e], bonus [H, d]; S [H, d, e] starts at zero (or `state`).  Returns (o, S)."""
    T, H, d = r.shape
    e = v.shape[2]
    S = np.zeros((H, d, e)) if state is None else np.array(state, dtype=np.float64)
    o = np.zeros((T, H, e))
    for t in range(T):
        kv = k[t][:, :, None] * v[t][:, None, :]
        o[t] = np.einsum("hd,hde->he", r[t], S + bonus[:, :, None] * kv)
        S = decay[t][:, :, None] * S + kv
    return o, S


def wkv_mixer(h, w, p, m, eps):
    """The time-mixing layer over one sequence from position 0; returns [T, width]."""
    T = h.shape[0]
    H, d = m["heads"], m["dim"]
    mix = {s: shifted_mix(h, w[p + "mu." + s]) for s in "rkvgw"}
    r = (mix["r"] @ w[p + "r"].T).reshape(T, H, d)
    k = (mix["k"] @ w[p + "k"].T).reshape(T, H, d)
    v = (mix["v"] @ w[p + "v"].T).reshape(T, H, d)
    gate = silu(mix["g"] @ w[p + "g"].T)
    decay = np.exp(-np.exp(np.tanh(mix["w"] @ w[p + "w1"].T) @ w[p + "w2"].T + w[p + "w0"])).reshape(T, H, d)
    o, _ = decayed_outer_recurrence(r, k, v, decay, w[p + "u"].reshape(H, d))
    o = rms_norm(o, None, eps).reshape(T, H * d) * w[p + "norm"] * gate
    return o @ w[p + "o"].T


def clamped_glu_ff(h, w, p, limit):
    """W_d (g sigmoid(1.702 g) (u + 1)) with g = min(W_g h + b, limit), u = clamp(W_u h + b, -limit, limit)."""
    g = np.minimum(h @ w[p + "gate"].T + w[p + "gate.b"], limit)
    u = np.clip(h @ w[p + "up"].T + w[p + "up.b"], -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].T + w[p + "down.b"]


def routed_ff(h, w, p, experts, top, margins=None):
    """Every token through its `top` experts with the largest router logits, weighted by the softmax over those
    logits only; an expert is W_d (silu(W_g h) * (W_u h)).  `margins` (a list) receives per token the distance
    between the last chosen logit and the first one left out (how close the choice was)."""
    z = h @ w[p + "router"].T + w[p + "router.b"]
    out = np.zeros_like(h)
    if margins is not None:
        srt = -np.sort(-z, axis=1)
        margins.append(srt[:, top - 1] - srt[:, top] if top < experts else np.full(h.shape[0], np.inf))
    for t in range(h.shape[0]):
        chosen = np.argsort(-z[t], kind="stable")[:top]
        a = np.exp(z[t, chosen] - z[t, chosen].max())
        a /= a.sum()
        for e, share in zip(chosen, a):
            q = f"{p}e{e}."
            out[t] += share * ((silu(h[t] @ w[q + "gate"].T) * (h[t] @ w[q + "up"].T)) @ w[q + "down"].T)
    return out


def feed_forward(h, w, p, mlp, margins=None):
    if mlp is None:
        return np.zeros_like(h)
    if mlp["kind"] == "dense":
        return clamped_glu_ff(h, w, p, float(mlp["limit"]))
    return routed_ff(h, w, p, mlp["router"]["experts"], mlp["router"]["top"], margins)


# ------------------------------------------------------------------ the model -------
def forward(cfg, w, tokens, return_layers=False, margins=None):
    """Logits [T, vocab] of one sequence from position 0 (and the residual rows after every layer).  `margins` (a
    list) receives one array per layer of routed experts, see `routed_ff`."""
    eps = float(cfg["norm"]["eps"])
    x = w["embed"][np.asarray(tokens)]
    kept, layers = {}, []
    for i, l in enumerate(cfg["layers"]):
        p, m = f"l{i}.", l["mixer"]
        h = rms_norm(x, w[p + "norm1"], eps)
        if l["type"] == "wkv":
            mixed = wkv_mixer(h, w, p + "mix.", m, eps)
        else:
            src = m.get("kv_from")
            mixed, rows = latent_attention_mixer(h, w, p + "mix.", m, eps, None if src is None else kept[src])
            if src is None:
                kept[i] = rows
        x = x + (mixed + feed_forward(h, w, p + "mlp.", l.get("mlp"), margins))
        layers.append(x.copy())
    logits = rms_norm(x, w["final.norm"], eps) @ w["embed"].T
    return (logits, np.stack(layers)) if return_layers else logits


def greedy_generate(cfg, w, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(np.argmax(forward(cfg, w, toks)[-1])))
    return toks[len(prompt):]


# ------------------------------------------------------------------ files -----------
def read_folder(folder):
    """(config dict, float64 tensors by name) of a model folder; bfloat16 and float32 tensors."""
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    w = {}
    with open(os.path.join(folder, "model.safetensors"), "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        head = json.loads(f.read(n))
        data = f.read()
    for name, t in head.items():
        if name == "__metadata__":
            continue
        a, b = t["data_offsets"]
        raw = data[a:b]
        if t["dtype"] == "BF16":
            arr = (np.frombuffer(raw, dtype="<u2").astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        elif t["dtype"] == "F32":
            arr = np.frombuffer(raw, dtype="<f4").astype(np.float64)
        elif t["dtype"] == "I32":
            arr = np.frombuffer(raw, dtype="<i4")
        else:
            raise ValueError(f"{name}: dtype {t['dtype']}")
        w[name] = arr.reshape(t["shape"])
    return cfg, w


def to_bf16(a):
    """Round float values to the nearest bfloat16 (ties to even), returned as float64."""
    u = np.ascontiguousarray(np.asarray(a, dtype=np.float32)).view(np.uint32)
    r = ((u + (((u >> 16) & 1) + 0x7FFF)) >> 16).astype(np.uint32) << 16
    return r.view(np.float32).astype(np.float64)


def write_folder(folder, cfg, w):
    """config.json and model.safetensors (bfloat16) of a configuration dict and float tensors."""
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    head, blobs, off = {}, [], 0
    for name, a in w.items():
        a32 = np.asarray(a, dtype=np.float32)
        u = np.ascontiguousarray(a32).reshape(-1).view(np.uint32)
        raw = ((u + (((u >> 16) & 1) + 0x7FFF)) >> 16).astype("<u2").tobytes()
        head[name] = {"dtype": "BF16", "shape": list(a32.shape), "data_offsets": [off, off + len(raw)]}
        off += len(raw)
        blobs.append(raw)
    hj = json.dumps(head).encode()
    hj += b" " * (-len(hj) % 8)
    with open(os.path.join(folder, "model.safetensors"), "wb") as f:
        f.write(struct.pack("<Q", len(hj)) + hj + b"".join(blobs))


def random_weights(cfg, seed, gain=1.0):
    """Random tensors (bfloat16 values) for a configuration dict: matrices N(0, gain^2 / fan-in), norm weights
    around 1, mixing shares in (0, 1), biases and sinks of the size of a logit."""
    rng = np.random.default_rng(seed)
    W, w = cfg["width"], {}

    def mat(o, i, g=gain):
        return to_bf16(rng.standard_normal((o, i)) * g / math.sqrt(i))

    def vec(n, around=1.0, spread=0.3):
        return to_bf16(around + spread * rng.standard_normal(n))
    w["embed"] = to_bf16(rng.standard_normal((cfg["vocab"], W)))
    for i, l in enumerate(cfg["layers"]):
        p, m = f"l{i}.", l["mixer"]
        w[p + "norm1"] = vec(W)
        H, d = m["heads"], m["dim"]
        q = p + "mix."
        if l["type"] == "latent_attention":
            dr, e, r, qr = m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            w[q + "dq"], w[q + "dq.norm"], w[q + "uq"] = mat(qr, W), vec(qr), mat(H * (d + dr), qr)
            if m.get("kv_from") is None:
                w[q + "dkv"], w[q + "dkv.norm"] = mat(r + dr, W), vec(r)
            w[q + "uk"], w[q + "uv"] = mat(H * d, r), mat(H * e, r)
            w[q + "sink"] = vec(H, 0.5, 1.0)
            w[q + "o"] = mat(W, H * e)
        else:
            for s in "rkvgw":
                w[q + "mu." + s] = to_bf16(rng.uniform(0.0, 1.0, W))
            for s in "rkvg":
                w[q + s] = mat(H * d, W)
            rank = m.get("decay_rank", 8)
            w[q + "w1"], w[q + "w2"] = mat(rank, W), mat(H * d, rank)
            w[q + "w0"] = to_bf16(rng.uniform(-3.0, 0.5, H * d))
            w[q + "u"] = to_bf16(rng.standard_normal((H, d)) * 0.5)
            w[q + "norm"], w[q + "o"] = vec(H * d), mat(W, H * d)
        mlp = l.get("mlp")
        q = p + "mlp."
        if mlp is None:
            continue
        if mlp["kind"] == "dense":
            F = mlp["ff"]
            w[q + "gate"], w[q + "gate.b"] = mat(F, W, 2.0 * gain), vec(F, 0.0)
            w[q + "up"], w[q + "up.b"] = mat(F, W, 2.0 * gain), vec(F, 0.0)
            w[q + "down"], w[q + "down.b"] = mat(W, F), vec(W, 0.0)
        else:
            F, E = mlp["expert"]["ff"], mlp["router"]["experts"]
            for e in range(E):
                w[f"{q}e{e}.gate"], w[f"{q}e{e}.up"], w[f"{q}e{e}.down"] = mat(F, W), mat(F, W), mat(W, F)
            w[q + "router"], w[q + "router.b"] = mat(E, W, 2.0 * gain), vec(E, 0.0, 0.5)
    w["final.norm"] = vec(W)
    return w
