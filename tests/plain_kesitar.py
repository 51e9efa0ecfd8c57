"""A plain, slow implementation of the Kesitar design in NumPy float64, one function per
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
def layer_norm(x, weight, eps):
    """(x - mean) / sqrt(var + eps) * weight over the last axis, var = mean squared deviation, no bias."""
    mu = x.mean(axis=-1, keepdims=True)
    d = x - mu
    var = (d * d).mean(axis=-1, keepdims=True)
    return d / np.sqrt(var + eps) * weight


def rms_norm(x, weight, eps):
    """x / sqrt(mean(x^2) + eps) * weight over the last axis."""
    ms = (x * x).mean(axis=-1, keepdims=True)
    return x / np.sqrt(ms + eps) * weight


def silu(z):
    return z / (1.0 + np.exp(-z))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def rotate(x, positions, dims, base):
    """Rotary positions on the first `dims` elements of the last axis of x [T, heads, d]:
    element i pairs with i + dims/2; angle = position * base^(-2i/dims)."""
    out = x.copy()
    half = dims // 2
    i = np.arange(half, dtype=np.float64)
    freq = base ** (-2.0 * i / dims)
    ang = np.asarray(positions, dtype=np.float64)[:, None] * freq[None, :]       # [T, half]
    c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def pooled_window_attention(q, k, v, scale, size, pool, sink=True):
    """q [T, H, d], k [T, G, d], v [T, G, e] of one sequence from position 0.  Query i sees the
    tokens j with 0 <= i - j < size and, for every block b of `pool` tokens with
    b*pool + pool - 1 <= i - size, one key and value: the block's means.  One softmax over both,
    with 1 added to its denominator when `sink`.  Returns [T, H, e]."""
    T, H, d = q.shape
    G, e = k.shape[1], v.shape[2]
    rep = H // G
    out = np.zeros((T, H, e))
    nb = T // pool if pool else 0
    kb = np.stack([k[b * pool:(b + 1) * pool].mean(axis=0) for b in range(nb)]) if nb else np.zeros((0, G, d))
    vb = np.stack([v[b * pool:(b + 1) * pool].mean(axis=0) for b in range(nb)]) if nb else np.zeros((0, G, e))
    for i in range(T):
        lo = max(0, i - size + 1)
        seen = [b for b in range(nb) if b * pool + pool - 1 <= i - size] if pool else []
        for h in range(H):
            g = h // rep
            keys = np.concatenate([kb[seen, g], k[lo:i + 1, g]], axis=0)
            vals = np.concatenate([vb[seen, g], v[lo:i + 1, g]], axis=0)
            s = keys @ q[i, h] * scale
            m = max(s.max(), 0.0) if sink else s.max()
            p = np.exp(s - m)
            den = p.sum() + (math.exp(-m) if sink else 0.0)
            out[i, h] = (p / den) @ vals
    return out


def gated_recurrence(q, f, v):
    """q, f [T, H, d], v [T, H, e]; per head S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T from S = 0,
    o_t = S_t^T q_t.  Returns o [T, H, e] and the last state [H, d, e]."""
    T, H, d = q.shape
    e = v.shape[2]
    S = np.zeros((H, d, e))
    o = np.zeros((T, H, e))
    for t in range(T):
        S = f[t][:, :, None] * S + (1.0 - f[t])[:, :, None] * v[t][:, None, :]
        o[t] = np.einsum("hde,hd->he", S, q[t])
    return o, S


def dense_ff(h, gate, up, down):
    return (silu(h @ gate.T) * (h @ up.T)) @ down.T


# ------------------------------------------------------------------ mixers ----------
def attention_mixer(h, w, p, m, eps, v_first):
    """h [T, width]; `p` the layer's tensor prefix, `m` its mixer's sizes.  Returns the mixer's
    output and the values that were cached (what a later value-mixing layer takes as v_first)."""
    T = h.shape[0]
    H, d, e = m["heads"], m["dim"], m["vdim"]
    G = m.get("kv_heads", H)
    q = (h @ w[p + "q"].T + w[p + "q.b"]).reshape(T, H, d)
    k = (h @ w[p + "k"].T + w[p + "k.b"]).reshape(T, G, d)
    v = (h @ w[p + "v"].T + w[p + "v.b"]).reshape(T, G, e)
    q = rms_norm(q, w[p + "q.norm"], eps)
    k = rms_norm(k, w[p + "k.norm"], eps)
    pos = np.arange(T)
    rot = m.get("rot")
    if rot:
        q = rotate(q, pos, rot["dims"], rot["base"])
        k = rotate(k, pos, rot["dims"], rot["base"])
    if m.get("v_mix") and v_first is not None:
        lam = float(w[p + "vmix"])
        v = (1.0 - lam) * v + lam * v_first
    scale = m["scale"] if m.get("scale") is not None else d ** -0.5
    o = pooled_window_attention(q, k, v, scale, m["mask"]["size"], m["mask"].get("pool") or 0)
    return o.reshape(T, H * e) @ w[p + "o"].T, v


def hgrn2_mixer(h, w, p, m, eps):
    T = h.shape[0]
    H, d, e = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w[p + "q"].T).reshape(T, H, d)
    v = (h @ w[p + "v"].T).reshape(T, H, e)
    low = w[p + "lower"]
    f = (low + (1.0 - low) * sigmoid(h @ w[p + "f"].T + w[p + "f.b"])).reshape(T, H, d)
    o, _ = gated_recurrence(q, f, v)
    o = rms_norm(o, w[p + "norm"], eps)
    return o.reshape(T, H * e) @ w[p + "o"].T


# ------------------------------------------------------------------ the model -------
def forward(cfg, w, tokens, return_layers=False):
    """Logits [T, vocab] of one sequence (and the residual rows after every layer)."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][np.asarray(tokens)] * cfg["embedding"]["scale"]
    v_first = None
    after = []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = layer_norm(x, w[p + "norm1"], eps)
        if layer["type"] == "attention":
            m = layer["mixer"]
            y, v = attention_mixer(h, w, p + "mix.", m, eps, v_first if m.get("v_mix") else None)
            if m.get("v_mix") and v_first is None:
                v_first = v
        elif layer["type"] == "hgrn2":
            y = hgrn2_mixer(h, w, p + "mix.", layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        x = x + layer_norm(y, w[p + "norm1b"], eps)
        if layer.get("mlp"):
            h = layer_norm(x, w[p + "norm2"], eps)
            y = dense_ff(h, w[p + "mlp.gate"], w[p + "mlp.up"], w[p + "mlp.down"])
            x = x + layer_norm(y, w[p + "norm2b"], eps)
        after.append(x.copy())
    hn = layer_norm(x, w["final.norm"], eps)
    logits = hn @ w["embed"].T * cfg["logit_scale"]
    return (logits, np.stack(after)) if return_layers else logits


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
            u = np.frombuffer(raw, dtype="<u2").astype(np.uint32) << 16
            arr = u.view(np.float32).astype(np.float64)
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
    u = np.asarray(a, dtype=np.float32).view(np.uint32)
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
    """Random tensors (bfloat16 values) for a configuration dict: matrices N(0, gain^2 / fan-in), norm
    weights around 1, biases N(0, 0.3^2), lower bounds in (0.05, 0.9), value mixing in (0.2, 0.8)."""
    rng = np.random.default_rng(seed)
    W, w = cfg["width"], {}

    def mat(o, i):
        return to_bf16(rng.standard_normal((o, i)) * gain / math.sqrt(i))

    def vec(n, around=1.0, spread=0.3):
        return to_bf16(around + spread * rng.standard_normal(n))
    w["embed"] = to_bf16(rng.standard_normal((cfg["vocab"], W)))
    for i, l in enumerate(cfg["layers"]):
        p, m = f"l{i}.", l["mixer"]
        for n in ["norm1", "norm1b"] + (["norm2", "norm2b"] if l.get("mlp") else []):
            w[p + n] = vec(W)
        H, d, e = m["heads"], m["dim"], m["vdim"]
        if l["type"] == "attention":
            G = m.get("kv_heads", H)
            w[p + "mix.q"], w[p + "mix.q.b"] = mat(H * d, W), vec(H * d, 0.0)
            w[p + "mix.k"], w[p + "mix.k.b"] = mat(G * d, W), vec(G * d, 0.0)
            w[p + "mix.v"], w[p + "mix.v.b"] = mat(G * e, W), vec(G * e, 0.0)
            w[p + "mix.q.norm"], w[p + "mix.k.norm"] = vec(d, 1.5), vec(d, 1.5)
            if m.get("v_mix"):
                w[p + "mix.vmix"] = to_bf16(rng.uniform(0.2, 0.8, ()))
            w[p + "mix.o"] = mat(W, H * e)
        else:
            w[p + "mix.q"], w[p + "mix.f"], w[p + "mix.f.b"] = mat(H * d, W), mat(H * d, W), vec(H * d, 0.0, 1.0)
            w[p + "mix.lower"] = to_bf16(rng.uniform(0.05, 0.9, H * d))
            w[p + "mix.v"], w[p + "mix.norm"], w[p + "mix.o"] = mat(H * e, W), vec(e), mat(W, H * e)
        if l.get("mlp"):
            F = l["mlp"]["ff"]
            w[p + "mlp.gate"], w[p + "mlp.up"], w[p + "mlp.down"] = mat(F, W), mat(F, W), mat(W, F)
    w["final.norm"] = vec(W)
    return w
