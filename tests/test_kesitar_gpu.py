"""The Kesitar design in the engine against the plain implementation (`plain_kesitar`): each
mechanism's kernels alone, whole prompts, portions, single tokens, batches, slots used again,
the edges of windows, pooled blocks and pages, and greedy generation through the engine's own
entry point.  Configurations and weights are made here; where random weights would hide a fault
(one far block among many, the sink, a window's edge) the inputs are made so that it shows."""
import math

import numpy as np
import pytest
import torch

import plain_kesitar as P

pytestmark = pytest.mark.gpu


def attention(heads, kv, dim, vdim, size, pool, rot=None, v_mix=False, scale=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else 1.3 / math.sqrt(dim),
         "v_mix": v_mix, "mask": {"size": size, "pool": pool}}
    if rot:
        m["rot"] = {"dims": rot[0], "base": rot[1]}
    return {"type": "attention", "mixer": m, "mlp": {"kind": "dense", "ff": mlp} if mlp else None}


def hgrn2(heads, dim, vdim, mlp=None):
    return {"type": "hgrn2", "mixer": {"heads": heads, "dim": dim, "vdim": vdim}, "mlp": {"kind": "dense", "ff": mlp} if mlp else None}


def model(width, vocab, layers, eps=1e-5, emb=0.8, out=1.7):
    return {"architecture": "Kesitar", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": emb},
            "logit_scale": out, "layers": layers}


CONFIGS = {
    # two value-mixing attention layers around recurrent ones; a window shorter than a page, blocks of 3
    "a": model(64, 211, [attention(4, 2, 32, 16, 7, 3, rot=(16, 1e4), v_mix=True, mlp=96), hgrn2(2, 16, 32, mlp=96),
                         attention(4, 2, 32, 16, 7, 3, rot=(16, 1e4), v_mix=True), hgrn2(2, 16, 32, mlp=80)]),
    # sizes the usual shapes make equal or 1: one kv head, heads == kv heads, dim == vdim, the whole head rotated,
    # blocks of one token, a window of one token, a window below the block's size, no pooling, scales of 1,
    # one recurrent head, value channels beyond 64 and not in steps of 64, query channels not in steps of 4
    "b": model(48, 97, [attention(3, 1, 16, 16, 5, 1, rot=(16, 50.0), mlp=64), hgrn2(1, 18, 80, mlp=64),
                        attention(2, 2, 24, 8, 1, 4, rot=(8, 1e6)), attention(2, 2, 16, 40, 3, 7, mlp=32),
                        attention(2, 1, 16, 16, 6, 0, rot=(4, 2.0), v_mix=True), hgrn2(3, 6, 8)], eps=1e-6, emb=1.0, out=1.0),
    # windows and blocks longer than a page of 64 tokens
    "c": model(32, 64, [attention(2, 1, 16, 16, 70, 66, rot=(8, 1e4), v_mix=True, mlp=48), hgrn2(2, 8, 8),
                        attention(2, 1, 16, 16, 130, 5, rot=(8, 1e4), v_mix=True, mlp=48)]),
    # recurrent layers first and last, the values' source in the middle of the stack, many query heads to a kv head,
    # a width that is no multiple of 4, value channels that are no multiple of 4, odd query channels
    "d": model(50, 131, [hgrn2(2, 9, 7, mlp=36), attention(8, 1, 8, 12, 11, 2, rot=(6, 300.0), v_mix=True, mlp=36),
                         attention(2, 1, 12, 12, 4, 6, v_mix=True), hgrn2(1, 33, 16, mlp=20)], emb=2.0, out=0.5),
    # recurrent layers only (no cache unit at all, no position encoding)
    "e": model(64, 101, [hgrn2(2, 16, 32, mlp=64), hgrn2(4, 8, 16)]),
    # attention only, keys wider than 128 and values of three blocks of 32; the second layer's config leaves out
    # kv_heads (= heads) and scale (= 1 / sqrt(dim))
    "f": model(128, 90, [attention(2, 1, 160, 96, 20, 4, rot=(64, 1e4), mlp=128), attention(4, 4, 16, 16, 9, 0, mlp=64)]),
}
for _k in ("kv_heads", "scale"):
    del CONFIGS["f"]["layers"][1]["mixer"][_k]


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, cfg in CONFIGS.items():
        d = str(tmp_path_factory.mktemp(f"kesitar_{name}"))
        w = P.random_weights(cfg, seed=100 + ord(name), gain=1.5)
        P.write_folder(d, cfg, w)
        out[name] = (d, cfg, w)
    return out


@pytest.fixture(scope="module")
def engines(folders):
    import braidinfer_amd as B
    made = {}

    def get(name, dtype, max_tokens=4096):
        if (name, dtype) not in made:
            made[(name, dtype)] = B.Engine.from_folder(folders[name][0], dtype=dtype, max_tokens=max_tokens)
        return made[(name, dtype)]
    return get


def close(got, want, dtype, what=""):
    """Logits against the plain ones: centred difference over the vocabulary, relative to the logits' spread."""
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want)
    d = got - want
    d = d - d.mean(axis=-1, keepdims=True)
    err = np.sqrt((d * d).mean(axis=-1)) / want.std()
    tol = 2e-4 if dtype == "float32" else 6e-2
    if dtype != "float32":
        # bfloat16 rounding is amplified where a narrow model's norm divides by a small spread: a row in fifty
        # may go up to three times the tolerance, none beyond
        assert (err > tol).sum() <= max(1, len(err) // 50) and err.max() < 3 * tol, \
            f"{what}: {int((err > tol).sum())} rows over {tol}, the worst (row {err.argmax()}) by {err.max():.3g}"
        return
    assert err.max() < tol, f"{what}: row {err.argmax()} differs by {err.max():.3g} (tolerance {tol})"


def run(eng, tokens, portions, want_all=True):
    """One sequence in the given portions; logits of every place."""
    import braidinfer_amd as B
    s = eng.alloc_slot()
    out, at = [], 0
    try:
        for n in portions:
            out.append(eng.step([B.StepEntry(s, tokens[at:at + n], list(range(n)))]).cpu().numpy())
            at += n
    finally:
        eng.free_slot(s)
    assert at == len(tokens)
    return np.concatenate(out)


def tokens_of(cfg, n, seed):
    return [int(t) for t in np.random.default_rng(seed).integers(0, cfg["vocab"], n)]


# ------------------------------------------------------------ mechanisms alone -------
def test_layer_norm_kernels():
    from braidinfer_amd import kernels as K
    rng = np.random.default_rng(0)
    for T, H in ((5, 48), (3, 100), (2, 2048), (4, 777)):
        x = (rng.standard_normal((T, H)) * 3 + 2).astype(np.float32)
        w = (1 + 0.3 * rng.standard_normal(H)).astype(np.float32)
        xd, wd = torch.tensor(x).cuda(), torch.tensor(w).cuda()
        for center, plain in ((True, P.layer_norm), (False, P.rms_norm)):
            want = plain(x.astype(np.float64), w.astype(np.float64), 1e-5)
            out = torch.empty_like(xd)
            K.layernorm(xd, wd, out, 1e-5, center=center)
            assert np.abs(out.cpu().numpy() - want).max() < 2e-5
            acc = torch.tensor(x[::-1].copy()).cuda()
            K.layernorm(xd, wd, acc, 1e-5, center=center, add=True)
            assert np.abs(acc.cpu().numpy() - (x[::-1] + want)).max() < 2e-5
            ob = torch.empty((T, H), dtype=torch.bfloat16, device="cuda")
            K.layernorm(xd, wd, ob, 1e-5, center=center)
            assert np.abs(ob.float().cpu().numpy() - want).max() < 0.02 * np.abs(want).max()
        rows = torch.tensor([T - 1, 0], dtype=torch.int32).cuda()
        out = torch.empty((2, H), dtype=torch.float32, device="cuda")
        K.layernorm(xd, wd, out, 1e-5, rows=rows)
        assert np.abs(out.cpu().numpy() - P.layer_norm(x[[T - 1, 0]].astype(np.float64), w, 1e-5)).max() < 2e-5


@pytest.mark.parametrize("H,d,e", [(2, 16, 32), (1, 18, 80), (3, 6, 8), (2, 128, 128), (1, 70, 200)])
def test_gated_recurrence_kernels(H, d, e):
    """scan (with its gates) and head norm against the plain recurrence: two sequences in unequal portions, the state
    carried in slots that are not neighbours, a padding sequence between them."""
    from braidinfer_amd import kernels as K
    rng = np.random.default_rng(d)
    lens = [37, 5]
    raw = [rng.standard_normal((n, 2 * H * d + H * e)).astype(np.float32) * 2 for n in lens]
    bias = rng.standard_normal(H * d).astype(np.float32)
    lower = rng.uniform(0.05, 0.9, H * d).astype(np.float32)
    nw = (1 + 0.3 * rng.standard_normal(e)).astype(np.float32)
    want = []
    for r in raw:
        r = r.astype(np.float64)
        q = P.silu(r[:, :H * d]).reshape(-1, H, d)
        f = (lower + (1 - lower) * P.sigmoid(r[:, H * d:2 * H * d] + bias)).reshape(-1, H, d)
        o, S = P.gated_recurrence(q, f, r[:, 2 * H * d:].reshape(-1, H, e))
        want.append((P.rms_norm(o, nw, 1e-5).reshape(-1, H * e), S))
    shape = K.glr_state_shape(H, d, e)                   # the state lies as the kernel's lanes hold it
    n_state = int(np.prod(shape))
    arena = torch.zeros((6, n_state + 8), dtype=torch.float32, device="cuda")      # slots with a gap between them
    state = arena[:, 4:4 + n_state].view(6, *shape)
    slots_of = [4, 1]
    got = [[], []]
    for portion in ([20, 3], [1, 1], [16, 1]):
        starts = [sum(len(x) for x in got[0]), sum(len(x) for x in got[1])]
        pieces = [raw[0][starts[0]:starts[0] + portion[0]], np.zeros((1, raw[0].shape[1]), np.float32),
                  raw[1][starts[1]:starts[1] + portion[1]]]
        rows = torch.tensor(np.concatenate(pieces)).cuda()
        cu = torch.tensor(np.cumsum([0, portion[0], 1, portion[1]]), dtype=torch.int32).cuda()
        slots = torch.tensor([slots_of[0], -1, slots_of[1]], dtype=torch.int32).cuda()
        o = torch.zeros((rows.shape[0], H * e), dtype=torch.float32, device="cuda")
        K.glr_scan(rows, torch.tensor(bias).cuda(), torch.tensor(lower).cuda(), o, state, cu, slots, 3, H, d, e)
        on = torch.empty_like(o)
        K.head_rmsnorm(o, torch.tensor(nw).cuda(), on, H, e, 1e-5)
        on = on.cpu().numpy()
        got[0].append(on[:portion[0]])
        got[1].append(on[portion[0] + 1:])
    for i in range(2):
        g = np.concatenate(got[i])
        assert np.abs(g - want[i][0][:len(g)]).max() < 3e-4 * max(1.0, np.abs(want[i][0]).max())
    full = K.glr_state_dense(state[slots_of[1]], H, d, e).cpu().numpy()      # the second sequence ran to its end
    assert np.abs(full - want[1][1]).max() < 1e-4 * max(1.0, np.abs(want[1][1]).max())
    assert float(arena[:, :4].abs().max()) == 0 and float(arena[[0, 2, 3, 5]].abs().max()) == 0


@pytest.mark.parametrize("H,d,e,pieces", [(2, 16, 32, 3), (1, 18, 80, 5), (2, 128, 128, 4), (1, 70, 200, 2)])
def test_recurrence_in_pieces(H, d, e, pieces):
    """Long prompts cut into pieces that are walked side by side, against the plain recurrence: from a state that is
    not zero, with a padding sequence, a sequence shorter than the number of pieces and one whose last pieces are empty."""
    from braidinfer_amd import kernels as K
    rng = np.random.default_rng(e)
    lens = [150, 3, 33]
    raw = [rng.standard_normal((n + 20, 2 * H * d + H * e)).astype(np.float32) * 2 for n in lens]
    bias = rng.standard_normal(H * d).astype(np.float32)
    lower = rng.uniform(0.05, 0.9, H * d).astype(np.float32)
    shape = K.glr_state_shape(H, d, e)
    state = torch.zeros((5,) + tuple(shape), dtype=torch.float32, device="cuda")
    slots_of = [3, 0, 4]
    dev = lambda a: torch.tensor(np.asarray(a), dtype=torch.int32).cuda()
    bd, ld = torch.tensor(bias).cuda(), torch.tensor(lower).cuda()
    # the first 20 tokens of each by the plain walk, so that the pieces start from a state
    first = torch.tensor(np.concatenate([r[:20] for r in raw])).cuda()
    o0 = torch.zeros((60, H * e), dtype=torch.float32, device="cuda")
    K.glr_scan(first, bd, ld, o0, state, dev([0, 20, 40, 60]), dev(slots_of), 3, H, d, e)
    rest = [r[20:] for r in raw]
    pad = np.zeros((1, raw[0].shape[1]), np.float32)
    rows = torch.tensor(np.concatenate([rest[0], pad, rest[1], rest[2]])).cuda()
    new = [lens[0], 1, lens[1], lens[2]]
    slots = [slots_of[0], -1, slots_of[1], slots_of[2]]
    cu, numbers, at = [0], [], 0
    for b, n in enumerate(new):
        run = -(-(-(-n // pieces)) // 16) * 16
        for c in range(pieces):
            cu.append(at + min(n, (c + 1) * run))
            numbers.append(b * pieces + c if slots[b] >= 0 else -1)
        at += n
    o = torch.zeros((rows.shape[0], H * e), dtype=torch.float32, device="cuda")
    piece_state = torch.full((4 * pieces,) + tuple(shape), 7.0, dtype=torch.float32, device="cuda")
    decay = torch.full((4 * pieces, H, 16 * K.glr_rows_per_lane(d)), 7.0, dtype=torch.float32, device="cuda")
    K.glr_scan_pieces(rows, bd, ld, o, state, dev(slots), dev(cu), dev(numbers), piece_state, decay, 4, pieces, H, d, e)
    o = o.cpu().numpy()
    offs = [0, lens[0] + 1, lens[0] + 1 + lens[1]]
    for i, r in enumerate(raw):
        r = r.astype(np.float64)
        q = P.silu(r[:, :H * d]).reshape(-1, H, d)
        f = (lower + (1 - lower) * P.sigmoid(r[:, H * d:2 * H * d] + bias)).reshape(-1, H, d)
        want, S = P.gated_recurrence(q, f, r[:, 2 * H * d:].reshape(-1, H, e))
        got = o[offs[i]:offs[i] + lens[i]]
        assert np.abs(got - want[20:].reshape(lens[i], -1)).max() < 3e-4 * max(1.0, np.abs(want).max())
        assert np.abs(K.glr_state_dense(state[slots_of[i]], H, d, e).cpu().numpy() - S).max() < 1e-4 * max(1.0, np.abs(S).max())
    assert float(state[[1, 2]].abs().max()) == 0


class HandCache:
    """A token unit and a pooled unit with block tables of shuffled pages, for the attention kernels alone."""

    def __init__(self, G, dk, dv, dtype, n_pages=24, slots=3, seed=0):
        self.G, self.dk, self.dv = G, dk, dv
        perm = np.random.default_rng(seed).permutation(n_pages)
        per = n_pages // slots
        self.table = torch.tensor(perm[:per * slots].reshape(slots, per), dtype=torch.int32).cuda()
        self.ptable = torch.tensor(np.random.default_rng(seed + 1).permutation(n_pages)[:per * slots].reshape(slots, per),
                                   dtype=torch.int32).cuda()
        self.unit = torch.full((n_pages, G * 64 * (dk + dv)), 1e4, dtype=dtype, device="cuda")     # stale rows would show
        self.pooled = torch.full((n_pages, G * 64 * (dk + dv)), 1e4, dtype=dtype, device="cuda")


def attend_in_portions(q, k, v, size, pool, scale, sink, portions, dtype=torch.float32, slot=1, matrix=False):
    """q [T, H, dk], k [T, G, dk], v [T, G, dv] through prepare (no bias, norm or rotation), pool and attend
    (`matrix`: portions of more than one token through the matrix-core kernel)."""
    from braidinfer_amd import kernels as K
    T, H, dk = q.shape
    G, dv = k.shape[1], v.shape[2]
    c = HandCache(G, dk, dv, dtype)
    rows = np.concatenate([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], axis=1).astype(np.float32)
    outs, at = [], 0
    for n in portions:
        dev = lambda a: torch.tensor(np.asarray(a), dtype=torch.int32).cuda()
        pos, sot = dev(np.arange(at, at + n)), dev(np.ones(n))            # the sequence is the batch's second; the first is padding
        slots, cu, ctx = dev([-1, slot]), dev([0, 0, n]), dev([0, at + n])
        qo = torch.empty((n, H * dk), dtype=dtype, device="cuda")
        K.pwa_prepare(torch.tensor(rows[at:at + n]).cuda(), None, None, None, 0.0, None, None, 0, pos, sot, slots, c.table, qo, c.unit,
                      None, None, 0, H, G, dk, dv, 64, True)
        if pool:
            K.pwa_pool(c.unit, c.table, c.pooled, c.ptable, cu, ctx, slots, 2, n, G, dk, dv, 64, pool)
        o = torch.empty((n, H * dv), dtype=dtype, device="cuda")
        if matrix and n == 1:
            K.pwa_decode_bf16(qo[:1].repeat(2, 1), o2 := torch.empty((2, H * dv), dtype=dtype, device="cuda"), slots, ctx, c.table,
                              c.unit, c.ptable if pool else None, c.pooled if pool else None, 2, H, G, dk, dv, 64, size, pool, scale, sink)
            o = o2[1:]                    # row b of a single-token step is sequence b: the first is padding
        elif matrix:
            K.pwa_prefill_bf16(qo, o, cu, slots, ctx, c.table, c.unit, c.ptable if pool else None, c.pooled if pool else None, 2, n,
                               H, G, dk, dv, 64, size, pool, scale, sink)
        else:
            K.pwa_attend(qo, o, pos, sot, slots, c.table, c.unit, c.ptable if pool else None, c.pooled if pool else None, H, G, dk,
                         dv, 64, size, pool, scale, sink)
        outs.append(o.float().cpu().numpy())
        at += n
    return np.concatenate(outs).reshape(T, H, dv)


@pytest.mark.parametrize("H,G,dk,dv,size,pool", [(4, 2, 32, 16, 7, 3), (3, 1, 16, 16, 5, 1), (2, 2, 24, 72, 1, 4),
                                                 (2, 1, 16, 8, 70, 66), (2, 2, 80, 16, 130, 5), (2, 1, 8, 8, 6, 0)])
def test_pooled_window_attention_kernels(H, G, dk, dv, size, pool):
    rng = np.random.default_rng(size * 100 + pool)
    T = 300
    q, k, v = (rng.standard_normal((T, n, w)) for n, w in ((H, dk), (G, dk), (G, dv)))
    for sink in (True, False):
        want = P.pooled_window_attention(q.astype(np.float32).astype(np.float64), k.astype(np.float32).astype(np.float64),
                                         v.astype(np.float32).astype(np.float64), 0.4, size, pool, sink)
        whole = attend_in_portions(q, k, v, size, pool, 0.4, sink, [T])
        assert np.abs(whole - want).max() < 2e-5
        cut = attend_in_portions(q, k, v, size, pool, 0.4, sink, [61, 2, 1, 1, 64, 65, 3] + [1] * 40 + [63])
        assert np.array_equal(cut, whole), "portions and single tokens must give the bits of the whole prompt"
    kb, vb = P.to_bf16(k), P.to_bf16(v)
    got = attend_in_portions(P.to_bf16(q), kb, vb, size, pool, 0.4, True, [100, 1, 1, 198], dtype=torch.bfloat16)
    # pooled rows are rounded to bfloat16 where they are kept, and so is the output
    want = P.pooled_window_attention(P.to_bf16(q), kb, vb, 0.4, size, pool, True)
    assert np.abs(got - want).max() < 0.03 * np.abs(want).max()
    for sink in (True, False):
        # the matrix-core kernel against the float one on the same cache: whole, and in portions whose edges
        # fall inside a block of 32 keys, at a page's border and just behind it
        plain = attend_in_portions(P.to_bf16(q), kb, vb, size, pool, 0.4, sink, [T], dtype=torch.bfloat16)
        for portions in ([T], [33, 31, 2, 63, 65, 100, 6], [129, 171], [T - 45] + [1] * 45):
            fast = attend_in_portions(P.to_bf16(q), kb, vb, size, pool, 0.4, sink, portions, dtype=torch.bfloat16, matrix=True)
            assert np.abs(fast - plain).max() < 0.03 * np.abs(plain).max()


def test_edges_that_random_inputs_would_hide():
    """One key made to stand out: just inside and just outside the window; a block that is just seen and not yet;
    a far block among a hundred; and the sink when every score is very negative."""
    H = G = 1
    dk, dv, size, pool, T = 8, 4, 10, 4, 460
    rng = np.random.default_rng(5)
    base_k = rng.standard_normal((T, G, dk)) * 0.1
    v = rng.standard_normal((T, G, dv))
    q = np.zeros((T, H, dk))
    q[:, 0, 0] = 1.0
    for loud in (5, 399, 449, 450, 451):           # tokens whose key answers every query loudly
        k = base_k.copy()
        k[loud, 0, 0] = 60.0
        want = P.pooled_window_attention(q, k, v, 1.0, size, pool, True)
        got = attend_in_portions(q, k, v, size, pool, 1.0, True, [T - 30] + [1] * 30)
        assert np.abs(got - want).max() < 2e-5
        fast = attend_in_portions(q, P.to_bf16(k), P.to_bf16(v), size, pool, 1.0, True, [T - 40, 40], dtype=torch.bfloat16, matrix=True)
        assert np.abs(fast - P.pooled_window_attention(q, P.to_bf16(k), P.to_bf16(v), 1.0, size, pool, True)).max() < 0.03
        i = T - 1
        inside = i - loud < size
        blk = loud // pool
        seen = blk * pool + pool - 1 <= i - size
        if inside:
            assert np.abs(want[i, 0] - v[loud, 0]).max() < 1e-3            # the loud token alone
        elif seen:
            assert np.abs(want[i, 0] - v[blk * pool:blk * pool + pool, 0].mean(axis=0)).max() < 1e-2   # its block's mean
        else:
            assert np.abs(want[i, 0]).max() < np.abs(v).max()              # neither: nothing stands out
        # the query at which the loud token leaves the window, and the one at which its block appears
        for j in (loud + size - 1, loud + size, blk * pool + pool - 1 + size - 1, blk * pool + pool - 1 + size):
            if j < T:
                assert np.abs(got[j] - want[j]).max() < 2e-5
    k = base_k.copy()
    qs = q * 0
    qs[:, 0, 1] = -40.0
    k[:, 0, 1] = 1.0                                # every score is -40: the sink takes the weight
    got = attend_in_portions(qs, k, v, size, pool, 1.0, True, [T])
    assert np.abs(got).max() < 1e-12
    got = attend_in_portions(qs, k, v, size, pool, 1.0, False, [T])
    assert np.abs(got - P.pooled_window_attention(qs, k, v, 1.0, size, pool, False)).max() < 2e-5 and np.abs(got[-1]).max() > 1e-3


def test_prepare_norm_rotation_and_value_mix():
    from braidinfer_amd import kernels as K
    rng = np.random.default_rng(9)
    H, G, dk, dv, T, rd = 3, 1, 24, 40, 70, 8
    rows = rng.standard_normal((T, H * dk + G * dk + G * dv)).astype(np.float32)
    bias = rng.standard_normal(rows.shape[1]).astype(np.float32)
    qn, kn = (1 + 0.3 * rng.standard_normal(dk)).astype(np.float32), (1 + 0.3 * rng.standard_normal(dk)).astype(np.float32)
    pos = np.arange(1000, 1000 + T)
    c = HandCache(G, dk, dv, torch.float32, n_pages=40, slots=2)
    inv = torch.tensor((37.0 ** (-2.0 * np.arange(rd // 2) / rd)).astype(np.float32)).cuda()
    cos, sin = torch.empty((T, rd // 2), device="cuda"), torch.empty((T, rd // 2), device="cuda")
    dev = lambda a: torch.tensor(np.asarray(a), dtype=torch.int32).cuda()
    K.rope_table(dev(pos), inv, cos, sin)
    x = rows.astype(np.float64) + bias
    q = P.rotate(P.rms_norm(x[:, :H * dk].reshape(T, H, dk), qn, 1e-5), pos, rd, 37.0)
    k = P.rotate(P.rms_norm(x[:, H * dk:H * dk + G * dk].reshape(T, G, dk), kn, 1e-5), pos, rd, 37.0)
    v = x[:, H * dk + G * dk:]
    qo = torch.empty((T, H * dk), device="cuda")
    vf = torch.zeros((T, G * dv), device="cuda")
    args = (torch.tensor(rows).cuda(), torch.tensor(bias).cuda(), torch.tensor(qn).cuda(), torch.tensor(kn).cuda(), 1e-5, cos, sin, rd,
            dev(pos), dev(np.zeros(T)), dev([1]), c.table, qo, c.unit)
    K.pwa_prepare(*args, vf, None, 1, H, G, dk, dv, 64, True)
    # angles are float products of position and frequency: at positions near 1000 they carry 6e-5 of rounding
    assert np.abs(qo.cpu().numpy().reshape(T, H, dk) - q).max() < 4e-4
    assert np.abs(vf.cpu().numpy() - v).max() < 1e-6

    def cached():
        unit = c.unit.cpu().numpy()
        table = c.table.cpu().numpy()
        ks, vs = [], []
        for p in pos:
            page = unit[table[1, p // 64]]
            ks.append(page[:G * 64 * dk].reshape(G, 64, dk)[:, p % 64])
            vs.append(page[G * 64 * dk:].reshape(G, dv, 64)[:, :, p % 64])      # values lie transposed in a page
        return np.stack(ks), np.stack(vs).reshape(T, -1)
    ck, cv = cached()
    assert np.abs(ck - k).max() < 4e-4 and np.abs(cv - v).max() < 1e-6
    other = rng.standard_normal((T, G * dv)).astype(np.float32)
    K.pwa_prepare(*args, torch.tensor(other).cuda(), torch.tensor([0.3], dtype=torch.float32).cuda(), 2, H, G, dk, dv, 64, True)
    assert np.abs(cached()[1] - (0.7 * v + np.float64(np.float32(0.3)) * other)).max() < 1e-5


# ------------------------------------------------------------ whole models -----------
@pytest.mark.parametrize("name", list(CONFIGS))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompt_against_plain(folders, engines, name, dtype):
    _, cfg, w = folders[name]
    toks = tokens_of(cfg, 150, 1)
    want = P.forward(cfg, w, toks)
    close(run(engines(name, dtype), toks, [150]), want, dtype, f"{name} {dtype}")
    close(run(engines(name, dtype), toks[:1], [1]), want[:1], dtype, "a sequence of one token")


@pytest.mark.parametrize("name", list(CONFIGS))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_portions_and_single_tokens(folders, engines, name, dtype):
    """A prompt in portions down to two tokens, then token by token across a page's border, against the plain
    logits and, in float32, against the whole prompt's own."""
    _, cfg, w = folders[name]
    n = 215
    toks = tokens_of(cfg, n, 2)
    want = P.forward(cfg, w, toks)
    eng = engines(name, dtype)
    whole = run(eng, toks, [n])
    for portions in ([2, 3, 59, 1, 63, 2, 64, 21], [17] + [1] * 198, [128, 2] + [1] * 85):
        got = run(eng, toks, portions)
        close(got, want, dtype, f"{name} {dtype} {portions[:4]}")
        if dtype == "float32":
            assert np.abs(got - whole).max() < 2e-4 * np.abs(whole).max()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_batch_against_each_alone(folders, engines, dtype):
    import braidinfer_amd as B
    _, cfg, w = folders["a"]
    eng = engines("a", dtype)
    lens = [1, 90, 33, 140, 7]
    prompts = [tokens_of(cfg, n + 20, 10 + n) for n in lens]
    slots = [eng.alloc_slot() for _ in lens]
    got = [[] for _ in lens]
    lg = eng.step([B.StepEntry(s, p[:n], list(range(n))) for s, p, n in zip(slots, prompts, lens)]).cpu().numpy()
    at = 0
    for i, n in enumerate(lens):
        got[i].append(lg[at:at + n])
        at += n
    live = list(range(len(lens)))
    for t in range(20):
        if t == 8:                                  # two requests end early; the batch goes on without them
            for i in (1, 4):
                eng.free_slot(slots[i])
                live.remove(i)
        lg = eng.step([B.StepEntry(slots[i], [prompts[i][lens[i] + t]], [0]) for i in live]).cpu().numpy()
        for r, i in enumerate(live):
            got[i].append(lg[r:r + 1])
    for i in live:
        eng.free_slot(slots[i])
    for i, p in enumerate(prompts):
        g = np.concatenate(got[i])
        close(g, P.forward(cfg, w, p)[:len(g)], dtype, f"request {i} of the batch")


def test_slots_and_pages_used_again(folders, engines):
    """Requests come and go through a cache of few pages: what a freed slot or a returned page held never shows."""
    import braidinfer_amd as B
    folder, cfg, w = folders["a"]
    eng = B.Engine.from_folder(folder, dtype="float32", max_tokens=704, max_seq_len=512, n_slots=3)
    free_before = [g.pool.free_count for g in eng.cache.groups]
    for r in range(6):
        toks = tokens_of(cfg, 100 + 37 * r, 50 + r)
        want = P.forward(cfg, w, toks)
        close(run(eng, toks, [len(toks) - 10] + [1] * 10), want, "float32", f"request {r}")
    assert [g.pool.free_count for g in eng.cache.groups] == free_before
    # a window's pages go back while the sequence runs on: the token unit of a long sequence stays small
    s = eng.alloc_slot()
    toks = tokens_of(cfg, 400, 77)
    eng.step([B.StepEntry(s, toks, [])])
    token_groups = [g for g in eng.cache.groups if g.need.tokens_per_row == 1]
    assert all(sum(p >= 0 for p in g.pages[s]) <= 2 for g in token_groups)
    eng.free_slot(s)


@pytest.mark.parametrize("name", ["a", "c"])
def test_long_decoding(folders, engines, name):
    """Three hundred single-token steps from a short prompt (recorded steps of the engine), past pages, windows and blocks."""
    _, cfg, w = folders[name]
    toks = tokens_of(cfg, 330, 3)
    want = P.forward(cfg, w, toks)
    for dtype in ("float32", "bfloat16"):
        close(run(engines(name, dtype), toks, [30] + [1] * 300), want, dtype, f"{name} {dtype}")


def test_greedy_generation_through_the_engine(folders, engines):
    _, cfg, w = folders["a"]
    prompts = [tokens_of(cfg, n, 20 + n) for n in (3, 41, 12, 70)]
    want = [P.greedy_generate(cfg, w, p, 12) for p in prompts]
    got = engines("a", "float32").generate(prompts, max_new_tokens=12, temperature=0.0, stop_token_ids=[])
    assert got == want
    got16 = engines("a", "bfloat16").generate(prompts, max_new_tokens=12, temperature=0.0, stop_token_ids=[])
    for g, wnt, p in zip(got16, want, prompts):
        for i, (a, b) in enumerate(zip(g, wnt)):
            if a != b:                              # bfloat16 may take the runner-up where two logits are nearly tied
                l = P.forward(cfg, w, p + wnt[:i])[-1]
                assert abs(l[a] - l[b]) < 0.05 * np.abs(l).max()
                break


def test_a_long_prompt_in_pieces(folders, engines):
    """A prompt long enough for the recurrent layers to walk it in pieces, whole and behind a first portion."""
    _, cfg, w = folders["a"]
    toks = tokens_of(cfg, 700, 8)
    want = P.forward(cfg, w, toks)
    for dtype in ("float32", "bfloat16"):
        eng = engines("a", dtype)
        hg = [l.mixer for l in eng.model.layers if type(l.mixer).__name__ == "HGRN2"]
        assert hg and all(m.MIN_PIECE * 4 <= 600 for m in hg)
        close(run(eng, toks, [700]), want, dtype, f"whole {dtype}")
        close(run(eng, toks, [100, 600]), want, dtype, f"behind a portion {dtype}")


def test_presets_run(tmp_path):
    """The tiny preset as a random-weights folder of the library's own making, against the plain implementation."""
    import braidinfer_amd as B
    cfg = B.any_preset("kesitar-tiny")
    folder = B.Engine.write_random_folder(str(tmp_path / "m"), cfg, seed=3, std=0.2, vector_jitter=0.3)
    pc, pw = P.read_folder(folder)
    toks = tokens_of(pc, 60, 4)
    eng = B.Engine.from_folder(folder, dtype="float32", max_tokens=512)
    close(run(eng, toks, [40] + [1] * 20), P.forward(pc, pw, toks), "float32", "preset")
