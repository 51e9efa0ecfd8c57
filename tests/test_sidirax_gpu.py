"""The Sidirax design in the engine against the plain implementation (`plain_sidirax`): each mechanism's
kernels alone, whole prompts, portions, single tokens, batches, slots used again, far keys, page borders,
the sink, and greedy generation through the engine's own entry point.  Configurations and weights are made
here; where random weights would hide a fault (one far key among hundreds, the sink) the inputs are made so
that it shows."""
import math

import numpy as np
import pytest
import torch

import plain_sidirax as P

pytestmark = pytest.mark.gpu


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, base=10000.0, scaling=None, kv_from=None, scale=None, dims=None, mlp=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
         "scale": scale if scale is not None else 1.3 / math.sqrt(dim + rot_dim)}
    if rot_dim:
        m["rot"] = {"dims": dims or rot_dim, "base": base}
        if scaling:
            m["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def wkv(heads, dim, rank, mlp=None, say_rank=True):
    m = {"heads": heads, "dim": dim}
    if say_rank:
        m["decay_rank"] = rank
    return {"type": "wkv", "mixer": m, "mlp": mlp, "_rank": rank}


def dense(ff, limit=2.5):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(ff, experts, top):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def model(width, vocab, layers, eps=1e-5):
    return {"architecture": "Sidirax", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


YARN = (4.0, 64, 16.0, 1.0)
CONFIGS = {
    # the usual stack: attention with rows of its own, recurrent layers, a second attention layer reading the first one's rows
    "a": model(64, 211, [latent(4, 16, 8, 16, 24, 24, scaling=YARN, mlp=dense(96)), wkv(2, 16, 4, mlp=moe(32, 6, 2)),
                         latent(4, 16, 8, 16, 24, 24, scaling=YARN, kv_from=0, mlp=moe(32, 6, 2)), wkv(2, 16, 4, mlp=moe(32, 6, 2))]),
    # sizes the usual shapes make equal or 1, and odd ones: a recurrent layer first, one head, head sizes that are no
    # multiples of 4 or 8, a cache row of 20 elements, all experts chosen, one expert chosen, a decay of rank 1 whose
    # rank only the tensor gives, no frequency scaling, rot.dims below rot_dim, two attention layers with rows of their
    # own and different sizes, a layer reading rows from a layer that is not the first, layers without feed-forward
    "b": model(50, 97, [wkv(3, 33, 1, mlp=dense(36, 0.7), say_rank=False), latent(1, 10, 6, 12, 9, 14, base=50.0, mlp=moe(20, 3, 3)),
                        latent(2, 12, 4, 6, 16, 10, base=1e6, dims=2, mlp=moe(24, 5, 1)), wkv(1, 6, 3),
                        latent(3, 8, 6, 10, 7, 14, base=50.0, kv_from=1), latent(2, 4, 4, 4, 4, 10, base=1e6, dims=2, kv_from=2, mlp=dense(20, 9.0))],
               eps=1e-6),
    # more heads than a matrix-core workgroup serves at once, a recurrent head wider than 64 channels, a cache row of 256
    "c": model(96, 150, [latent(40, 8, 16, 8, 48, 240, scaling=(8.0, 128, 32.0, 2.0), mlp=moe(40, 9, 4)), wkv(1, 80, 5, mlp=dense(64)),
                         latent(2, 16, 16, 24, 32, 240, scaling=(8.0, 128, 32.0, 2.0), kv_from=0)]),
    # recurrent layers only (no cache unit at all, no position encoding)
    "d": model(64, 101, [wkv(2, 16, 8, mlp=dense(64)), wkv(4, 8, 2, mlp=moe(16, 4, 2))]),
    # attention only; every width equal, a scale of 1, two experts
    "e": model(32, 64, [latent(2, 16, 16, 16, 16, 16, scale=1.0, mlp=moe(16, 2, 1)), latent(2, 16, 16, 16, 16, 16, scale=1.0, mlp=dense(16, 1.0))]),
}


# The size of the random matrices: large enough for every layer to move the logits, small enough where a scale of 1
# or a head of few channels would otherwise make a softmax so sharp that it amplifies bfloat16 rounding a hundredfold.
GAINS = {"a": 1.5, "b": 1.0, "c": 1.5, "d": 1.5, "e": 0.7}


def plain_cfg(cfg):
    """The configuration as the plain implementation and config.json get it (the test's own notes taken out)."""
    out = {k: v for k, v in cfg.items() if k != "layers"}
    out["layers"] = []
    for l in cfg["layers"]:
        l2 = {k: v for k, v in l.items() if not k.startswith("_")}
        out["layers"].append(l2)
    return out


def calm_routing(cfg, w, seed):
    """The same weights with routers whose choice is clear: small router matrices under biases 2.5 apart (in an order
    of the layer's own).  Activations rounded to bfloat16 move a router logit by a few hundredths, and a token that
    takes another expert than the plain implementation differs by far more than rounding, also in what later tokens
    read of it; so the bfloat16 runs of whole models use these, and the float32 runs the lively routers."""
    rng = np.random.default_rng(seed)
    out = dict(w)
    for i, l in enumerate(cfg["layers"]):
        if l.get("mlp") and l["mlp"]["kind"] == "moe":
            E = l["mlp"]["router"]["experts"]
            out[f"l{i}.mlp.router"] = P.to_bf16(w[f"l{i}.mlp.router"] * 0.1)
            out[f"l{i}.mlp.router.b"] = P.to_bf16(2.5 * rng.permutation(E) - 1.25 * E)
    return out


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    """(name, dtype) -> (folder, configuration, weights); see `calm_routing` for what differs between the dtypes."""
    out = {}
    for name, cfg in CONFIGS.items():
        gen = plain_cfg(cfg)
        for l, src in zip(gen["layers"], cfg["layers"]):      # the generator needs every rank; config.json may leave one out
            if l["type"] == "wkv":
                l["mixer"] = dict(l["mixer"], decay_rank=src["_rank"])
        lively = P.random_weights(gen, seed=100 + ord(name), gain=GAINS[name])
        for dtype, w in (("float32", lively), ("bfloat16", calm_routing(gen, lively, ord(name)))):
            d = str(tmp_path_factory.mktemp(f"sidirax_{name}_{dtype}"))
            P.write_folder(d, plain_cfg(cfg), w)
            out[(name, dtype)] = (d, plain_cfg(cfg), w)
    return out


@pytest.fixture(scope="module")
def engines(folders):
    import braidinfer_amd as B
    made = {}

    def get(name, dtype, max_tokens=4096):
        if (name, dtype) not in made:
            made[(name, dtype)] = B.Engine.from_folder(folders[(name, dtype)][0], dtype=dtype, max_tokens=max_tokens)
        return made[(name, dtype)]
    return get


def plain(cfg, w, toks):
    """The plain logits, and per token whether every choice of experts on its way was a clear one: the distance
    between the last chosen router logit and the first one left out, smallest over the layers."""
    margins = []
    want = P.forward(cfg, w, toks, margins=margins)
    return want, (np.min(margins, axis=0) if margins else np.full(len(toks), np.inf))


CLOSE_CALL = 0.1         # router logits closer than this may fall the other way once activations are rounded to bfloat16


def close(got, want, dtype, what="", margins=None):
    """Logits against the plain ones: centred difference over the vocabulary, relative to the logits' spread.  In
    bfloat16 a token whose choice of experts was a close call in the plain implementation may have taken the other
    expert; such rows are left out (float32 holds them like all others)."""
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want)
    d = got - want
    d = d - d.mean(axis=-1, keepdims=True)
    err = np.sqrt((d * d).mean(axis=-1)) / want.std()
    tol = 2e-4 if dtype == "float32" else 6e-2
    if dtype != "float32":
        if margins is not None:
            clear = np.asarray(margins)[:len(err)] >= CLOSE_CALL
            assert clear.sum() >= 0.9 * len(err), f"{what}: many choices of experts are close calls; the test's weights are at fault"
            err = err[clear]
        assert (err > tol).sum() <= max(1, len(err) // 50) and err.max() < 3 * tol, \
            f"{what}: {int((err > tol).sum())} rows over {tol}, the worst (row {err.argmax()}) by {err.max():.3g}"
        return
    assert err.max() < tol, f"{what}: row {err.argmax()} differs by {err.max():.3g} (tolerance {tol})"


def run(eng, tokens, portions):
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


def dev_i(a):
    return torch.tensor(np.asarray(a), dtype=torch.int32).cuda()


def dev_f(a):
    return torch.tensor(np.asarray(a, dtype=np.float32)).cuda()


# ------------------------------------------------------------ mechanisms alone -------
def test_scaled_frequencies_and_tables():
    """The rotary part's frequencies with and without scaling, and its tables with the factor on cos and sin."""
    from braidinfer_amd.parts.rope import RotaryEncoding
    from braidinfer_amd.parts import Runtime
    from braidinfer_amd.engine.step import Workspace, pack_step
    rt = Runtime(torch.device("cuda"), torch.float32)
    for dims, base, sc in ((16, 250.0, (4.0, 64, 16.0, 1.0)), (6, 1e4, None), (32, 5e5, (16.0, 4096, 32.0, 1.0)), (2, 7.0, (2.0, 8, 1.0, 0.5))):
        scaling = dict(zip(("factor", "original", "fast", "slow"), sc)) if sc else None
        enc = RotaryEncoding(dims, base, "adjacent", scaling)
        enc.load({}, "", rt)
        f, mag = P.scaled_frequencies(dims, base, scaling)
        assert np.allclose(enc.inv_freq.cpu().numpy(), f, rtol=1e-6, atol=0)
        assert abs(enc.magnitude - mag) < 1e-12
        if sc:
            plain = base ** (-2.0 * np.arange(dims // 2) / dims)
            assert np.all(f <= plain * (1 + 1e-12)) and np.all(f >= plain / sc[0] * (1 - 1e-12))
        step = pack_step([0], [list(range(50))], [3], "cuda", Workspace("cuda"))
        t = enc.prepare(step)
        ang = (np.arange(3, 53)[:, None] * f[None, :])
        assert np.abs(t.cos.cpu().numpy() - np.cos(ang) * mag).max() < 3e-5 and np.abs(t.sin.cpu().numpy() - np.sin(ang) * mag).max() < 3e-5


@pytest.mark.parametrize("H,d", [(2, 16), (3, 33), (1, 80), (2, 64), (1, 6), (1, 200)])
def test_decayed_recurrence_kernel(H, d):
    """The scan with its decay against the plain recurrence: two sequences in unequal portions, the state carried in
    slots that are not neighbours and lie inside wider rows, a padding sequence between them."""
    from braidinfer_amd import kernels as K
    rng = np.random.default_rng(d)
    lens, hd = [37, 5], H * d
    raw = [rng.standard_normal((n, 5 * hd)).astype(np.float32) for n in lens]
    w0 = rng.uniform(-3.0, 0.5, hd).astype(np.float32)
    u = rng.standard_normal(hd).astype(np.float32)
    want = []
    for r in raw:
        r = r.astype(np.float64)
        rr, kk, vv = (r[:, i * hd:(i + 1) * hd].reshape(-1, H, d) for i in range(3))
        decay = np.exp(-np.exp(r[:, 3 * hd:4 * hd] + w0)).reshape(-1, H, d)
        want.append(P.decayed_outer_recurrence(rr, kk, vv, decay, u.astype(np.float64).reshape(H, d)))
    n_state = int(np.prod(K.glr_state_shape(H, d, d)))
    arena = torch.zeros((6, n_state + 24), dtype=torch.float32, device="cuda")
    state = arena[:, 4:4 + n_state + 10]                     # a slot's row is wider than the heads' states
    slots_of = [4, 1]
    got = [[], []]
    for portion in ([20, 3], [1, 1], [16, 1]):
        starts = [sum(len(x) for x in got[0]), sum(len(x) for x in got[1])]
        pieces = [raw[0][starts[0]:starts[0] + portion[0]], np.zeros((1, 5 * hd), np.float32), raw[1][starts[1]:starts[1] + portion[1]]]
        rows = torch.tensor(np.concatenate(pieces)).cuda()
        o = torch.zeros((rows.shape[0], hd), dtype=torch.float32, device="cuda")
        K.wkv_scan(rows, dev_f(w0), dev_f(u), o, state, dev_i(np.cumsum([0, portion[0], 1, portion[1]])), dev_i([slots_of[0], -1, slots_of[1]]),
                   3, H, d, d)
        o = o.cpu().numpy()
        got[0].append(o[:portion[0]])
        got[1].append(o[portion[0] + 1:])
    for i in range(2):
        g = np.concatenate(got[i])
        wnt = want[i][0].reshape(-1, hd)[:len(g)]
        assert np.abs(g - wnt).max() < 3e-4 * max(1.0, np.abs(wnt).max())
    full = K.glr_state_dense(state[slots_of[1], :n_state].reshape(K.glr_state_shape(H, d, d)), H, d, d).cpu().numpy()
    assert np.abs(full - want[1][1]).max() < 1e-4 * max(1.0, np.abs(want[1][1]).max())
    assert float(arena[:, :4].abs().max()) == 0 and float(arena[[0, 2, 3, 5]].abs().max()) == 0 and float(arena[:, 4 + n_state:].abs().max()) == 0


def test_the_bonus_and_the_order_of_output_and_update():
    """A single token: the output is the bonus term alone; two tokens: the second sees the first without decay of its
    own and without the bonus."""
    from braidinfer_amd import kernels as K
    H, d = 1, 4
    rows = np.zeros((2, 5 * d), np.float32)
    r, k, v = np.array([1, 2, 0, 0.5]), np.array([0.5, -1, 3, 2.0]), np.array([1, -2, 0.25, 4.0])
    rows[0, :d], rows[0, d:2 * d], rows[0, 2 * d:3 * d] = r, k, v
    rows[1, :d], rows[1, d:2 * d], rows[1, 2 * d:3 * d] = r[::-1], k * 0, v * 0
    rows[:, 3 * d:4 * d] = 50.0                                  # decay exp(-exp(50 + w0)): with w0 = -50, 1 / e; with w0 = 0, nothing stays
    u = np.array([2.0, 0.0, 1.0, -1.0], np.float32)
    for w0, keep in ((-50.0, math.exp(-1.0)), (0.0, 0.0)):
        state = torch.zeros((1, int(np.prod(K.glr_state_shape(H, d, d)))), dtype=torch.float32, device="cuda")
        o = torch.zeros((2, d), dtype=torch.float32, device="cuda")
        K.wkv_scan(dev_f(rows), dev_f(np.full(d, w0)), dev_f(u), o, state, dev_i([0, 2]), dev_i([0]), 1, H, d, d)
        o = o.cpu().numpy()
        assert np.allclose(o[0], (r * u * k).sum() * v, rtol=1e-6)
        assert np.allclose(o[1], (r[::-1] * k).sum() * v, rtol=1e-6)          # S_1 = k v^T: the first token's decay never touched it
        S = K.glr_state_dense(state[0].reshape(K.glr_state_shape(H, d, d)), H, d, d).cpu().numpy()[0]
        assert np.allclose(S, keep * np.outer(k, v), rtol=1e-5, atol=1e-30)


def test_shifted_mixes_and_the_kept_row():
    from braidinfer_amd import kernels as K
    rng = np.random.default_rng(3)
    W, n = 50, 5
    mu = rng.uniform(0, 1, (n, W)).astype(np.float32)
    seqs = [rng.standard_normal((23, W)).astype(np.float32), rng.standard_normal((9, W)).astype(np.float32)]
    want = [np.stack([P.shifted_mix(s.astype(np.float64), mu[i].astype(np.float64)) for i in range(n)]) for s in seqs]
    arena = torch.zeros((4, W + 7), dtype=torch.float32, device="cuda")
    kept = arena[:, 3:]
    at = [0, 0]
    for portion in ([10, 1], [1, 1], [2, 7], [10, 0]):
        live = [i for i in (0, 1) if portion[i]]
        hs = [seqs[i][at[i]:at[i] + portion[i]] for i in live]
        pad = np.full((1, W), 9.0, np.float32)
        h = torch.tensor(np.concatenate([hs[0], pad] + hs[1:])).cuda()
        new = [portion[live[0]], 1] + [portion[i] for i in live[1:]]
        slots = [[2, 0][live[0]], -1] + [[2, 0][i] for i in live[1:]]
        T = sum(new)
        out = torch.zeros((n, T, W), dtype=torch.float32, device="cuda")
        K.shift_mix(h, dev_f(mu), out, kept, dev_i(np.repeat(np.arange(len(new)), new)), dev_i(np.cumsum([0] + new)), dev_i(slots), len(new),
                    all(x == 1 for x in new))
        out = out.cpu().numpy()
        o = 0
        for j, i in enumerate(live):
            if j == 1:
                o += 1
            got = out[:, o:o + portion[i]]
            assert np.abs(got - want[i][:, at[i]:at[i] + portion[i]]).max() < 1e-6
            o += portion[i]
            at[i] += portion[i]
    assert np.array_equal(kept[2].cpu().numpy()[:W], seqs[0][-1]) and np.array_equal(kept[0].cpu().numpy()[:W], seqs[1][-1])
    assert float(arena[[1, 3]].abs().max()) == 0 and float(arena[:, :3].abs().max()) == 0
    # bfloat16 rows: differences in float, the result rounded once
    hb = torch.tensor(seqs[0]).cuda().to(torch.bfloat16)
    ob = torch.zeros((n, 23, W), dtype=torch.bfloat16, device="cuda")
    K.shift_mix(hb, dev_f(mu), ob, torch.zeros((1, W), device="cuda"), dev_i(np.zeros(23)), dev_i([0, 23]), dev_i([0]), 1, False)
    wb = np.stack([P.shifted_mix(hb.float().cpu().numpy().astype(np.float64), mu[i].astype(np.float64)) for i in range(n)])
    assert np.abs(ob.float().cpu().numpy() - wb).max() < 0.01 * np.abs(wb).max()


def test_head_norm_weight_and_gate():
    from braidinfer_amd import kernels as K
    rng = np.random.default_rng(4)
    for T, H, e in ((7, 3, 33), (2, 1, 80), (5, 4, 16)):
        o = rng.standard_normal((T, H * e)).astype(np.float32) * 3
        w = (1 + 0.3 * rng.standard_normal(H * e)).astype(np.float32)
        wide = rng.standard_normal((T, 3 * H * e)).astype(np.float32)
        gate = torch.tensor(wide).cuda()[:, H * e:2 * H * e]
        g = wide[:, H * e:2 * H * e].astype(np.float64)
        want = P.rms_norm(o.astype(np.float64).reshape(T, H, e), None, 1e-5).reshape(T, H * e) * w * P.silu(g)
        y = torch.empty((T, H * e), dtype=torch.float32, device="cuda")
        K.head_norm_gate(dev_f(o), dev_f(w), gate, y, H, e, 1e-5)
        assert np.abs(y.cpu().numpy() - want).max() < 1e-5 * max(1.0, np.abs(want).max())


def test_routing_and_experts():
    from braidinfer_amd import kernels as K
    rng = np.random.default_rng(5)
    for T, W, F, E, top, dtype in ((9, 50, 20, 7, 3, torch.float32), (4, 64, 24, 70, 5, torch.float32), (3, 32, 16, 2, 2, torch.float32),
                                   (6, 64, 32, 8, 1, torch.bfloat16), (70, 72, 40, 5, 3, torch.bfloat16), (700, 136, 200, 3, 2, torch.bfloat16)):
        h = P.to_bf16(rng.standard_normal((T, W)))
        w = {"router": P.to_bf16(rng.standard_normal((E, W))), "router.b": P.to_bf16(rng.standard_normal(E))}
        w["router"][1] = w["router"][0]                       # two experts that always tie: the lower number goes first
        w["router.b"][1] = w["router.b"][0]
        for e in range(E):
            w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = (P.to_bf16(rng.standard_normal(s) * 0.3) for s in ((F, W), (F, W), (W, F)))
        want = P.routed_ff(h, w, "", E, top)
        scores = dev_f(h @ w["router"].T)
        chosen = torch.zeros((T, top), dtype=torch.int32, device="cuda")
        share = torch.zeros((T, top), dtype=torch.float32, device="cuda")
        K.route_topk(scores, dev_f(w["router.b"]), chosen, share, top)
        z = h @ w["router"].T + w["router.b"]
        order = np.argsort(-z, axis=1, kind="stable")[:, :top]
        assert np.array_equal(chosen.cpu().numpy(), order)
        zz = np.take_along_axis(z, order, axis=1)
        sm = np.exp(zz - zz.max(axis=1, keepdims=True))
        assert np.abs(share.cpu().numpy() - sm / sm.sum(axis=1, keepdims=True)).max() < 1e-5
        stack = lambda n: torch.tensor(np.stack([w[f"e{e}.{n}"] for e in range(E)]), dtype=torch.float32).cuda().to(dtype)
        hd = torch.tensor(h, dtype=torch.float32).cuda().to(dtype)
        y = torch.zeros((T, top, F), dtype=dtype, device="cuda")
        w_gu = torch.cat([stack("gate"), stack("up")], dim=1).contiguous()
        K.experts_up(hd, w_gu, chosen, y)
        x0 = rng.standard_normal((T, W)).astype(np.float32)
        x = torch.tensor(x0).cuda()
        K.experts_down(y, stack("down"), chosen, share, x)
        tol = 2e-5 if dtype == torch.float32 else 2e-2
        assert np.abs(x.cpu().numpy() - x0 - want).max() < tol * max(1.0, np.abs(want).max())
        if K.experts_grouped_takes(dtype, W, F):
            # the same through the kernels that read every expert once
            n = T * top
            first, order, place = (torch.zeros(k, dtype=torch.int32, device="cuda") for k in (E + 1, n, n))
            K.experts_sort(chosen, first, order, place, E)
            y2 = torch.zeros((n, F), dtype=dtype, device="cuda")
            K.experts_up_grouped(hd, w_gu, first, order, y2, top)
            assert np.abs(y2[place.long()].float().cpu().numpy().reshape(T, top, F) - y.float().cpu().numpy()).max() < 0.02 * float(y.float().abs().max())
            out = torch.zeros((n, W), dtype=torch.float32, device="cuda")
            K.experts_down_grouped(y2, stack("down"), first, out)
            x2 = torch.tensor(x0).cuda()
            K.experts_combine(out, place, share, x2)
            assert np.abs(x2.cpu().numpy() - x0 - want).max() < tol * max(1.0, np.abs(want).max())
            # and through the one launch a product for steps of many tokens
            rows = torch.zeros((n, W), dtype=dtype, device="cuda")
            K.experts_gather(hd, order, rows, top)
            gu = torch.zeros((n, 2 * F), dtype=dtype, device="cuda")
            K.experts_gemm(rows, w_gu, first, gu)
            act = torch.zeros((n, F), dtype=dtype, device="cuda")
            K.silu_mul(gu, act)
            assert np.abs(act.float().cpu().numpy() - y2.float().cpu().numpy()).max() < 0.03 * float(y2.float().abs().max())
            out3 = torch.zeros((n, W), dtype=torch.float32, device="cuda")
            K.experts_gemm(act, stack("down"), first, out3)
            x3 = torch.tensor(x0).cuda()
            K.experts_combine(out3, place, share, x3)
            assert np.abs(x3.cpu().numpy() - x0 - want).max() < 1.5 * tol * max(1.0, np.abs(want).max())


def test_experts_in_their_order():
    """The pairs of (token, slot) grouped by expert, their rows gathered, and the weighted outputs added back."""
    from braidinfer_amd import kernels as K
    rng = np.random.default_rng(8)
    T, top, E, W = 130, 3, 7, 20
    chosen = np.stack([rng.permutation(E)[:top] for _ in range(T)]).astype(np.int32)
    chosen[chosen == 6] = chosen[0, 0]              # no token takes expert 6 (a token may take an expert twice here)
    n = T * top
    first = torch.zeros(E + 1, dtype=torch.int32, device="cuda")
    order = torch.zeros(n, dtype=torch.int32, device="cuda")
    place = torch.zeros(n, dtype=torch.int32, device="cuda")
    K.experts_sort(dev_i(chosen), first, order, place, E)
    f, o, p = first.cpu().numpy(), order.cpu().numpy(), place.cpu().numpy()
    flat = chosen.reshape(-1)
    assert f[0] == 0 and f[E] == n and np.array_equal(np.diff(f), np.bincount(flat, minlength=E))
    assert sorted(o.tolist()) == list(range(n)) and np.array_equal(o[p], np.arange(n))
    for e in range(E):
        assert np.all(flat[o[f[e]:f[e + 1]]] == e)
    h = rng.standard_normal((T, W)).astype(np.float32)
    rows = torch.zeros((n, W), dtype=torch.float32, device="cuda")
    K.experts_gather(dev_f(h), order, rows, top)
    assert np.array_equal(rows.cpu().numpy(), h[o // top])
    out = rng.standard_normal((n, W)).astype(np.float32)
    share = rng.uniform(0, 1, (T, top)).astype(np.float32)
    x0 = rng.standard_normal((T, W)).astype(np.float32)
    x = dev_f(x0)
    K.experts_combine(dev_f(out), place, dev_f(share), x)
    want = x0 + (share[:, :, None].astype(np.float64) * out[p].reshape(T, top, W)).sum(axis=1)
    assert np.abs(x.cpu().numpy() - want).max() < 1e-5


def test_a_product_head_by_head():
    from braidinfer_amd import kernels as K
    rng = np.random.default_rng(9)
    for T, H, N, K_, dtype, pad in ((70, 3, 40, 24, torch.bfloat16, 8), (5, 2, 130, 16, torch.bfloat16, 0), (33, 4, 10, 12, torch.bfloat16, 2),
                                    (9, 5, 7, 13, torch.float32, 3), (1, 1, 96, 64, torch.bfloat16, 16)):
        a = P.to_bf16(rng.standard_normal((T, H, K_ + pad)))
        w = P.to_bf16(rng.standard_normal((H, N, K_)))
        ad = torch.tensor(a, dtype=torch.float32).cuda().to(dtype)
        od = torch.full((T, H, N + 5), 7.0, dtype=dtype, device="cuda")
        K.head_linear(ad[:, :, :K_], torch.tensor(w, dtype=torch.float32).cuda().to(dtype), od[:, :, 2:2 + N])
        want = np.einsum("thk,hnk->thn", a[:, :, :K_], w)
        got = od.float().cpu().numpy()
        assert np.abs(got[:, :, 2:2 + N] - want).max() < (1e-5 if dtype == torch.float32 else 0.01) * np.abs(want).max()
        assert np.all(got[:, :, :2] == 7.0) and np.all(got[:, :, 2 + N:] == 7.0)          # nothing beside the view is touched


def test_clamped_gated_unit():
    from braidinfer_amd import kernels as K
    rng = np.random.default_rng(6)
    T, F = 5, 37
    gu = (rng.standard_normal((T, 2 * F)) * 3).astype(np.float32)
    b = rng.standard_normal(2 * F).astype(np.float32)
    for limit in (0.5, 2.0, 100.0):
        g = np.minimum(gu[:, :F].astype(np.float64) + b[:F], limit)
        u = np.clip(gu[:, F:].astype(np.float64) + b[F:], -limit, limit)
        want = g * P.sigmoid(1.702 * g) * (u + 1)
        a = torch.empty((T, F), dtype=torch.float32, device="cuda")
        K.clamped_glu(dev_f(gu), dev_f(b), a, limit, 1.702)
        assert np.abs(a.cpu().numpy() - want).max() < 1e-5 * max(1.0, np.abs(want).max())
    x = dev_f(gu)
    K.add_bias_rows(x, dev_f(b))
    assert np.abs(x.cpu().numpy() - (gu + b)).max() < 1e-6


class LatentCache:
    """One cache unit of latent rows with a block table of shuffled pages, for the kernels alone."""

    def __init__(self, R, DR, dtype, n_pages=24, slots=3, seed=0):
        perm = np.random.default_rng(seed).permutation(n_pages)
        per = n_pages // slots
        self.table = torch.tensor(perm[:per * slots].reshape(slots, per), dtype=torch.int32).cuda()
        self.unit = torch.full((n_pages, 64 * (2 * R + DR)), 1e4, dtype=dtype, device="cuda")      # stale rows would show


def latent_in_portions(q, dkv, cw, sinks, H, D, DR, R, rot, freqs, mag, scale, portions, dtype=torch.float32, matrix=False, slot=1,
                       absorb=None):
    """q [T, H (D + DR)] and dkv [T, R + DR] float sums through prepare and the attention kernels; `absorb` [H, R, D]
    takes the plain query parts to the latent (None: the first R of D elements as they are, D >= R not needed).
    Returns the mixed latents [T, H, R]."""
    from braidinfer_amd import kernels as K
    T = q.shape[0]
    c = LatentCache(R, DR, dtype)
    wide = R + DR
    outs, at = [], 0
    for n in portions:
        pos = np.arange(at, at + n)
        ang = pos[:, None] * np.asarray(freqs)[None, :] if rot else np.zeros((n, 0))
        cos, sin = dev_f(np.cos(ang) * mag), dev_f(np.sin(ang) * mag)
        slots, cu, ctx = dev_i([-1, slot]), dev_i([0, 0, n]), dev_i([0, at + n])
        q_plain = torch.zeros((n, H * D), dtype=dtype, device="cuda")
        q_wide = torch.zeros((n, H * wide), dtype=dtype, device="cuda")
        K.latent_prepare(dev_f(q[at:at + n]), dev_f(dkv[at:at + n]), dev_f(cw), 1e-5, cos if rot else None, sin if rot else None, rot,
                         dev_i(pos), dev_i(np.ones(n)), slots, c.table, c.unit, q_plain, q_wide, H, D, DR, R, 64)
        qp = q_plain.float().cpu().numpy().reshape(n, H, D)
        lat = np.einsum("hrd,thd->thr", absorb, qp)
        qw = q_wide.float().cpu().numpy().reshape(n, H, wide)
        qw[:, :, :R] = lat
        q_wide = torch.tensor(qw.reshape(n, -1), dtype=torch.float32).cuda().to(dtype)
        o = torch.empty((n, H * R), dtype=dtype, device="cuda")
        sk = dev_f(sinks) if sinks is not None else None
        if matrix and n == 1:
            o2 = torch.empty((2, H * R), dtype=dtype, device="cuda")
            blocks = next(b for b in range(1, H + 1) if H % b == 0 and K.pwa_decode_takes(dtype, H, b, wide, R, 64))
            K.pwa_decode_bf16(q_wide[:1].repeat(2, 1), o2, slots, ctx, c.table, c.unit, None, None, 2, H, blocks, wide, R, 64, 1 << 30, 0, scale,
                              sinks is not None, sk, cache_heads=1)
            o = o2[1:]
        elif matrix:
            K.pwa_prefill_bf16(q_wide, o, cu, slots, ctx, c.table, c.unit, None, None, 2, n, H, 1, wide, R, 64, 1 << 30, 0, scale,
                               sinks is not None, sk)
        else:
            K.pwa_attend(q_wide, o, dev_i(pos), dev_i(np.ones(n)), slots, c.table, c.unit, None, None, H, 1, wide, R, 64, 1 << 30, 0, scale,
                         sinks is not None, sk)
        outs.append(o.float().cpu().numpy())
        at += n
    return np.concatenate(outs).reshape(T, H, R)


def plain_latent(q, dkv, cw, sinks, H, D, DR, R, freqs, mag, scale, absorb):
    """The same by the plain functions: keys [W c | k_r] head by head with W = absorb^T, values c."""
    T = q.shape[0]
    pos = np.arange(T)
    c = P.rms_norm(dkv[:, :R], cw, 1e-5)
    kr = P.rotate_pairs(dkv[:, R:], pos, np.asarray(freqs), mag) if len(freqs) else dkv[:, R:]
    q = q.reshape(T, H, D + DR)
    qr = P.rotate_pairs(q[..., D:], pos, np.asarray(freqs), mag) if len(freqs) else q[..., D:]
    qq = np.concatenate([q[..., :D], qr], axis=-1)
    k = np.concatenate([np.einsum("hrd,tr->thd", absorb, c), np.repeat(kr[:, None, :], H, axis=1)], axis=-1)
    v = np.repeat(c[:, None, :], H, axis=1)
    return P.sink_softmax_attention(qq, k, v, scale, sinks)


@pytest.mark.parametrize("H,D,DR,R,rot", [(4, 16, 8, 24, 8), (1, 10, 6, 14, 6), (3, 12, 4, 10, 2), (2, 8, 16, 40, 16), (2, 5, 0, 8, 0),
                                          (16, 8, 32, 160, 32), (48, 4, 8, 64, 8), (32, 4, 32, 224, 32)])
def test_latent_attention_kernels(H, D, DR, R, rot):
    """prepare (norm, rotation, cache rows) and the attention kernels with a learnt sink a head, against the plain
    attention with expanded keys: whole, in portions across page borders, and token by token."""
    rng = np.random.default_rng(H * 100 + R)
    T = 200
    q = rng.standard_normal((T, H * (D + DR))).astype(np.float32).astype(np.float64)
    dkv = (rng.standard_normal((T, R + DR)) * 2).astype(np.float32).astype(np.float64)
    cw = (1 + 0.3 * rng.standard_normal(R)).astype(np.float32).astype(np.float64)
    absorb = rng.standard_normal((H, R, D)) / math.sqrt(D)
    freqs, mag = P.scaled_frequencies(rot, 300.0, {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}) if rot else ([], 1.0)
    for sinks in (rng.standard_normal(H).astype(np.float32).astype(np.float64) * 2, None):
        want = plain_latent(q, dkv, cw, sinks, H, D, DR, R, freqs, mag, 0.3, absorb)
        whole = latent_in_portions(q, dkv, cw, sinks, H, D, DR, R, rot, freqs, mag, 0.3, [T], absorb=absorb)
        assert np.abs(whole - want).max() < 1e-4 * max(1.0, np.abs(want).max())
        cut = latent_in_portions(q, dkv, cw, sinks, H, D, DR, R, rot, freqs, mag, 0.3, [61, 2, 1, 1, 64, 65] + [1] * 6, absorb=absorb)
        assert np.abs(cut - whole).max() < 1e-5 * max(1.0, np.abs(want).max())
    if (R + DR) % 8 == 0 and R % 4 == 0:
        sinks = rng.standard_normal(H) * 2
        plain = latent_in_portions(q, dkv, cw, sinks, H, D, DR, R, rot, freqs, mag, 0.3, [T], dtype=torch.bfloat16, absorb=absorb)
        for portions in ([T], [33, 31, 2, 63, 65, 6], [T - 45] + [1] * 45):
            fast = latent_in_portions(q, dkv, cw, sinks, H, D, DR, R, rot, freqs, mag, 0.3, portions, dtype=torch.bfloat16, matrix=True, absorb=absorb)
            assert np.abs(fast - plain).max() < 0.03 * np.abs(plain).max()


def test_a_far_key_and_the_sink_show():
    """One key made to stand out among hundreds, at a page's border and far back, in prompts and single tokens; the
    sink when it outweighs every score and when it weighs nothing."""
    H, D, DR, R, T = 2, 8, 0, 8, 460
    rng = np.random.default_rng(5)
    absorb = np.stack([np.eye(R, D)] * H)
    cw = np.ones(R)
    q = np.zeros((T, H * D))
    q[:, 0] = q[:, D] = 1.0
    base = rng.standard_normal((T, R)) * 0.1
    for loud in (0, 5, 63, 64, 399):
        dkv = base.copy()
        dkv[:, 1:] += rng.standard_normal((T, R - 1))           # the latents differ, so a mix-up of rows shows
        dkv[loud] *= 0.05
        dkv[loud, 0] = 50.0                                     # after the norm: first element sqrt(R), all others tiny
        want = plain_latent(q, dkv, cw, np.zeros(H), H, D, DR, R, [], 1.0, 8.0, absorb)
        c_loud = P.rms_norm(dkv[loud:loud + 1, :R], cw, 1e-5)[0]
        assert np.abs(want[T - 1, 0] - c_loud).max() < 1e-3     # the last query sees the loud token alone
        got = latent_in_portions(q, dkv, cw, np.zeros(H), H, D, DR, R, 0, [], 1.0, 8.0, [T - 30] + [1] * 30, absorb=absorb)
        assert np.abs(got - want).max() < 2e-5
        fast = latent_in_portions(q, dkv, cw, np.zeros(H), H, D, DR, R, 0, [], 1.0, 8.0, [T - 30] + [1] * 30, dtype=torch.bfloat16,
                                  matrix=True, absorb=absorb)
        assert np.abs(fast[T - 1, 0] - c_loud).max() < 0.03 * np.abs(c_loud).max()
    dkv = base + rng.standard_normal((T, R))
    heavy = latent_in_portions(q, dkv, cw, np.array([60.0, -60.0]), H, D, DR, R, 0, [], 1.0, 1.0, [T], absorb=absorb)
    none = latent_in_portions(q, dkv, cw, None, H, D, DR, R, 0, [], 1.0, 1.0, [T], absorb=absorb)
    assert np.abs(heavy[:, 0]).max() < 1e-12                    # the first head's sink takes all the weight
    assert np.abs(heavy[:, 1] - none[:, 1]).max() < 1e-6 and np.abs(none[-1, 1]).max() > 1e-3      # the second head's takes none


# ------------------------------------------------------------ whole models -----------
@pytest.mark.parametrize("name", list(CONFIGS))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompt_against_plain(folders, engines, name, dtype):
    _, cfg, w = folders[(name, dtype)]
    toks = tokens_of(cfg, 150, 1)
    want, m = plain(cfg, w, toks)
    close(run(engines(name, dtype), toks, [150]), want, dtype, f"{name} {dtype}", m)
    close(run(engines(name, dtype), toks[:1], [1]), want[:1], dtype, "a sequence of one token")
    close(run(engines(name, dtype), toks[:3], [1, 1, 1]), want[:3], dtype, "the first tokens one by one")


def test_residual_rows_after_every_layer(folders, engines):
    import braidinfer_amd as B
    _, cfg, w = folders[("a", "float32")]
    toks = tokens_of(cfg, 40, 9)
    _, layers = P.forward(cfg, w, toks, return_layers=True)
    eng = engines("a", "float32")
    seen = {}
    s = eng.alloc_slot()
    eng.step([B.StepEntry(s, toks, [])], probe=lambda n, t: seen.__setitem__(n, t.float().cpu().numpy().copy()))
    eng.free_slot(s)
    for i in range(len(cfg["layers"])):
        assert np.abs(seen[f"L{i}.post_ffn"] - layers[i]).max() < 2e-4 * np.abs(layers[i]).max()


@pytest.mark.parametrize("name", list(CONFIGS))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_portions_and_single_tokens(folders, engines, name, dtype):
    """A prompt in portions down to two tokens, then token by token across a page's border, against the plain
    logits and, in float32, against the whole prompt's own."""
    _, cfg, w = folders[(name, dtype)]
    n = 215
    toks = tokens_of(cfg, n, 2)
    want, m = plain(cfg, w, toks)
    eng = engines(name, dtype)
    whole = run(eng, toks, [n])
    for portions in ([2, 3, 59, 1, 63, 2, 64, 21], [17] + [1] * 198, [128, 2] + [1] * 85):
        got = run(eng, toks, portions)
        close(got, want, dtype, f"{name} {dtype} {portions[:4]}", m)
        if dtype == "float32":
            assert np.abs(got - whole).max() < 2e-4 * np.abs(whole).max()


@pytest.mark.parametrize("name", ["a", "b"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_batch_against_each_alone(folders, engines, name, dtype):
    import braidinfer_amd as B
    _, cfg, w = folders[(name, dtype)]
    eng = engines(name, dtype)
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
        want, m = plain(cfg, w, p)
        close(g, want[:len(g)], dtype, f"request {i} of the batch", m)


def test_slots_and_pages_used_again(folders):
    """Requests come and go through a cache of few pages and slots: what a freed slot's state or a returned page held
    never shows."""
    import braidinfer_amd as B
    folder, cfg, w = folders[("a", "float32")]
    eng = B.Engine.from_folder(folder, dtype="float32", max_tokens=704, max_seq_len=512, n_slots=2)
    free_before = [g.pool.free_count for g in eng.cache.groups]
    for r in range(6):
        toks = tokens_of(cfg, 100 + 37 * r, 50 + r)
        want = P.forward(cfg, w, toks)
        close(run(eng, toks, [len(toks) - 10] + [1] * 10), want, "float32", f"request {r}")
    assert [g.pool.free_count for g in eng.cache.groups] == free_before
    # the layers that read another layer's rows own no cache unit
    assert sorted(eng.cache.group_of_unit) == [0]


@pytest.mark.parametrize("name", ["a", "b"])
def test_long_decoding(folders, engines, name):
    """Three hundred single-token steps from a short prompt (recorded steps of the engine), past page borders."""
    for dtype in ("float32", "bfloat16"):
        _, cfg, w = folders[(name, dtype)]
        toks = tokens_of(cfg, 330, 3)
        want, m = plain(cfg, w, toks)
        close(run(engines(name, dtype), toks, [30] + [1] * 300), want, dtype, f"{name} {dtype}", m)


def test_a_long_prompt(folders, engines):
    for dtype in ("float32", "bfloat16"):
        _, cfg, w = folders[("a", dtype)]
        toks = tokens_of(cfg, 700, 8)
        want, m = plain(cfg, w, toks)
        close(run(engines("a", dtype), toks, [700]), want, dtype, f"whole {dtype}", m)
        close(run(engines("a", dtype), toks, [100, 600]), want, dtype, f"behind a portion {dtype}", m)


def test_greedy_generation_through_the_engine(folders, engines):
    _, cfg, w = folders[("a", "float32")]
    prompts = [tokens_of(cfg, n, 20 + n) for n in (3, 41, 12, 70)]
    want = [P.greedy_generate(cfg, w, p, 12) for p in prompts]
    got = engines("a", "float32").generate(prompts, max_new_tokens=12, temperature=0.0, stop_token_ids=[])
    assert got == want
    _, cfg, w = folders[("a", "bfloat16")]
    want = [P.greedy_generate(cfg, w, p, 12) for p in prompts]
    got16 = engines("a", "bfloat16").generate(prompts, max_new_tokens=12, temperature=0.0, stop_token_ids=[])
    for g, wnt, p in zip(got16, want, prompts):
        for i, (a, b) in enumerate(zip(g, wnt)):
            if a != b:                              # bfloat16 may take the runner-up where two logits are nearly tied
                l = P.forward(cfg, w, p + wnt[:i])[-1]
                assert abs(l[a] - l[b]) < 0.05 * np.abs(l).max()
                break


def test_presets_run(tmp_path):
    """The tiny preset as a random-weights folder of the library's own making, against the plain implementation."""
    import braidinfer_amd as B
    cfg = B.any_preset("sidirax-tiny")
    folder = B.Engine.write_random_folder(str(tmp_path / "m"), cfg, seed=3, std=0.2, vector_jitter=0.3)
    pc, pw = P.read_folder(folder)
    toks = tokens_of(pc, 60, 4)
    eng = B.Engine.from_folder(folder, dtype="float32", max_tokens=512)
    close(run(eng, toks, [40] + [1] * 20), P.forward(pc, pw, toks), "float32", "preset")


def test_replay_of_given_tokens_through_the_command(folders, tmp_path):
    """`bin/trace_run` as a child process on a Sidirax folder (one whose config.json leaves a size to a tensor): requests
    whole, with their last tokens one by one, and two of unequal length in one batch, against the plain logits."""
    import json
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder, cfg, w = folders[("b", "float32")]
    V = cfg["vocab"]
    seqs = [tokens_of(cfg, n, 60 + n) for n in (90, 41)]
    refs = [P.forward(cfg, w, s) for s in seqs]
    out = str(tmp_path / "out")
    p = subprocess.Popen([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out", out,
                          "--max-tokens", "512"], stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    n = [0]

    def step(entries, end=()):
        p.stdin.write(json.dumps({"step": n[0], "entries": entries, "end": list(end)}) + "\n")
        p.stdin.flush()
        line = p.stdout.readline().strip()
        assert line == f"done {n[0]}", f"trace_run said {line!r} (exit {p.poll()})"
        path = os.path.join(out, f"{n[0]}.f32")
        n[0] += 1
        return np.fromfile(path, dtype="<f4").reshape(-1, V) if os.path.exists(path) else None

    got = step([{"id": "w", "tokens": seqs[0], "want": [0, 63, 64, 89]}], end=["w"])
    close(got, refs[0][[0, 63, 64, 89]], "float32", "whole")
    assert step([{"id": "d", "tokens": seqs[0][:60], "want": []}]) is None
    for t in range(60, 90):
        got = step([{"id": "d", "tokens": [seqs[0][t]], "want": [0]}], end=["d"] if t == 89 else [])
        close(got, refs[0][t:t + 1], "float32", f"one by one at {t}")
    got = step([{"id": "a", "tokens": seqs[0][:80], "want": [79]}, {"id": "b", "tokens": seqs[1][:35], "want": [3, 34]}])
    close(got, np.stack([refs[0][79], refs[1][3], refs[1][34]]), "float32", "a batch's prompts")
    for t in range(6):
        ending = ["b"] if t == 5 else []
        got = step([{"id": "a", "tokens": [seqs[0][80 + t]], "want": [0]}, {"id": "b", "tokens": [seqs[1][35 + t]], "want": [0]}], end=ending)
        close(got, np.stack([refs[0][80 + t], refs[1][35 + t]]), "float32", f"a batch's token {t}")
    got = step([{"id": "a", "tokens": [seqs[0][86]], "want": [0]}], end=["a"])
    close(got, refs[0][86:87], "float32", "the batch's longer request alone")
    p.stdin.close()
    assert p.wait(timeout=60) == 0
