"""WKV time mixing: a linear recurrence with a decay per key channel that depends on the token, a bonus
for the current token, and inputs mixed with the token before.

With n the mixer's input and n' the input of the token before in the sequence (zeros before the first), each
of five branches s in (r, k, v, g, w) reads its own mix m_s = n + (n' - n) * mu_s.  Per head of d channels:
r, k, v = W_r m_r, W_k m_k, W_v m_v, the gate silu(W_g m_g), and the decay
    w = exp(-exp(W_w2 tanh(W_w1 m_w) + w0))      (a low-rank projection; in (0, 1) per head and key channel)
drive
    o_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t,      S_t = diag(w_t) S_(t-1) + k_t v_t^T
with the bonus u [heads, d] for the current token only.  Every head's o is divided by its root mean square,
the heads are concatenated, multiplied by a weight [heads * d] and by the gate, and projected by W_o.

What a sequence keeps is fixed in size: S [heads, d, d] (zero at first) and the last token's n, both float in
both precisions, in the sequence's slot of the cache's state area (`StateNeed`; S laid out as the scan kernel's
lanes hold it, n behind it).  The five products leave float sums, so decay, gate, recurrence and head norm work
on unrounded projections; the mixes and tanh's output have the products' type.  The reference has no recurrent
mixer.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import kernels as K
from ..cache import StateNeed
from ..errors import ConfigError, StepError
from ..weights import TensorSpec
from .base import Mixer, MixerContext, Runtime, register_part
from .gated_recurrence import HGRN2, pieces_for
from .linear import linear, stream_layout

BRANCHES = ("r", "k", "v", "g", "w")


class WKVTimeMix(Mixer):
    graph_safe = True

    NAMES = {"mu_r": "mu.r", "mu_k": "mu.k", "mu_v": "mu.v", "mu_g": "mu.g", "mu_w": "mu.w", "r": "r", "k": "k", "v": "v",
             "g": "g", "w1": "w1", "w2": "w2", "w0": "w0", "u": "u", "norm": "norm", "o": "o"}

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, decay_rank: int, norm_eps: float,
                 names: Optional[Dict[str, str]] = None):
        if num_heads <= 0 or not 0 < head_dim <= 512 or decay_rank <= 0:
            raise ConfigError(f"wkv: {num_heads} heads of {head_dim} channels with a decay of rank {decay_rank} "
                              "(all positive, at most 512 channels a head)")
        self.H, self.nh, self.d, self.rank = int(hidden_size), int(num_heads), int(head_dim), int(decay_rank)
        self.eps = float(norm_eps)
        self.names = dict(self.NAMES, **(names or {}))
        self.mu = self.w = self.w0 = self.u = self.norm_w = self.w_o = None
        self.state_floats = 1
        for n in K.glr_state_shape(self.nh, self.d, self.d):
            self.state_floats *= n

    def weight_specs(self, prefix: str) -> List[TensorSpec]:
        n, hd = self.names, self.nh * self.d
        out = [TensorSpec(prefix + n["mu_" + s], (self.H,), kind="vector", init="normal") for s in BRANCHES]
        out += [TensorSpec(prefix + n["r"], (hd, self.H)), TensorSpec(prefix + n["k"], (hd, self.H)),
                TensorSpec(prefix + n["v"], (hd, self.H)), TensorSpec(prefix + n["g"], (hd, self.H)),
                TensorSpec(prefix + n["w1"], (self.rank, self.H)), TensorSpec(prefix + n["w2"], (hd, self.rank)),
                TensorSpec(prefix + n["w0"], (hd,), kind="vector", init="normal"),
                TensorSpec(prefix + n["u"], (self.nh, self.d), kind="vector", init="normal"),
                TensorSpec(prefix + n["norm"], (hd,), kind="vector", init="ones"),
                TensorSpec(prefix + n["o"], (self.H, hd))]
        return out

    def load(self, tensors: Dict[str, torch.Tensor], prefix: str, rt: Runtime) -> None:
        self.rt = rt
        n = self.names
        mu = rt.empty((len(BRANCHES), self.H), torch.float32)
        for i, s in enumerate(BRANCHES):
            mu[i].copy_(tensors[prefix + n["mu_" + s]].to(torch.float32).reshape(-1))
        self.mu = mu
        self.w = {s: stream_layout(tensors[prefix + n[s]], rt) for s in ("r", "k", "v", "g", "w1", "w2")}
        self.w_o = stream_layout(tensors[prefix + n["o"]], rt)
        self.w0 = rt.own(tensors[prefix + n["w0"]].to(torch.float32).reshape(-1))
        self.u = rt.own(tensors[prefix + n["u"]].to(torch.float32).reshape(-1))
        self.norm_w = rt.own(tensors[prefix + n["norm"]].to(torch.float32).reshape(-1))

    MIN_PIECE = 128          # tokens: shorter pieces do not pay for the second walk

    def state_need(self) -> StateNeed:
        # the heads' states as the scan keeps them, then the last token's input
        return StateNeed((self.state_floats + self.H,), torch.float32)

    def forward(self, h, x, step, ctx: MixerContext) -> None:
        T, hd, dt = step.n_tokens, self.nh * self.d, self.rt.dtype
        if ctx.state is None:
            raise StepError("wkv: the cache gave this mixer no state")
        state = ctx.state
        kept = state[:, self.state_floats:]
        mixes = step.ws.get("wkv_mix", (len(BRANCHES), T, self.H), dt)
        K.shift_mix(h, self.mu, mixes, kept, step.seq_of_token, step.cu_seqlens, step.slots, step.n_seqs, step.is_decode)
        # float sums r | k | v | z | g side by side
        rows = step.ws.get("wkv_rows", (T, 5 * hd), torch.float32)
        for i, s in enumerate(("r", "k", "v")):
            linear(mixes[i], self.w[s], rows[:, i * hd:(i + 1) * hd], step.ws)
        linear(mixes[3], self.w["g"], rows[:, 4 * hd:5 * hd], step.ws)
        low = step.ws.get("wkv_low", (T, self.rank), torch.float32)
        linear(mixes[4], self.w["w1"], low, step.ws)
        low_t = step.ws.get("wkv_low_t", (T, self.rank), dt)
        K.tanh(low, low_t)
        linear(low_t, self.w["w2"], rows[:, 3 * hd:4 * hd], step.ws)
        o = step.ws.get("wkv_o", (T, hd), torch.float32)
        pieces = pieces_for(step, self.nh * -(-self.d // 16), self.MIN_PIECE)
        if pieces > 1:
            # long prompts: every sequence cut into pieces that are walked side by side, twice
            cu, numbers = HGRN2._piece_arrays(step, pieces)
            n = step.n_seqs * pieces
            piece_state = step.ws.get("wkv_piece_state", (n,) + tuple(K.glr_state_shape(self.nh, self.d, self.d)), torch.float32)
            decay = step.ws.get("wkv_decay", (n, self.nh, 16 * K.glr_rows_per_lane(self.d)), torch.float32)
            K.wkv_scan_pieces(rows, self.w0, self.u, o, state, step.slots, cu, numbers, piece_state, decay, step.n_seqs, pieces,
                              self.nh, self.d, self.d)
        else:
            K.wkv_scan(rows, self.w0, self.u, o, state, step.cu_seqlens, step.slots, step.n_seqs, self.nh, self.d, self.d)
        y = step.ws.get("wkv_y", (T, hd), dt)
        K.head_norm_gate(o, self.norm_w, rows[:, 4 * hd:5 * hd], y, self.nh, self.d, self.eps)
        linear(y, self.w_o, x, step.ws, accumulate=True)


register_part("mixer", "wkv", WKVTimeMix, replace=True)
