"""HGRN2: linear attention whose forget gate also decides what is written.

Per token and head (d query channels, e value channels): q = silu(W_q n), v = W_v n,
f = lower + (1 - lower) * sigmoid(W_f n + b) per channel with a learnt lower bound, then
    S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T,     o_t = S_t^T q_t
(the gate acts on the rows of S that belong to q's channels; no key, no other scale).  Every
head's o is RMS-normed over its e channels with one weight shared by the heads, the heads are
concatenated and projected by W_o.

The state S [heads, d, e] starts at zero, lives in float in both precisions and is carried from
step to step in the sequence's slot of the cache's state area (`StateNeed`); gates, the
recurrence and the head norm are float.  Prompts are walked token by token inside one kernel,
the state in registers.  The reference has no recurrent mixer of this form.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import kernels as K
from ..cache import StateNeed
from ..errors import ConfigError, StepError
from ..weights import TensorSpec
from .base import Mixer, MixerContext, Runtime, register_part
from .linear import fused_layout, linear, stream_layout


class HGRN2(Mixer):
    graph_safe = True
    through_linear_only = True

    NAMES = {"q": "q_proj.weight", "f": "f_proj.weight", "f_bias": "f_proj.bias", "v": "v_proj.weight",
             "lower": "lower_bound", "norm": "g_norm.weight", "o": "o_proj.weight"}

    def __init__(self, hidden_size: int, num_heads: int, key_dim: int, value_dim: int, norm_eps: float,
                 names: Optional[Dict[str, str]] = None):
        if num_heads <= 0 or not 0 < key_dim <= 512 or value_dim <= 0:
            raise ConfigError(f"hgrn2: {num_heads} heads of {key_dim} query and {value_dim} value channels "
                              "(heads and widths must be positive, at most 512 query channels a head)")
        self.H, self.nh, self.d, self.e = int(hidden_size), int(num_heads), int(key_dim), int(value_dim)
        self.eps = float(norm_eps)
        self.names = dict(self.NAMES, **(names or {}))
        self.w_qfv = self.w_o = self.f_bias = self.lower = self.norm_w = None

    def weight_specs(self, prefix: str) -> List[TensorSpec]:
        n, hd = self.names, self.nh * self.d
        return [TensorSpec(prefix + n["q"], (hd, self.H)),
                TensorSpec(prefix + n["f"], (hd, self.H)),
                TensorSpec(prefix + n["f_bias"], (hd,), kind="vector", init="normal"),
                TensorSpec(prefix + n["lower"], (hd,), kind="vector", init="normal"),
                TensorSpec(prefix + n["v"], (self.nh * self.e, self.H)),
                TensorSpec(prefix + n["norm"], (self.e,), kind="vector", init="ones"),
                TensorSpec(prefix + n["o"], (self.H, self.nh * self.e))]

    def load(self, tensors: Dict[str, torch.Tensor], prefix: str, rt: Runtime) -> None:
        self.rt = rt
        n = self.names
        self.w_qfv = fused_layout([tensors[prefix + n[x]] for x in ("q", "f", "v")], rt)
        self.w_o = stream_layout(tensors[prefix + n["o"]], rt)
        self.f_bias = rt.own(tensors[prefix + n["f_bias"]].to(torch.float32))
        self.lower = rt.own(tensors[prefix + n["lower"]].to(torch.float32))
        self.norm_w = rt.own(tensors[prefix + n["norm"]].to(torch.float32))

    def state_need(self) -> StateNeed:
        return StateNeed((self.nh, self.d, self.e), torch.float32)

    def forward(self, h, x, step, ctx: MixerContext) -> None:
        T, nh, d, e = step.n_tokens, self.nh, self.d, self.e
        if ctx.state is None:
            raise StepError("hgrn2: the cache gave this mixer no state")
        # float sums of the three projections: the gates and the recurrence work on them unrounded
        rows = step.ws.get("glr_qfv", (T, 2 * nh * d + nh * e), torch.float32)
        linear(h, self.w_qfv, rows, step.ws)
        K.glr_gates(rows, self.f_bias, self.lower, nh * d)
        o = step.ws.get("glr_o", (T, nh * e), torch.float32)
        K.glr_scan(rows, o, ctx.state, step.cu_seqlens, step.slots, step.n_seqs, nh, d, e)
        on = step.ws.get("glr_on", (T, nh * e), self.rt.dtype)
        K.head_rmsnorm(o, self.norm_w, on, nh, e, self.eps)
        linear(on, self.w_o, x, step.ws, accumulate=True)


register_part("mixer", "hgrn2", HGRN2, replace=True)
