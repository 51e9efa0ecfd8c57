"""HGRN2: linear attention whose forget gate also decides what is written.

Per token and head (d query channels, e value channels): q = silu(W_q n), v = W_v n,
f = lower + (1 - lower) * sigmoid(W_f n + b) per channel with a learnt lower bound, then
    S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T,     o_t = S_t^T q_t
(the gate acts on the rows of S that belong to q's channels; no key, no other scale).  Every
head's o is RMS-normed over its e channels with one weight shared by the heads, the heads are
concatenated and projected by W_o.

The state S [heads, d, e] starts at zero, lives in float in both precisions and is carried from
step to step in the sequence's slot of the cache's state area (`StateNeed`, laid out as the scan
kernel's lanes hold it); the gates' activations, the recurrence and the head norm are float.
Prompts are walked token by token inside one kernel, a workgroup per 16 columns of a head's state
with the state in registers and the tokens' rows staged through LDS a chunk ahead; long prompts that
would leave the chip idle are cut into pieces that are walked side by side (`pieces_for`).  The reference has no recurrent mixer of this form.
"""
from __future__ import annotations

import os
from typing import Dict, List, Optional

import torch

from .. import kernels as K
from ..cache import StateNeed
from ..errors import ConfigError, StepError
from ..weights import TensorSpec
from .base import Mixer, MixerContext, Runtime, register_part
from .linear import fused_layout, linear, stream_layout


def pieces_for(step, units_per_sequence: int, min_piece: int) -> int:
    """Into how many pieces a step's sequences are cut so that a recurrence's walk fills the chip: a workgroup walks 16
    columns of a head's state for one sequence (`units_per_sequence` of them a sequence), and a lone prompt of a small
    model has a few dozen.  One piece (the plain walk) for single tokens, short steps and batches that fill the chip."""
    if step.is_decode or step.max_new < 4 * min_piece:
        return 1
    # a workgroup is four waves, one to a SIMD, and a lone wave waits out every latency of its token loop, so
    # pieces are asked for until four workgroups share a compute unit (BRAIDINFER_GLR_FILL, for measurements;
    # a prompt of 8,192 tokens through 8 HGRN2 layers of width 2,048 / 4,096: 17.8 / 43.3 ms at 1, 13.7 / 40.2 at 2,
    # 12.9 / 38.4 at 4, 12.8 / 38.1 at 8)
    units = step.n_seqs * units_per_sequence
    want = (int(os.environ.get("BRAIDINFER_GLR_FILL", "4")) * K.device_cus()) // max(1, units)
    return max(1, min(want, step.max_new // min_piece, 16, 65535 // max(1, step.n_seqs)))


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
        return StateNeed(K.glr_state_shape(self.nh, self.d, self.e), torch.float32)

    MIN_PIECE = 128          # tokens: shorter pieces do not pay for the second walk

    def pieces_for(self, step) -> int:
        return pieces_for(step, self.nh * -(-self.e // 16), self.MIN_PIECE)

    @staticmethod
    def _piece_arrays(step, pieces: int):
        """(cuts of the packed tokens [B * pieces + 1], piece numbers [B * pieces]) on the device, made once per step
        and number of pieces: sequence b's tokens in `pieces` runs of equal length (a multiple of 16), the last ones
        shorter or empty."""
        key = ("glr_pieces", pieces)
        if key not in step.extras:
            cu, numbers, at = [0], [], 0
            for b, n in enumerate(step.host_new):
                run = -(-(-(-n // pieces)) // 16) * 16
                for c in range(pieces):
                    cu.append(at + min(n, (c + 1) * run))
                    numbers.append(b * pieces + c if step.host_slots[b] >= 0 else -1)
                at += n
            dev = torch.tensor(cu + numbers, dtype=torch.int32).to(step.tokens.device)
            step.extras[key] = (dev[:len(cu)], dev[len(cu):])
        return step.extras[key]

    def forward(self, h, x, step, ctx: MixerContext) -> None:
        T, nh, d, e = step.n_tokens, self.nh, self.d, self.e
        if ctx.state is None:
            raise StepError("hgrn2: the cache gave this mixer no state")
        # float sums of the three projections: the gates and the recurrence work on them unrounded
        rows = step.ws.get("glr_qfv", (T, 2 * nh * d + nh * e), torch.float32)
        linear(h, self.w_qfv, rows, step.ws)
        o = step.ws.get("glr_o", (T, nh * e), torch.float32)
        pieces = self.pieces_for(step)
        if pieces > 1:
            cu, numbers = self._piece_arrays(step, pieces)
            n = step.n_seqs * pieces
            piece_state = step.ws.get("glr_piece_state", (n,) + tuple(K.glr_state_shape(nh, d, e)), torch.float32)
            decay = step.ws.get("glr_decay", (n, nh, 16 * K.glr_rows_per_lane(d)), torch.float32)
            K.glr_scan_pieces(rows, self.f_bias, self.lower, o, ctx.state, step.slots, cu, numbers, piece_state, decay,
                              step.n_seqs, pieces, nh, d, e)
        else:
            K.glr_scan(rows, self.f_bias, self.lower, o, ctx.state, step.cu_seqlens, step.slots, step.n_seqs, nh, d, e)
        on = step.ws.get("glr_on", (T, nh * e), self.rt.dtype)
        K.head_rmsnorm(o, self.norm_w, on, nh, e, self.eps)
        linear(on, self.w_o, x, step.ws, accumulate=True)


register_part("mixer", "hgrn2", HGRN2, replace=True)
