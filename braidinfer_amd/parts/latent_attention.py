"""Attention through a latent: queries and keys/values each pass a narrow normed projection, and the cache
keeps per token only the key/value latent and one rotated key part shared by all heads.

Per token, with n the mixer's input: c_q = rms_norm(W_dq n) * g_q and q = W_uq c_q, laid out head by head as
[`dim` plain | `rot_dim` rotated] elements; W_dkv n has `kv_rank` + `rot_dim` rows, of which the first `kv_rank`,
normed (c = rms_norm(.) * g_kv), are the latent and the last `rot_dim`, rotated, are the key part k_r that every
head shares.  A head's key is [W_uk c | k_r] and its value W_uv c; scores are (q_plain . k_plain + q_rot . k_rot) *
scale over all tokens up to the query's own, in a softmax whose denominator may also hold exp(sink_h), a learnt
score per head with no value.  The heads' outputs, concatenated, go through W_o.

The cache row of a token is [c | k_r] (after norm and rotation); keys and values are never expanded.  Since
q_plain . (W_uk c) = (W_uk^T q_plain) . c and sum_j p_j W_uv c_j = W_uv sum_j p_j c_j, the step takes every head's
plain query part through W_uk^T, runs attention of all heads over the one row per token (keys `kv_rank` +
`rot_dim` wide, values the first `kv_rank` of the same row) and takes the result through W_uv: the work per cached
token does not grow with `dim` or the number of key heads, and a step reads the cache once for all heads.

A layer may read the rows another layer keeps (`own_rows=False`): it has no W_dkv and no norm weight of its
own; its run-order entry names that layer's cache unit with `writes_cache=False`.

Rotation is the position encoding the mixer names (pairs of neighbouring elements); norms, angles, scores and
softmax are float in both precisions, the three narrow products leave float sums.  The attention kernels are
those of `pooled_window_attention` with one kv head, no window and no pooled blocks, which want a page's
values transposed: a page keeps the latent twice, once in the key rows and once transposed.  The reference's
attention keeps full keys and values per kv head (kernels/megakernel_ops.hip:2150-2343).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import kernels as K
from ..cache import CacheNeed
from ..errors import ConfigError, StepError
from ..weights import TensorSpec
from .base import Mixer, MixerContext, RotaryTables, Runtime, register_part
from .linear import linear, stream_layout

NO_WINDOW = 1 << 30       # a window no sequence reaches: the attention kernels then see every earlier token
MAX_WIDTH = 512           # of a cache row's key part or latent: the attention kernels' limit


class LatentAttention(Mixer):
    graph_safe = True

    NAMES = {"dq": "dq", "dq_norm": "dq.norm", "uq": "uq", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk", "uv": "uv",
             "sink": "sink", "o": "o"}

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, rot_dim: int, value_dim: int, q_rank: int,
                 kv_rank: int, scale: float, norm_eps: float, position: Optional[str] = None, sink: bool = True,
                 own_rows: bool = True, names: Optional[Dict[str, str]] = None):
        if min(num_heads, head_dim, value_dim, q_rank, kv_rank) <= 0 or rot_dim < 0:
            raise ConfigError(f"latent attention: heads {num_heads}, widths {head_dim} + {rot_dim} and {value_dim}, ranks "
                              f"{q_rank} and {kv_rank} must be positive (the rotated part may be empty)")
        if kv_rank + rot_dim > MAX_WIDTH:
            raise ConfigError(f"latent attention: a cache row of {kv_rank} + {rot_dim} elements is beyond the attention "
                              f"kernels' {MAX_WIDTH}")
        self.H, self.nh, self.d, self.dr, self.e = int(hidden_size), int(num_heads), int(head_dim), int(rot_dim), int(value_dim)
        self.qr, self.r = int(q_rank), int(kv_rank)
        self.scale, self.eps = float(scale), float(norm_eps)
        self.position, self.sink, self.own_rows = position, bool(sink), bool(own_rows)
        self.names = dict(self.NAMES, **(names or {}))
        self.w_dq = self.w_dkv = self.w_uq = self.w_uk_t = self.w_uv = self.w_o = None
        self.q_norm_w = self.c_norm_w = self.sinks = None
        self.rot = 0
        self.force_simple = False          # tests set it to run the float kernel in bfloat16 too
        self._blocks = {}

    # ---- weights -----------------------------------------------------------------------
    def weight_specs(self, prefix: str) -> List[TensorSpec]:
        n = self.names
        out = [TensorSpec(prefix + n["dq"], (self.qr, self.H)),
               TensorSpec(prefix + n["dq_norm"], (self.qr,), kind="vector", init="ones"),
               TensorSpec(prefix + n["uq"], (self.nh * (self.d + self.dr), self.qr))]
        if self.own_rows:
            out += [TensorSpec(prefix + n["dkv"], (self.r + self.dr, self.H)),
                    TensorSpec(prefix + n["dkv_norm"], (self.r,), kind="vector", init="ones")]
        out += [TensorSpec(prefix + n["uk"], (self.nh * self.d, self.r)),
                TensorSpec(prefix + n["uv"], (self.nh * self.e, self.r))]
        if self.sink:
            out.append(TensorSpec(prefix + n["sink"], (self.nh,), kind="vector", init="normal"))
        out.append(TensorSpec(prefix + n["o"], (self.H, self.nh * self.e)))
        return out

    def load(self, tensors: Dict[str, torch.Tensor], prefix: str, rt: Runtime) -> None:
        self.rt = rt
        n = self.names
        self.w_dq = stream_layout(tensors[prefix + n["dq"]], rt)
        self.w_dkv = stream_layout(tensors[prefix + n["dkv"]], rt) if self.own_rows else None
        self.w_uq = stream_layout(tensors[prefix + n["uq"]], rt)
        # W_uk head by head, transposed: [heads, kv_rank, dim], the matrices that take a plain query part to the latent
        uk = tensors[prefix + n["uk"]]
        uk_t = rt.empty((self.nh, self.r, self.d), uk.dtype)
        uk_t.copy_(uk.reshape(self.nh, self.d, self.r).transpose(1, 2))
        self.w_uk_t = uk_t
        self.w_uv = rt.own(tensors[prefix + n["uv"]]).view(self.nh, self.e, self.r)
        self.w_o = stream_layout(tensors[prefix + n["o"]], rt)
        self.q_norm_w = rt.own(tensors[prefix + n["dq_norm"]].to(torch.float32))
        if self.own_rows:
            self.c_norm_w = rt.own(tensors[prefix + n["dkv_norm"]].to(torch.float32))
        if self.sink:
            self.sinks = rt.own(tensors[prefix + n["sink"]].to(torch.float32).reshape(-1))

    # ---- what it keeps -----------------------------------------------------------------
    def cache_need(self) -> CacheNeed:
        return CacheNeed(kv_heads=1, head_dim=self.r + self.dr, value_dim=self.r)

    def check_positions(self, encodings) -> None:
        if self.position is None:
            return
        enc = encodings.get(self.position)
        if enc is None:
            raise ConfigError(f"latent attention asks for the position encoding {self.position!r}, the model has {sorted(encodings)}")
        if getattr(enc, "gives", None) != "rotary" or getattr(enc, "pairing", None) != "adjacent" or enc.rotary_dim > self.dr:
            raise ConfigError(f"latent attention rotates up to {self.dr} elements in pairs of neighbours; the encoding "
                              f"{self.position!r} gives {getattr(enc, 'gives', None)!r} over {getattr(enc, 'rotary_dim', None)} "
                              f"elements in {getattr(enc, 'pairing', None)!r} pairs")
        self.rot = int(enc.rotary_dim)

    # ---- one step ----------------------------------------------------------------------
    def forward(self, h, x, step, ctx: MixerContext) -> None:
        T, nh, d, dr, e, r, qr = step.n_tokens, self.nh, self.d, self.dr, self.e, self.r, self.qr
        dt = self.rt.dtype
        tables = step.position_data.get(self.position) if self.position else None
        if self.rot and not isinstance(tables, RotaryTables):
            raise StepError(f"latent attention: the position encoding {self.position!r} gave {type(tables).__name__}, "
                            "rotary tables were expected")
        if ctx.keys is None or ctx.block_table is None:
            raise StepError("latent attention: the run order gave this mixer no cache unit")
        if self.own_rows != bool(ctx.writes_cache):
            raise StepError("latent attention: a layer with rows of its own writes its cache unit, one without reads another's")
        wide = r + dr
        # the narrow projections' float sums: the query latent, and [latent | key part] where the layer keeps rows
        cq_raw = step.ws.get("la_cq_raw", (T, qr), torch.float32)
        linear(h, self.w_dq, cq_raw, step.ws)
        dkv = None
        if self.own_rows:
            dkv = step.ws.get("la_dkv", (T, wide), torch.float32)
            linear(h, self.w_dkv, dkv, step.ws)
        cq = step.ws.get("la_cq", (T, qr), dt)
        K.rmsnorm(cq_raw, self.q_norm_w, cq, self.eps)
        q = step.ws.get("la_q", (T, nh * (d + dr)), torch.float32)
        linear(cq, self.w_uq, q, step.ws)
        q_plain = step.ws.get("la_q_plain", (T, nh * d), dt)
        q_wide = step.ws.get("la_q_wide", (T, nh * wide), dt)
        unit = self._unit(ctx)
        K.latent_prepare(q, dkv, self.c_norm_w, self.eps,
                         tables.cos if self.rot else None, tables.sin if self.rot else None, self.rot,
                         step.positions, step.seq_of_token, step.slots, ctx.block_table, unit if self.own_rows else None,
                         q_plain, q_wide, nh, d, dr, r, ctx.page_tokens)
        # every head's plain part through its W_uk^T into the first kv_rank elements of its wide query
        K.head_linear(q_plain.view(T, nh, d), self.w_uk_t, q_wide.view(T, nh, wide)[:, :, :r])
        o_lat = step.ws.get("la_o_lat", (T, nh * r), dt)
        sinks = self.sinks if self.sink else None
        if not step.is_decode and not self.force_simple and K.pwa_prefill_takes(dt, wide, r, ctx.page_tokens):
            K.pwa_prefill_bf16(q_wide, o_lat, step.cu_seqlens, step.slots, step.ctx_lens, ctx.block_table, unit, None, None,
                               step.n_seqs, step.max_new, nh, 1, wide, r, ctx.page_tokens, NO_WINDOW, 0, self.scale, self.sink, sinks)
        elif step.is_decode and not self.force_simple and self._decode_blocks(dt, ctx.page_tokens):
            # all heads read the one row a token: dealt to as few workgroups a sequence as the kernel's merge allows
            K.pwa_decode_bf16(q_wide, o_lat, step.slots, step.ctx_lens, ctx.block_table, unit, None, None, step.n_seqs,
                              nh, self._decode_blocks(dt, ctx.page_tokens), wide, r, ctx.page_tokens, NO_WINDOW, 0, self.scale,
                              self.sink, sinks, cache_heads=1)
        else:
            K.pwa_attend(q_wide, o_lat, step.positions, step.seq_of_token, step.slots, ctx.block_table, unit, None, None,
                         nh, 1, wide, r, ctx.page_tokens, NO_WINDOW, 0, self.scale, self.sink, sinks)
        # and every head's mixed latent through its W_uv
        o = step.ws.get("la_o", (T, nh * e), dt)
        K.head_linear(o_lat.view(T, nh, r), self.w_uv, o.view(T, nh, e))
        linear(o, self.w_o, x, step.ws, accumulate=True)

    def _decode_blocks(self, dt, page: int) -> int:
        """Into how many blocks of heads the single-token kernel takes this mixer's heads (0: it does not)."""
        key = (dt, page)
        if key not in self._blocks:
            self._blocks[key] = next((b for b in range(1, self.nh + 1)
                                      if self.nh % b == 0 and K.pwa_decode_takes(dt, self.nh, b, self.r + self.dr, self.r, page)), 0)
        return self._blocks[key]

    @staticmethod
    def _unit(ctx: MixerContext) -> torch.Tensor:
        """The cache unit as the kernels take it: [pages, elements of a page]."""
        s = ctx.storage
        return s if s.dim() == 2 else s.reshape(s.shape[0], -1)


register_part("mixer", "latent_attention", LatentAttention, replace=True)
