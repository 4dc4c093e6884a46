"""Attention whose cache holds one low-rank vector and one rotated key part per
token instead of keys and values per head ("latent attention").

Per token, from the mixer's input x:

    q_h = [qn_h (plain_dim) | qr_h (rot_dim)]       = rows of W_q x, head by head
    [c_raw (rank) | kr (rot_dim)]                   = W_dkv x
    c  = c_raw / rms(c_raw) * w_norm                 (eps inside the root)
    qr_h, kr rotated by position (the leading rot.dim elements; element i with i + rot.dim/2, or with rot_pairs =
    "neighbours" element 2i with 2i + 1); kr is shared by all heads
    k_h = [W_uk,h c | kr],  v_h = W_uv,h c
    score_h(i, j) = scale * q_h(i) . k_h(j),  j seen from i  <=>  0 <= i - j < window (window 0: every j <= i)
    p = softmax over the seen keys, with exp(sink_h) added to the denominator if the mixer has sinks
    out = W_o ( concat_h(sum_j p_hj v_h(j)) * sigmoid(W_g x) )        (no gate: without the factor)

Only c and kr are cached, and k_h, v_h are never formed: since qn . (W_uk c) = (W_uk^T qn) . c and
sum_j p_j W_uv c_j = W_uv sum_j p_j c_j, the attention runs over ONE key/value head whose keys are [c | kr] and whose
values are c, with queries [W_uk,h^T qn_h | qr_h] of size rank + rot_dim, through the same kernels as
`MaskedAttention`; the two small per-head products stand in front of it and behind it (`ops.head_linear`).  A page
holds the keys as [1][slot][rank + rot_dim] and c once more transposed, [1][rank][slot], as those kernels read values.
"""
from __future__ import annotations

import math
from typing import Callable, Dict, Optional

import numpy as np
import torch

from ..config.base import PartSpec
from ..kernels import ops
from .base import MIXERS, POSITIONS, CacheNeed, PageTensor, Part, Runtime, StateNeed, TensorDecl
from .linear import can_add_residual, linear
from .masked_attention import plan_tiles, run_masked_attention


@MIXERS.register("latent_attention")
class LatentAttention(Part):
    replayable = True       # a decoding step's launches depend on the number of entries only

    def __init__(self, *, rt: Runtime, width: int, prefix: str, num_heads: int, plain_dim: int, rot_dim: int,
                 value_dim: int, rank: int, norm_eps: float, position: Optional[PartSpec] = None,
                 scale: Optional[float] = None, window: int = 0, sink: bool = False, out_gate: bool = False,
                 shared: Optional[dict] = None, names: Optional[Dict[str, str]] = None, rot_pairs: str = "halves"):
        """plain_dim / rot_dim: a query head's unrotated and rotated elements; value_dim: a head's values; rank: the
        low-rank vector's size; norm_eps: eps of its RMS norm; position: a rotary encoding of at most rot_dim
        elements (None: nothing is rotated); window: 0 or how many positions back a token sees, itself included;
        sink: a learned number per head in the softmax's denominator; out_gate: the heads' outputs times
        sigmoid(W_g x), element by element; names: tensor names behind the prefix for q, dkv, dkv_norm, uk, uv, o,
        g, sink; rot_pairs: which elements of the rotated part turn together, "halves" (i with i + dims/2) or
        "neighbours" (2i with 2i + 1).  A score is a sum over the elements of q and k alike, so neighbours are
        served by the same kernels: the rows of W_q and W_dkv that make the rotated parts are put into the
        half-split order once, when they are loaded (pair i's two elements to places i and i + dims/2)."""
        if rot_pairs not in ("halves", "neighbours"):
            raise ValueError(f"rot_pairs '{rot_pairs}' is not known ('halves' and 'neighbours' are)")
        self.rot_pairs = rot_pairs
        self.rt, self.width = rt, int(width)
        self.nh, self.dn, self.dr = int(num_heads), int(plain_dim), int(rot_dim)
        self.dv, self.rank = int(value_dim), int(rank)
        if min(self.nh, self.dn, self.dv, self.rank) <= 0 or self.dr < 0:
            raise ValueError("latent attention: heads and sizes must be positive")
        self.dk = self.rank + self.dr
        # (beyond 256 the matrix-core kernels do not take them: the kernel with a block per (token, head) does it all)
        if self.dk > ops.ATTN_MASKED_MAX_KEY_DIM or self.rank > ops.MASKED_MAX_VALUE_DIM:
            raise ValueError(f"latent attention: rank {self.rank} + {self.dr} rotated elements: the attention kernels take keys "
                             f"up to {ops.ATTN_MASKED_MAX_KEY_DIM} and values up to {ops.MASKED_MAX_VALUE_DIM}")
        self.eps = float(norm_eps)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.dn + self.dr)
        self.window = int(window)
        if self.window < 0:
            raise ValueError("window must not be negative (0: every earlier token is seen)")
        self.has_sink, self.out_gate = bool(sink), bool(out_gate)
        n = {"q": "q_proj.weight", "dkv": "kv_a_proj.weight", "dkv_norm": "kv_a_norm.weight", "uk": "k_b_proj.weight",
             "uv": "v_b_proj.weight", "o": "o_proj.weight", "g": "g_proj.weight", "sink": "sink"}
        n.update(names or {})
        self.names = {k: prefix + v for k, v in n.items()}
        pos_spec = position or PartSpec("none", {})
        shared = shared if shared is not None else {}
        key = "position:" + pos_spec.key()
        if key not in shared:
            shared[key] = POSITIONS.build(pos_spec, rt=rt)
        self.position = shared[key]
        if getattr(self.position, "dim", 0) > self.dr:
            raise ValueError(f"{self.position.dim} rotated elements in a part of {self.dr}")
        if getattr(self.position, "dim", 0) and not hasattr(self.position, "rotary_tables"):
            raise ValueError("this mixer takes rotary position encodings (or none)")
        self.w_in = self.p_in = self.w_o = self.p_o = self.w_uk = self.w_uv = self.norm_w = self.sink = None

    # columns of the input projection: the heads' queries, the low-rank part, the gate
    @property
    def _c_column(self) -> int:
        return self.nh * (self.dn + self.dr)

    @property
    def _gate_column(self) -> int:
        return self._c_column + self.dk

    def cache_need(self) -> Optional[CacheNeed]:
        return CacheNeed((PageTensor("k", (1, self.dk), slot_axis=1), PageTensor("v", (1, self.rank), slot_axis=2)),
                         window=self.window, page_multiple=16 if self._matrix_cores() else 1)

    def state_need(self) -> Optional[StateNeed]:
        return None

    def _matrix_cores(self) -> bool:
        return self.rt.lowp and ops.attention_masked_mfma_takes(self.dk, self.rank, 16)

    def prepare_step(self, ctx) -> Optional[Dict[tuple, np.ndarray]]:
        return plan_tiles(ctx) if self._matrix_cores() else None

    def tensors(self) -> Dict[str, TensorDecl]:
        nm = self.names
        t = {
            nm["q"]: TensorDecl((self.nh * (self.dn + self.dr), self.width), "matrix"),
            nm["dkv"]: TensorDecl((self.dk, self.width), "matrix"),
            nm["dkv_norm"]: TensorDecl((self.rank,), "gain"),
            nm["uk"]: TensorDecl((self.nh * self.dn, self.rank), "matrix"),
            nm["uv"]: TensorDecl((self.nh * self.dv, self.rank), "matrix"),
            nm["o"]: TensorDecl((self.width, self.nh * self.dv), "matrix"),
        }
        if self.out_gate:
            t[nm["g"]] = TensorDecl((self.nh * self.dv, self.width), "matrix")
        if self.has_sink:
            t[nm["sink"]] = TensorDecl((self.nh,), "bias")
        return t

    def load(self, get: Callable[[str], torch.Tensor], rt: Runtime) -> None:
        nm = self.names
        mats = [rt.place(get(nm[k]), "matrix") for k in (("q", "dkv", "g") if self.out_gate else ("q", "dkv"))]
        dims = int(getattr(self.position, "dim", 0))
        if self.rot_pairs == "neighbours" and dims:
            # rows of the rotated parts: pair i's elements from places 2i and 2i + 1 to places i and i + dims/2
            order = torch.cat([torch.arange(0, dims, 2), torch.arange(1, dims, 2), torch.arange(dims, self.dr)]).to(mats[0].device)
            per_head = self.dn + self.dr
            q_rows = torch.cat([torch.cat([torch.arange(self.dn, device=order.device), self.dn + order]) + h * per_head
                                for h in range(self.nh)])
            mats[0] = mats[0].index_select(0, q_rows)
            mats[1] = mats[1].index_select(0, torch.cat([torch.arange(self.rank, device=order.device), self.rank + order]))
        self.w_in = torch.cat(mats, dim=0).contiguous()
        self.w_o = rt.place(get(nm["o"]), "matrix")
        # W_uk is only ever used transposed (queries go through it, not the cache): kept as [H][rank][plain_dim], so
        # that both per-head products read a matrix row by row
        w_uk = rt.place(get(nm["uk"]), "matrix")
        self.w_uk = w_uk.view(self.nh, self.dn, self.rank).transpose(1, 2).contiguous().view(self.nh * self.rank, self.dn)
        self.w_uv = rt.place(get(nm["uv"]), "matrix")
        self.norm_w = rt.place(get(nm["dkv_norm"]), "gain")
        if self.has_sink:
            self.sink = rt.place(get(nm["sink"]), "bias")
        self.p_in, self.p_o = rt.pack(self.w_in), rt.pack(self.w_o)
        self.w_in, self.w_o = rt.row_major(self.w_in, self.p_in), rt.row_major(self.w_o, self.p_o)

    takes_normed_input = True     # the input product applies the norm in front of it when the rows are few
    hands_norm_on = True          # ... and the output product prepares the norm behind it

    def adds_residual(self, rows: int) -> bool:
        return can_add_residual(self.rt, rows, self.width, self.nh * self.dv)

    def forward(self, x, ctx, cache, state=None, residual: Optional[torch.Tensor] = None, hand_on=None):
        rt, nh, dn, dr, dv, rank, dk = self.rt, self.nh, self.dn, self.dr, self.dv, self.rank, self.dk
        n = x.shape[0]
        if not cache.writes:
            raise RuntimeError("this mixer does not read another layer's cache")
        y = linear(rt, x, self.w_in, None, "lattn.in", packed=self.p_in)
        tables = self.position.rotary_tables(ctx.n_positions) if getattr(self.position, "dim", 0) else None
        cos, sin = tables if tables is not None else (None, None)
        q = rt.buffer("lattn.q", (n, nh * dk), rt.dtype)
        ops.latent_prepare(y, 0, self._c_column, self.norm_w, self.eps, cos, sin, ctx.positions, ctx.tok_entry,
                           cache.block_table, q, cache["k"], cache["v"], nh, dn, dr, rank)
        # the unrotated query parts through W_uk^T, into the query rows in front of the rotated parts
        ops.head_linear(y, 0, dn + dr, self.w_uk, False, q, 0, dk, nh, dn, rank)
        mixed = rt.buffer("lattn.mixed", (n, nh * rank), rt.dtype)
        run_masked_attention(rt, ctx, cache, q, mixed, nh, 1, dk, rank, self.scale, window=self.window, sink=self.sink)
        # the heads' mixed low-rank vectors through W_uv, times the gate
        out = rt.buffer("lattn.out", (n, nh * dv), rt.dtype)
        ops.head_linear(mixed, 0, rank, self.w_uv, False, out, 0, dv, nh, rank, dv,
                        gate=y if self.out_gate else None, gate_column=self._gate_column)
        return linear(rt, out, self.w_o, None, "lattn.o", packed=self.p_o, residual=residual, hand_on=hand_on)
