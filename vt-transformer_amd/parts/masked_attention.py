"""Attention mixer for heads that `PagedAttention`'s kernels do not take: keys
and values of different sizes, rotation of part of the head, queries and
keys scaled to unit root mean square, queries that grow with the logarithm of
the position, scores capped by a tanh or lowered by a slope times the
distance, keys masked by a window or by chunks of positions, a learned sink in
the softmax's denominator, values mixed with those of an earlier layer, and
one sigmoid gate per head (or per element) on the output, a gain on the
unit-RMS queries and keys, a bias that grows with the logarithm of the
distance, a learned shift of every score per head, weights that are sigmoids of
the scores instead of a softmax, neighbouring elements rotated together, a bias
on the output projection.  Every one of these is a constructor parameter that
can be left out.

Per token: q, k, v (and the gates' logits) in one matrix product with the
biases; rotation, unit scaling and the write into the pages in one kernel;
scores, cap, mask, float32 softmax, weighted sum and gate in one kernel that
reads the pages; output projection.

    q_i = temp(i) * (W_q x_i),  temp(i) = 1 + coef * ln(floor((i + 1) / every) + 1)           (no q_temp: 1)
    score(i, j) = cap * tanh(scale * q_i . k_j / cap) - slope_h * (i - j)                     (cap 0: scale * q_i . k_j)
    slope_h = 2^(-distance_slopes * (h + 1) / H)                                              (no distance_slopes: 0)
    j is seen from i  <=>  j <= i,  i - j < window (if window > 0),  floor(j / chunk) = floor(i / chunk) (if chunk > 0)
    p_ij = exp(score(i, j)) / (sum_j' exp(score(i, j')) + exp(sink_h))                        (no sink: the plain softmax)
    out_i[h] = sigmoid(gate_i[h]) * sum_j p_ij v_j

    distance_log:  score(i, j) -= r1_h * ln(1 + r2_h * (i - j))        r1, r2 learned, one each per head
    score_shift:   score(i, j) += shift_h                              learned, one per head
    weights "sigmoid":  p_ij = sigmoid(score(i, j)) for every seen j, not normalized (no sink)
    out_gate:      out_i[h][d] *= sigmoid((W_g x_i)[h][d])             one logit per output element instead of per head
    qk_gain:       after the unit-RMS scaling q and k are multiplied by a learned gain per element (shared by heads)

Value mixing ties layers together: the first layer of a model that says value_mix="source" leaves the step's values
in a buffer, and every layer that says value_mix="mix" keeps (1 - lambda) v + lambda v_source in its pages instead
of its own v, with lambda a learned number of its own.

Chunks are counted from position 0 of the sequence.  A key that no later
position can see is dead for the cache manager: the pages' window is the
mask's reach.
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


TILE_ROWS = 16
TILES_KEY = ("masked_attention.tiles", TILE_ROWS)


def plan_tiles(ctx) -> Optional[Dict[tuple, np.ndarray]]:
    """The work of `ops.attention_masked_mfma` for a step that brings more than single tokens: runs of up to 16
    consecutive tokens of one request, (first row, rows).  One list serves every layer whose mixer goes through that
    kernel; it is found as ctx.extra[TILES_KEY]."""
    if ctx.single_token or TILES_KEY in ctx.extra_host:
        return None
    start = np.asarray(ctx.h_entry_start, dtype=np.int64)
    tiles = []
    for e in range(len(start) - 1):
        for first in range(int(start[e]), int(start[e + 1]), TILE_ROWS):
            tiles.append((first, min(TILE_ROWS, int(start[e + 1]) - first)))
    return {TILES_KEY: np.asarray(tiles, dtype=np.int32).reshape(-1)}


def run_masked_attention(rt: Runtime, ctx, cache, q: torch.Tensor, out: torch.Tensor, nh: int, nkv: int, d: int, dv: int,
                         scale: float, softcap: float = 0.0, window: int = 0, chunk: int = 0, gate=None,
                         gate_column: int = 0, sink=None, slopes=None, dist_log=None, score_shift=None,
                         sigmoid_weights: bool = False, gate_wide: bool = False) -> torch.Tensor:
    """The attention itself over a layer's pages, by the kernel that suits the step: in the 16-bit types with heads
    in multiples of 16, steps of single tokens go to the matrix-core kernel whose rows are the heads of a key/value
    group and whose keys are dealt out to many waves, steps with portions of prompts to the one whose rows are tokens
    (tiles planned by `plan_tiles`); everything else, and float32 always, to the kernel with a block per (token, head)."""
    cores = rt.lowp and ops.attention_masked_mfma_takes(d, dv, cache["k"].shape[2])
    kw = dict(gate=gate, gate_column=gate_column, sink=sink, slopes=slopes, dist_log=dist_log, score_shift=score_shift,
              sigmoid_weights=sigmoid_weights, gate_wide=gate_wide)
    if cores and ctx.single_token:
        n = q.shape[0]
        splits = ops.attention_masked_decode_splits(n, nh, nkv, ctx.n_positions)
        part = rt.buffer("mattn.decode_parts", (ops.attention_masked_decode_scratch(n, nh, nkv, dv, splits),), torch.float32)
        return ops.attention_masked_decode(q, cache["k"], cache["v"], ctx.positions, ctx.tok_entry, cache.block_table, out,
                                           part, splits, nh, nkv, d, dv, scale, softcap, window, chunk, **kw)
    tiles = ctx.extra.get(TILES_KEY) if cores and not ctx.single_token else None
    if tiles is not None:
        return ops.attention_masked_mfma(q, cache["k"], cache["v"], ctx.positions, ctx.tok_entry, cache.block_table, tiles,
                                         out, nh, nkv, d, dv, scale, softcap, window, chunk, **kw)
    return ops.attention_masked(q, cache["k"], cache["v"], ctx.positions, ctx.tok_entry, cache.block_table, out, nh, nkv,
                                d, dv, scale, softcap, window, chunk, **kw)


def head_slopes(n_heads: int, steepness: float) -> np.ndarray:
    """slope_h = 2^(-steepness (h + 1) / H), float32."""
    return np.power(2.0, -float(steepness) * (np.arange(n_heads, dtype=np.float64) + 1.0) / n_heads).astype(np.float32)


@MIXERS.register("masked_attention")
class MaskedAttention(Part):
    replayable = True       # a decoding step's launches depend on the number of entries only

    def __init__(self, *, rt: Runtime, width: int, prefix: str, num_heads: int, num_kv_heads: int, key_dim: int,
                 value_dim: Optional[int] = None, qkv_bias: bool = False, position: Optional[PartSpec] = None,
                 scale: Optional[float] = None, softcap: float = 0.0, window: int = 0, chunk: int = 0,
                 unit_rms_eps: Optional[float] = None, head_gate: bool = False, shared: Optional[dict] = None,
                 names: Optional[Dict[str, str]] = None, sink: bool = False, distance_slopes: Optional[float] = None,
                 q_temp: Optional[Dict[str, float]] = None, value_mix: Optional[str] = None, fuse_norms: bool = False,
                 rot_pairs: str = "halves", qk_gain: bool = False, distance_log: bool = False, score_shift: bool = False,
                 weights: str = "softmax", out_gate: bool = False, o_bias: bool = False):
        """key_dim / value_dim: sizes of a head's queries and keys / of its values (default: the same);
        position: a rotary encoding whose `dim` may be smaller than key_dim (the rest of a head passes unchanged);
        unit_rms_eps: queries and keys are divided by their root mean square per head after the rotation, with
        this eps inside the root (None: they are not); head_gate: one sigmoid gate per head from a projection of
        the mixer's input; names: tensor names behind the prefix for q, k, v, o, g, sink, vmix and the biases q_bias,
        k_bias, v_bias; sink: one learned number per head whose exponential joins the softmax's denominator;
        distance_slopes: s > 0 takes 2^(-s (h + 1) / H) times the distance off head h's scores; q_temp {coef, every}:
        the queries' factor by position; value_mix: "source" (this layer's values are what later layers mix in),
        "mix" (this layer keeps (1 - lambda) v + lambda v_source, lambda its tensor `vmix`), "off" (neither, in a
        model whose checkpoints may hold a `vmix` for such a layer all the same: it is tolerated and not read) or
        None; fuse_norms: with
        few rows in bfloat16 the input product applies the norm in front of the mixer and the output product adds to
        the residual stream and prepares the norm behind (as `PagedAttention` does; it rounds the stream times the
        norm's gains to 16 bits before the division by the root instead of after it);
        rot_pairs: "halves" (element i turns with element i + dims/2) or "neighbours" (element 2i with 2i + 1: the
        rows of W_q and W_k and their biases are reordered when they are loaded, after which the kernels' half-split
        rotation is the neighbouring one, and a score, a sum over the elements of q and k alike, does not see the
        order); qk_gain (with unit_rms_eps): tensors q_norm, k_norm [key_dim]; distance_log: tensors r1, r2 [heads];
        score_shift: tensor shift [heads]; weights: "softmax" or "sigmoid"; out_gate: an elementwise sigmoid gate from
        a projection g [heads * value_dim, width] (head_gate's tensor name; not both); o_bias: tensor o_bias [width]."""
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads are not a multiple of {num_kv_heads} key/value heads")
        self.rt, self.width = rt, int(width)
        self.nh, self.nkv, self.d = int(num_heads), int(num_kv_heads), int(key_dim)
        self.dv = int(value_dim) if value_dim is not None else self.d
        if not 1 <= self.d <= ops.MASKED_MAX_KEY_DIM or not 1 <= self.dv <= ops.MASKED_MAX_VALUE_DIM:
            raise ValueError(f"head sizes {self.d}/{self.dv}: the kernels take keys up to {ops.MASKED_MAX_KEY_DIM} and "
                             f"values up to {ops.MASKED_MAX_VALUE_DIM}")
        self.qkv_bias, self.head_gate = bool(qkv_bias), bool(head_gate)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.d)
        self.softcap, self.window, self.chunk = float(softcap), int(window), int(chunk)
        if self.softcap < 0 or self.window < 0 or self.chunk < 0:
            raise ValueError("softcap, window and chunk must not be negative (0 switches each off)")
        self.unit_rms_eps = None if unit_rms_eps is None else float(unit_rms_eps)
        self.has_sink = bool(sink)
        self.distance_slopes = None if not distance_slopes else float(distance_slopes)
        if self.distance_slopes is not None and self.distance_slopes < 0:
            raise ValueError("distance_slopes must be positive (None switches the slopes off)")
        self.q_temp = None
        if q_temp:
            self.q_temp = (float(q_temp["coef"]), int(q_temp["every"]))
            if self.q_temp[1] <= 0:
                raise ValueError(f"q_temp.every {self.q_temp[1]} must be positive")
        if value_mix not in (None, "off", "source", "mix"):
            raise ValueError(f"value_mix {value_mix!r} ('source', 'mix', 'off' or None)")
        self.value_mix = value_mix
        if rot_pairs not in ("halves", "neighbours"):
            raise ValueError(f"rot_pairs {rot_pairs!r} ('halves' or 'neighbours')")
        if weights not in ("softmax", "sigmoid"):
            raise ValueError(f"weights {weights!r} ('softmax' or 'sigmoid')")
        self.rot_pairs, self.sigmoid_weights = rot_pairs, weights == "sigmoid"
        self.qk_gain, self.distance_log, self.score_shift = bool(qk_gain), bool(distance_log), bool(score_shift)
        self.out_gate, self.o_bias = bool(out_gate), bool(o_bias)
        if self.qk_gain and self.unit_rms_eps is None:
            raise ValueError("qk_gain is a gain on unit-RMS queries and keys: give unit_rms_eps")
        if self.qk_gain and rot_pairs == "neighbours" and position is not None:
            raise ValueError("a gain per element and reordered rotated elements are not combined")
        if self.out_gate and self.head_gate:
            raise ValueError("one gate on the output: per head or per element")
        if self.sigmoid_weights and self.has_sink:
            raise ValueError("sigmoid weights have no denominator for a sink to join")
        # what the block asks for (parts/block.py)
        self.takes_normed_input = self.hands_norm_on = bool(fuse_norms)
        n = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight", "g": "g_proj.weight",
             "q_bias": "q_proj.bias", "k_bias": "k_proj.bias", "v_bias": "v_proj.bias", "sink": "sink", "vmix": "vmix",
             "q_norm": "q_norm.weight", "k_norm": "k_norm.weight", "r1": "r1", "r2": "r2", "shift": "shift",
             "o_bias": "o_proj.bias"}
        n.update(names or {})
        self.names = {k: prefix + v for k, v in n.items()}
        pos_spec = position or PartSpec("none", {})
        shared = shared if shared is not None else {}
        key = "position:" + pos_spec.key()
        if key not in shared:
            shared[key] = POSITIONS.build(pos_spec, rt=rt)
        self.position = shared[key]
        if getattr(self.position, "dim", 0) > self.d:
            raise ValueError(f"{self.position.dim} rotated elements in heads of {self.d}")
        if getattr(self.position, "dim", 0) and not hasattr(self.position, "rotary_tables"):
            raise ValueError("this mixer takes rotary position encodings (or none)")
        self.w_in = self.b_in = self.b_in_lowp = self.p_in = self.w_o = self.p_o = None
        self.sink = self.slopes = self.v_lambda = None
        self.q_gain = self.k_gain = self.r1 = self.r2 = self.shift = self.b_o = self.b_o_lowp = None

    # columns of the input projection: queries, keys, values, gates
    @property
    def _gate_column(self) -> int:
        return (self.nh + self.nkv) * self.d + self.nkv * self.dv

    def cache_need(self) -> Optional[CacheNeed]:
        """Keys [kv head][slot][D] and values transposed, [kv head][Dv][slot] (the matrix-core kernel reads four keys of
        one value element with one load), in the runtime's dtype.  The mask's reach bounds how long a key lives: with
        chunks, a key is never seen from `chunk` or more positions later."""
        reach = [w for w in (self.window, self.chunk) if w > 0]
        return CacheNeed((PageTensor("k", (self.nkv, self.d), slot_axis=1), PageTensor("v", (self.nkv, self.dv), slot_axis=2)),
                         window=min(reach) if reach else 0, page_multiple=16 if self._matrix_cores() else 1)

    def _matrix_cores(self) -> bool:
        """Whether portions of prompts go to the matrix-core kernel: a 16-bit runtime and heads in multiples of 16."""
        return self.rt.lowp and ops.attention_masked_mfma_takes(self.d, self.dv, 16)

    TILE_ROWS = TILE_ROWS

    def prepare_step(self, ctx) -> Optional[Dict[tuple, np.ndarray]]:
        """The matrix-core kernel's work for a step that brings more than single tokens (`plan_tiles`)."""
        if not self._matrix_cores():
            return None
        return plan_tiles(ctx)

    def state_need(self) -> Optional[StateNeed]:
        return None

    def tensors(self) -> Dict[str, TensorDecl]:
        nm = self.names
        t = {
            nm["q"]: TensorDecl((self.nh * self.d, self.width), "matrix"),
            nm["k"]: TensorDecl((self.nkv * self.d, self.width), "matrix"),
            nm["v"]: TensorDecl((self.nkv * self.dv, self.width), "matrix"),
            nm["o"]: TensorDecl((self.width, self.nh * self.dv), "matrix"),
        }
        if self.qkv_bias:
            t[nm["q_bias"]] = TensorDecl((self.nh * self.d,), "bias")
            t[nm["k_bias"]] = TensorDecl((self.nkv * self.d,), "bias")
            t[nm["v_bias"]] = TensorDecl((self.nkv * self.dv,), "bias")
        if self.head_gate:
            t[nm["g"]] = TensorDecl((self.nh, self.width), "matrix")
        if self.out_gate:
            t[nm["g"]] = TensorDecl((self.nh * self.dv, self.width), "matrix")
        if self.qk_gain:
            t[nm["q_norm"]] = TensorDecl((self.d,), "gain")
            t[nm["k_norm"]] = TensorDecl((self.d,), "gain")
        if self.distance_log:
            t[nm["r1"]] = TensorDecl((self.nh,), "bias")
            # (r2 multiplies the distance inside the logarithm: a model with random weights draws it around 1)
            t[nm["r2"]] = TensorDecl((self.nh,), "gain")
        if self.score_shift:
            t[nm["shift"]] = TensorDecl((self.nh,), "bias")
        if self.o_bias:
            t[nm["o_bias"]] = TensorDecl((self.width,), "bias")
        if self.has_sink:
            t[nm["sink"]] = TensorDecl((self.nh,), "bias")
        if self.value_mix is not None:
            # (the source layer's number is part of the checkpoint and is not used)
            t[nm["vmix"]] = TensorDecl((), "bias", optional=self.value_mix != "mix")
        return t

    def _pair_order(self, t: torch.Tensor, heads: int) -> torch.Tensor:
        """Rows (or elements) of the heads of a query or key projection in the order in which the kernels' half-split
        rotation is the neighbouring one: of a head's first `dims` elements, element 2i goes to place i and element
        2i + 1 to place i + dims/2."""
        dims = int(getattr(self.position, "dim", 0))
        if self.rot_pairs != "neighbours" or dims == 0:
            return t
        order = torch.cat([torch.arange(0, dims, 2), torch.arange(1, dims, 2), torch.arange(dims, self.d)])
        index = (torch.arange(heads)[:, None] * self.d + order[None, :]).reshape(-1).to(t.device)
        return t.index_select(0, index)

    def load(self, get: Callable[[str], torch.Tensor], rt: Runtime) -> None:
        nm = self.names
        gated = self.head_gate or self.out_gate
        mats = [rt.place(get(nm[k]), "matrix") for k in (("q", "k", "v", "g") if gated else ("q", "k", "v"))]
        mats[0], mats[1] = self._pair_order(mats[0], self.nh), self._pair_order(mats[1], self.nkv)
        self.w_in = torch.cat(mats, dim=0).contiguous()
        if self.qkv_bias:
            b = [rt.place(get(nm[k]), "bias") for k in ("q_bias", "k_bias", "v_bias")]
            b[0], b[1] = self._pair_order(b[0], self.nh), self._pair_order(b[1], self.nkv)
            if gated:
                b.append(torch.zeros(mats[3].shape[0], dtype=torch.float32, device=rt.device))
            self.b_in = torch.cat(b, dim=0).contiguous()
            self.b_in_lowp = self.b_in.to(rt.dtype)
        if self.qk_gain:
            self.q_gain, self.k_gain = rt.place(get(nm["q_norm"]), "gain"), rt.place(get(nm["k_norm"]), "gain")
        if self.distance_log:
            self.r1, self.r2 = rt.place(get(nm["r1"]), "bias"), rt.place(get(nm["r2"]), "gain")
        if self.score_shift:
            self.shift = rt.place(get(nm["shift"]), "bias")
        if self.o_bias:
            self.b_o = rt.place(get(nm["o_bias"]), "bias")
            self.b_o_lowp = self.b_o.to(rt.dtype)
        self.w_o = rt.place(get(nm["o"]), "matrix")
        if self.has_sink:
            self.sink = rt.place(get(nm["sink"]), "bias")
        if self.distance_slopes is not None:
            self.slopes = torch.from_numpy(head_slopes(self.nh, self.distance_slopes)).to(rt.device)
        if self.value_mix == "mix":
            self.v_lambda = rt.place(get(nm["vmix"]), "bias").reshape(1)
        self.p_in, self.p_o = rt.pack(self.w_in), rt.pack(self.w_o)
        self.w_in, self.w_o = rt.row_major(self.w_in, self.p_in), rt.row_major(self.w_o, self.p_o)

    def adds_residual(self, rows: int) -> bool:
        """Whether the output product adds to the residual stream itself at this many rows."""
        return self.takes_normed_input and can_add_residual(self.rt, rows, self.width, self.nh * self.dv)

    def forward(self, x, ctx, cache, state=None, residual: Optional[torch.Tensor] = None, hand_on=None):
        rt, nh, nkv, d, dv = self.rt, self.nh, self.nkv, self.d, self.dv
        n = x.shape[0]
        if not cache.writes:
            raise RuntimeError("this mixer does not read another layer's keys and values")
        y = linear(rt, x, self.w_in, self.b_in, "mattn.in", bias_lowp=self.b_in_lowp, packed=self.p_in)
        tables = self.position.rotary_tables(ctx.n_positions) if getattr(self.position, "dim", 0) else None
        cos, sin = tables if tables is not None else (None, None)
        q = rt.buffer("mattn.q", (n, nh * d), rt.dtype)
        # the values that layers mix: one buffer per model and step, written by the source layer, read by the others
        v_first = rt.buffer("mattn.v_first", (n, nkv * dv), torch.float32) if self.value_mix in ("source", "mix") else None
        ops.qk_prepare(y, cos, sin, ctx.positions, ctx.tok_entry, cache.block_table, q, cache["k"], cache["v"], nh, nkv,
                       d, dv, self.unit_rms_eps, q_temp=self.q_temp, v_first=v_first, v_lambda=self.v_lambda,
                       q_gain=self.q_gain, k_gain=self.k_gain)
        out = rt.buffer("mattn.out", (n, nh * dv), rt.dtype)
        run_masked_attention(rt, ctx, cache, q, out, nh, nkv, d, dv, self.scale, self.softcap, self.window, self.chunk,
                             gate=y if (self.head_gate or self.out_gate) else None, gate_column=self._gate_column,
                             sink=self.sink, slopes=self.slopes, dist_log=(self.r1, self.r2) if self.distance_log else None,
                             score_shift=self.shift, sigmoid_weights=self.sigmoid_weights, gate_wide=self.out_gate)
        return linear(rt, out, self.w_o, self.b_o, "mattn.o", bias_lowp=self.b_o_lowp, packed=self.p_o, residual=residual,
                      hand_on=hand_on)
