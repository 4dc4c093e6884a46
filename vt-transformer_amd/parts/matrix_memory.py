"""Matrix memory (the mLSTM cell of xLSTM): a token mixer with a matrix state per
head, exponential gates and a running maximum that keeps them in range.

Per head, with S [D, Dv], a normalizer n [D] and a maximum m carried from token to token in float32 (all zero at
the start of a sequence) and x the mixer's input:

    q = W_q x * D^-1/2,  k = W_k x  (D each),   v = W_v x  (Dv)
    i = cap * tanh((W_i x + b_i) / cap)                         log of the input gate, capped
    f = logsigmoid(cap * tanh((W_f x + b_f) / cap))             log of the forget gate
    m' = max(f + m, i)
    S <- exp(f + m - m') S + exp(i - m') k v^T
    n <- exp(f + m - m') n + exp(i - m') k
    o  = S^T q / (max(|n . q|, exp(-m')) + 1e-6)

Behind it every head's o is divided by its root mean square, the concatenated heads are multiplied by a gain per
channel and by sigmoid(W_g x), and projected back to the model's width.  Gates, maximum, state and read-out are
float32 whatever the runtime's dtype.

A request's state slot holds the heads' matrices, normalizers and maxima (`ops.matrix_memory_state_floats`); the
mixer has no pages.
"""
from __future__ import annotations

from typing import Callable, Dict, Optional

import torch

from ..kernels import ops
from .base import MIXERS, CacheNeed, Part, Runtime, StateNeed, TensorDecl
from .linear import linear


@MIXERS.register("matrix_memory")
class MatrixMemoryMixer(Part):
    replayable = True       # a decoding step's launches depend on the number of entries only; the state lies in device
                            # memory and is found by the slots of the step's metadata

    def __init__(self, *, rt: Runtime, width: int, prefix: str, num_heads: int, key_dim: int, norm_eps: float,
                 value_dim: Optional[int] = None, gate_cap: float = 0.0, shared: Optional[dict] = None,
                 names: Optional[Dict[str, str]] = None):
        """num_heads heads with queries and keys of key_dim and values of value_dim (default: the same); gate_cap: the
        bound of the gates' logits (0: none); norm_eps: eps of the output's norm per head; names: tensor names behind
        the prefix for q, k, v, g, o, i, f (matrices; i and f have one row per head), i_bias, f_bias (per head) and
        norm (per value channel of all heads)."""
        self.rt, self.width = rt, int(width)
        self.nh, self.d = int(num_heads), int(key_dim)
        self.dv = int(value_dim) if value_dim is not None else self.d
        if min(self.nh, self.d, self.dv) <= 0:
            raise ValueError("matrix memory: heads and sizes must be positive")
        if self.d > ops.DELTA_MAX_KEY_DIM:
            raise ValueError(f"key size {self.d}: the kernel takes up to {ops.DELTA_MAX_KEY_DIM}")
        self.eps, self.cap = float(norm_eps), float(gate_cap)
        if self.cap < 0:
            raise ValueError("gate_cap must not be negative (0: the gates' logits are not bounded)")
        n = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "i": "i", "f": "f", "i_bias": "i.b", "f_bias": "f.b", "norm": "norm"}
        n.update(names or {})
        self.names = {k: prefix + v for k, v in n.items()}
        kd, vd = self.nh * self.d, self.nh * self.dv
        # columns of the input product: queries, keys, values, the output's gate, the two gates' logits
        self.col = {"q": 0, "k": kd, "v": 2 * kd, "g": 2 * kd + vd, "i": 2 * kd + 2 * vd, "f": 2 * kd + 2 * vd + self.nh}
        self.state_floats = ops.matrix_memory_state_floats(self.nh, self.d, self.dv)
        self.w_in = self.p_in = self.w_o = self.p_o = self.i_bias = self.f_bias = self.norm_w = None

    def cache_need(self) -> Optional[CacheNeed]:
        return None

    def state_need(self) -> Optional[StateNeed]:
        """One float32 row per request: matrices [H][Dv][D], then normalizers and maxima per block of value columns."""
        return StateNeed((self.state_floats,), torch.float32)

    def tensors(self) -> Dict[str, TensorDecl]:
        nm, kd, vd = self.names, self.nh * self.d, self.nh * self.dv
        return {
            nm["q"]: TensorDecl((kd, self.width), "matrix"),
            nm["k"]: TensorDecl((kd, self.width), "matrix"),
            nm["v"]: TensorDecl((vd, self.width), "matrix"),
            nm["g"]: TensorDecl((vd, self.width), "matrix"),
            nm["i"]: TensorDecl((self.nh, self.width), "matrix"),
            nm["f"]: TensorDecl((self.nh, self.width), "matrix"),
            nm["i_bias"]: TensorDecl((self.nh,), "bias"),
            nm["f_bias"]: TensorDecl((self.nh,), "bias"),
            nm["norm"]: TensorDecl((vd,), "gain"),
            nm["o"]: TensorDecl((self.width, vd), "matrix"),
        }

    def load(self, get: Callable[[str], torch.Tensor], rt: Runtime) -> None:
        nm = self.names
        # one product for everything that reads the mixer's input
        self.w_in = torch.cat([rt.place(get(nm[k]), "matrix") for k in ("q", "k", "v", "g", "i", "f")], dim=0).contiguous()
        self.w_o = rt.place(get(nm["o"]), "matrix")
        self.p_in, self.p_o = rt.pack(self.w_in), rt.pack(self.w_o)
        self.w_in, self.w_o = rt.row_major(self.w_in, self.p_in), rt.row_major(self.w_o, self.p_o)
        self.i_bias, self.f_bias = rt.place(get(nm["i_bias"]), "bias"), rt.place(get(nm["f_bias"]), "bias")
        self.norm_w = rt.place(get(nm["norm"]), "gain")

    def forward(self, x, ctx, cache, state):
        rt, c = self.rt, self.col
        n = x.shape[0]
        if state is None or state.dim() != 2 or state.shape[1] != self.state_floats:
            raise RuntimeError("the matrix memory mixer was given no state of its shape")
        y = linear(rt, x, self.w_in, None, "memory.in", packed=self.p_in)       # q, k, v, gate, the two gates' logits
        o = rt.buffer("memory.o", (n, self.nh * self.dv), torch.float32)
        ops.matrix_memory(y, c["q"], c["k"], c["v"], c["i"], c["f"], self.i_bias, self.f_bias, state, ctx.entry_start,
                          ctx.state_slots, o, self.nh, self.d, self.dv, self.cap, self.d ** -0.5)
        gated = rt.buffer("memory.gated", (n, self.nh * self.dv), rt.dtype)
        ops.gated_rmsnorm(o, self.norm_w, y, c["g"], gated, self.nh, self.dv, self.eps, gate_kind="sigmoid")
        return linear(rt, gated, self.w_o, None, "memory.o_proj", packed=self.p_o)
