"""Generalized delta rule: a token mixer with a matrix state per head whose decay
is a vector (one factor per key channel) and whose removal lies along the unit
key, scaled per channel.

Per head, with S [D, Dv] (float32) carried from token to token and x the mixer's input:

    r, k = W_r x, W_k x  (D each),   v = W_v x  (Dv)
    w = exp(-c * sigmoid(W_w2 tanh(W_w1 x) + w0))      decay per key channel, in (exp(-c), 1); c = `decay_scale`
    a = sigmoid(W_a x + a_bias)                        removal rate per key channel
    u = k / sqrt(|k|^2 + key_eps)                      the unit key
    S <- diag(w) S - (a * u)(u^T S) + k v^T            (decay and removal both read the old S)
    o = S^T r

Behind it every head's o is divided by its root mean square, multiplied by a gain (one per channel of all heads) and
by sigmoid(W_g x), and projected back to the model's width.  Decay, removal rate, unit key and state are float32
whatever the runtime's dtype; the decay's logits come out of their low-rank projection in float32 as well (one
kernel: tanh, the small product and the bias).

A request's state slot holds the heads' matrices ([H][Dv][D]); the mixer has no pages.
"""
from __future__ import annotations

import math
from typing import Callable, Dict, Optional

import torch

from ..kernels import ops
from .base import MIXERS, CacheNeed, Part, Runtime, StateNeed, TensorDecl
from .linear import linear


@MIXERS.register("general_delta")
class GeneralDeltaMixer(Part):
    replayable = True       # a decoding step's launches depend on the number of entries only; the state lies in device
                            # memory and is found by the slots of the step's metadata

    def __init__(self, *, rt: Runtime, width: int, prefix: str, num_heads: int, key_dim: int, decay_rank: int, norm_eps: float,
                 value_dim: Optional[int] = None, decay_scale: float = math.exp(-0.5), key_eps: float = 1e-6,
                 shared: Optional[dict] = None, names: Optional[Dict[str, str]] = None):
        """num_heads heads with keys of key_dim and values of value_dim (default: the same); decay_rank: the size of
        the low-rank projection that the decay's logits go through; norm_eps: eps of the output's norm per head;
        decay_scale, key_eps: the constants c and key_eps above; names: tensor names behind the prefix for r, k, v, g,
        a, o, w1, w2 (matrices), a_bias, w0 (per key channel of all heads) and norm (per value channel of all heads)."""
        self.rt, self.width = rt, int(width)
        self.nh, self.d = int(num_heads), int(key_dim)
        self.dv = int(value_dim) if value_dim is not None else self.d
        self.low = int(decay_rank)
        if min(self.nh, self.d, self.dv, self.low) <= 0:
            raise ValueError("general delta rule: heads and sizes must be positive")
        if self.d > ops.DELTA_MAX_KEY_DIM:
            raise ValueError(f"key size {self.d}: the kernel takes up to {ops.DELTA_MAX_KEY_DIM}")
        self.eps, self.decay_scale, self.key_eps = float(norm_eps), float(decay_scale), float(key_eps)
        if not self.decay_scale > 0 or self.key_eps < 0:
            raise ValueError("decay_scale must be positive and key_eps not negative")
        n = {"r": "r", "k": "k", "v": "v", "g": "g", "a": "a", "o": "o", "w1": "w1", "w2": "w2", "a_bias": "a.b", "w0": "w0",
             "norm": "norm"}
        n.update(names or {})
        self.names = {k: prefix + v for k, v in n.items()}
        kd, vd = self.nh * self.d, self.nh * self.dv
        # columns of the input product: read-out vectors, keys, values, the output's gate, removal logits, the decay's
        # low-rank part
        self.col = {"r": 0, "k": kd, "v": 2 * kd, "g": 2 * kd + vd, "a": 2 * kd + 2 * vd, "w1": 3 * kd + 2 * vd}
        self.w_in = self.p_in = self.w_o = self.p_o = self.w2 = self.w0 = self.a_bias = self.norm_w = None

    def cache_need(self) -> Optional[CacheNeed]:
        return None

    def state_need(self) -> Optional[StateNeed]:
        """One float32 row per request: the heads' matrices [H][Dv][D]."""
        return StateNeed((self.nh * self.d * self.dv,), torch.float32)

    def tensors(self) -> Dict[str, TensorDecl]:
        nm, kd, vd = self.names, self.nh * self.d, self.nh * self.dv
        return {
            nm["r"]: TensorDecl((kd, self.width), "matrix"),
            nm["k"]: TensorDecl((kd, self.width), "matrix"),
            nm["v"]: TensorDecl((vd, self.width), "matrix"),
            nm["g"]: TensorDecl((vd, self.width), "matrix"),
            nm["a"]: TensorDecl((kd, self.width), "matrix"),
            nm["a_bias"]: TensorDecl((kd,), "bias"),
            nm["w1"]: TensorDecl((self.low, self.width), "matrix"),
            nm["w2"]: TensorDecl((kd, self.low), "matrix"),
            nm["w0"]: TensorDecl((kd,), "bias"),
            nm["norm"]: TensorDecl((vd,), "gain"),
            nm["o"]: TensorDecl((self.width, vd), "matrix"),
        }

    def load(self, get: Callable[[str], torch.Tensor], rt: Runtime) -> None:
        nm = self.names
        # one product for everything that reads the mixer's input
        self.w_in = torch.cat([rt.place(get(nm[k]), "matrix") for k in ("r", "k", "v", "g", "a", "w1")], dim=0).contiguous()
        self.w_o = rt.place(get(nm["o"]), "matrix")
        self.p_in, self.p_o = rt.pack(self.w_in), rt.pack(self.w_o)
        self.w_in, self.w_o = rt.row_major(self.w_in, self.p_in), rt.row_major(self.w_o, self.p_o)
        self.w2 = rt.place(get(nm["w2"]), "matrix")
        self.w0, self.a_bias = rt.place(get(nm["w0"]), "bias"), rt.place(get(nm["a_bias"]), "bias")
        self.norm_w = rt.place(get(nm["norm"]), "gain")

    def forward(self, x, ctx, cache, state):
        rt, c = self.rt, self.col
        n = x.shape[0]
        need = self.nh * self.d * self.dv
        if state is None or state.dim() != 2 or state.shape[1] != need:
            raise RuntimeError("the general delta mixer was given no state of its shape")
        y = linear(rt, x, self.w_in, None, "gdelta.in", packed=self.p_in)       # r, k, v, gate, removal logits, low-rank part
        z = ops.lowrank_tanh(y, c["w1"], self.w2, self.w0, rt.buffer("gdelta.decay", (n, self.nh * self.d), torch.float32))
        o = rt.buffer("gdelta.o", (n, self.nh * self.dv), torch.float32)
        ops.general_delta(y, c["r"], c["k"], c["v"], c["a"], z, self.a_bias, state, ctx.entry_start, ctx.state_slots, o,
                          self.nh, self.d, self.dv, self.decay_scale, self.key_eps)
        gated = rt.buffer("gdelta.gated", (n, self.nh * self.dv), rt.dtype)
        ops.gated_rmsnorm(o, self.norm_w, y, c["g"], gated, self.nh, self.dv, self.eps, gate_kind="sigmoid")
        return linear(rt, gated, self.w_o, None, "gdelta.o_proj", packed=self.p_o)
