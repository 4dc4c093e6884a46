"""Gated delta rule: a token mixer with a matrix state per head instead of a
cache of keys and values.

For every value head the mixer carries S [D, Dv] (float32) from token to token:

    S <- g S                      decay, g = exp(-exp(A_log) * softplus(a + dt_bias)) in (0, 1)
    u  = beta (v - S^T k)         what the state gets wrong about this key, times beta = sigmoid(b)
    S <- S + k u^T                corrected towards v
    o  = S^T q                    read out after the write

q and k (shared by the value heads of a group) are unit vectors, q also times
D^-1/2.  In front, q, k and v pass a short causal convolution over time per
channel and a SiLU; behind, each head's o is divided by its root mean square,
multiplied by a gain shared by the heads and by silu of a gate projection, and
projected back to the model's width.  Decay, beta, the unit lengths and the
state are float32 whatever the runtime's dtype.

A request's state slot holds the convolution's last taps - 1 inputs and the
heads' matrices; it has no pages.

Variants, each a constructor parameter: the decay may be one factor per key
channel, g[d] = exp(-exp(A_log) * softplus(z[d])), whose logits z come out of a
low-rank projection W_a2 (W_a1 x) + dt_bias (decay="channel"); the output's
gate may come out of a low-rank projection too (gate_rank) and may be a sigmoid
instead of a SiLU (gate_act).  The second halves of the low-rank projections
add up in float32.
"""
from __future__ import annotations

from typing import Callable, Dict, Optional

import torch

from ..kernels import ops
from .base import MIXERS, CacheNeed, Part, Runtime, StateNeed, TensorDecl
from .linear import linear


@MIXERS.register("gated_delta")
class GatedDeltaMixer(Part):
    replayable = True       # a decoding step's launches depend on the number of entries only; its state lies in device
                            # memory and is found by the slots of the step's metadata

    def __init__(self, *, rt: Runtime, width: int, prefix: str, num_heads: int, num_kv_heads: int, key_dim: int,
                 value_dim: int, conv_taps: int, norm_eps: float, shared: Optional[dict] = None,
                 names: Optional[Dict[str, str]] = None, decay: str = "head", decay_rank: int = 0, gate_rank: int = 0,
                 gate_act: str = "silu"):
        """num_heads value heads of value_dim, num_kv_heads query/key heads of key_dim (value head h reads query/key
        head h // (num_heads / num_kv_heads)); conv_taps: length of the convolutions (1: a factor per channel); norm_eps: eps of
        the output's norm; names: tensor names behind the prefix for q, k, v, g, o (matrices), q_conv, k_conv, v_conv
        ([channels, taps], the last column is the current token's), b and a (write strength and decay, one row per
        head), A_log, dt_bias (per head) and norm (per value channel).
        decay "channel": no `a`; a1 [decay_rank, width], a2 [heads * key_dim, decay_rank] and dt_bias per head and key
        channel instead.  gate_rank > 0: no `g`; g1 [gate_rank, width] and g2 [heads * value_dim, gate_rank] instead.
        gate_act: "silu" or "sigmoid"."""
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} value heads are not a multiple of {num_kv_heads} query/key heads")
        self.rt, self.width = rt, int(width)
        self.nh, self.nkv, self.d, self.dv = int(num_heads), int(num_kv_heads), int(key_dim), int(value_dim)
        self.taps = int(conv_taps)
        self.eps = float(norm_eps)
        if decay not in ("head", "channel"):
            raise ValueError(f"decay {decay!r} ('head': one factor per head; 'channel': one per key channel)")
        if gate_act not in ("silu", "sigmoid"):
            raise ValueError(f"gate_act {gate_act!r} ('silu' or 'sigmoid')")
        self.channel_decay, self.decay_rank, self.gate_rank, self.gate_act = decay == "channel", int(decay_rank), int(gate_rank), gate_act
        if self.channel_decay and self.decay_rank <= 0:
            raise ValueError("a decay per key channel comes out of a low-rank projection: give decay_rank")
        if self.gate_rank < 0:
            raise ValueError("gate_rank must not be negative (0: the gate's projection is one matrix)")
        if not 1 <= self.d <= ops.DELTA_MAX_KEY_DIM:
            raise ValueError(f"key size {self.d}: the kernel takes up to {ops.DELTA_MAX_KEY_DIM}")
        if not 1 <= self.taps <= ops.CONV_MAX_TAPS:
            raise ValueError(f"{self.taps} taps: the convolution takes 1 to {ops.CONV_MAX_TAPS}")
        n = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "g": "g_proj.weight", "o": "o_proj.weight",
             "q_conv": "q_conv.weight", "k_conv": "k_conv.weight", "v_conv": "v_conv.weight", "b": "b_proj.weight",
             "a": "a_proj.weight", "A_log": "A_log", "dt_bias": "dt_bias", "norm": "norm.weight",
             "a1": "a1", "a2": "a2", "g1": "g1", "g2": "g2"}
        n.update(names or {})
        self.names = {k: prefix + v for k, v in n.items()}
        self.channels = 2 * self.nkv * self.d + self.nh * self.dv      # what the convolutions run over: q, k, v
        self.conv_floats = (self.taps - 1) * self.channels
        self.rule_floats = self.nh * self.d * self.dv
        self.w_in = self.p_in = self.w_o = self.p_o = None
        self.conv_w = self.a_log = self.dt_bias = self.norm_w = self.w_a2 = self.w_g2 = None
        # columns of the input product: q, k, v (what the convolutions run over), then the gate (or its low-rank
        # part), the write strength's logits, the decay's logits (or their low-rank part)
        gate_cols = self.gate_rank if self.gate_rank else self.nh * self.dv
        self.col_gate = self.channels
        self.col_beta = self.col_gate + gate_cols
        self.col_decay = self.col_beta + self.nh

    def cache_need(self) -> Optional[CacheNeed]:
        return None

    def state_need(self) -> Optional[StateNeed]:
        """One float32 row per request: the convolutions' last taps - 1 inputs [taps - 1][channels], then the heads'
        matrices [H][Dv][D]."""
        return StateNeed((self.conv_floats + self.rule_floats,), torch.float32)

    def tensors(self) -> Dict[str, TensorDecl]:
        nm, kd, vd = self.names, self.nkv * self.d, self.nh * self.dv
        # (the order of a dict is the order in which a model's tensors are listed and drawn)
        t = {
            nm["q"]: TensorDecl((kd, self.width), "matrix"),
            nm["k"]: TensorDecl((kd, self.width), "matrix"),
            nm["v"]: TensorDecl((vd, self.width), "matrix"),
        }
        if self.gate_rank:
            t[nm["g1"]] = TensorDecl((self.gate_rank, self.width), "matrix")
            t[nm["g2"]] = TensorDecl((vd, self.gate_rank), "matrix")
        else:
            t[nm["g"]] = TensorDecl((vd, self.width), "matrix")
        t[nm["o"]] = TensorDecl((self.width, vd), "matrix")
        t[nm["b"]] = TensorDecl((self.nh, self.width), "matrix")
        if self.channel_decay:
            t[nm["a1"]] = TensorDecl((self.decay_rank, self.width), "matrix")
            t[nm["a2"]] = TensorDecl((self.nh * self.d, self.decay_rank), "matrix")
        else:
            t[nm["a"]] = TensorDecl((self.nh, self.width), "matrix")
        t[nm["A_log"]] = TensorDecl((self.nh,), "bias")
        t[nm["dt_bias"]] = TensorDecl((self.nh * self.d if self.channel_decay else self.nh,), "bias")
        t[nm["norm"]] = TensorDecl((self.dv,), "gain")
        # (with one tap the "convolution" is a factor per channel: the tensors are there all the same)
        t[nm["q_conv"]] = TensorDecl((kd, self.taps), "bias")
        t[nm["k_conv"]] = TensorDecl((kd, self.taps), "bias")
        t[nm["v_conv"]] = TensorDecl((vd, self.taps), "bias")
        return t

    def load(self, get: Callable[[str], torch.Tensor], rt: Runtime) -> None:
        nm = self.names
        # one product for everything that reads the mixer's input: q, k, v, the output's gate, and the logits of the
        # write strength and of the decay (what is computed from those two is float32)
        order = ("q", "k", "v", "g1" if self.gate_rank else "g", "b", "a1" if self.channel_decay else "a")
        self.w_in = torch.cat([rt.place(get(nm[k]), "matrix") for k in order], dim=0).contiguous()
        if self.gate_rank:
            self.w_g2 = rt.place(get(nm["g2"]), "matrix")
        if self.channel_decay:
            self.w_a2 = rt.place(get(nm["a2"]), "matrix")
        self.w_o = rt.place(get(nm["o"]), "matrix")
        self.p_in, self.p_o = rt.pack(self.w_in), rt.pack(self.w_o)
        self.w_in, self.w_o = rt.row_major(self.w_in, self.p_in), rt.row_major(self.w_o, self.p_o)
        self.conv_w = torch.cat([rt.place(get(nm[k]), "bias") for k in ("q_conv", "k_conv", "v_conv")], dim=0).contiguous()
        self.a_log, self.dt_bias = rt.place(get(nm["A_log"]), "bias"), rt.place(get(nm["dt_bias"]), "bias")
        self.norm_w = rt.place(get(nm["norm"]), "gain")

    def forward(self, x, ctx, cache, state):
        rt, c = self.rt, self.channels
        n = x.shape[0]
        if state is None or state.dim() != 2 or state.shape[1] != self.conv_floats + self.rule_floats:
            raise RuntimeError("the gated delta mixer was given no state of its shape")
        conv_state, rule_state = state[:, :self.conv_floats], state[:, self.conv_floats:]
        y = linear(rt, x, self.w_in, None, "delta.in", packed=self.p_in)            # q, k, v, gate, b, a
        qkv = rt.buffer("delta.qkv", (n, c), rt.dtype)
        ops.short_conv(y, c, self.conv_w, conv_state, ctx.tok_entry, ctx.entry_start, ctx.state_slots, qkv)
        if self.taps > 1:
            ops.short_conv_carry(y, c, self.taps, conv_state, ctx.entry_start, ctx.state_slots)
        o = rt.buffer("delta.o", (n, self.nh * self.dv), torch.float32)
        if self.channel_decay:
            # (the decays of all tokens at once, so that the recurrence only multiplies by them)
            decays = ops.lowrank_tanh(y, self.col_decay, self.w_a2, self.dt_bias,
                                      rt.buffer("delta.decay", (n, self.nh * self.d), torch.float32), tanh=False,
                                      decay=(self.a_log, self.d))
            ops.delta_rule_channel(qkv, y, self.col_beta, decays, rule_state, ctx.entry_start, ctx.state_slots, o,
                                   self.nh, self.nkv, self.d, self.dv)
        else:
            ops.delta_rule(qkv, y, self.col_beta, self.a_log, self.dt_bias, rule_state, ctx.entry_start, ctx.state_slots, o,
                           self.nh, self.nkv, self.d, self.dv)
        gate, gate_col = y, self.col_gate
        if self.gate_rank:
            gate, gate_col = ops.lowrank_tanh(y, self.col_gate, self.w_g2, None,
                                              rt.buffer("delta.gate", (n, self.nh * self.dv), torch.float32), tanh=False), 0
        z = rt.buffer("delta.gated", (n, self.nh * self.dv), rt.dtype)
        ops.gated_rmsnorm(o, self.norm_w, gate, gate_col, z, self.nh, self.dv, self.eps, gate_kind=self.gate_act)
        return linear(rt, z, self.w_o, None, "delta.o_proj", packed=self.p_o)
