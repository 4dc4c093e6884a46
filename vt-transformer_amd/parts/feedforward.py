"""Gated feed-forward: down( act(gate(x)) * up(x) ).

The reference's order (v1/models/qwen2-7b/inference_fp16.dag:333-337): up
projection (mlp.w2), gate projection (mlp.w1), silu(gate) * up
(v1/tensortype/hip_kernels/silu_product.cpp:8-16), down projection
(mlp.o_proj); w1 = gate_proj, w2 = up_proj, o_proj = down_proj
(v1/models/qwen2-7b/dump_from_huggingface.py:89-99).  Gate and up are one
matrix here (gate rows, then up rows); with few tokens the gating is applied
to the fp32 accumulators inside the product's kernel.

The gate's form has parameters: with g = gate(x) and u = up(x), both with their
biases if the model has them,

    g <- min(g, limit),  u <- clamp(u, -limit, limit)        (limit 0: no bounds)
    act = g * sigmoid(alpha * g * (1 + cubic * g^2)) * (u + up_shift)

alpha 1, no bounds, no shift and cubic 0 is SiLU gating, the reference's.  activation "relu" is max(g, 0) * (u +
up_shift), the form's limit for alpha -> infinity, which the kernels compute as such.  activation "gelu_tanh" is the tanh form of
GELU, 0.5 g (1 + tanh(sqrt(2 / pi) (g + 0.044715 g^3))): since (1 + tanh z) / 2 = sigmoid(2 z) it is the same form
with alpha = 2 sqrt(2 / pi) and cubic = 0.044715.
"""
from __future__ import annotations

import math
from typing import Callable, Dict, Optional

import torch

from ..kernels import ops
from .base import FEED_FORWARDS, Part, Runtime, TensorDecl
from .base import NormedInput
from .linear import GATED_MAX_ROWS, UNPACK_MIN_ROWS, can_add_residual, can_fuse, linear, takes_prepared_norm


@FEED_FORWARDS.register("gated_mlp")
class GatedMLP(Part):
    replayable = True

    def __init__(self, *, rt: Runtime, width: int, prefix: str, intermediate_size: int, activation: str = "silu",
                 names: Optional[Dict[str, str]] = None, weight_suffix: str = ".weight",
                 bias_suffix: Optional[str] = None, act_alpha: float = 1.0, act_limit: float = 0.0, up_shift: float = 0.0,
                 act_cubic: float = 0.0):
        """names: the three matrices' names behind the prefix; weight_suffix: what follows a matrix's name in its
        tensor's name ("" where the tensor is called as the matrix); bias_suffix: likewise for the three biases
        (None: the projections have none); activation: "silu" or "gelu_tanh"; act_alpha, act_limit, up_shift, act_cubic:
        the gate's form (module docstring; "gelu_tanh" sets alpha and cubic itself)."""
        if activation == "gelu_tanh":
            if act_alpha != 1.0 or act_cubic != 0.0:
                raise ValueError("activation 'gelu_tanh' fixes act_alpha and act_cubic")
            act_alpha, act_cubic = 2.0 * math.sqrt(2.0 / math.pi), 0.044715
        elif activation == "relu":
            if act_alpha != 1.0 or act_cubic != 0.0:
                raise ValueError("activation 'relu' fixes act_alpha and act_cubic")
            act_alpha = math.inf        # the sigmoid of the gate's form as a step (the kernels test for it)
        elif activation != "silu":
            raise ValueError(f"activation '{activation}' is not supported ('silu', whose form act_alpha, act_limit, "
                             f"up_shift and act_cubic change, 'gelu_tanh' and 'relu' are)")
        if not act_alpha > 0 or act_limit < 0:
            raise ValueError("act_alpha must be positive and act_limit not negative (0: no bounds)")
        self.alpha, self.limit, self.shift, self.cubic = float(act_alpha), float(act_limit), float(up_shift), float(act_cubic)
        self.plain_silu = self.alpha == 1.0 and self.limit == 0.0 and self.shift == 0.0 and self.cubic == 0.0
        self.bias_suffix = bias_suffix
        self.b_gu = self.b_gu_lowp = self.b_down = self.b_down_lowp = None
        self.rt = rt
        self.width = int(width)
        self.inter = int(intermediate_size)
        n = {"gate": "gate_proj", "up": "up_proj", "down": "down_proj"}
        n.update(names or {})
        self.names = {k: prefix + v for k, v in n.items()}
        self.suffix = weight_suffix
        self.w_gu = self.w_down = self.p_gu = self.p_down = None

    def tensors(self) -> Dict[str, TensorDecl]:
        nm = self.names
        t = {
            nm["gate"] + self.suffix: TensorDecl((self.inter, self.width), "matrix"),
            nm["up"] + self.suffix: TensorDecl((self.inter, self.width), "matrix"),
            nm["down"] + self.suffix: TensorDecl((self.width, self.inter), "matrix"),
        }
        if self.bias_suffix is not None:
            t[nm["gate"] + self.bias_suffix] = TensorDecl((self.inter,), "bias")
            t[nm["up"] + self.bias_suffix] = TensorDecl((self.inter,), "bias")
            t[nm["down"] + self.bias_suffix] = TensorDecl((self.width,), "bias")
        return t

    def load(self, get: Callable[[str], torch.Tensor], rt: Runtime) -> None:
        nm = self.names
        self.w_gu = torch.cat([rt.place(get(nm["gate"] + self.suffix), "matrix"),
                               rt.place(get(nm["up"] + self.suffix), "matrix")], dim=0).contiguous()
        self.w_down = rt.place(get(nm["down"] + self.suffix), "matrix")
        if self.bias_suffix is not None:
            self.b_gu = torch.cat([rt.place(get(nm["gate"] + self.bias_suffix), "bias"),
                                   rt.place(get(nm["up"] + self.bias_suffix), "bias")], dim=0).contiguous()
            self.b_down = rt.place(get(nm["down"] + self.bias_suffix), "bias")
            self.b_gu_lowp, self.b_down_lowp = self.b_gu.to(rt.dtype), self.b_down.to(rt.dtype)
        self.p_down = rt.pack(self.w_down)
        self.p_gu = rt.pack(self.w_gu, halves=2)           # gate and up side by side for the kernel that gates on its way
        self.w_gu = rt.row_major(self.w_gu, self.p_gu)
        self.w_down = rt.row_major(self.w_down, self.p_down)

    takes_normed_input = True     # the gate/up product applies the norm in front of it when the rows are few
    hands_norm_on = True          # ... and the down product prepares the norm behind it

    def adds_residual(self, rows: int) -> bool:
        """Whether the down product adds to the residual stream itself at this many rows."""
        return can_add_residual(self.rt, rows, self.width, self.inter)

    def _forward_formed(self, x, act, residual, hand_on):
        """The gate in another form than SiLU's, or with biases.  Few rows in a 16-bit type: the gated product's kernel
        takes biases and form (and the norm in front, as for SiLU).  Otherwise the plain product of both matrices
        with the biases, the gate as a kernel of its own, and the down product."""
        rt = self.rt
        n = x.shape[0]
        normed = isinstance(x, NormedInput)
        if rt.lowp and self.p_gu is not None and (n <= GATED_MAX_ROWS or self.w_gu is None):
            if normed:
                ok = takes_prepared_norm(rt, n, self.width) if x.prepared else (can_fuse(rt, n) and self.width % 8 == 0)
                if not ok:
                    x, normed = x.materialize(), False
            if normed and x.prepared:
                ops.gated_linear_bf16_form(x.xn, self.p_gu, self.b_gu, act, self.alpha, self.limit, self.shift,
                                           norm_eps=x.eps, ssq_in=x.ssq, cubic=self.cubic)
            elif normed:
                ops.gated_linear_bf16_form(x.h, self.p_gu, self.b_gu, act, self.alpha, self.limit, self.shift,
                                           norm_gain=x.gain, norm_eps=x.eps, cubic=self.cubic)
            else:
                ops.gated_linear_bf16_form(x, self.p_gu, self.b_gu, act, self.alpha, self.limit, self.shift, cubic=self.cubic)
        else:
            gu = linear(rt, x, self.w_gu, self.b_gu, "mlp.gu", bias_lowp=self.b_gu_lowp)
            ops.gated_act(gu, act, self.alpha, self.limit, self.shift, self.cubic)
        return linear(rt, act, self.w_down, self.b_down, "mlp.down", bias_lowp=self.b_down_lowp, packed=self.p_down,
                      residual=residual, hand_on=hand_on)

    def forward(self, x, ctx=None, residual: Optional[torch.Tensor] = None, hand_on=None):
        rt = self.rt
        n = x.shape[0]
        act = rt.buffer("mlp.act", (n, self.inter), rt.dtype)
        if not self.plain_silu or self.b_gu is not None:
            return self._forward_formed(x, act, residual, hand_on)
        normed = isinstance(x, NormedInput)
        if normed:
            ok = (takes_prepared_norm(rt, n, self.width) and self.p_gu is not None) if x.prepared else \
                (can_fuse(rt, n) and self.width % 8 == 0)
            if not ok:
                x, normed = x.materialize(), False
        if rt.lowp and (n <= GATED_MAX_ROWS or (self.w_gu is None and (rt.keep_row_major or n < UNPACK_MIN_ROWS))):
            w = self.p_gu if self.p_gu is not None else self.w_gu
            if normed and x.prepared:
                ops.gated_linear_bf16_link(x.xn, w, act, x.ssq, x.eps)
            elif normed:
                ops.gated_linear_bf16(x.h, w, act, norm_gain=x.gain, norm_eps=x.eps)
            else:
                ops.gated_linear_bf16(x, w, act)
        else:
            gu = linear(rt, x, self.w_gu, None, "mlp.gu", packed=self.p_gu if self.w_gu is None else None)
            ops.silu_mul(gu, act)
        return linear(rt, act, self.w_down, None, "mlp.down", packed=self.p_down, residual=residual, hand_on=hand_on)
