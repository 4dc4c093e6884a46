"""A feed-forward made of many small gated ones ("experts"), of which a router
chooses a few for every token.

    z = W_router x                                  in float32 (the router's matrix is kept in float32)
    s = sigmoid(z)   or   softmax(z)                `score`
    the `top` experts with the largest s are chosen (the lower index among equals); their weights are their scores,
    divided by their sum if `renormalize`
    weight_on "input":   out = sum_e expert_e(s_e * x)
    weight_on "output":  out = sum_e s_e * expert_e(x)
    expert_e(x) = W_down,e ( f(W_gate,e x) * (W_up,e x) ),   f = SiLU or the tanh form of GELU; no biases

The experts' matrices are stacked when they are loaded ([E, 2 F, W] with an expert's gate rows in front of its up rows,
and [E, W, F]), so a kernel finds an expert by its index.  Nothing of a step's routing reaches the host: the launches
depend on the number of tokens alone.
"""
from __future__ import annotations

import math
from typing import Callable, Dict, Optional

import torch

from ..kernels import ops
from .base import FEED_FORWARDS, NormedInput, Part, Runtime, TensorDecl


@FEED_FORWARDS.register("expert_mixture")
class ExpertMixture(Part):
    replayable = True

    def __init__(self, *, rt: Runtime, width: int, prefix: str, num_experts: int, top: int, intermediate_size: int,
                 score: str = "sigmoid", renormalize: bool = False, weight_on: str = "input", activation: str = "silu",
                 names: Optional[Dict[str, str]] = None):
        """num_experts experts of intermediate_size, `top` of them per token; score, renormalize, weight_on: module
        docstring; activation: "silu" or "gelu_tanh"; names: tensor names behind the prefix for the router and, with
        {} standing for an expert's index, for an expert's gate, up and down matrices."""
        self.rt, self.width = rt, int(width)
        self.ne, self.top, self.inter = int(num_experts), int(top), int(intermediate_size)
        if not 1 <= self.top <= self.ne or self.inter <= 0:
            raise ValueError(f"{self.top} of {self.ne} experts of {self.inter}")
        if score not in ("sigmoid", "softmax"):
            raise ValueError(f"score '{score}' is not known ('sigmoid' and 'softmax' are)")
        if weight_on not in ("input", "output"):
            raise ValueError(f"weight_on '{weight_on}' is not known ('input' and 'output' are)")
        if activation == "silu":
            self.alpha, self.cubic = 1.0, 0.0
        elif activation == "gelu_tanh":
            self.alpha, self.cubic = 2.0 * math.sqrt(2.0 / math.pi), 0.044715      # (1 + tanh z) / 2 = sigmoid(2 z)
        else:
            raise ValueError(f"activation '{activation}' is not supported ('silu' and 'gelu_tanh' are)")
        self.score, self.renormalize, self.weight_on = score, bool(renormalize), weight_on
        n = {"router": "router", "gate": "e{}.gate", "up": "e{}.up", "down": "e{}.down"}
        n.update(names or {})
        self.names = {k: prefix + v for k, v in n.items()}
        self.router = self.w_gu = self.w_down = None
        # pairs (token, choice) from which the experts' products run on the matrix cores, sorted by expert (16-bit types
        # with sizes in multiples of 8: few pairs 16 rows of a matrix to a block, many in tiles of 128 x 128)
        self.grouped_from = 1

    def tensors(self) -> Dict[str, TensorDecl]:
        nm = self.names
        t = {nm["router"]: TensorDecl((self.ne, self.width), "matrix32")}
        for e in range(self.ne):
            t[nm["gate"].format(e)] = TensorDecl((self.inter, self.width), "matrix")
            t[nm["up"].format(e)] = TensorDecl((self.inter, self.width), "matrix")
            t[nm["down"].format(e)] = TensorDecl((self.width, self.inter), "matrix")
        return t

    def load(self, get: Callable[[str], torch.Tensor], rt: Runtime) -> None:
        nm = self.names
        self.router = rt.place(get(nm["router"]), "matrix32")
        self.w_gu = torch.empty((self.ne, 2 * self.inter, self.width), dtype=rt.dtype, device=rt.device)
        self.w_down = torch.empty((self.ne, self.width, self.inter), dtype=rt.dtype, device=rt.device)
        for e in range(self.ne):
            self.w_gu[e, :self.inter].copy_(rt.place(get(nm["gate"].format(e)), "matrix"))
            self.w_gu[e, self.inter:].copy_(rt.place(get(nm["up"].format(e)), "matrix"))
            self.w_down[e].copy_(rt.place(get(nm["down"].format(e)), "matrix"))

    def forward(self, x, ctx=None):
        rt = self.rt
        if isinstance(x, NormedInput):
            x = x.materialize()
        n = x.shape[0]
        ids = rt.buffer("moe.ids", (n, self.top), torch.int32)
        wts = rt.buffer("moe.weights", (n, self.top), torch.float32)
        ops.moe_route(x, self.router, ids, wts, self.score, self.renormalize)
        act = rt.buffer("moe.act", (n * self.top, self.inter), rt.dtype)
        out = rt.buffer("moe.out", (n, self.width), torch.float32)
        if n * self.top >= self.grouped_from and ops.moe_grouped_ok(x, self.ne, self.width, self.inter):
            plan = rt.buffer("moe.plan", (ops.moe_plan_size(n * self.top, self.ne),), torch.int32)
            ops.moe_sort(ids, plan, self.ne)
            ops.moe_gate_up_grouped(x, self.w_gu, plan, wts, act, self.top, self.weight_on == "input", self.alpha, self.cubic)
            scratch = rt.buffer("moe.choices", (n * self.top, self.width), torch.float32) if self.top > 1 else None
            return ops.moe_down_grouped(act, self.w_down, plan, wts, out, scratch, self.weight_on == "output")
        ops.moe_gate_up(x, self.w_gu, ids, wts, act, self.weight_on == "input", self.alpha, self.cubic)
        return ops.moe_down(act, self.w_down, ids, wts, out, self.weight_on == "output")
