"""RMSNorm, fused with the residual addition that precedes it.

out = (w * x) * 1/sqrt(mean(x^2) + eps), all in fp32, one rounding to the
output dtype (v1/tensortype/hip_kernels/rmsnorm.cpp:7-44: the sum of squares
divided by the width, eps inside the root, product evaluated (w*x)*r).
x = h + delta is the reference's fp32 residual addition
(v1/tensortype/hip_kernels/pointwise.cpp:51-57).
"""
from __future__ import annotations

from typing import Callable, Dict, Optional

import torch

from ..kernels import ops
from .base import NORMS, Part, Runtime, TensorDecl


@NORMS.register("rmsnorm")
class RMSNorm(Part):
    replayable = True
    # out = (gain * x) / sqrt(mean(x^2) + eps) with `gain` and `eps` as attributes: a matrix product can apply it on
    # the way (NormedInput); any norm of that form may say so
    rms_fusable = True

    def __init__(self, *, rt: Runtime, width: int, prefix: str, eps: float, name: str = "weight", scratch: str = "norm",
                 unit_offset: bool = False):
        """unit_offset: the tensor holds w = gain - 1 (the one is added once, in float32, when it is loaded)."""
        self.rt = rt
        self.width = int(width)
        self.eps = float(eps)
        self.name = prefix + name
        self.scratch = scratch
        self.unit_offset = bool(unit_offset)
        self.gain: Optional[torch.Tensor] = None

    def tensors(self) -> Dict[str, TensorDecl]:
        # (a gain less one is drawn like a bias where a model gets random weights)
        return {self.name: TensorDecl((self.width,), "bias" if self.unit_offset else "gain")}

    def load(self, get: Callable[[str], torch.Tensor], rt: Runtime) -> None:
        self.gain = rt.place(get(self.name), "gain")
        if self.unit_offset:
            self.gain = (self.gain + 1.0).contiguous()

    def forward_streams(self, x: torch.Tensor, w_in: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """The norm of a weighted sum of several residual streams: x [N, S, H] float32, w_in [S] float32 -> normed
        [N or R, H] in the runtime's dtype (one kernel: the sum is never written)."""
        n = rows.numel() if rows is not None else x.shape[0]
        out = self.rt.buffer(self.scratch + (".rows" if rows is not None else ""), (n, self.width), self.rt.dtype)
        return ops.streams_read(x, w_in, self.gain, out, self.eps, rows=rows)

    def forward(self, h: torch.Tensor, delta: Optional[torch.Tensor] = None,
                rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        n = rows.numel() if rows is not None else h.shape[0]
        out = self.rt.buffer(self.scratch + (".rows" if rows is not None else ""), (n, self.width), self.rt.dtype)
        return ops.rmsnorm(h, delta, self.gain, out, self.eps, rows=rows)


@NORMS.register("layernorm")
class LayerNorm(Part):
    """Layer norm with a gain and (optionally) a bias: out = (x - mean) / sqrt(var + eps) * gain + bias, the variance
    the mean of the squared deviations, all in float32, fused with the residual additions in front of it.  Beside
    `delta` it takes `delta2`: with both, x = h + (delta + delta2), the sum of two sublayers that ran side by side."""

    replayable = True
    takes_pair = True       # forward(h, delta, delta2=): two addends of one type in front of the norm

    def __init__(self, *, rt: Runtime, width: int, prefix: str, eps: float, name: str = "weight", bias_name: Optional[str] = None,
                 scratch: str = "norm"):
        """name / bias_name: the tensors' names behind the prefix (bias_name None: no bias)."""
        self.rt = rt
        self.width = int(width)
        self.eps = float(eps)
        self.name = prefix + name
        self.bias_name = prefix + bias_name if bias_name is not None else None
        self.scratch = scratch
        self.gain: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None

    def tensors(self) -> Dict[str, TensorDecl]:
        t = {self.name: TensorDecl((self.width,), "gain")}
        if self.bias_name is not None:
            t[self.bias_name] = TensorDecl((self.width,), "bias")
        return t

    def load(self, get: Callable[[str], torch.Tensor], rt: Runtime) -> None:
        self.gain = rt.place(get(self.name), "gain")
        if self.bias_name is not None:
            self.bias = rt.place(get(self.bias_name), "bias")

    def forward(self, h: torch.Tensor, delta: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None,
                delta2: Optional[torch.Tensor] = None) -> torch.Tensor:
        n = rows.numel() if rows is not None else h.shape[0]
        out = self.rt.buffer(self.scratch + (".rows" if rows is not None else ""), (n, self.width), self.rt.dtype)
        return ops.layernorm(h, delta, self.gain, self.bias, out, self.eps, rows=rows, delta2=delta2)
