"""Arrangement of a layer's parts around the residual stream.

"prenorm" is the reference's layer (v1/models/qwen2-7b/inference_fp16.dag:287-345):
norm -> mixer -> add -> norm -> feed-forward -> add.  The residual stream h is
fp32.  A layer hands its last output on unadded (`delta`), so the next norm
adds it in the same kernel that normalises.

With few rows in bfloat16 (decoding) the norms and additions are not kernels of
their own: a mixer or feed-forward that says so takes the residual stream with
the norm still to be applied (`NormedInput`: its first matrix product applies
it) and adds its result to the stream itself (`residual=`: its last matrix
product does; `adds_residual(rows)` says for how many rows it can, which reaches
up to 64 for matrices that fill the GPU without splitting k over blocks).  A part
that `hands_norm_on` is also told which norm comes behind it (`hand_on=`) and
may return that norm prepared (a NormedInput with `xn` and `ssq`), which the
part behind the norm then takes as its input.
"""
from __future__ import annotations

from typing import Callable, Dict, Optional, Tuple

import torch

from ..kernels import ops
from .base import BLOCKS, NormedInput, Part, Runtime, StateNeed, TensorDecl
from .linear import can_fuse, linear


@BLOCKS.register("prenorm")
class PreNormBlock(Part):
    norm_roles = ("input", "post_mixer")
    replayable = True
    takes_next_norm = True      # forward(..., next_norm=): the norm that the layer behind this one starts with

    def __init__(self, *, rt: Runtime, norms, mixer, feed_forward, prefix: str = "", width: int = 0):
        self.rt = rt
        self.norm_in = norms["input"]
        self.mixer = mixer
        # a layer without a feed-forward has only the first sublayer (and no second norm)
        self.feed_forward = feed_forward
        self.norm_post = norms["post_mixer"] if feed_forward is not None else None

    def parts(self):
        if self.feed_forward is None:
            return [self.norm_in, self.mixer]
        return [self.norm_in, self.mixer, self.norm_post, self.feed_forward]

    @property
    def first_norm(self):
        """The norm that this layer applies to the stream it is given (what the layer in front may prepare)."""
        return self.norm_in

    def forward(self, h: torch.Tensor, delta, ctx, cache, state, next_norm=None) -> Tuple[torch.Tensor, object]:
        """delta: what is still to be added to h (a tensor), None, or this layer's first norm as the layer in front
        has prepared it (a NormedInput; its addition is done).  Returns (h, delta) in the same terms."""
        fuse = can_fuse(self.rt, h.shape[0]) and h.shape[1] % 8 == 0
        if self.feed_forward is None:
            return h, self._run(self.mixer, self.norm_in, h, delta, fuse, next_norm, ctx, cache, state)
        y = self._run(self.mixer, self.norm_in, h, delta, fuse, self.norm_post, ctx, cache, state)
        z = self._run(self.feed_forward, self.norm_post, h, y, fuse, next_norm, ctx)
        return h, z

    def _run(self, part, norm, h, delta, fuse, norm_behind, *args):
        """norm (of h + delta), then the part; returns what is still to be added to h (None: the part added it; a
        NormedInput: it added it and prepared `norm_behind`)."""
        takes = getattr(part, "takes_normed_input", False)
        if isinstance(delta, NormedInput):
            x = delta if (delta.norm is norm and takes) else norm.forward(h, None)
        elif fuse and delta is None and getattr(norm, "rms_fusable", False) and takes:
            x = NormedInput(h, norm)
        else:
            x = norm.forward(h, delta)
        adds = getattr(part, "adds_residual", None)
        if adds is not None and adds(h.shape[0]):
            if norm_behind is not None and getattr(part, "hands_norm_on", False):
                r = part.forward(x, *args, residual=h, hand_on=norm_behind)
                return r if isinstance(r, NormedInput) else None
            part.forward(x, *args, residual=h)
            return None
        return part.forward(x, *args)


@BLOCKS.register("parallel")
class ParallelBlock(Part):
    """One norm whose output the mixer and the feed-forward both read; their results join the stream in one sum:

        h = norm(x);   x <- x + (mixer(h) + feed_forward(h))

    The block hands both results on unadded (a pair), so that the norm of the layer behind it adds them in the kernel
    that normalises (a norm with `delta2`); whoever cannot take a pair gets them added first (`settle`).  A layer
    without a feed-forward hands the mixer's result on alone."""

    norm_roles = ("input",)
    replayable = True
    takes_pair = True       # forward(h, delta, ...) with delta a pair of tensors: both are still to be added to h

    def __init__(self, *, rt: Runtime, norms, mixer, feed_forward, prefix: str = "", width: int = 0):
        self.rt = rt
        self.norm_in = norms["input"]
        self.mixer = mixer
        self.feed_forward = feed_forward

    def parts(self):
        return [self.norm_in, self.mixer] + ([self.feed_forward] if self.feed_forward is not None else [])

    @staticmethod
    def settle(h: torch.Tensor, delta):
        """Adds what is still to be added to the stream (a tensor, a pair of tensors or None); returns h."""
        if isinstance(delta, tuple):
            return ops.residual_add2(h, delta[0], delta[1])
        if isinstance(delta, torch.Tensor):
            return ops.residual_add(h, delta)
        return h

    def forward(self, h: torch.Tensor, delta, ctx, cache, state) -> Tuple[torch.Tensor, object]:
        if isinstance(delta, NormedInput):
            delta = None            # (its addition is done; this block applies its own norm)
        if isinstance(delta, tuple) and not getattr(self.norm_in, "takes_pair", False):
            h, delta = self.settle(h, delta), None
        if isinstance(delta, tuple):
            x = self.norm_in.forward(h, delta[0], delta2=delta[1])
        else:
            x = self.norm_in.forward(h, delta)
        y = self.mixer.forward(x, ctx, cache, state)
        if self.feed_forward is None:
            return h, y
        z = self.feed_forward.forward(x, ctx)
        if y.dtype != z.dtype:
            # (results of different types are joined in the stream one after the other)
            ops.residual_add(h, y)
            return h, z
        return h, (y, z)


@BLOCKS.register("hyper")
class HyperBlock(Part):
    """Pre-norm sublayers around S residual streams x_1 .. x_S (float32, [tokens, S, width]) instead of one.  For
    sublayer q (1: the mixer, 2: the feed-forward) with its learned numbers in_q [S], out_q [S] and mix_q [S, S]:

        u   = sum_s in_q[s] x_s
        h   = norm_q(u)
        y   = sublayer(h') * sigmoid(W_rg,q h + b_rg,q)        residual_gate; without it y = sublayer(h')
        x_t <- sum_s mix_q[s, t] x_s + out_q[t] y              all streams at once from the old ones

    h' is h, or for the mixer with token_shift the blend h + (h_prev - h) * mu with the previous token's h (as it was
    before blending; zeros in front of a sequence's first token), mu one number per channel.  The previous h of a
    request's last token is part of its state: the block declares one float32 row per request that holds it in front
    of whatever the mixer keeps there.  The weighted sum and the norm are one kernel, and so are the gate, the mixing
    and the addition.  With learned_streams False there is one stream with in = out = mix = 1 and no tensors for
    them: the plain residual sum.
    """

    norm_roles = ("input", "post_mixer")
    replayable = True

    def __init__(self, *, rt: Runtime, norms, mixer, feed_forward, prefix: str = "", width: int = 0, streams: int = 1,
                 learned_streams: bool = True, token_shift: bool = False, residual_gate: bool = False,
                 names: Optional[Dict[str, str]] = None):
        """names: tensor names behind the layer's prefix, with {} standing for the sublayer's number, for in, out, mix
        (the streams' numbers), gate and gate_bias (the residual gate's matrix and bias), for shift (mu), and for
        idle_norm (the second norm's tensor of a layer without a feed-forward, where a checkpoint holds one)."""
        self.rt, self.width, self.s = rt, int(width), int(streams)
        if not 1 <= self.s <= ops.STREAMS_MAX:
            raise ValueError(f"{self.s} residual streams (1 to {ops.STREAMS_MAX})")
        if not learned_streams and self.s != 1:
            raise ValueError("streams without learned numbers are one stream")
        self.learned, self.shift, self.gated = bool(learned_streams), bool(token_shift), bool(residual_gate)
        self.norm_in = norms["input"]
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norm_post = norms["post_mixer"] if feed_forward is not None else None
        n = {"in": "hc{}.in", "out": "hc{}.out", "mix": "hc{}.mix", "gate": "rg{}", "gate_bias": "rg{}.b", "shift": "shift",
             "idle_norm": "norm2"}
        n.update(names or {})
        self.names = {k: prefix + v for k, v in n.items()}
        self.n_sub = 1 if feed_forward is None else 2
        self.w_in = [None, None]
        self.w_out = [None, None]
        self.w_mix = [None, None]
        self.w_gate, self.p_gate, self.b_gate, self.b_gate_lowp = [None, None], [None, None], [None, None], [None, None]
        self.mu = None
        inner = mixer.state_need() if hasattr(mixer, "state_need") else None
        if inner is not None and (inner.dtype != torch.float32 or len(inner.shape) != 1):
            raise ValueError("a mixer inside this block keeps its state as one float32 row per request")
        self.inner_floats = int(inner.shape[0]) if inner is not None else 0
        self.own_floats = self.width if self.shift else 0

    def parts(self):
        if self.feed_forward is None:
            return [self, self.norm_in, self.mixer]
        return [self, self.norm_in, self.mixer, self.norm_post, self.feed_forward]

    def state_need(self) -> Optional[StateNeed]:
        """One float32 row per request: the previous token's mixer input (if token_shift), then the mixer's state."""
        total = self.own_floats + self.inner_floats
        return StateNeed((total,), torch.float32) if total else None

    def tensors(self) -> Dict[str, TensorDecl]:
        """A layer without a feed-forward has no second sublayer; a checkpoint that holds the second sublayer's
        numbers for it all the same is tolerated, and they are not read."""
        nm, t = self.names, {}
        for q in (1, 2):
            idle = q > self.n_sub
            if self.learned:
                t[nm["in"].format(q)] = TensorDecl((self.s,), "gain", optional=idle)
                t[nm["out"].format(q)] = TensorDecl((self.s,), "gain", optional=idle)
                t[nm["mix"].format(q)] = TensorDecl((self.s, self.s), "stream_mix", optional=idle)
            if self.gated:
                t[nm["gate"].format(q)] = TensorDecl((self.width, self.width), "matrix", optional=idle)
                t[nm["gate_bias"].format(q)] = TensorDecl((self.width,), "bias", optional=idle)
        if self.n_sub == 1:
            t[nm["idle_norm"]] = TensorDecl((self.width,), "gain", optional=True)
        if self.shift:
            t[nm["shift"]] = TensorDecl((self.width,), "bias")
        return t

    def load(self, get: Callable[[str], torch.Tensor], rt: Runtime) -> None:
        nm = self.names
        for i in range(self.n_sub):
            q = i + 1
            if self.learned:
                self.w_in[i] = rt.place(get(nm["in"].format(q)), "gain")
                self.w_out[i] = rt.place(get(nm["out"].format(q)), "gain")
                self.w_mix[i] = rt.place(get(nm["mix"].format(q)), "stream_mix")
            else:
                one = torch.ones(1, dtype=torch.float32, device=rt.device)
                self.w_in[i], self.w_out[i], self.w_mix[i] = one, one, one.view(1, 1)
            if self.gated:
                w = rt.place(get(nm["gate"].format(q)), "matrix")
                self.b_gate[i] = rt.place(get(nm["gate_bias"].format(q)), "bias")
                self.b_gate_lowp[i] = self.b_gate[i].to(rt.dtype)
                self.p_gate[i] = rt.pack(w)
                self.w_gate[i] = rt.row_major(w, self.p_gate[i])
        if self.shift:
            self.mu = rt.place(get(nm["shift"]), "bias")

    def _sublayer(self, i: int, part, norm, x, ctx, shift_state, *args):
        rt = self.rt
        h = norm.forward_streams(x, self.w_in[i])
        gate = None
        if self.gated:
            gate = linear(rt, h, self.w_gate[i], self.b_gate[i], f"hyper.gate{i}", bias_lowp=self.b_gate_lowp[i],
                          packed=self.p_gate[i])
        if shift_state is not None:
            h = ops.token_shift(h, self.mu, shift_state, ctx.tok_entry, ctx.entry_start, ctx.state_slots,
                                rt.buffer("hyper.shifted", tuple(h.shape), h.dtype))
        y = part.forward(h, ctx, *args)
        ops.streams_write(x, self.w_mix[i], self.w_out[i], y, gate)

    def forward(self, x: torch.Tensor, delta, ctx, cache, state) -> Tuple[torch.Tensor, object]:
        """x [tokens, S, width] float32, changed in place; nothing is left to be added (`delta` stays None)."""
        if x.dim() != 3 or x.shape[1] != self.s or delta is not None:
            raise RuntimeError(f"this block works on {self.s} residual streams [tokens, {self.s}, width]")
        shift_state = inner_state = None
        if self.own_floats or self.inner_floats:
            if state is None or state.dim() != 2 or state.shape[1] != self.own_floats + self.inner_floats:
                raise RuntimeError("the block was given no state of its shape")
            shift_state = state[:, :self.own_floats] if self.own_floats else None
            inner_state = state[:, self.own_floats:] if self.inner_floats else None
        self._sublayer(0, self.mixer, self.norm_in, x, ctx, shift_state, cache, inner_state)
        if self.feed_forward is not None:
            self._sublayer(1, self.feed_forward, self.norm_post, x, ctx, None)
        return x, None
