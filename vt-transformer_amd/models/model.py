"""A decoder put together from a `ModelSpec`: embedding, layers, the order in
which they run, final norm and head.  It is the same class for every
architecture; what differs is the spec.

The reference's counterpart is the outer program gpu_main
(v1/models/qwen2-7b/inference_fp16.dag:368-396): embed, 28 x layer_forward,
final norm over the rows, logits where the mask asks for them.
"""
from __future__ import annotations

from typing import Callable, Dict, List, Optional

import torch

from ..config.base import LayerSpec, ModelSpec, PartSpec
from ..kernels import ops
from ..parts.linear import linear
from ..parts.base import (BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, NormedInput, Part, Registry,
                          Runtime, TensorDecl)


def settle(h: torch.Tensor, delta):
    """Adds what a layer has handed on unadded (a tensor, a pair of tensors, or nothing) to the stream."""
    if isinstance(delta, tuple):
        return ops.residual_add2(h, delta[0], delta[1])
    if isinstance(delta, torch.Tensor):
        return ops.residual_add(h, delta)
    return h


def build_part(registry: Registry, spec: PartSpec, prefix: str, **context):
    params = dict(spec.params)
    local = params.pop("prefix", "")
    return registry.build(PartSpec(spec.kind, params), prefix=prefix + local, **context)


class DecoderModel:
    def __init__(self, spec: ModelSpec, rt: Runtime):
        spec.validate()
        self.spec = spec
        self.rt = rt
        width = spec.hidden_size
        shared: dict = {}  # parts that several layers hold one instance of (position tables)
        self.embedding = EMBEDDINGS.build(spec.embedding, rt=rt, width=width, vocab_size=spec.vocab_size)
        self.layers = [self._build_layer(ls, shared) for ls in spec.layers]
        self.final_norm = build_part(NORMS, spec.final_norm, "", rt=rt, width=width)
        self.head = HEADS.build(spec.head, rt=rt, width=width, vocab_size=spec.vocab_size)
        self.schedule = list(spec.schedule)
        # vectors that schedule entries add to the whole stream before they run (a repeated run of layers tells its
        # passes apart by them)
        self.offsets_name: Optional[str] = spec.stream_offsets["name"] if spec.stream_offsets else None
        self.offsets_rows = int(spec.stream_offsets["rows"]) if spec.stream_offsets else 0
        self.offsets: Optional[torch.Tensor] = None
        # the matrix W [width, 2 width] of x <- W [x; x0] in front of the schedule entries that say `inject`
        self.inject_name: Optional[str] = spec.stream_inject["name"] if spec.stream_inject else None
        self.w_inject = self.p_inject = None
        # several residual streams: [tokens, streams, width] between the embedding and the final norm
        self.streams = int(spec.streams)
        self._stream_ones: Optional[torch.Tensor] = None

    def _build_layer(self, ls: LayerSpec, shared: dict):
        rt, width = self.rt, self.spec.hidden_size
        norms = {role: build_part(NORMS, ns, ls.prefix, rt=rt, width=width) for role, ns in ls.norms.items()}
        mixer = build_part(MIXERS, ls.mixer, ls.prefix, rt=rt, width=width, shared=shared)
        ffn = build_part(FEED_FORWARDS, ls.feed_forward, ls.prefix, rt=rt, width=width) if ls.feed_forward is not None else None
        return build_part(BLOCKS, ls.block, ls.prefix, rt=rt, width=width, norms=norms, mixer=mixer, feed_forward=ffn)

    # ------------------------------------------------------------------
    def parts(self) -> List[Part]:
        out: List[Part] = [self.embedding]
        for layer in self.layers:
            out.extend(layer.parts())
        out.extend([self.final_norm, self.head])
        return out

    def tensors(self) -> Dict[str, TensorDecl]:
        out: Dict[str, TensorDecl] = {}
        for p in self.parts():
            for name, decl in p.tensors().items():
                if name in out and out[name].shape != decl.shape:
                    raise ValueError(f"tensor '{name}' is declared twice with shapes {out[name].shape} and {decl.shape}")
                if name not in out or not decl.optional:
                    out[name] = decl
        if self.offsets_name:
            out[self.offsets_name] = TensorDecl((self.offsets_rows, self.spec.hidden_size), "bias")
        if self.inject_name:
            out[self.inject_name] = TensorDecl((self.spec.hidden_size, 2 * self.spec.hidden_size), "matrix")
        return out

    def load(self, get: Callable[[str], torch.Tensor]) -> None:
        self.embedding.load(get, self.rt)
        for layer in self.layers:
            for p in layer.parts():
                p.load(get, self.rt)
        self.final_norm.load(get, self.rt)
        if self.offsets_name:
            self.offsets = self.rt.place(get(self.offsets_name), "bias")
        if self.inject_name:
            w = self.rt.place(get(self.inject_name), "matrix")
            self.p_inject = self.rt.pack(w)
            self.w_inject = self.rt.row_major(w, self.p_inject)
        # a head's loader takes `shared`: tensors by name that other parts have already placed on the device (the
        # embedding's table, which a tied head multiplies by)
        shared = {}
        if getattr(self.embedding, "table", None) is not None:
            shared[self.embedding.name] = self.embedding.table
        self.head.load(get, self.rt, shared=shared)

    # ------------------------------------------------------------------
    def forward(self, ctx, caches, states) -> Optional[torch.Tensor]:
        """Run the tokens of one step.  caches[i] / states[i] belong to schedule entry i.
        Returns fp32 logits [rows wanted, vocab], or None if no row is wanted."""
        h = self.embedding.forward(ctx.token_ids)
        if self.streams:
            # every stream starts as the embedding's output
            h = ops.streams_fill(h, self.rt.buffer("streams", (h.shape[0], self.streams, h.shape[1]), torch.float32))
        delta = None
        first = None
        if self.inject_name:
            # the embedding's output is kept: passes of a repeated run of layers start from it again
            first = ops.set_plus_row(self.rt.buffer("h.first", tuple(h.shape), torch.float32), h, None)
        last = len(self.schedule) - 1
        for i, entry in enumerate(self.schedule):
            block = self.layers[entry.layer]
            if isinstance(delta, tuple) and (entry.inject or entry.offset_row is not None
                                             or not getattr(block, "takes_pair", False)):
                h, delta = settle(h, delta), None
            if entry.inject:
                # x <- W [x; x0] (+ the entry's offset): one product over the joined rows, its result is the new stream
                h = settle(h, delta)
                delta = None
                width = h.shape[1]
                joined = ops.concat_cast(h, first, self.rt.buffer("h.joined", (h.shape[0], 2 * width), self.rt.dtype))
                y = linear(self.rt, joined, self.w_inject, None, "h.injected", packed=self.p_inject)
                ops.set_plus_row(h, y, self.offsets[entry.offset_row] if entry.offset_row is not None else None)
            elif entry.offset_row is not None:
                # what is still to be added goes in with the offset, in one pass over the stream
                ops.add_row(h, delta if isinstance(delta, torch.Tensor) else None, self.offsets[entry.offset_row])
                delta = None
            if getattr(block, "takes_next_norm", False):
                # the norm that the layer behind starts with, which this layer's last product may prepare (not if
                # the stream still changes in between)
                behind = self.schedule[i + 1] if i < last else None
                nxt = (getattr(self.layers[behind.layer], "first_norm", None)
                       if behind is not None and behind.offset_row is None and not behind.inject else None)
                h, delta = block.forward(h, delta, ctx, caches[i], states[i], next_norm=nxt)
            else:
                if isinstance(delta, NormedInput):
                    delta = None            # (its addition is done; this block applies its own norm)
                h, delta = block.forward(h, delta, ctx, caches[i], states[i])
        if ctx.n_logit_rows == 0:
            return None
        if isinstance(delta, NormedInput):
            delta = None
        if isinstance(delta, tuple):
            if getattr(self.final_norm, "takes_pair", False) and not self.streams:
                return self.head.forward(self.final_norm.forward(h, delta[0], rows=ctx.logit_rows, delta2=delta[1]))
            h, delta = settle(h, delta), None
        if self.streams:
            # the streams' sum, for the wanted rows only, inside the final norm's kernel
            if self._stream_ones is None:
                self._stream_ones = torch.ones(self.streams, dtype=torch.float32, device=self.rt.device)
            x = self.final_norm.forward_streams(h, self._stream_ones, rows=ctx.logit_rows)
        else:
            x = self.final_norm.forward(h, delta, rows=ctx.logit_rows)
        return self.head.forward(x)
