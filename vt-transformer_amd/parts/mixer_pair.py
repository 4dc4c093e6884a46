"""Two mixers side by side: both read the same input, and the result is a
weighted sum of theirs with two constants,

    out = left_scale * left(x) + right_scale * right(x)

Either may be any registered mixer.  What they want of the cache manager is
passed through: pages for at most one of them (a layer has one set of pages),
and their per-request states one behind the other in one float32 row.
"""
from __future__ import annotations

from typing import Callable, Dict, Optional

import numpy as np
import torch

from ..config.base import PartSpec
from ..kernels import ops
from .base import MIXERS, CacheNeed, Part, Runtime, StateNeed, TensorDecl


@MIXERS.register("mixer_pair")
class MixerPair(Part):
    def __init__(self, *, rt: Runtime, width: int, prefix: str, left: PartSpec, right: PartSpec, left_scale: float = 1.0,
                 right_scale: float = 1.0, shared: Optional[dict] = None):
        """left, right: the two mixers' specs (a `prefix` among their params stands behind this part's own)."""
        self.rt, self.width = rt, int(width)
        self.scales = (float(left_scale), float(right_scale))
        if left.kind == right.kind:
            # (a kind's scratch buffers are keyed by name: the second member would overwrite the first one's result)
            raise ValueError(f"two mixers of one kind ('{left.kind}') side by side are not supported")
        self.members = []
        for spec in (left, right):
            params = dict(spec.params)
            local = params.pop("prefix", "")
            self.members.append(MIXERS.build(PartSpec(spec.kind, params), rt=rt, width=width, prefix=prefix + local, shared=shared))
        with_pages = [m for m in self.members if self._cache_need(m) is not None]
        if len(with_pages) > 1:
            raise ValueError("of two mixers side by side at most one keeps pages")
        self.paged = with_pages[0] if with_pages else None
        self.state_floats = []
        for m in self.members:
            need = m.state_need() if hasattr(m, "state_need") else None
            if need is not None and (need.dtype != torch.float32 or len(need.shape) != 1):
                raise ValueError("a mixer beside another keeps its state as one float32 row per request")
            self.state_floats.append(int(need.shape[0]) if need is not None else 0)
        # a decoding step can be recorded and replayed if both members' can
        self.replayable = all(getattr(m, "replayable", False) for m in self.members)

    @staticmethod
    def _cache_need(m) -> Optional[CacheNeed]:
        return m.cache_need() if hasattr(m, "cache_need") else None

    def cache_need(self) -> Optional[CacheNeed]:
        return self._cache_need(self.paged) if self.paged is not None else None

    def state_need(self) -> Optional[StateNeed]:
        total = sum(self.state_floats)
        return StateNeed((total,), torch.float32) if total else None

    def prepare_step(self, ctx) -> Optional[Dict[tuple, np.ndarray]]:
        out: Dict[tuple, np.ndarray] = {}
        for m in self.members:
            extra = m.prepare_step(ctx) if hasattr(m, "prepare_step") else None
            if extra:
                out.update(extra)
        return out or None

    def tensors(self) -> Dict[str, TensorDecl]:
        t: Dict[str, TensorDecl] = {}
        for m in self.members:
            t.update(m.tensors())
        return t

    def load(self, get: Callable[[str], torch.Tensor], rt: Runtime) -> None:
        for m in self.members:
            m.load(get, rt)

    def forward(self, x, ctx, cache, state):
        if sum(self.state_floats) and (state is None or state.dim() != 2 or state.shape[1] != sum(self.state_floats)):
            raise RuntimeError("the pair of mixers was given no state of its shape")
        results, at = [], 0
        for m, floats in zip(self.members, self.state_floats):
            own_state = state[:, at:at + floats] if floats else None
            at += floats
            y = m.forward(x, ctx, cache if m is self.paged else None, own_state)
            results.append(y)
        out = self.rt.buffer("pair.out", tuple(results[0].shape), torch.float32)
        return ops.scaled_sum(results[0], self.scales[0], results[1], self.scales[1], out)
