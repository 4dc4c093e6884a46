"""Kigalix: typed configuration read from the keys of its config.json.

A Kigalix model keeps `streams` copies of the float32 residual stream.  Every sublayer reads a learned weighted sum
of them through an RMS norm whose tensor holds the gain less one, and its result, times a sigmoid gate computed from
the sublayer's normed input, goes back into every stream with a learned weight while a small learned matrix mixes the
streams (`parts/block.py`: "hyper").  A mixer reads its input blended with the previous token's.  Three mixers:

"latent_attention": the cache holds one low-rank vector and one rotated key part per token; per head the unrotated
keys and the values are projections of the low-rank vector; a query head is [dim unrotated | rot_dim rotated];
neighbouring elements are rotated together; every earlier token is seen (`parts/latent_attention.py`).

"latent_attention_2": the same with frequencies stretched for longer contexts (`rot.scaling`) and an elementwise
sigmoid gate on the heads' outputs.

"general_delta": a matrix state per head, a decay per key channel from a low-rank projection, a removal along the
unit key (`parts/general_delta.py`).

The feed-forward is dense (a gated unit with the tanh form of GELU) or a mixture of experts (SiLU experts, sigmoid
scores that multiply the chosen experts' inputs and are not renormalized: `parts/moe.py`).

config.json:
  architecture            "Kigalix"
  vocab, width            sizes of the vocabulary and of the stream
  streams                 number of residual streams (absent: one, with no learned numbers)
  norm.eps                eps of every RMS norm of the model
  layers[i].type          "latent_attention" | "latent_attention_2" | "general_delta"
  layers[i].mixer         latent attention: heads, dim, rot_dim, vdim, kv_rank, scale, rot.{dims, base, scaling.{factor,
                                            original, fast, slow}}
                          general_delta:    heads, dim (the size of the decay's low-rank projection is the number of rows
                                            of the layer's tensor mix.w1; `decay_rank` says it where there is no tensor)
  layers[i].mlp           null | {kind: "dense", ff} | {kind: "moe", expert.ff, router.{experts, top}}

Tensor names: embed, head, final.norm, and per layer l<i>.norm1, l<i>.norm2, l<i>.mix.*, l<i>.mlp.* (experts
l<i>.mlp.e<j>.*), l<i>.hc<q>.{in, out, mix}, l<i>.rg<q>, l<i>.rg<q>.b, l<i>.shift; a bias is the matrix's name with ".b".

Fixed by the architecture: the norms' tensors hold the gains less one (but the plain gains of the low-rank vector's norm and
of the delta rule's output norm); the token shift in front of every mixer and the gates on every sublayer's result;
rotation of neighbouring pairs over the whole rotated part; the decay's constant exp(-1/2) and the unit key's 1e-6.
"""
from __future__ import annotations

import copy
import math
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .base import (ConfigError, LayerSpec, ModelConfig, ModelSpec, PartSpec, ScheduleEntry, read_key, require_positive)

_LATENT_NAMES = {"q": "q", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk", "uv": "uv", "o": "o", "g": "g"}
_MLP_NAMES = {"gate": "gate", "up": "up", "down": "down"}
_LATENT_TYPES = ("latent_attention", "latent_attention_2")

DECAY_SCALE = math.exp(-0.5)    # decay = exp(-DECAY_SCALE * sigmoid(logit))
UNIT_KEY_EPS = 1e-6
DEFAULT_DECAY_RANK = 16         # where neither a tensor nor the configuration says it (a model with random weights)


def _sub(d: Dict[str, Any], key: str, where: str, optional: bool = False) -> Optional[Dict[str, Any]]:
    v = d.get(key)
    if v is None:
        if optional:
            return None
        raise ConfigError(f"{where}: required key '{key}' is missing")
    if not isinstance(v, dict):
        raise ConfigError(f"{where}: key '{key}' must be an object, got {v!r}")
    return v


@dataclass
class KigalixConfig(ModelConfig):
    vocab: int
    width: int
    norm_eps: float
    layers: List[Dict[str, Any]]
    streams: Optional[int] = None         # None: config.json has no 'streams' (one stream, no learned numbers)
    max_positions: int = 1 << 20          # the design sets no limit; the engine's max_seq_len bounds what is run
    eos_token_id: List[int] = field(default_factory=list)

    architecture = "Kigalix"

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "KigalixConfig":
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers or not all(isinstance(x, dict) for x in layers):
            raise ConfigError("config.json: key 'layers' must be a non-empty list of objects")
        eos = d.get("eos_token_id")
        eos_list = [] if eos is None else ([eos] if isinstance(eos, int) else list(eos))
        cfg = cls(
            vocab=read_key(d, "vocab", int),
            width=read_key(d, "width", int),
            norm_eps=read_key(_sub(d, "norm", "config.json"), "eps", float, where="config.json: norm"),
            layers=copy.deepcopy(layers),
            streams=read_key(d, "streams", int, None),
            max_positions=read_key(d, "max_positions", int, 1 << 20),
            eos_token_id=eos_list,
        )
        cfg.check()
        return cfg

    # ------------------------------------------------------------------
    def check(self) -> None:
        require_positive("vocab", self.vocab)
        require_positive("width", self.width)
        require_positive("norm.eps", self.norm_eps)
        if self.streams is not None and not 1 <= self.streams <= 8:
            raise ConfigError(f"config.json: streams {self.streams} (1 to 8)")
        for i, L in enumerate(self.layers):
            where = f"config.json: layers[{i}]"
            kind = read_key(L, "type", str, where=where)
            m = _sub(L, "mixer", where)
            mw = where + ".mixer"
            for key in ("heads", "dim"):
                require_positive(f"layers[{i}].mixer.{key}", read_key(m, key, int, where=mw))
            if kind in _LATENT_TYPES:
                for key in ("vdim", "kv_rank"):
                    require_positive(f"layers[{i}].mixer.{key}", read_key(m, key, int, where=mw))
                require_positive(f"layers[{i}].mixer.scale", read_key(m, "scale", float, where=mw))
                rot_dim = read_key(m, "rot_dim", int, where=mw)
                if rot_dim < 0 or rot_dim % 2:
                    raise ConfigError(f"{mw}: rot_dim {rot_dim} must be even and not negative")
                rot = _sub(m, "rot", mw, optional=rot_dim == 0)
                if rot is not None and rot_dim:
                    dims = read_key(rot, "dims", int, where=mw + ".rot")
                    if dims <= 0 or dims % 2 or dims > rot_dim:
                        raise ConfigError(f"{mw}.rot: dims {dims} must be even, positive and at most rot_dim {rot_dim}")
                    require_positive(f"layers[{i}].mixer.rot.base", read_key(rot, "base", float, where=mw + ".rot"))
                    sc = _sub(rot, "scaling", mw + ".rot", optional=True)
                    if sc is not None:
                        for key in ("factor", "original", "fast", "slow"):
                            require_positive(f"layers[{i}].mixer.rot.scaling.{key}",
                                             read_key(sc, key, float, where=mw + ".rot.scaling"))
            elif kind == "general_delta":
                rank = read_key(m, "decay_rank", int, None, where=mw)
                if rank is not None:
                    require_positive(f"layers[{i}].mixer.decay_rank", rank)
            else:
                raise ConfigError(f"{where}: mixer type '{kind}' is not known ('latent_attention', 'latent_attention_2' "
                                  f"and 'general_delta' are)")
            mlp = _sub(L, "mlp", where, optional=True)
            if mlp is not None:
                mk = read_key(mlp, "kind", str, where=where + ".mlp")
                if mk == "dense":
                    require_positive(f"layers[{i}].mlp.ff", read_key(mlp, "ff", int, where=where + ".mlp"))
                elif mk == "moe":
                    ex, ro = _sub(mlp, "expert", where + ".mlp"), _sub(mlp, "router", where + ".mlp")
                    require_positive(f"layers[{i}].mlp.expert.ff", read_key(ex, "ff", int, where=where + ".mlp.expert"))
                    n = read_key(ro, "experts", int, where=where + ".mlp.router")
                    top = read_key(ro, "top", int, where=where + ".mlp.router")
                    if not 1 <= top <= n:
                        raise ConfigError(f"{where}.mlp.router: top {top} of {n} experts")
                else:
                    raise ConfigError(f"{where}.mlp: kind '{mk}' is not known ('dense' and 'moe' are)")

    def take_tensor_shapes(self, shapes: Dict[str, Any]) -> None:
        """The size of a delta layer's low-rank decay projection is the number of rows of its tensor mix.w1."""
        for i, L in enumerate(self.layers):
            if L["type"] == "general_delta":
                shape = shapes.get(f"l{i}.mix.w1")
                if shape is not None and len(shape) == 2:
                    said = L["mixer"].get("decay_rank")
                    if said is not None and int(said) != int(shape[0]):
                        raise ConfigError(f"config.json: layers[{i}].mixer.decay_rank is {said}, the tensor l{i}.mix.w1 has "
                                          f"{shape[0]} rows")
                    L["mixer"]["decay_rank"] = int(shape[0])

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {
            "architecture": self.architecture, "vocab": self.vocab, "width": self.width,
            "norm": {"eps": self.norm_eps}, "layers": copy.deepcopy(self.layers),
        }
        if self.streams is not None:
            d["streams"] = self.streams
        if self.max_positions != 1 << 20:
            d["max_positions"] = self.max_positions
        if self.eos_token_id:
            d["eos_token_id"] = list(self.eos_token_id)
        return d

    # ------------------------------------------------------------------
    def _mixer_spec(self, L: Dict[str, Any]) -> PartSpec:
        m = L["mixer"]
        if L["type"] in _LATENT_TYPES:
            rot = m.get("rot")
            position = None
            if rot is not None and int(m["rot_dim"]) > 0:
                sc = rot.get("scaling")
                scaling = {k: float(sc[k]) for k in ("factor", "original", "fast", "slow")} if sc else None
                position = PartSpec("rotary", {"theta": float(rot["base"]), "dim": int(rot["dims"]), "scaling": scaling})
            return PartSpec("latent_attention", {
                "num_heads": int(m["heads"]), "plain_dim": int(m["dim"]), "rot_dim": int(m["rot_dim"]),
                "value_dim": int(m["vdim"]), "rank": int(m["kv_rank"]), "norm_eps": self.norm_eps, "position": position,
                "scale": float(m["scale"]), "window": 0, "sink": False, "out_gate": L["type"] == "latent_attention_2",
                "rot_pairs": "neighbours", "names": dict(_LATENT_NAMES), "prefix": "mix.",
            })
        return PartSpec("general_delta", {
            "num_heads": int(m["heads"]), "key_dim": int(m["dim"]), "decay_rank": int(m.get("decay_rank") or DEFAULT_DECAY_RANK),
            "norm_eps": self.norm_eps, "decay_scale": DECAY_SCALE, "key_eps": UNIT_KEY_EPS, "prefix": "mix.",
        })

    def _mlp_spec(self, mlp: Dict[str, Any]) -> PartSpec:
        if mlp["kind"] == "dense":
            return PartSpec("gated_mlp", {"intermediate_size": int(mlp["ff"]), "activation": "gelu_tanh",
                                          "names": dict(_MLP_NAMES), "weight_suffix": "", "prefix": "mlp."})
        return PartSpec("expert_mixture", {
            "num_experts": int(mlp["router"]["experts"]), "top": int(mlp["router"]["top"]),
            "intermediate_size": int(mlp["expert"]["ff"]), "score": "sigmoid", "renormalize": False, "weight_on": "input",
            "activation": "silu", "prefix": "mlp.",
        })

    def to_spec(self) -> ModelSpec:
        layers = []
        learned = self.streams is not None
        n_streams = self.streams if learned else 1
        for i, L in enumerate(self.layers):
            mlp = L.get("mlp")
            norms = {"input": PartSpec("rmsnorm", {"eps": self.norm_eps, "name": "norm1", "unit_offset": True})}
            ffn = None
            if mlp is not None:
                norms["post_mixer"] = PartSpec("rmsnorm", {"eps": self.norm_eps, "name": "norm2", "unit_offset": True})
                ffn = self._mlp_spec(mlp)
            block = PartSpec("hyper", {"streams": n_streams, "learned_streams": learned, "token_shift": True,
                                       "residual_gate": True})
            layers.append(LayerSpec(block=block, mixer=self._mixer_spec(L), feed_forward=ffn, norms=norms, prefix=f"l{i}."))
        spec = ModelSpec(
            architecture=self.architecture,
            vocab_size=self.vocab,
            hidden_size=self.width,
            embedding=PartSpec("embedding", {"name": "embed"}),
            layers=layers,
            schedule=[ScheduleEntry(i) for i in range(len(layers))],
            final_norm=PartSpec("rmsnorm", {"eps": self.norm_eps, "name": "final.norm", "unit_offset": True}),
            head=PartSpec("linear_head", {"name": "head", "tied_to": None}),
            max_positions=self.max_positions,
            eos_token_ids=list(self.eos_token_id),
            streams=n_streams,
        )
        spec.validate()
        return spec
