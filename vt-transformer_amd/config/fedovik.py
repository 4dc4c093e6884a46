"""Fedovik: typed configuration read from the keys of its config.json.

A Fedovik model is a list of parallel layers around a float32 residual stream:
one layer norm (gain and bias) feeds the mixer and the feed-forward alike, and
their results join the stream in one sum.  Three mixers: "attention" (weights
that are sigmoids of the scores with a learned shift per head, neighbouring
elements rotated together, biases on every projection, an elementwise sigmoid
gate), "parallel" (two mixers side by side with a constant factor each:
windowed softmax attention with normed queries and keys and a bias that grows
with the logarithm of the distance, and a gated delta rule whose decay has one
factor per key channel) and "mlstm" (the matrix memory of xLSTM with capped
gates).  The feed-forward is a gated unit with ReLU.  A run of layers can be
repeated with shared weights; every pass has caches and state of its own and
starts from W_in [x; x0], the stream joined with the embedding's output, plus
its own row of `loop.step`.  The logits come from the embedding's table.

config.json:
  architecture            "Fedovik"
  vocab, width            sizes of the vocabulary and of the stream
  embedding.scale         factor on the embedding rows
  norm.eps                eps of every norm of the model (also of the mixers' own)
  layers[i].type          "attention" | "parallel" | "mlstm"
  layers[i].mixer         attention: heads, kv_heads, dim, vdim, scale, rot.{dims, base}
                          parallel:  left_scale, right_scale,
                                     left.{heads, kv_heads, dim, vdim, scale, mask.size},
                                     right.{heads, kv_heads, dim, vdim, conv} (and optionally a_rank, g_rank)
                          mlstm:     heads, dim, vdim, gate_cap
  layers[i].mlp           null | {kind: "dense", ff}
  loop                    null | {start, stop, times}

The sizes of the delta rule's two low-rank projections are the rows of its tensors a1 and g1; a config.json that is
written for random weights says them as right.a_rank and right.g_rank.

Tensor names: embed, final.norm, final.norm.b, loop.in, loop.step, and per layer l<i>.norm1, l<i>.norm1.b,
l<i>.mix.*, l<i>.mlp.*; a bias is the matrix's name with ".b", a convolution's taps the matrix's name with ".conv".

Fixed by the architecture: which projections have biases; rotation of neighbouring pairs; sigmoid gates; ReLU;
1e-6 inside the root of the delta rule's unit vectors and in the matrix memory's denominator (in the kernels).
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .base import (ConfigError, LayerSpec, ModelConfig, ModelSpec, PartSpec, ScheduleEntry, read_key, require_positive)

_ATTENTION_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "g": "g", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b",
                    "o_bias": "o.b", "shift": "pb"}
_LEFT_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b",
               "q_norm": "q.norm", "k_norm": "k.norm", "r1": "r1", "r2": "r2"}
_RIGHT_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv",
                "b": "b", "a1": "a1", "a2": "a2", "g1": "g1", "g2": "g2", "A_log": "A_log", "dt_bias": "dt_bias", "norm": "norm"}
_MEMORY_NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "i": "i", "f": "f", "i_bias": "i.b", "f_bias": "f.b",
                 "norm": "norm"}
_MLP_NAMES = {"gate": "gate", "up": "up", "down": "down"}


def _sub(d: Dict[str, Any], key: str, where: str, optional: bool = False) -> Optional[Dict[str, Any]]:
    v = d.get(key)
    if v is None:
        if optional:
            return None
        raise ConfigError(f"{where}: required key '{key}' is missing")
    if not isinstance(v, dict):
        raise ConfigError(f"{where}: key '{key}' must be an object, got {v!r}")
    return v


def _heads(m: Dict[str, Any], where: str, grouped: bool) -> None:
    heads = read_key(m, "heads", int, where=where)
    kv = read_key(m, "kv_heads", int, where=where) if grouped else heads
    for key in ("dim", "vdim"):
        require_positive(f"{where}.{key}", read_key(m, key, int, where=where))
    if heads <= 0 or kv <= 0 or heads % kv:
        raise ConfigError(f"{where}: heads {heads} must be a positive multiple of kv_heads {kv}")


@dataclass
class FedovikConfig(ModelConfig):
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    layers: List[Dict[str, Any]]
    loop: Optional[Dict[str, int]] = None
    max_positions: int = 1 << 20          # the design sets no limit; the engine's max_seq_len bounds what is run
    eos_token_id: List[int] = field(default_factory=list)

    architecture = "Fedovik"

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "FedovikConfig":
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers or not all(isinstance(x, dict) for x in layers):
            raise ConfigError("config.json: key 'layers' must be a non-empty list of objects")
        eos = d.get("eos_token_id")
        eos_list = [] if eos is None else ([eos] if isinstance(eos, int) else list(eos))
        cfg = cls(
            vocab=read_key(d, "vocab", int),
            width=read_key(d, "width", int),
            embedding_scale=read_key(_sub(d, "embedding", "config.json", optional=True) or {}, "scale", float, 1.0,
                                     where="config.json: embedding"),
            norm_eps=read_key(_sub(d, "norm", "config.json"), "eps", float, where="config.json: norm"),
            layers=copy.deepcopy(layers),
            loop=copy.deepcopy(_sub(d, "loop", "config.json", optional=True)),
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
        for i, L in enumerate(self.layers):
            where = f"config.json: layers[{i}]"
            kind = read_key(L, "type", str, where=where)
            m = _sub(L, "mixer", where)
            mw = where + ".mixer"
            if kind == "attention":
                _heads(m, mw, grouped=True)
                require_positive(f"layers[{i}].mixer.scale", read_key(m, "scale", float, where=mw))
                rot = _sub(m, "rot", mw, optional=True)
                if rot is not None:
                    dims = read_key(rot, "dims", int, where=mw + ".rot")
                    if dims <= 0 or dims % 2 or dims > m["dim"]:
                        raise ConfigError(f"{mw}.rot: dims {dims} must be even, positive and at most dim {m['dim']}")
                    require_positive(f"layers[{i}].mixer.rot.base", read_key(rot, "base", float, where=mw + ".rot"))
            elif kind == "parallel":
                left, right = _sub(m, "left", mw), _sub(m, "right", mw)
                _heads(left, mw + ".left", grouped=True)
                _heads(right, mw + ".right", grouped=True)
                require_positive(f"layers[{i}].mixer.left.scale", read_key(left, "scale", float, where=mw + ".left"))
                mask = _sub(left, "mask", mw + ".left", optional=True)
                if mask is not None:
                    require_positive(f"layers[{i}].mixer.left.mask.size", read_key(mask, "size", int, where=mw + ".left.mask"))
                require_positive(f"layers[{i}].mixer.right.conv", read_key(right, "conv", int, where=mw + ".right"))
                for key in ("a_rank", "g_rank"):
                    if right.get(key) is not None:
                        require_positive(f"layers[{i}].mixer.right.{key}", read_key(right, key, int, where=mw + ".right"))
                read_key(m, "left_scale", float, 1.0, where=mw)
                read_key(m, "right_scale", float, 1.0, where=mw)
            elif kind == "mlstm":
                _heads(m, mw, grouped=False)
                if read_key(m, "gate_cap", float, 0.0, where=mw) < 0:
                    raise ConfigError(f"{mw}: gate_cap must not be negative")
            else:
                raise ConfigError(f"{where}: mixer type '{kind}' is not known ('attention', 'parallel' and 'mlstm' are)")
            mlp = _sub(L, "mlp", where, optional=True)
            if mlp is not None:
                if read_key(mlp, "kind", str, "dense", where=where + ".mlp") != "dense":
                    raise ConfigError(f"{where}.mlp: kind '{mlp['kind']}' is not known ('dense' is)")
                require_positive(f"layers[{i}].mlp.ff", read_key(mlp, "ff", int, where=where + ".mlp"))
        if self.loop is not None:
            a, b = read_key(self.loop, "start", int, where="config.json: loop"), read_key(self.loop, "stop", int, where="config.json: loop")
            t = read_key(self.loop, "times", int, where="config.json: loop")
            if not (0 <= a < b <= len(self.layers)) or t < 1:
                raise ConfigError(f"config.json: loop {self.loop!r} does not name a run of the {len(self.layers)} layers "
                                  f"(0 <= start < stop <= layers, times >= 1)")

    def take_tensor_shapes(self, shapes: Dict[str, Any]) -> None:
        """The sizes of a delta rule's low-rank projections are the rows of its tensors a1 (decay) and g1 (gate)."""
        for i, L in enumerate(self.layers):
            if L["type"] != "parallel":
                continue
            right = L["mixer"]["right"]
            for key, tensor in (("a_rank", f"l{i}.mix.right.a1"), ("g_rank", f"l{i}.mix.right.g1")):
                shape = shapes.get(tensor)
                if shape is not None and len(shape) == 2:
                    said = right.get(key)
                    if said is not None and int(said) != int(shape[0]):
                        raise ConfigError(f"config.json: layers[{i}].mixer.right.{key} is {said}, the tensor {tensor} has "
                                          f"{shape[0]} rows")
                    right[key] = int(shape[0])

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {
            "architecture": self.architecture, "vocab": self.vocab, "width": self.width,
            "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps},
            "layers": copy.deepcopy(self.layers), "loop": copy.deepcopy(self.loop),
        }
        if self.max_positions != 1 << 20:
            d["max_positions"] = self.max_positions
        if self.eos_token_id:
            d["eos_token_id"] = list(self.eos_token_id)
        return d

    # ------------------------------------------------------------------
    def _mixer_spec(self, i: int, L: Dict[str, Any]) -> PartSpec:
        m = L["mixer"]
        if L["type"] == "attention":
            rot = m.get("rot")
            position = PartSpec("rotary", {"theta": float(rot["base"]), "dim": int(rot["dims"]), "scaling": None}) if rot else None
            return PartSpec("masked_attention", {
                "num_heads": int(m["heads"]), "num_kv_heads": int(m["kv_heads"]), "key_dim": int(m["dim"]),
                "value_dim": int(m["vdim"]), "qkv_bias": True, "o_bias": True, "position": position,
                "rot_pairs": "neighbours", "scale": float(m["scale"]), "weights": "sigmoid", "score_shift": True,
                "out_gate": True, "names": dict(_ATTENTION_NAMES), "prefix": "mix.",
            })
        if L["type"] == "mlstm":
            return PartSpec("matrix_memory", {
                "num_heads": int(m["heads"]), "key_dim": int(m["dim"]), "value_dim": int(m["vdim"]),
                "gate_cap": float(m.get("gate_cap") or 0.0), "norm_eps": self.norm_eps, "names": dict(_MEMORY_NAMES),
                "prefix": "mix.",
            })
        left, right = m["left"], m["right"]
        if right.get("a_rank") is None or right.get("g_rank") is None:
            raise ConfigError(f"config.json: layers[{i}].mixer.right: the sizes of the low-rank projections are not known "
                              f"(the tensors l{i}.mix.right.a1 and g1 give them, or the keys a_rank and g_rank)")
        mask = left.get("mask")
        left_spec = PartSpec("masked_attention", {
            "num_heads": int(left["heads"]), "num_kv_heads": int(left["kv_heads"]), "key_dim": int(left["dim"]),
            "value_dim": int(left["vdim"]), "qkv_bias": True, "position": None, "scale": float(left["scale"]),
            "window": int(mask["size"]) if mask else 0, "unit_rms_eps": self.norm_eps, "qk_gain": True, "distance_log": True,
            "names": dict(_LEFT_NAMES), "prefix": "left.",
        })
        right_spec = PartSpec("gated_delta", {
            "num_heads": int(right["heads"]), "num_kv_heads": int(right["kv_heads"]), "key_dim": int(right["dim"]),
            "value_dim": int(right["vdim"]), "conv_taps": int(right["conv"]), "norm_eps": self.norm_eps,
            "decay": "channel", "decay_rank": int(right["a_rank"]), "gate_rank": int(right["g_rank"]), "gate_act": "sigmoid",
            "names": dict(_RIGHT_NAMES), "prefix": "right.",
        })
        return PartSpec("mixer_pair", {"left": left_spec, "right": right_spec, "left_scale": float(m.get("left_scale", 1.0)),
                                       "right_scale": float(m.get("right_scale", 1.0)), "prefix": "mix."})

    def run_order(self) -> List[ScheduleEntry]:
        """The layers in the order they run: those in front of the loop, the looped run `times` times (each pass
        opens by re-entering the embedding's output and adding its row of the offsets), the rest."""
        n = len(self.layers)
        if self.loop is None:
            return [ScheduleEntry(i) for i in range(n)]
        a, b, times = int(self.loop["start"]), int(self.loop["stop"]), int(self.loop["times"])
        order = [ScheduleEntry(i) for i in range(a)]
        for t in range(times):
            order += [ScheduleEntry(i, offset_row=t if i == a else None, inject=i == a) for i in range(a, b)]
        return order + [ScheduleEntry(i) for i in range(b, n)]

    def to_spec(self) -> ModelSpec:
        layers = []
        for i, L in enumerate(self.layers):
            mlp = L.get("mlp")
            norms = {"input": PartSpec("layernorm", {"eps": self.norm_eps, "name": "norm1", "bias_name": "norm1.b"})}
            ffn = None
            if mlp is not None:
                ffn = PartSpec("gated_mlp", {"intermediate_size": int(mlp["ff"]), "activation": "relu",
                                             "names": dict(_MLP_NAMES), "weight_suffix": "", "prefix": "mlp."})
            layers.append(LayerSpec(block=PartSpec("parallel", {}), mixer=self._mixer_spec(i, L), feed_forward=ffn,
                                    norms=norms, prefix=f"l{i}."))
        looped = self.loop is not None
        spec = ModelSpec(
            architecture=self.architecture,
            vocab_size=self.vocab,
            hidden_size=self.width,
            embedding=PartSpec("embedding", {"name": "embed", "scale": self.embedding_scale}),
            layers=layers,
            schedule=self.run_order(),
            final_norm=PartSpec("layernorm", {"eps": self.norm_eps, "name": "final.norm", "bias_name": "final.norm.b"}),
            head=PartSpec("linear_head", {"name": "head", "tied_to": "embed"}),
            max_positions=self.max_positions,
            eos_token_ids=list(self.eos_token_id),
            stream_offsets={"name": "loop.step", "rows": int(self.loop["times"])} if looped else None,
            stream_inject={"name": "loop.in"} if looped else None,
        )
        spec.validate()
        return spec
