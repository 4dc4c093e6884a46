"""Small Kigalix configurations, weights that make every mechanism matter, and the comparison of logits with the
plain implementation (plain_kigalix.py)."""
from __future__ import annotations

import copy
import json
import os
from typing import Dict, List

import numpy as np
import torch

import plain_kigalix as pk

# root mean square of a row's error (its mean taken off) over the root mean square of the row's logits (theirs too)
TOL = {"float32": 5e-5, "bfloat16": 3e-2}
# bfloat16: a token whose choice of experts hangs on less than this (in units of its router logits' spread) may go to
# other experts in the engine than in the plain implementation, which rounds nothing, and every later token of its
# sequence reads what it left: a sequence is compared up to its first such token (float32 compares everything, and
# `without_experts` gives the same layers with dense feed-forwards, which bfloat16 compares to the end)
CLOSE_CALL = 0.15


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def latent_layer(heads=4, dim=16, rot_dim=16, vdim=24, rank=32, scale=0.2, base=10000.0, scaling=None, gated=False, mlp=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": scale}
    if rot_dim:
        m["rot"] = {"dims": rot_dim, "base": base}
        if scaling:
            m["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return {"type": "latent_attention_2" if gated else "latent_attention", "mixer": m, "mlp": mlp}


def delta_layer(heads=2, dim=16, rank=8, mlp=None):
    return {"type": "general_delta", "mixer": {"heads": heads, "dim": dim, "decay_rank": rank}, "mlp": mlp}


# three streams; a delta layer first with a key size that is no multiple of 16 and experts of which two are chosen; latent
# layers whose cache suits the matrix-core kernels (32 + 16) and one whose sizes are no multiples of 16, with stretched
# frequencies; a layer without a feed-forward; one head with a state of 64 x 64
CFG_A = {"architecture": "Kigalix", "vocab": 211, "width": 96, "streams": 3, "norm": {"eps": 1e-5},
         "layers": [delta_layer(heads=3, dim=20, rank=12, mlp=moe(5, 2, 40)),
                    latent_layer(heads=4, dim=16, rot_dim=16, vdim=24, rank=32, mlp=dense(80)),
                    latent_layer(heads=3, dim=20, rot_dim=12, vdim=10, rank=24, scaling=(4.0, 64, 16.0, 2.0), gated=True),
                    delta_layer(heads=1, dim=64, rank=4, mlp=dense(56)),
                    latent_layer(heads=8, dim=8, rot_dim=32, vdim=16, rank=32, base=500.0, scaling=(8.0, 32, 4.0, 1.0),
                                 gated=True, mlp=moe(3, 1, 64))]}
# one stream with learned numbers; a latent layer first; every expert chosen; nothing rotated in one layer
CFG_B = {"architecture": "Kigalix", "vocab": 131, "width": 80, "streams": 1, "norm": {"eps": 1e-6},
         "layers": [latent_layer(heads=1, dim=8, rot_dim=16, vdim=8, rank=16, mlp=moe(4, 4, 24)),
                    delta_layer(heads=5, dim=16, rank=16, mlp=moe(9, 3, 32)),
                    latent_layer(heads=2, dim=24, rot_dim=0, vdim=40, rank=48, gated=True, mlp=dense(112))]}
# no 'streams' at all (the plain residual sum); four streams is CFG_D
CFG_C = {"architecture": "Kigalix", "vocab": 97, "width": 64, "norm": {"eps": 1e-5},
         "layers": [delta_layer(heads=2, dim=32, rank=8, mlp=dense(96)),
                    latent_layer(heads=2, dim=16, rot_dim=8, vdim=16, rank=40, mlp=moe(6, 2, 48))]}
CFG_D = {"architecture": "Kigalix", "vocab": 150, "width": 128, "streams": 4, "norm": {"eps": 1e-6},
         "layers": [latent_layer(heads=16, dim=16, rot_dim=32, vdim=8, rank=32, gated=True, scaling=(2.0, 40, 8.0, 1.0),
                                 mlp=moe(16, 4, 16)),
                    delta_layer(heads=2, dim=128, rank=32, mlp=moe(2, 1, 200))]}
CONFIGS = {"A": CFG_A, "B": CFG_B, "C": CFG_C, "D": CFG_D}


def without_experts(cfg: dict) -> dict:
    """The same model with a dense feed-forward of a token's experts' size wherever it has a mixture of experts."""
    cfg = copy.deepcopy(cfg)
    for layer in cfg["layers"]:
        mlp = layer.get("mlp")
        if mlp is not None and mlp["kind"] == "moe":
            layer["mlp"] = dense(mlp["expert"]["ff"] * mlp["router"]["top"])
    return cfg


def make_weights(cfg: dict, seed: int, idle: bool = False) -> Dict[str, torch.Tensor]:
    """Weights at scales at which every mechanism shows in the logits (projections that keep activations near 1,
    streams that are read, written and mixed with numbers well away from 0 and 1, shifts between 0 and 1, routers that
    spread their scores, gains away from 1), rounded to bfloat16.  idle: also the second sublayer's tensors of layers
    without a feed-forward, which a model tolerates and does not read."""
    from vt_transformer_amd.config import config_from_dict
    from vt_transformer_amd.weights.random_init import declared_tensors
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, decl in declared_tensors(config_from_dict(copy.deepcopy(cfg))).items():
        shape = tuple(decl.shape)
        leaf = name.split(".")[-1]
        if decl.optional and not idle:
            continue
        if leaf == "shift":
            t = torch.rand(shape, generator=g)
        elif decl.role == "stream_mix":
            t = torch.eye(shape[0]) * 0.8 + torch.randn(shape, generator=g) * 0.25
        elif ".hc" in name:
            t = 0.4 + torch.rand(shape, generator=g) * 0.9
        elif decl.role == "matrix32":
            t = torch.randn(shape, generator=g) * 2.0 / shape[-1] ** 0.5
        elif decl.role == "gain":
            t = 1.0 + torch.randn(shape, generator=g) * 0.3
        elif decl.role == "bias":
            t = torch.randn(shape, generator=g) * (0.8 if leaf in ("w0", "b") else 0.3)
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        elif leaf in ("w1", "w2"):
            t = torch.randn(shape, generator=g) * 2.0 / shape[-1] ** 0.5
        else:
            t = torch.randn(shape, generator=g) / shape[-1] ** 0.5
        out[name] = t.to(torch.bfloat16)
    return out


def write_model(cfg: dict, folder: str, seed: int, keep_rank: bool = False, idle: bool = False) -> str:
    """config.json without the delta layers' `decay_rank` (the tensors say it) unless keep_rank."""
    from vt_transformer_amd.weights.safetensors_io import write_safetensors
    os.makedirs(folder, exist_ok=True)
    weights = make_weights(cfg, seed, idle)
    cfg = copy.deepcopy(cfg)
    if not keep_rank:
        for layer in cfg["layers"]:
            layer["mixer"].pop("decay_rank", None)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_safetensors(os.path.join(folder, "model.safetensors"), weights.items(), metadata={"format": "pt"})
    return folder


def _row_errors(got: np.ndarray, ref: np.ndarray) -> np.ndarray:
    """Per row: root mean square of the difference (its mean taken off) over that of the reference (its mean too)."""
    d = got.astype(np.float64) - ref
    d = d - d.mean(axis=-1, keepdims=True)
    c = ref - ref.mean(axis=-1, keepdims=True)
    return np.sqrt((d * d).mean(axis=-1)) / np.maximum(np.sqrt((c * c).mean(axis=-1)), 1e-30)


def check_logits(model_dir: str, reqs: Dict[str, List[int]], steps: List[dict], got: Dict[int, np.ndarray], dtype: str,
                 cache: dict = None) -> float:
    """Every wanted row against the plain implementation's logits at that place; raises at the first row beyond
    tolerance, naming step, request and position.  Returns the worst error."""
    cfg, w = pk.read_folder(model_dir)
    cache = cache if cache is not None else {}
    ref = {}
    close, limit = {}, {}
    for rid, toks in reqs.items():
        key = (model_dir, tuple(toks))
        if key not in cache:
            margins = []
            logits = pk.forward(cfg, w, toks, margins=margins).numpy()
            least = torch.stack(margins).min(dim=0).values.numpy() if margins else np.full(len(toks), np.inf)
            first = np.nonzero(least < CLOSE_CALL)[0]
            # what rounding alone does to every position of this model (a model of few channels and many heads, or a
            # delta layer whose output is divided by a size near zero, moves further than the tolerance): bfloat16 may
            # differ by three times that where it is more than the tolerance
            moved = _row_errors(pk.forward(cfg, w, toks, rounded=True).numpy(), logits)
            cache[key] = (logits, int(first[0]) if len(first) else len(toks), np.maximum(TOL["bfloat16"], 3.0 * moved))
        ref[rid], close[rid], limit[rid] = cache[key]
    pos = {r: 0 for r in reqs}
    worst, over, count, skipped, far = 0.0, 0, 0, 0, []
    for s in steps:
        row = 0
        for e in s["entries"]:
            for wi in e["want"]:
                p = pos[e["id"]] + wi
                r = ref[e["id"]][p]
                gl = got[s["step"]][row].astype(np.float64)
                assert np.isfinite(gl).all(), f"step {s['step']} request {e['id']} position {p}: logits are not finite"
                row += 1
                if dtype != "float32" and p >= close[e["id"]]:
                    skipped += 1
                    continue
                err = float(_row_errors(gl[None], r[None])[0])
                lim = TOL[dtype] if dtype == "float32" else float(limit[e["id"]][p])
                # float32: every position within the tolerance
                if dtype == "float32":
                    assert err < TOL[dtype], (f"step {s['step']} request {e['id']} position {p} "
                                              f"(portion starts at {pos[e['id']]}): error {err:.3e} > {TOL[dtype]:.1e}")
                elif err >= 1.5 * lim:
                    far.append((s["step"], e["id"], p, pos[e["id"]], round(err, 4), round(lim, 4)))
                over += err >= lim
                count += 1
                worst = max(worst, err)
            pos[e["id"]] += len(e["tokens"])
    # bfloat16: rounding alone moves a few positions a long way (a delta layer's output is divided by its size, which
    # the first tokens of a sequence can leave near zero), while a lost state, a missed key or a wrong edge moves every
    # position behind it: one position in ten may be over the tolerance, one in forty (or two) half again over it
    assert over <= max(2, count // 10), f"{over} of {count} positions are over their limit (worst {worst:.3e})"
    assert len(far) <= max(2, count // 40), f"{len(far)} of {count} positions are far over their limit: {far[:8]}"
    return worst
