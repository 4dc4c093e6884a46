"""Small Fedovik configurations, weights that make every mechanism matter, and the comparison of logits with the
plain implementation (plain_fedovik.py)."""
from __future__ import annotations

import copy
import json
import os
from typing import Dict, List

import numpy as np
import torch

import plain_fedovik as pf

# root mean square of a row's error (its mean taken off) over the root mean square of the row's logits (theirs too):
# bfloat16 rounds every activation to eight bits, about 4e-3 each, through up to eleven layer runs of these weights
TOL = {"float32": 4e-5, "bfloat16": 4e-2}


def _mlp(ff):
    return {"kind": "dense", "ff": ff} if ff else None


def attention_layer(heads=4, kv_heads=2, dim=32, vdim=48, scale=0.2, rot_dims=8, base=10000.0, ff=None):
    return {"type": "attention",
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
                      "rot": {"dims": rot_dims, "base": base}},
            "mlp": _mlp(ff)}


def pair_layer(heads=4, kv_heads=2, dim=16, vdim=24, scale=0.3, window=12, r_heads=2, r_kv=1, r_dim=16, r_vdim=24, conv=3,
               a_rank=6, g_rank=5, left_scale=0.8, right_scale=1.3, ff=None):
    return {"type": "parallel",
            "mixer": {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
                               "mask": {"size": window}},
                      "right": {"heads": r_heads, "kv_heads": r_kv, "dim": r_dim, "vdim": r_vdim, "conv": conv,
                                "a_rank": a_rank, "g_rank": g_rank},
                      "left_scale": left_scale, "right_scale": right_scale},
            "mlp": _mlp(ff)}


def memory_layer(heads=2, dim=16, vdim=24, gate_cap=12.0, ff=None):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": gate_cap}, "mlp": _mlp(ff)}


# a loop from layer 0 run three times with the pair first, grouped heads everywhere, a window that is no multiple of a
# page, a layer without a feed-forward
CFG_A = {"architecture": "Fedovik", "vocab": 203, "width": 96, "embedding": {"scale": 2.5}, "norm": {"eps": 1e-5},
         "layers": [pair_layer(ff=80), memory_layer(ff=64), attention_layer(ff=72), memory_layer(heads=3, dim=20, vdim=8)],
         "loop": {"start": 0, "stop": 2, "times": 3}}
# no loop; as many key heads as query heads and one key head for all; the whole head rotated; a window of one
# position and one longer than the requests; two taps; scales, embedding factor and mixing factors of 1
CFG_B = {"architecture": "Fedovik", "vocab": 131, "width": 80, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-6},
         "layers": [attention_layer(heads=3, kv_heads=3, dim=16, vdim=16, scale=1.0, rot_dims=16, base=500.0, ff=112),
                    pair_layer(heads=3, kv_heads=3, dim=8, vdim=40, scale=1.0, window=1, r_heads=3, r_kv=3, r_dim=64,
                               r_vdim=16, conv=2, a_rank=1, g_rank=12, left_scale=1.0, right_scale=1.0, ff=64),
                    attention_layer(heads=5, kv_heads=1, dim=48, vdim=80, scale=0.05, rot_dims=24),
                    memory_layer(heads=1, dim=8, vdim=8, gate_cap=4.0, ff=48),
                    pair_layer(heads=2, kv_heads=1, dim=64, vdim=16, window=500, r_heads=1, r_kv=1, r_dim=8, r_vdim=8, conv=4)],
         "loop": None}
# a loop in the middle that runs once, then layers behind it; heads in multiples of 16 (the matrix-core kernels)
CFG_C = {"architecture": "Fedovik", "vocab": 97, "width": 64, "embedding": {"scale": 6.0}, "norm": {"eps": 1e-5},
         "layers": [attention_layer(heads=2, kv_heads=1, dim=32, vdim=16, rot_dims=4, ff=96),
                    pair_layer(heads=4, kv_heads=1, dim=16, vdim=32, window=33, r_heads=4, r_kv=4, r_dim=12, r_vdim=20, conv=4),
                    memory_layer(heads=4, dim=12, vdim=20, ff=48)],
         "loop": {"start": 1, "stop": 2, "times": 1}}
CONFIGS = {"A": CFG_A, "B": CFG_B, "C": CFG_C}


def make_weights(cfg: dict, seed: int) -> Dict[str, torch.Tensor]:
    """Weights at scales at which every mechanism shows in the logits (projections that keep activations near 1,
    biases, decays spread between 0.5 and 0.999, shifts that keep a sum of sigmoids over many keys near 1, forget gates
    that mostly keep, gains away from 1), rounded to bfloat16."""
    from vt_transformer_amd.config import config_from_dict
    from vt_transformer_amd.weights.random_init import declared_tensors
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, decl in declared_tensors(config_from_dict(copy.deepcopy(cfg))).items():
        if decl.optional:
            continue            # (a tied head has no tensor of its own)
        shape = tuple(decl.shape)
        leaf = name.split(".")[-1]
        tail = ".".join(name.split(".")[-2:])
        if leaf == "A_log":
            t = torch.log(torch.rand(shape, generator=g) * 2.0 + 0.01)
        elif leaf == "dt_bias":
            t = torch.randn(shape, generator=g) * 1.0 - 2.0
        elif leaf == "conv":
            t = torch.randn(shape, generator=g) * 0.6
        elif leaf == "step":
            t = torch.randn(shape, generator=g) * 0.5
        elif leaf == "pb":
            t = torch.randn(shape, generator=g) * 0.5 - 3.5
        elif leaf == "r1":
            t = torch.rand(shape, generator=g) * 2.0
        elif leaf == "r2":
            t = torch.rand(shape, generator=g) * 0.6 + 0.02
        elif tail == "f.b":
            t = torch.rand(shape, generator=g) * 4.0 + 1.0
        elif decl.role == "gain":
            t = 1.0 + torch.randn(shape, generator=g) * 0.3
        elif decl.role == "bias":
            t = torch.randn(shape, generator=g) * 0.3
        elif name == "embed":
            t = torch.randn(shape, generator=g) * 0.5
        else:
            t = torch.randn(shape, generator=g) / shape[-1] ** 0.5
        out[name] = t.to(torch.bfloat16)
    return out


def write_model(cfg: dict, folder: str, seed: int, keep_ranks: bool = False) -> str:
    """The folder as a checkpoint has it: the sizes of the low-rank projections are not in config.json (the tensors'
    shapes say them) unless keep_ranks."""
    from vt_transformer_amd.weights.safetensors_io import write_safetensors
    os.makedirs(folder, exist_ok=True)
    weights = make_weights(cfg, seed)
    stored = copy.deepcopy(cfg)
    if not keep_ranks:
        for L in stored["layers"]:
            if L["type"] == "parallel":
                L["mixer"]["right"].pop("a_rank", None)
                L["mixer"]["right"].pop("g_rank", None)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(stored, f)
    write_safetensors(os.path.join(folder, "model.safetensors"), weights.items(), metadata={"format": "pt"})
    return folder


def row_error(got: np.ndarray, ref: np.ndarray) -> float:
    diff = got.astype(np.float64) - ref
    return float(np.sqrt(np.mean((diff - diff.mean()) ** 2)) / max(np.sqrt(np.mean((ref - ref.mean()) ** 2)), 1e-30))


def check_logits(model_dir: str, reqs: Dict[str, List[int]], steps: List[dict], got: Dict[int, np.ndarray], dtype: str,
                 cache: dict = None) -> float:
    """Every wanted row against the plain implementation's logits at that place; raises at the first row beyond
    tolerance, naming step, request and position.  Returns the worst error."""
    cfg, w = pf.read_folder(model_dir)
    cache = cache if cache is not None else {}
    ref, limit = {}, {}
    for rid, toks in reqs.items():
        key = (model_dir, tuple(toks))
        if key not in cache:
            logits = pf.forward(cfg, w, toks).numpy()
            # what rounding alone does to every position of this model (a recurrent layer's read-out is divided by its
            # size, which the first tokens of a sequence can leave near zero; a normalizer can cancel): bfloat16 may
            # differ by three times that where it is more than the tolerance
            moved = np.array([row_error(a, b) for a, b in zip(pf.forward(cfg, w, toks, rounded=True).numpy(), logits)])
            cache[key] = (logits, np.maximum(TOL["bfloat16"], 3.0 * moved))
        ref[rid], limit[rid] = cache[key]
    pos = {r: 0 for r in reqs}
    worst, over, count, far = 0.0, 0, 0, []
    for s in steps:
        row = 0
        for e in s["entries"]:
            for wi in e["want"]:
                p = pos[e["id"]] + wi
                gl = got[s["step"]][row]
                assert np.isfinite(gl).all(), f"step {s['step']} request {e['id']} position {p}: logits are not finite"
                err = row_error(gl, ref[e["id"]][p])
                row += 1
                if dtype == "float32":
                    # every position within the tolerance
                    assert err < TOL[dtype], (f"step {s['step']} request {e['id']} position {p} "
                                              f"(portion starts at {pos[e['id']]}): error {err:.3e} > {TOL[dtype]:.1e}")
                else:
                    lim = float(limit[e["id"]][p])
                    over += err >= lim
                    if err >= 1.5 * lim:
                        far.append((s["step"], e["id"], p, pos[e["id"]], round(err, 4), round(lim, 4)))
                count += 1
                worst = max(worst, err)
            pos[e["id"]] += len(e["tokens"])
    # bfloat16: rounding alone moves a few positions a long way, while a lost state, a missed key or a wrong edge moves
    # every position behind it: one position in twenty (or two) may be over its limit, one in fifty (or one) half again
    assert over <= max(2, count // 20), f"{over} of {count} positions are over their limit (worst {worst:.3e})"
    assert len(far) <= max(1, count // 50), f"{len(far)} of {count} positions are far over their limit: {far[:8]}"
    return worst
