"""Plain, slow implementation of the Kigalix decoder: whole sequences, no
cache, one function per mechanism, in float64 on the CPU.  It shares no code
with the engine; the tests compare the engine against it.

Kigalix keeps several copies of the residual stream ("streams").  A sublayer
reads a weighted sum of them, and its result, times a sigmoid gate computed
from the sublayer's input, goes back into every stream with a weight of its
own while the streams are mixed among themselves by a small matrix.  A mixer
reads its normed input blended with the previous token's.  Three mixers:
latent attention (one low-rank vector and one rotated key part per token,
rotation of neighbouring pairs), the same with stretched frequencies and an
elementwise output gate, and a generalized delta rule with a matrix state per
head, a decay per key channel and a removal along the unit key.  The
feed-forward is dense (tanh-form GELU gate) or a mixture of experts whose
router's sigmoid scores scale the chosen experts' inputs.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

from plain_model import read_folder  # noqa: F401  (own safetensors reader of the tests)

DT = torch.float64

DECAY_SCALE = math.exp(-0.5)
UNIT_KEY_EPS = 1e-6


def offset_rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) * (1 + w): what is stored is the gain less one."""
    return x * torch.rsqrt((x * x).mean(dim=-1, keepdim=True) + eps) * (1.0 + w)


def plain_rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return x * torch.rsqrt((x * x).mean(dim=-1, keepdim=True) + eps) * w


def token_shift(h: torch.Tensor, mu: torch.Tensor) -> torch.Tensor:
    """h [T, width]: every token blended with the one before it (zeros before the first), h + (h_prev - h) mu."""
    prev = torch.cat([torch.zeros_like(h[:1]), h[:-1]], dim=0)
    return h + (prev - h) * mu


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def pair_frequencies(dims: int, base: float, scaling: Optional[dict]):
    """Frequencies of the dims/2 rotated pairs and the factor on cosine and sine."""
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    mag = 1.0
    if scaling:
        factor, orig = float(scaling["factor"]), float(scaling["original"])

        def index_of(turns):
            return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
        lo = max(math.floor(index_of(float(scaling["fast"]))), 0)
        hi = min(math.ceil(index_of(float(scaling["slow"]))), dims - 1)
        out = []
        for i, fi in enumerate(f):
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            out.append(fi / factor * ramp + fi * (1.0 - ramp))
        f = out
        mag = 0.1 * math.log(factor) + 1.0
    return torch.tensor(f, dtype=DT), mag


def rotate_neighbours(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float, scaling: Optional[dict]) -> torch.Tensor:
    """x [T, ..., D]: among the first `dims` elements of the last axis, element 2i is rotated with element 2i + 1 by
    the angle position * f_i; the rest passes."""
    f, mag = pair_frequencies(dims, base, scaling)
    ang = positions.to(DT)[:, None] * f[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [dims // 2]
    c, s = (torch.cos(ang) * mag).reshape(shape), (torch.sin(ang) * mag).reshape(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def latent_attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float,
                           positions: torch.Tensor, gated: bool) -> torch.Tensor:
    """h [T, width] -> [T, width].  Every head's keys and values are made from the low-rank vectors here."""
    t = h.shape[0]
    heads, dim, rot_dim, vdim, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    rot = m.get("rot") or {}
    q = (h @ w[p + "q"].T).reshape(t, heads, dim + rot_dim)
    q_plain, q_rot = q[..., :dim], q[..., dim:]
    dkv = h @ w[p + "dkv"].T
    c = plain_rmsnorm(dkv[:, :rank], w[p + "dkv.norm"], eps)
    k_rot = dkv[:, rank:]
    if rot and rot_dim:
        q_rot = rotate_neighbours(q_rot, positions, int(rot["dims"]), float(rot["base"]), rot.get("scaling"))
        k_rot = rotate_neighbours(k_rot, positions, int(rot["dims"]), float(rot["base"]), rot.get("scaling"))
    k_plain = (c @ w[p + "uk"].T).reshape(t, heads, dim)
    v = (c @ w[p + "uv"].T).reshape(t, heads, vdim)
    scores = (torch.einsum("ihd,jhd->hij", q_plain, k_plain) + torch.einsum("ihd,jd->hij", q_rot, k_rot)) * m["scale"]
    seen = (positions[:, None] - positions[None, :]) >= 0
    a = torch.softmax(scores.masked_fill(~seen[None], -math.inf), dim=-1)
    o = torch.einsum("hij,jhd->ihd", a, v).reshape(t, heads * vdim)
    if gated:
        o = o * torch.sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def general_delta_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    """h [T, width] -> [T, width].  Per head a state S [key channel, value channel] from zero:
    S <- diag(decay) S - (a u)(u^T S) + k v^T, both read the old S; o = S^T r."""
    t = h.shape[0]
    heads, d = m["heads"], m["dim"]
    r = (h @ w[p + "r"].T).reshape(t, heads, d)
    k = (h @ w[p + "k"].T).reshape(t, heads, d)
    v = (h @ w[p + "v"].T).reshape(t, heads, d)
    decay = torch.exp(-DECAY_SCALE * torch.sigmoid(torch.tanh(h @ w[p + "w1"].T) @ w[p + "w2"].T + w[p + "w0"])).reshape(t, heads, d)
    a = torch.sigmoid(h @ w[p + "a"].T + w[p + "a.b"]).reshape(t, heads, d)
    u = k / torch.sqrt((k * k).sum(dim=-1, keepdim=True) + UNIT_KEY_EPS)
    out = torch.zeros(t, heads, d, dtype=DT)
    for hd in range(heads):
        S = torch.zeros(d, d, dtype=DT)
        for i in range(t):
            seen = u[i, hd] @ S                              # [value channel]
            S = decay[i, hd][:, None] * S - torch.outer(a[i, hd] * u[i, hd], seen) + torch.outer(k[i, hd], v[i, hd])
            out[i, hd] = S.T @ r[i, hd]
    out = out * torch.rsqrt((out * out).mean(dim=-1, keepdim=True) + eps)
    o = out.reshape(t, heads * d) * w[p + "norm"] * torch.sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def dense_mlp(x: torch.Tensor, w: Dict[str, torch.Tensor], p: str) -> torch.Tensor:
    return (gelu_tanh(x @ w[p + "gate"].T) * (x @ w[p + "up"].T)) @ w[p + "down"].T


def expert_mixture(x: torch.Tensor, w: Dict[str, torch.Tensor], p: str, experts: int, top: int,
                   margins: Optional[list] = None) -> torch.Tensor:
    """Every token goes to the `top` experts with the largest sigmoid scores; a chosen expert's score multiplies its
    input, and the experts' outputs are added.  margins: a list that receives, per token, how far the last chosen
    expert's logit lies above the first one left out, in units of the logits' spread (a choice that rounding may turn
    has a small one)."""
    logits = x @ w[p + "router"].T
    scores = torch.sigmoid(logits)
    if margins is not None and top < experts:
        ranked = torch.sort(logits, dim=-1, descending=True).values
        margins.append((ranked[:, top - 1] - ranked[:, top]) / logits.std(dim=-1).clamp_min(1e-30))
    out = torch.zeros_like(x)
    chosen = torch.topk(scores, top, dim=-1).indices
    for t in range(x.shape[0]):
        for e in chosen[t].tolist():
            xe = scores[t, e] * x[t]
            g = xe @ w[f"{p}e{e}.gate"].T
            out[t] += ((g * torch.sigmoid(g)) * (xe @ w[f"{p}e{e}.up"].T)) @ w[f"{p}e{e}.down"].T
    return out


def forward(cfg: dict, w: Dict[str, torch.Tensor], ids: List[int], streams: Optional[list] = None,
            margins: Optional[list] = None, rounded: bool = False) -> torch.Tensor:
    """Logits [T, vocab] of one sequence from position 0.  streams: a list that receives the sum of the residual
    streams after every layer; margins: a list that receives every expert layer's margins (expert_mixture); rounded:
    every sublayer's input and result and the last norm's output are rounded to bfloat16, which shows how far rounding
    alone moves this model's logits."""
    def r16(x):
        return x.to(torch.bfloat16).to(DT) if rounded else x

    w = {k: v.to(DT) for k, v in w.items()}
    eps = float(cfg["norm"]["eps"])
    n_streams = int(cfg.get("streams", 1))
    positions = torch.arange(len(ids))
    x0 = w["embed"][torch.tensor(ids, dtype=torch.long)]
    xs = [x0.clone() for _ in range(n_streams)]

    def sublayer(q: int, p: str, fn):
        nonlocal xs
        hc = f"{p}hc{q}."
        if "streams" in cfg:
            w_in, w_out, w_mix = w[hc + "in"], w[hc + "out"], w[hc + "mix"]
        else:                                   # one stream and no numbers for it: x <- x + y
            w_in, w_out, w_mix = torch.ones(1, dtype=DT), torch.ones(1, dtype=DT), torch.ones(1, 1, dtype=DT)
        read = sum(w_in[s] * xs[s] for s in range(n_streams))
        h = r16(offset_rmsnorm(read, w[f"{p}norm{q}"], eps))
        y = r16(r16(fn(h)) * torch.sigmoid(r16(h @ w[f"{p}rg{q}"].T + w[f"{p}rg{q}.b"])))
        xs = [sum(w_mix[s, t] * xs[s] for s in range(n_streams)) + w_out[t] * y for t in range(n_streams)]

    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        kind, m = layer["type"], layer["mixer"]
        if kind in ("latent_attention", "latent_attention_2"):
            sublayer(1, p, lambda h: latent_attention_mixer(token_shift(h, w[p + "shift"]), w, p + "mix.", m, eps, positions,
                                                            gated=kind == "latent_attention_2"))
        elif kind == "general_delta":
            sublayer(1, p, lambda h: general_delta_mixer(token_shift(h, w[p + "shift"]), w, p + "mix.", m, eps))
        else:
            raise ValueError(f"layer type {kind!r}")
        mlp = layer.get("mlp")
        if mlp is not None:
            if mlp["kind"] == "dense":
                sublayer(2, p, lambda h: dense_mlp(h, w, p + "mlp."))
            elif mlp["kind"] == "moe":
                sublayer(2, p, lambda h: expert_mixture(h, w, p + "mlp.", int(mlp["router"]["experts"]), int(mlp["router"]["top"]),
                                                     margins))
            else:
                raise ValueError(f"feed-forward kind {mlp['kind']!r}")
        if streams is not None:
            streams.append(sum(xs).clone())
    return r16(offset_rmsnorm(sum(xs), w["final.norm"], eps)) @ w["head"].T


def greedy(cfg: dict, w: Dict[str, torch.Tensor], prompt: List[int], n_new: int) -> List[int]:
    ids = list(prompt)
    for _ in range(n_new):
        ids.append(int(torch.argmax(forward(cfg, w, ids)[-1])))
    return ids[len(prompt):]
