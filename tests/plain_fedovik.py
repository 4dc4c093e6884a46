"""Plain, slow implementation of the Fedovik decoder: whole sequences, no
cache, one function per mechanism, in float64 on the CPU.  It shares no code
with the engine; the tests compare the engine against it.

Fedovik's layers are parallel: one layer norm (gain and bias) feeds the mixer
and the feed-forward alike and both results join the residual stream in one
sum.  Three mixers: attention whose weights are sigmoids of the scores (no
softmax; a learned shift per head; neighbouring elements rotated together;
biases on all four projections; an elementwise sigmoid gate); a pair of mixers
side by side (windowed softmax attention with normed queries and keys and a
bias that grows with the logarithm of the distance, beside a gated delta rule
whose decay has one factor per key channel); and the matrix memory of xLSTM
with capped gates and a running maximum.  A run of layers may be repeated with
shared weights; every pass starts from a projection of the stream joined with
the embedding's output, plus a vector of its own.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

from plain_model import read_folder  # noqa: F401  (own safetensors reader of the tests)

DT = torch.float64


def layer_norm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float) -> torch.Tensor:
    mu = x.mean(dim=-1, keepdim=True)
    var = ((x - mu) ** 2).mean(dim=-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def silu(x: torch.Tensor) -> torch.Tensor:
    return x * torch.sigmoid(x)


def softplus(x: torch.Tensor) -> torch.Tensor:
    return torch.where(x > 30, x, torch.log1p(torch.exp(torch.clamp(x, max=30))))


def log_sigmoid(x: torch.Tensor) -> torch.Tensor:
    return -softplus(-x)


def rotate_neighbours(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [T, heads, D]: of the first `dims` elements of each head, element 2i turns with element 2i + 1 by the
    angle position * base^(-2i/dims)."""
    i = torch.arange(dims // 2, dtype=DT)
    ang = positions.to(DT)[:, None] * torch.pow(torch.tensor(base, dtype=DT), -2.0 * i / dims)[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def sigmoid_attention(q, k, v, positions, scale: float, shift: torch.Tensor) -> torch.Tensor:
    """q [T, H, D], k [T, G, D], v [T, G, Dv]; the weight of key j <= i is sigmoid(scale q_i.k_j + shift_h), and the
    weights are not normalized.  -> [T, H, Dv]"""
    t, h, _ = q.shape
    g = k.shape[1]
    out = torch.zeros(t, h, v.shape[-1], dtype=DT)
    seen = positions[None, :] <= positions[:, None]
    for a in range(h):
        kv = a // (h // g)
        s = (q[:, a] @ k[:, kv].t()) * scale + shift[a]
        out[:, a] = (torch.sigmoid(s) * seen) @ v[:, kv]
    return out


def window_attention(q, k, v, positions, scale: float, window: int, r1: torch.Tensor, r2: torch.Tensor) -> torch.Tensor:
    """Softmax attention over the keys with 0 <= i - j < window; r1_h ln(1 + r2_h (i - j)) is taken off the score."""
    t, h, _ = q.shape
    g = k.shape[1]
    out = torch.zeros(t, h, v.shape[-1], dtype=DT)
    dist = (positions[:, None] - positions[None, :]).to(DT)
    seen = (dist >= 0) & (dist < window)
    for a in range(h):
        kv = a // (h // g)
        s = (q[:, a] @ k[:, kv].t()) * scale - r1[a] * torch.log1p(r2[a] * dist.clamp(min=0))
        s = s.masked_fill(~seen, float("-inf"))
        out[:, a] = torch.softmax(s, dim=-1) @ v[:, kv]
    return out


def attention_mixer(x, w: Dict[str, torch.Tensor], p: str, m: dict, positions) -> torch.Tensor:
    t = x.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (x @ w[p + "q"].t() + w[p + "q.b"]).reshape(t, H, D)
    k = (x @ w[p + "k"].t() + w[p + "k.b"]).reshape(t, G, D)
    v = (x @ w[p + "v"].t() + w[p + "v.b"]).reshape(t, G, Dv)
    rot = m.get("rot")
    if rot:
        q = rotate_neighbours(q, positions, rot["dims"], rot["base"])
        k = rotate_neighbours(k, positions, rot["dims"], rot["base"])
    o = sigmoid_attention(q, k, v, positions, m["scale"], w[p + "pb"]).reshape(t, H * Dv)
    o = o * torch.sigmoid(x @ w[p + "g"].t())
    return o @ w[p + "o"].t() + w[p + "o.b"]


def left_mixer(x, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float, positions) -> torch.Tensor:
    t = x.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (x @ w[p + "q"].t() + w[p + "q.b"]).reshape(t, H, D)
    k = (x @ w[p + "k"].t() + w[p + "k.b"]).reshape(t, G, D)
    v = (x @ w[p + "v"].t() + w[p + "v.b"]).reshape(t, G, Dv)
    q = rms_unit(q, eps) * w[p + "q.norm"]
    k = rms_unit(k, eps) * w[p + "k.norm"]
    o = window_attention(q, k, v, positions, m["scale"], m["mask"]["size"], w[p + "r1"], w[p + "r2"])
    return o.reshape(t, H * Dv) @ w[p + "o"].t()


def causal_conv(x: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """x [T, C], taps [C, K] with the last column the current token's; zeros in front of the sequence."""
    t, c = x.shape
    kk = taps.shape[1]
    padded = torch.cat([torch.zeros(kk - 1, c, dtype=DT), x], dim=0)
    out = torch.zeros(t, c, dtype=DT)
    for j in range(kk):
        out += padded[j:j + t] * taps[:, j]
    return out


def channel_delta_rule(q, k, v, beta, g) -> torch.Tensor:
    """q, k [T, H, D] (already unit vectors), v [T, H, Dv], beta [T, H], g [T, H, D] (a decay per key channel).
    S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q.  -> [T, H, Dv]"""
    t, h, d = q.shape
    dv = v.shape[-1]
    out = torch.zeros(t, h, dv, dtype=DT)
    for a in range(h):
        S = torch.zeros(d, dv, dtype=DT)
        for i in range(t):
            S = g[i, a][:, None] * S
            u = beta[i, a] * (v[i, a] - S.t() @ k[i, a])
            S = S + torch.outer(k[i, a], u)
            out[i, a] = S.t() @ q[i, a]
    return out


def right_mixer(x, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    t = x.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(x @ w[p + "q"].t(), w[p + "q.conv"])).reshape(t, G, D)
    k = silu(causal_conv(x @ w[p + "k"].t(), w[p + "k.conv"])).reshape(t, G, D)
    v = silu(causal_conv(x @ w[p + "v"].t(), w[p + "v.conv"])).reshape(t, H, Dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    rep = H // G
    q, k = q.repeat_interleave(rep, dim=1), k.repeat_interleave(rep, dim=1)
    beta = torch.sigmoid(x @ w[p + "b"].t())
    z = (x @ w[p + "a1"].t()) @ w[p + "a2"].t() + w[p + "dt_bias"]
    g = torch.exp(-torch.exp(w[p + "A_log"])[None, :, None] * softplus(z).reshape(t, H, D))
    o = channel_delta_rule(q, k, v, beta, g)
    o = rms_unit(o, eps) * w[p + "norm"]
    o = o * torch.sigmoid((x @ w[p + "g1"].t()) @ w[p + "g2"].t()).reshape(t, H, Dv)
    return o.reshape(t, H * Dv) @ w[p + "o"].t()


def pair_mixer(x, w, p: str, m: dict, eps: float, positions) -> torch.Tensor:
    return (m["left_scale"] * left_mixer(x, w, p + "left.", m["left"], eps, positions)
            + m["right_scale"] * right_mixer(x, w, p + "right.", m["right"], eps))


def matrix_memory(q, k, v, i_gate, f_gate) -> torch.Tensor:
    """q (already scaled), k [T, H, D], v [T, H, Dv], log gates [T, H].  With m_0 = 0, S_0 = 0, n_0 = 0:
    m_t = max(f + m, i); S_t = e^(f + m - m_t) S + e^(i - m_t) k v^T; n_t likewise with k;
    o = S_t^T q / (max(|n_t . q|, e^(-m_t)) + 1e-6)."""
    t, h, d = q.shape
    dv = v.shape[-1]
    out = torch.zeros(t, h, dv, dtype=DT)
    for a in range(h):
        S, n, m = torch.zeros(d, dv, dtype=DT), torch.zeros(d, dtype=DT), 0.0
        for j in range(t):
            f, i = float(f_gate[j, a]), float(i_gate[j, a])
            m_new = max(f + m, i)
            S = math.exp(f + m - m_new) * S + math.exp(i - m_new) * torch.outer(k[j, a], v[j, a])
            n = math.exp(f + m - m_new) * n + math.exp(i - m_new) * k[j, a]
            m = m_new
            out[j, a] = S.t() @ q[j, a] / (max(abs(float(n @ q[j, a])), math.exp(-m)) + 1e-6)
    return out


def mlstm_mixer(x, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    t = x.shape[0]
    H, D, Dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (x @ w[p + "q"].t()).reshape(t, H, D) * D ** -0.5
    k = (x @ w[p + "k"].t()).reshape(t, H, D)
    v = (x @ w[p + "v"].t()).reshape(t, H, Dv)
    i_gate = cap * torch.tanh((x @ w[p + "i"].t() + w[p + "i.b"]) / cap)
    f_gate = log_sigmoid(cap * torch.tanh((x @ w[p + "f"].t() + w[p + "f.b"]) / cap))
    o = rms_unit(matrix_memory(q, k, v, i_gate, f_gate), eps).reshape(t, H * Dv)
    o = o * w[p + "norm"] * torch.sigmoid(x @ w[p + "g"].t())
    return o @ w[p + "o"].t()


def relu_mlp(x, w: Dict[str, torch.Tensor], p: str) -> torch.Tensor:
    return (torch.relu(x @ w[p + "gate"].t()) * (x @ w[p + "up"].t())) @ w[p + "down"].t()


def layer_runs(cfg: dict) -> List[tuple]:
    """[(layer index, pass number or None if the layer starts no pass)] in the order they run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    runs = [(i, None) for i in range(a)]
    for t in range(times):
        runs += [(i, t if i == a else None) for i in range(a, b)]
    return runs + [(i, None) for i in range(b, n)]


def mixer(L: dict, h, w, p: str, eps: float, pos) -> torch.Tensor:
    if L["type"] == "attention":
        return attention_mixer(h, w, p, L["mixer"], pos)
    if L["type"] == "parallel":
        return pair_mixer(h, w, p, L["mixer"], eps, pos)
    if L["type"] == "mlstm":
        return mlstm_mixer(h, w, p, L["mixer"], eps)
    raise ValueError(L["type"])


def forward(cfg: dict, w: Dict[str, torch.Tensor], ids: List[int], streams: Optional[list] = None,
            rounded: bool = False) -> torch.Tensor:
    """Logits [T, vocab] of one sequence from position 0.  streams: a list that gets the residual stream after every
    layer run.  rounded: what the sublayers and the re-entry read is rounded to bfloat16 first, everything else stays
    float64: how far rounding alone moves the logits of this model."""
    def r16(t):
        return t.to(torch.bfloat16).to(DT) if rounded else t
    w = {k: v.to(DT) for k, v in w.items()}
    eps = cfg["norm"]["eps"]
    pos = torch.arange(len(ids))
    x0 = w["embed"][torch.tensor(ids, dtype=torch.long)] * (cfg.get("embedding") or {}).get("scale", 1.0)
    x = x0
    for i, t in layer_runs(cfg):
        if t is not None:
            x = r16(torch.cat([x, x0], dim=-1)) @ w["loop.in"].t() + w["loop.step"][t]
        L, p = cfg["layers"][i], f"l{i}."
        h = r16(layer_norm(x, w[p + "norm1"], w[p + "norm1.b"], eps))
        y = mixer(L, h, w, p + "mix.", eps, pos)
        if L.get("mlp"):
            y = y + relu_mlp(h, w, p + "mlp.")
        x = x + y
        if streams is not None:
            streams.append(x.clone())
    return r16(layer_norm(x, w["final.norm"], w["final.norm.b"], eps)) @ w["embed"].t()


def greedy(cfg: dict, w: Dict[str, torch.Tensor], prompt: List[int], n_new: int) -> List[int]:
    ids, out = list(prompt), []
    for _ in range(n_new):
        t = int(torch.argmax(forward(cfg, w, ids)[-1]))
        out.append(t)
        ids.append(t)
    return out
