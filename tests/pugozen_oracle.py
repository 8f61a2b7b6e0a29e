"""Plain whole-sequence implementation of the Pugozen design, for tests.

One function per mechanism, float64, token by token where the design is a
recurrence; no cache, no batching, no chunking, and no code shared with the
serving path (bee2bee_amd.*). Inputs: the parsed config.json dict and a dict
of checkpoint-named tensors.

Notation: unit(x) = x / sqrt(mean(x^2) + eps) over the last axis.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F64 = torch.float64


def unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(x: torch.Tensor) -> torch.Tensor:
    return x / (1.0 + torch.exp(-x))


def softplus(x: torch.Tensor) -> torch.Tensor:
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


def rotate(x: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [T, heads, D]; row t is position t. Coordinate i < dims/2 pairs
    with i + dims/2; the angle is t * base^(-2i/dims)."""
    T = x.shape[0]
    half = dims // 2
    out = x.clone()
    for t in range(T):
        for i in range(half):
            a = t * base ** (-2.0 * i / dims)
            c, s = math.cos(a), math.sin(a)
            u, v = x[t, :, i], x[t, :, i + half]
            out[t, :, i] = u * c - v * s
            out[t, :, i + half] = v * c + u * s
    return out


def causal_conv_silu(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """x [T, C]; w [C, taps], last column multiplies the current row."""
    T, C = x.shape
    taps = w.shape[1]
    y = torch.zeros_like(x)
    for t in range(T):
        for j in range(taps):
            src = t - (taps - 1 - j)
            if src >= 0:
                y[t] += w[:, j] * x[src]
    return silu(y)


def retention_mixer(h, P: Dict[str, torch.Tensor], m: dict, eps: float):
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ P["q"].T).view(T, H, D)
    k = (h @ P["k"].T).view(T, H, D)
    v = (h @ P["v"].T).view(T, H, Dv)
    rot = m.get("rot")
    if rot:
        q = rotate(q, rot["dims"], rot["base"])
        k = rotate(k, rot["dims"], rot["base"])
    k = k * D ** -0.5
    o = torch.zeros(T, H, Dv, dtype=F64)
    for hh in range(H):
        S = torch.zeros(D, Dv, dtype=F64)
        for t in range(T):
            S = m["decay"][hh] * S + torch.outer(k[t, hh], v[t, hh])
            o[t, hh] = S.T @ q[t, hh]
    o = unit(o, eps).reshape(T, H * Dv)
    return (o * silu(h @ P["g"].T)) @ P["o"].T


def delta_recurrence(q, k, v, beta, g):
    """q,k [T,H,D] (already per value head), v [T,H,Dv], beta [T,H],
    g [T,H] or [T,H,D] (per key channel -> rows of S)."""
    T, H, D = q.shape
    Dv = v.shape[-1]
    o = torch.zeros(T, H, Dv, dtype=F64)
    for hh in range(H):
        S = torch.zeros(D, Dv, dtype=F64)
        for t in range(T):
            gt = g[t, hh]
            S = (gt[:, None] if gt.dim() == 1 else gt) * S
            u = beta[t, hh] * (v[t, hh] - S.T @ k[t, hh])
            S = S + torch.outer(k[t, hh], u)
            o[t, hh] = S.T @ q[t, hh]
    return o


def delta_mixer(h, P: Dict[str, torch.Tensor], m: dict, eps: float,
                low_rank: bool):
    """low_rank=False: scalar decay per head from '.a', silu gate from '.g'.
    low_rank=True: per-key-channel decay from '.a2 .a1', sigmoid gate from
    '.g2 .g1'."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = causal_conv_silu(h @ P["q"].T, P["q.conv"]).view(T, G, D)
    k = causal_conv_silu(h @ P["k"].T, P["k.conv"]).view(T, G, D)
    v = causal_conv_silu(h @ P["v"].T, P["v.conv"]).view(T, H, Dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    rep = H // G
    q = q.repeat_interleave(rep, dim=1)
    k = k.repeat_interleave(rep, dim=1)
    beta = torch.sigmoid(h @ P["b"].T)
    A = torch.exp(P["A_log"])
    if low_rank:
        a = ((h @ P["a1"].T) @ P["a2"].T + P["dt_bias"]).view(T, H, D)
        g = torch.exp(-A[None, :, None] * softplus(a))
        gate = torch.sigmoid((h @ P["g1"].T) @ P["g2"].T)
    else:
        a = h @ P["a"].T + P["dt_bias"]
        g = torch.exp(-A[None, :] * softplus(a))
        gate = silu(h @ P["g"].T)
    o = delta_recurrence(q, k, v, beta, g)
    o = unit(o, eps) * P["norm"]
    return (o.reshape(T, H * Dv) * gate) @ P["o"].T


def sink_attention(h, P: Dict[str, torch.Tensor], m: dict, eps: float):
    T = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ P["q"].T).view(T, H, D)
    k = (h @ P["k"].T).view(T, G, D)
    v = k.clone()                       # values are the keys as projected
    q = unit(q, eps) * P["q.norm"]
    k = unit(k, eps) * P["k.norm"]
    rot = m.get("rot")
    if rot:
        q = rotate(q, rot["dims"], rot["base"])
        k = rotate(k, rot["dims"], rot["base"])
    out = torch.zeros(T, H, v.shape[-1], dtype=F64)
    for hh in range(H):
        g = hh // (H // G)
        for t in range(T):
            s = (k[: t + 1, g] @ q[t, hh]) * m["scale"] * P["temp"][hh]
            mx = max(float(s.max()), float(P["sink"][hh]))
            e = torch.exp(s - mx)
            den = e.sum() + math.exp(float(P["sink"][hh]) - mx)
            out[t, hh] = (e / den) @ v[: t + 1, g]
    return out.reshape(T, -1) @ P["o"].T


def parallel_mixer(h, P, m: dict, eps: float):
    left = sink_attention(h, sub(P, "left."), m["left"], eps)
    right = delta_mixer(h, sub(P, "right."), m["right"], eps, low_rank=True)
    return m["left_scale"] * left + m["right_scale"] * right


def dense_ff(h, P, f: Optional[dict]):
    if f is None:
        return torch.zeros_like(h)
    if f.get("kind", "dense") != "dense":
        raise ValueError(f["kind"])
    z = torch.relu(h @ P["up"].T)
    return (z * z) @ P["down"].T


def sub(P: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v for k, v in P.items() if k.startswith(prefix)}


def forward(tokens: List[int], cfg: dict, tensors: Dict[str, torch.Tensor],
            layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] (float64) of one whole sequence."""
    P = {k: v.to(F64) for k, v in tensors.items()}
    eps = cfg["norm"]["eps"]
    x = P["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
    for i, l in enumerate(cfg["layers"]):
        src = l.get("weights_of", i)
        L = sub(P, f"l{src}.")
        h = unit(x, eps) * L["norm1"]
        kind, m = l["type"], l["mixer"]
        if kind == "retention":
            y = retention_mixer(h, sub(L, "mix."), m, eps)
        elif kind == "delta":
            y = delta_mixer(h, sub(L, "mix."), m, eps, low_rank=False)
        elif kind == "parallel":
            y = parallel_mixer(h, sub(L, "mix."), m, eps)
        else:
            raise ValueError(kind)
        x = x + (y + dense_ff(h, sub(L, "mlp."), l.get("mlp")))
        if layers_out is not None:
            layers_out.append(x.clone())
    x = unit(x, eps) * P["final.norm"]
    return x @ P["head"].T
