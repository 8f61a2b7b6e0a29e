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
    o = unit(retention_core(q, k, v, m["decay"]), eps).reshape(T, H * Dv)
    return (o * silu(h @ P["g"].T)) @ P["o"].T


def retention_core(q, k, v, decay):
    """Memory M <- lam_h M + k v^T per token, read-out M^T q; q,k [T,H,D]."""
    T, H, D = q.shape
    Dv = v.shape[-1]
    o = torch.zeros(T, H, Dv, dtype=F64)
    for hh in range(H):
        S = torch.zeros(D, Dv, dtype=F64)
        for t in range(T):
            S = decay[hh] * S + torch.outer(k[t, hh], v[t, hh])
            o[t, hh] = S.T @ q[t, hh]
    return o


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
    out = softmax_sink_core(q, k, v, m["scale"], P["temp"], P["sink"])
    return out.reshape(T, -1) @ P["o"].T


def softmax_sink_core(q, k, v, scale, temp, sink, window=0):
    """Causal attention, q [T,H,D], k [T,G,D], v [T,G,Dv]; score =
    q.k * scale * temp_h; the denominator also holds exp(sink_h), once."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[-1], dtype=F64)
    for hh in range(H):
        g = hh // (H // G)
        for t in range(T):
            lo = max(0, t - window + 1) if window else 0
            s = (k[lo : t + 1, g] @ q[t, hh]) * scale * float(temp[hh])
            mx = max(float(s.max()), float(sink[hh]))
            e = torch.exp(s - mx)
            den = e.sum() + math.exp(float(sink[hh]) - mx)
            out[t, hh] = (e / den) @ v[lo : t + 1, g]
    return out


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


# ------------------------------------------------- small random checkpoints

def make_config(order=("parallel", "retention", "delta"), shared=(), *,
                vocab=61, width=40, ff=56, eps=1e-5, emb_scale=2.0,
                heads=4, kv_heads=2, dim=12, rot_dims=6, rot_base=5000.0,
                scale=0.3, left_scale=0.7, right_scale=0.6,
                r_heads=2, r_kv_heads=1, r_dim=10, r_vdim=14, r_conv=3,
                ret_heads=3, ret_dim=8, ret_vdim=10, ret_rot=8,
                ret_decay=(0.9, 0.97, 0.99),
                d_heads=4, d_kv_heads=2, d_dim=6, d_vdim=10, d_conv=4):
    """config.json dict; `shared` lists (layer, source) pairs: the layer runs
    the source layer's tensors."""
    def mixer(kind):
        if kind == "retention":
            return {"heads": ret_heads, "dim": ret_dim, "vdim": ret_vdim,
                    "decay": list(ret_decay),
                    "rot": {"base": rot_base * 3, "dims": ret_rot}}
        if kind == "delta":
            return {"heads": d_heads, "kv_heads": d_kv_heads, "dim": d_dim,
                    "vdim": d_vdim, "conv": d_conv}
        return {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim,
                         "vdim": dim, "scale": scale,
                         "rot": {"base": rot_base, "dims": rot_dims}},
                "right": {"heads": r_heads, "kv_heads": r_kv_heads,
                          "dim": r_dim, "vdim": r_vdim, "conv": r_conv},
                "left_scale": left_scale, "right_scale": right_scale}

    layers = [{"type": k, "mixer": mixer(k),
               "mlp": {"kind": "dense", "ff": ff}} for k in order]
    for i, j in shared:
        layers[i] = dict(layers[j], weights_of=j)
    return {"architecture": "Pugozen", "vocab": vocab, "width": width,
            "embedding": {"scale": emb_scale}, "norm": {"eps": eps},
            "layers": layers}


def random_weights(cfg, seed=0, rank=5):
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]

    def rnd(*shape, std=1.0, mean=0.0):
        t = mean + std * torch.randn(*shape, generator=g)
        return t.to(torch.bfloat16)

    def delta(p, m, low_rank):
        H, G, D, Dv, taps = (m["heads"], m["kv_heads"], m["dim"], m["vdim"],
                             m["conv"])
        t = {p + "q": rnd(G * D, W, std=W ** -0.5),
             p + "k": rnd(G * D, W, std=W ** -0.5),
             p + "v": rnd(H * Dv, W, std=W ** -0.5),
             p + "q.conv": rnd(G * D, taps, std=0.5),
             p + "k.conv": rnd(G * D, taps, std=0.5),
             p + "v.conv": rnd(H * Dv, taps, std=0.5),
             p + "b": rnd(H, W, std=W ** -0.5),
             p + "A_log": rnd(H, std=0.5, mean=-1.0),
             p + "norm": rnd(Dv, std=0.2, mean=1.0),
             p + "o": rnd(W, H * Dv, std=(H * Dv) ** -0.5)}
        if low_rank:
            t.update({p + "a1": rnd(rank, W, std=W ** -0.5),
                      p + "a2": rnd(H * D, rank, std=rank ** -0.5),
                      p + "dt_bias": rnd(H * D, std=0.7),
                      p + "g1": rnd(rank + 1, W, std=W ** -0.5),
                      p + "g2": rnd(H * Dv, rank + 1, std=rank ** -0.5)})
        else:
            t.update({p + "a": rnd(H, W, std=W ** -0.5),
                      p + "dt_bias": rnd(H, std=0.7),
                      p + "g": rnd(H * Dv, W, std=W ** -0.5)})
        return t

    out = {"embed": rnd(V, W, std=0.7), "head": rnd(V, W, std=W ** -0.5),
           "final.norm": rnd(W, std=0.2, mean=1.0)}
    for i, l in enumerate(cfg["layers"]):
        if "weights_of" in l:
            continue
        p, m = f"l{i}.", l["mixer"]
        out[p + "norm1"] = rnd(W, std=0.2, mean=1.0)
        if l["type"] == "retention":
            H, D, Dv = m["heads"], m["dim"], m["vdim"]
            out.update({p + "mix.q": rnd(H * D, W, std=W ** -0.5),
                        p + "mix.k": rnd(H * D, W, std=W ** -0.5),
                        p + "mix.v": rnd(H * Dv, W, std=W ** -0.5),
                        p + "mix.g": rnd(H * Dv, W, std=W ** -0.5),
                        p + "mix.o": rnd(W, H * Dv, std=(H * Dv) ** -0.5)})
        elif l["type"] == "delta":
            out.update(delta(p + "mix.", m, False))
        else:
            a = m["left"]
            H, G, D = a["heads"], a["kv_heads"], a["dim"]
            q = p + "mix.left."
            out.update({q + "q": rnd(H * D, W, std=W ** -0.5),
                        q + "k": rnd(G * D, W, std=W ** -0.5),
                        q + "q.norm": rnd(D, std=0.2, mean=1.0),
                        q + "k.norm": rnd(D, std=0.2, mean=1.0),
                        q + "temp": rnd(H, std=0.3, mean=1.2),
                        # sinks heavy enough that leaving them out shows
                        q + "sink": rnd(H, std=1.5, mean=1.0),
                        q + "o": rnd(W, H * a["vdim"],
                                     std=(H * a["vdim"]) ** -0.5)})
            out.update(delta(p + "mix.right.", m["right"], True))
        if l.get("mlp"):
            ff = l["mlp"]["ff"]
            out[p + "mlp.up"] = rnd(ff, W, std=W ** -0.5)
            out[p + "mlp.down"] = rnd(W, ff, std=ff ** -0.5)
    return out


def save_checkpoint(path, cfg, tensors):
    import json
    import os

    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    save_file({k: v.contiguous() for k, v in tensors.items()},
              os.path.join(path, "model.safetensors"))
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
