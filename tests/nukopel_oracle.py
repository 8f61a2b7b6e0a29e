"""Plain, slow whole-sequence implementation of the Nukopel design, written
from its equations with one function per mechanism. It shares no code with
the serving path: no cache, no paging, no batching — every call recomputes a
whole sequence from position 0 in one dtype (float64 by default).

Weights are a dict keyed by checkpoint tensor names ('l3.mix.q', ...), the
config is the parsed config.json dict.
"""
from __future__ import annotations

import math
from typing import Dict, List, Tuple

import torch

Tensors = Dict[str, torch.Tensor]


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def scalar_norm(x: torch.Tensor, g: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm whose gain is ONE number shared by all coordinates."""
    return unit_rms(x, eps) * g.reshape(())


def weighted_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return unit_rms(x, eps) * w


def causal_channel_conv(h: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """h [T, C], w [C, taps]: out_t = sum_j w[:, j] * h_(t - taps + 1 + j),
    with zeros for times before 0."""
    T, C = h.shape
    taps = w.shape[1]
    out = torch.zeros_like(h)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += w[:, j] * h[s]
    return out


def rotate_pairs(x: torch.Tensor, pos: torch.Tensor, base: float,
                 dims: int) -> torch.Tensor:
    """x [T, ..., D]: rotate the first `dims` coordinates, pairing i with
    i + dims/2; angle = pos * base**(-2i/dims)."""
    half = dims // 2
    out = x.clone()
    for i in range(half):
        f = base ** (-2.0 * i / dims)
        a = pos.to(x.dtype) * f
        shape = [x.shape[0]] + [1] * (x.dim() - 2)
        c, s = torch.cos(a).reshape(shape), torch.sin(a).reshape(shape)
        u, v = x[..., i], x[..., i + half]
        out[..., i] = u * c - v * s
        out[..., i + half] = v * c + u * s
    return out


def windowed_softmax_attention(q: torch.Tensor, k: torch.Tensor,
                               v: torch.Tensor, scale: float,
                               window: int) -> torch.Tensor:
    """q,k [T, H, Dk], v [T, H, Dv]; query i sees keys j, 0 <= i-j < window."""
    T, H, _ = q.shape
    out = torch.zeros(T, H, v.shape[-1], dtype=q.dtype)
    for i in range(T):
        lo = max(0, i - window + 1)
        for h in range(H):
            s = (k[lo:i + 1, h] @ q[i, h]) * scale
            p = torch.softmax(s, dim=0)
            out[i, h] = p @ v[lo:i + 1, h]
    return out


def latent_attention(h: torch.Tensor, W: Tensors, pfx: str, m: dict,
                     eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, D, R, Dv, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    q = (h @ W[pfx + "q"].T).reshape(T, H, D + R)
    dkv = h @ W[pfx + "dkv"].T
    c = weighted_norm(dkv[:, :C], W[pfx + "dkv.norm"], eps)
    k_rot = dkv[:, C:].reshape(T, 1, R)
    base, dims = m["rot"]["base"], m["rot"]["dims"]
    q_rot = rotate_pairs(q[..., D:], pos, base, dims)
    k_rot = rotate_pairs(k_rot, pos, base, dims).expand(T, H, R)
    k_un = (c @ W[pfx + "uk"].T).reshape(T, H, D)
    v = (c @ W[pfx + "uv"].T).reshape(T, H, Dv)
    qq = torch.cat([q[..., :D], q_rot], -1)
    kk = torch.cat([k_un, k_rot], -1)
    o = windowed_softmax_attention(qq, kk, v, m["scale"], m["mask"]["size"])
    gate = torch.sigmoid(h @ W[pfx + "g"].T)            # [T, H]
    o = o * gate[..., None]
    return o.reshape(T, H * Dv) @ W[pfx + "o"].T


def silu(x: torch.Tensor) -> torch.Tensor:
    return x * torch.sigmoid(x)


def lightning(h: torch.Tensor, W: Tensors, pfx: str, m: dict,
              eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ W[pfx + "q"].T).reshape(T, H, D)
    k = silu(h @ W[pfx + "k"].T).reshape(T, H, D)
    v = silu(h @ W[pfx + "v"].T).reshape(T, H, Dv)
    o = torch.zeros(T, H, Dv, dtype=h.dtype)
    for hd in range(H):
        S = torch.zeros(D, Dv, dtype=h.dtype)
        lam = m["decay"][hd]
        for t in range(T):
            S = lam * S + torch.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
    o = weighted_norm(o.reshape(T, H * Dv), W[pfx + "norm"], eps)
    o = o * torch.sigmoid(h @ W[pfx + "g"].T)
    return o @ W[pfx + "o"].T


def expert(h: torch.Tensor, W: Tensors, pfx: str, limit: float) -> torch.Tensor:
    g = torch.clamp(h @ W[pfx + "gate"].T, max=limit)
    u = torch.clamp(h @ W[pfx + "up"].T, min=-limit, max=limit)
    y = g * torch.sigmoid(1.702 * g) * (u + 1.0)
    return y @ W[pfx + "down"].T


def route(h: torch.Tensor, w_router: torch.Tensor,
          top: int) -> Tuple[torch.Tensor, torch.Tensor]:
    z = h @ w_router.T
    vals, idx = torch.topk(z, top, dim=-1)
    return torch.softmax(vals, dim=-1), idx


def moe(h: torch.Tensor, W: Tensors, pfx: str, f: dict) -> torch.Tensor:
    T = h.shape[0]
    wts, idx = route(h, W[pfx + "router"], f["router"]["top"])
    out = torch.zeros(T, W[pfx + "e0.down"].shape[0], dtype=h.dtype)
    for t in range(T):
        for j in range(idx.shape[1]):
            e = int(idx[t, j])
            out[t] += wts[t, j] * expert(h[t:t + 1], W, f"{pfx}e{e}.",
                                         f["expert"]["limit"])[0]
    if f.get("shared"):
        out = out + expert(h, W, pfx + "shared.", f["shared"]["limit"])
    return out


def forward(tokens: List[int], W: Tensors, cfg: dict,
            dtype=torch.float64) -> Tuple[torch.Tensor, torch.Tensor]:
    """-> (logits [T, vocab], residual stream after each layer [L, T, width])"""
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
    per_layer = []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = scalar_norm(x, W[p + "norm1"], eps)
        h = h + causal_channel_conv(h, W[p + "canon1"])
        if layer["type"] == "latent_attention":
            y = latent_attention(h, W, p + "mix.", layer["mixer"], eps)
        elif layer["type"] == "lightning":
            y = lightning(h, W, p + "mix.", layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        x = x + scalar_norm(y, W[p + "norm1b"], eps)
        if layer.get("mlp"):
            h = scalar_norm(x, W[p + "norm2"], eps)
            y = moe(h, W, p + "mlp.", layer["mlp"])
            x = x + scalar_norm(y, W[p + "norm2b"], eps)
        per_layer.append(x)
    x = scalar_norm(x, W["final.norm"], eps)
    return x @ W["head"].T, torch.stack(per_layer)


def random_weights(cfg: dict, seed: int = 0, std: float = 0.05) -> Tensors:
    """Random bf16-representable weights under the checkpoint's names."""
    g = torch.Generator().manual_seed(seed)

    def rnd(*shape, s=std):
        return (torch.randn(*shape, generator=g) * s).bfloat16()

    def gain():
        return (1.0 + 0.2 * torch.randn((), generator=g)).bfloat16()

    Wd, V = cfg["width"], cfg["vocab"]
    W: Tensors = {"embed": rnd(V, Wd, s=0.3), "head": rnd(V, Wd, s=0.08),
                  "final.norm": gain()}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        for n in ("norm1", "norm1b", "norm2", "norm2b"):
            W[p + n] = gain()
        W[p + "canon1"] = rnd(Wd, cfg["canon"]["taps"], s=0.3)
        H = m["heads"]
        if layer["type"] == "latent_attention":
            D, R, Dv, C = m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            W[p + "mix.q"] = rnd(H * (D + R), Wd, s=2.0 / math.sqrt(Wd))
            W[p + "mix.dkv"] = rnd(C + R, Wd, s=2.0 / math.sqrt(Wd))
            W[p + "mix.dkv.norm"] = (1.0 + 0.2 * torch.randn(C, generator=g)).bfloat16()
            W[p + "mix.uk"] = rnd(H * D, C, s=2.0 / math.sqrt(C))
            W[p + "mix.uv"] = rnd(H * Dv, C, s=1.0 / math.sqrt(C))
            W[p + "mix.g"] = rnd(H, Wd, s=1.0 / math.sqrt(Wd))
            W[p + "mix.o"] = rnd(Wd, H * Dv, s=1.0 / math.sqrt(H * Dv))
        else:
            D, Dv = m["dim"], m["vdim"]
            for n, rows in (("q", H * D), ("k", H * D), ("v", H * Dv),
                            ("g", H * Dv)):
                W[p + "mix." + n] = rnd(rows, Wd, s=1.5 / math.sqrt(Wd))
            W[p + "mix.norm"] = (1.0 + 0.2 * torch.randn(H * Dv, generator=g)).bfloat16()
            W[p + "mix.o"] = rnd(Wd, H * Dv, s=1.0 / math.sqrt(H * Dv))
        f = layer.get("mlp")
        if f:
            E, ff = f["router"]["experts"], f["expert"]["ff"]
            W[p + "mlp.router"] = rnd(E, Wd, s=2.0 / math.sqrt(Wd))
            blocks = [(f"e{e}.", ff) for e in range(E)]
            if f.get("shared"):
                blocks.append(("shared.", f["shared"]["ff"]))
            for name, width in blocks:
                W[p + "mlp." + name + "gate"] = rnd(width, Wd, s=1.5 / math.sqrt(Wd))
                W[p + "mlp." + name + "up"] = rnd(width, Wd, s=1.5 / math.sqrt(Wd))
                W[p + "mlp." + name + "down"] = rnd(Wd, width, s=1.0 / math.sqrt(width))
    return W


def make_config(vocab=96, width=48, taps=3, eps=1e-5, emb_scale=3.0,
                order=("lightning", "latent_attention"), heads_la=3, dim=8,
                rot_dim=4, vdim=12, kv_rank=20, window=7, base=10000.0,
                heads_li=2, li_dim=8, li_vdim=12, decay=(0.8, 0.97),
                experts=5, top=2, ff=16, limit=1.2, shared_ff=24,
                shared_limit=1.7, scale=None) -> dict:
    """A small config in the design's config.json form; every size differs
    from every other where the design lets them."""
    mlp = {"kind": "moe", "expert": {"ff": ff, "limit": limit},
           "router": {"experts": experts, "top": top},
           "shared": {"ff": shared_ff, "limit": shared_limit}}
    layers = []
    for t in order:
        if t == "latent_attention":
            mixer = {"heads": heads_la, "dim": dim, "rot_dim": rot_dim,
                     "vdim": vdim, "kv_rank": kv_rank,
                     "mask": {"size": window},
                     "rot": {"base": base, "dims": rot_dim},
                     "scale": scale if scale is not None
                     else 1.0 / math.sqrt(dim + rot_dim)}
        else:
            mixer = {"heads": heads_li, "dim": li_dim, "vdim": li_vdim,
                     "decay": list(decay)}
        layers.append({"type": t, "mixer": mixer, "mlp": mlp})
    return {"architecture": "Nukopel", "vocab": vocab, "width": width,
            "canon": {"taps": taps}, "embedding": {"scale": emb_scale},
            "norm": {"eps": eps}, "layers": layers}


def save_checkpoint(path: str, cfg: dict, W: Tensors) -> None:
    import json
    import os

    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in W.items()},
              os.path.join(path, "model.safetensors"))
