"""Per-layer specs for hybrid decoder stacks: models whose layers differ in
mixer kind (softmax attention over a compressed latent cache, linear
attention with a decayed recurrent state) and carry their own feed-forward
sizes. A ModelSpec with `layer_specs` set is executed by the Runner's hybrid
path (engine/runner.py), cached by PagedKV's latent pages and state slots
(engine/kv.py), and its mechanisms are ops beside the dense-attention ones
(ops/__init__.py: latent_attn, lightning_attn, canon_conv, scalar norms,
clamped GLU).

Every constant a checkpoint's config.json may vary is a field here; nothing
below assumes particular sizes, head counts, window lengths or layer order.

Nukopel config.json keys (the family served through this path):
  architecture, vocab, width, canon.taps, embedding.scale, norm.eps,
  layers[i].type in {latent_attention, lightning},
  layers[i].mixer.{heads, dim, vdim, ...}, layers[i].mlp (or null).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple


@dataclass
class LatentAttnSpec:
    """Multi-head attention whose keys/values are up-projections of one
    shared low-rank latent per token. Cached per token: the normed latent
    (kv_rank) and ONE rotated key part (rot_dim) shared by all heads."""
    heads: int
    dim: int            # unrotated query/key dims per head
    rot_dim: int        # rotated query/key dims per head
    vdim: int
    kv_rank: int
    window: int         # query i sees keys j with 0 <= i - j < window
    rope_base: float
    rope_dims: int      # leading dims of the rot part that rotate
    scale: float

    kind = "latent_attention"

    @property
    def q_size(self) -> int:
        return self.heads * (self.dim + self.rot_dim)

    @property
    def cache_dim(self) -> int:
        return self.kv_rank + self.rot_dim


@dataclass
class LightningSpec:
    """Linear attention with a per-head scalar decay:
    S_t = decay_h S_(t-1) + k_t v_t^T,  o_t = S_t^T q_t."""
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]

    kind = "lightning"


@dataclass
class MoEFFNSpec:
    """Routed experts (+ optional always-on shared expert) with the clamped
    GLU activation: g = min(gate, limit), u = clamp(up, +-limit),
    y = g * sigmoid(alpha g) * (u + 1)."""
    n_experts: int
    top_k: int
    ff: int
    limit: float
    shared_ff: int = 0
    shared_limit: float = 0.0
    alpha: float = 1.702


@dataclass
class LayerSpec:
    mixer: Any                      # LatentAttnSpec | LightningSpec
    ffn: Optional[MoEFFNSpec] = None

    @property
    def kind(self) -> str:
        return self.mixer.kind


def _mixer_from_cfg(kind: str, m: Dict[str, Any]):
    if kind == "latent_attention":
        rot = m.get("rot") or {}
        rot_dim = int(m["rot_dim"])
        return LatentAttnSpec(
            heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=rot_dim,
            vdim=int(m["vdim"]), kv_rank=int(m["kv_rank"]),
            window=int(m["mask"]["size"]),
            rope_base=float(rot.get("base", 10000.0)),
            rope_dims=int(rot.get("dims", rot_dim)),
            scale=float(m["scale"]),
        )
    if kind == "lightning":
        decay = tuple(float(d) for d in m["decay"])
        if len(decay) != int(m["heads"]):
            raise ValueError("lightning mixer needs one decay per head")
        return LightningSpec(heads=int(m["heads"]), dim=int(m["dim"]),
                             vdim=int(m["vdim"]), decay=decay)
    raise ValueError(f"unknown mixer type {kind!r}")


def _ffn_from_cfg(f: Optional[Dict[str, Any]]) -> Optional[MoEFFNSpec]:
    if not f:
        return None
    if f.get("kind", "moe") != "moe":
        raise ValueError(f"unknown feed-forward kind {f.get('kind')!r}")
    shared = f.get("shared") or {}
    return MoEFFNSpec(
        n_experts=int(f["router"]["experts"]), top_k=int(f["router"]["top"]),
        ff=int(f["expert"]["ff"]), limit=float(f["expert"]["limit"]),
        shared_ff=int(shared.get("ff", 0)),
        shared_limit=float(shared.get("limit", 0.0)),
    )


def layer_specs_from_cfg(layers: List[Dict[str, Any]]) -> List[LayerSpec]:
    return [LayerSpec(mixer=_mixer_from_cfg(l["type"], l["mixer"]),
                      ffn=_ffn_from_cfg(l.get("mlp"))) for l in layers]


def hybrid_n_params(width: int, vocab: int, taps: int,
                    layers: List[LayerSpec], active_only: bool = False) -> int:
    n = 2 * vocab * width + 1
    for l in layers:
        m = l.mixer
        n += 4 + width * taps
        if m.kind == "latent_attention":
            n += width * (m.q_size + m.cache_dim + m.heads) + m.kv_rank
            n += m.kv_rank * m.heads * (m.dim + m.vdim) + m.heads * m.vdim * width
        else:
            n += width * m.heads * (2 * m.dim + 2 * m.vdim)
            n += m.heads * m.vdim * (1 + width)
        f = l.ffn
        if f is not None:
            e = f.top_k if active_only else f.n_experts
            n += width * f.n_experts + 3 * width * (e * f.ff + f.shared_ff)
    return n


def nukopel_layers(n_layers: int, width: int, *, attn_every: int = 4,
                   heads: int = 16, dim: int = 128, rot_dim: int = 64,
                   vdim: int = 128, kv_rank: int = 512, window: int = 4096,
                   li_heads: int = 16, li_dim: int = 128, li_vdim: int = 128,
                   experts: int = 8, top_k: int = 2, ff: int = 2048,
                   shared_ff: int = 2048, limit: float = 7.0
                   ) -> List[LayerSpec]:
    """A synthetic Nukopel stack for benchmarks: lightning layers with a
    latent-attention layer every `attn_every`-th position."""
    out = []
    for i in range(n_layers):
        if (i + 1) % attn_every == 0:
            mixer: Any = LatentAttnSpec(
                heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim,
                kv_rank=kv_rank, window=window, rope_base=1e6,
                rope_dims=rot_dim, scale=(dim + rot_dim) ** -0.5)
        else:
            decay = tuple(1.0 - 2.0 ** (-5.0 - 3.0 * h / max(1, li_heads - 1))
                          for h in range(li_heads))
            mixer = LightningSpec(heads=li_heads, dim=li_dim, vdim=li_vdim,
                                  decay=decay)
        out.append(LayerSpec(mixer=mixer, ffn=MoEFFNSpec(
            n_experts=experts, top_k=top_k, ff=ff, limit=limit,
            shared_ff=shared_ff, shared_limit=limit)))
    return out
