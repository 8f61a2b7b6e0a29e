"""Pugozen (parallel-form layers: retention, gated delta rule, attention with
a sink beside a delta rule) on the CPU path (fp32 torch ops) against the
plain oracle in tests/pugozen_oracle.py: each mechanism alone, then the
served model through the engine's forced-token entry, its scheduler and the
trace replay."""
import io
import json
import sys

import pytest
import torch

from bee2bee_amd.models.spec import pugozen_spec
from bee2bee_amd.ops import reference as ref
from tests import pugozen_oracle as O
from tests.pugozen_util import (assert_logits, chunk_schedule, make_engine,
                                oracle_logits, random_tokens, rel_err, replay)

F32 = torch.float32
F64 = torch.float64


def i32(x):
    return torch.tensor(x, dtype=torch.int32)


def portions(total, cuts):
    """(start, n) pairs of the cuts (cycled) over `total` rows."""
    out, at, i = [], 0, 0
    while at < total:
        n = min(cuts[i % len(cuts)], total - at)
        out.append((at, n))
        at += n
        i += 1
    return out


# ------------------------------------------------------------- mechanisms

def test_weighted_norm_and_residual_add():
    torch.manual_seed(0)
    x, y, w = torch.randn(5, 37) * 4, torch.randn(5, 37), torch.randn(37)
    want = O.unit(x.double(), 1e-5) * w.double()
    assert torch.allclose(ref.rmsnorm_f32(x, w, 1e-5, F32).double(), want,
                          atol=1e-5)
    r = x.clone()
    out = ref.add_rmsnorm_f32(r, y, w, 1e-5, F32)
    assert torch.allclose(r.double(), x.double() + y.double(), atol=1e-6)
    assert torch.allclose(out.double(), O.unit(
        x.double() + y.double(), 1e-5) * w.double(), atol=1e-5)
    assert ref.add_rmsnorm_f32(r, y, None, 1e-5, F32) is None


def test_relu2_feed_forward():
    torch.manual_seed(1)
    h = torch.randn(6, 10)
    P = {"up": torch.randn(14, 10), "down": torch.randn(10, 14)}
    buf = torch.zeros(6, 30)
    ref.relu2((h @ P["up"].T), buf[:, 8:22])
    got = buf[:, 8:22] @ P["down"].T
    want = O.dense_ff(h.double(), {k: v.double() for k, v in P.items()},
                      {"kind": "dense", "ff": 14})
    assert torch.allclose(got.double(), want, atol=1e-4)
    assert float(buf[:, :8].abs().sum() + buf[:, 22:].abs().sum()) == 0.0


@pytest.mark.parametrize("taps", [1, 2, 3, 5])
@pytest.mark.parametrize("cuts", [[12], [2, 2, 1, 7], [1] * 12, [5, 7]])
def test_short_conv_portions_carry_state(taps, cuts):
    torch.manual_seed(taps)
    C, T = 9, 12
    wide = torch.randn(T, C + 6)
    x = wide[:, 3 : 3 + C]                       # a column slice
    w = torch.randn(C, taps)
    want = O.causal_conv_silu(x.double(), w.double())
    # the slot starts full of NaN: nothing before position 0 may be read
    state = torch.full((3, taps - 1, C), float("nan"))
    got = [ref.short_conv(x[a : a + n], w.t().contiguous(), state, i32([2]),
                          i32([0, n]), i32([0] * n), i32(range(a, a + n)))
           for a, n in portions(T, cuts)]
    assert torch.allclose(torch.cat(got).double(), want, atol=1e-5)


def test_short_conv_batch_of_unequal_chunks():
    torch.manual_seed(1)
    C, taps = 6, 4
    w = torch.randn(C, taps)
    seqs = [torch.randn(n, C) for n in (7, 3, 10)]
    want = [O.causal_conv_silu(s.double(), w.double()) for s in seqs]
    state = torch.full((4, taps - 1, C), float("nan"))
    slots = i32([3, 0, 1])
    outs, at = [[], [], []], [0, 0, 0]
    for takes in ([4, 1, 2], [3, 2, 8]):
        hs, cu, sidx, pos = [], [0], [], []
        for b, n in enumerate(takes):
            hs.append(seqs[b][at[b] : at[b] + n])
            cu.append(cu[-1] + n)
            sidx += [b] * n
            pos += list(range(at[b], at[b] + n))
        o = ref.short_conv(torch.cat(hs), w.t().contiguous(), state, slots,
                           i32(cu), i32(sidx), i32(pos))
        for b, n in enumerate(takes):
            outs[b].append(o[cu[b] : cu[b + 1]])
            at[b] += n
    for b in range(3):
        assert torch.allclose(torch.cat(outs[b]).double(), want[b], atol=1e-5)


@pytest.mark.parametrize("chan", [False, True])
def test_delta_gates_match_formulas(chan):
    torch.manual_seed(2)
    T, G, H, D = 7, 2, 4, 6
    qk = torch.randn(T, 2 * G * D + 3)
    b = torch.randn(T, H)
    a = torch.randn(T, H * (D if chan else 1)) * 3
    dt_bias = torch.randn(H * (D if chan else 1))
    A_log = torch.randn(H) * 0.5
    q0 = qk[:, : G * D].double().view(T, G, D)
    k0 = qk[:, G * D : 2 * G * D].double().view(T, G, D)
    tail = qk[:, 2 * G * D :].clone()
    beta, g = ref.delta_gates(qk, G, D, b, a, dt_bias, torch.exp(A_log), chan)
    want_q = q0 / torch.sqrt((q0 * q0).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    want_k = k0 / torch.sqrt((k0 * k0).sum(-1, keepdim=True) + 1e-6)
    assert torch.allclose(qk[:, : G * D].double().view(T, G, D), want_q,
                          atol=1e-6)
    assert torch.allclose(qk[:, G * D : 2 * G * D].double().view(T, G, D),
                          want_k, atol=1e-6)
    assert torch.equal(qk[:, 2 * G * D :], tail)
    assert torch.allclose(beta.double(), torch.sigmoid(b.double()), atol=1e-6)
    sp = O.softplus(a.double() + dt_bias.double())
    rate = torch.exp(A_log.double())
    want_g = torch.exp(-(rate[None, :, None] * sp.view(T, H, -1))).view(T, -1)
    assert torch.allclose(g.double(), want_g, atol=1e-6)


@pytest.mark.parametrize("chan", [False, True])
@pytest.mark.parametrize("cuts", [[40], [2, 3, 1, 16], [1] * 40, [7, 33]])
def test_delta_rule_portions_match_recurrence(chan, cuts):
    torch.manual_seed(3)
    T, G, H, D, Dv = 40, 2, 4, 6, 5
    q = torch.nn.functional.normalize(torch.randn(T, G, D), dim=-1) * D ** -0.5
    k = torch.nn.functional.normalize(torch.randn(T, G, D), dim=-1)
    v = torch.randn(T, H, Dv)
    beta = torch.rand(T, H)
    g = torch.rand(T, H * (D if chan else 1)) * 0.4 + 0.6
    rep = H // G
    want = O.delta_recurrence(
        q.double().repeat_interleave(rep, 1), k.double().repeat_interleave(rep, 1),
        v.double(), beta.double(),
        g.double().view(T, H, D) if chan else g.double())
    state = torch.full((3, H, D, Dv), float("nan"))
    got = [ref.delta_rule(q[a : a + n], k[a : a + n], v[a : a + n],
                          beta[a : a + n], g[a : a + n], state, i32([1]),
                          i32([0, n]), i32(range(a, a + n)))
           for a, n in portions(T, cuts)]
    assert torch.allclose(torch.cat(got).double(), want, atol=1e-5)


def test_delta_rule_overwrites_a_key():
    """Writing (k, v1) then (k, v2) with beta = 1 and no decay must read back
    v2 alone, hundreds of tokens later: the rule removes what the key held."""
    torch.manual_seed(4)
    T, D, Dv = 300, 16, 4
    k = torch.zeros(T, 1, D)
    v = torch.zeros(T, 1, Dv)
    beta = torch.zeros(T, 1)
    key = torch.nn.functional.normalize(torch.randn(D), dim=0)
    for t, val in ((5, 1.0), (9, -3.0)):
        k[t, 0], v[t, 0], beta[t, 0] = key, val, 1.0
    q = torch.zeros(T, 1, D)
    q[T - 1, 0] = key
    g = torch.ones(T, 1)
    state = torch.zeros(1, 1, D, Dv)
    parts = [ref.delta_rule(q[a : a + n], k[a : a + n], v[a : a + n],
                            beta[a : a + n], g[a : a + n], state, i32([0]),
                            i32([0, n]), i32(range(a, a + n)))
             for a, n in portions(T, [7, 64, 1, 1, 100])]
    out = torch.cat(parts)
    assert torch.allclose(out[T - 1, 0], torch.full((Dv,), -3.0), atol=1e-5)


@pytest.mark.parametrize("dims", [0, 4, 8])
@pytest.mark.parametrize("cuts", [[70], [2, 5, 1, 64], [1] * 70])
def test_retention_portions_match_recurrence(dims, cuts):
    torch.manual_seed(5)
    T, H, D, Dv = 70, 3, 8, 5
    q, k, v = torch.randn(T, H, D), torch.randn(T, H, D), torch.randn(T, H, Dv)
    decay = torch.tensor([0.8, 0.99, 1.0])
    qd, kd = q.double(), k.double()
    if dims:
        qd, kd = O.rotate(qd, dims, 777.0), O.rotate(kd, dims, 777.0)
    want = O.retention_core(qd, kd * D ** -0.5, v.double(), decay.tolist())
    cos = sin = None
    if dims:
        cos, sin = ref.rope_tables_f64(128, dims, 777.0, "cpu")
    state = torch.full((2, H, D, Dv), float("nan"))
    got = [ref.retention_attn(q[a : a + n], k[a : a + n], v[a : a + n], decay,
                              dims, cos, sin, D ** -0.5, state, i32([1]),
                              i32([0, n]), i32(range(a, a + n)))
           for a, n in portions(T, cuts)]
    assert torch.allclose(torch.cat(got).view(T, H, Dv).double(), want,
                          atol=1e-4)


def test_retention_far_token_is_remembered():
    """One early token writes a strong key; a query 400 tokens later, across
    many portions, must read it back with decay^distance."""
    T, D, Dv, lam = 420, 4, 3, 0.995
    q, k, v = torch.zeros(T, 1, D), torch.zeros(T, 1, D), torch.zeros(T, 1, Dv)
    k[11, 0, 2], v[11, 0] = 2.0, torch.tensor([1.0, -2.0, 0.5])
    q[411, 0, 2] = 1.0
    state = torch.zeros(1, 1, D, Dv)
    outs = [ref.retention_attn(q[a : a + n], k[a : a + n], v[a : a + n],
                               torch.tensor([lam]), 0, None, None, 1.0, state,
                               i32([0]), i32([0, n]), i32(range(a, a + n)))
            for a, n in portions(T, [64, 1, 100, 2])]
    got = torch.cat(outs)[411]
    assert torch.allclose(got, 2.0 * lam ** 400 * v[11, 0], rtol=1e-4)


def _paged(seq_len, bs, n_blocks, seed):
    g = torch.Generator().manual_seed(seed)
    need = -(-seq_len // bs)
    return torch.randperm(n_blocks, generator=g)[:need].to(torch.int32)


def _attend(q, k, v, wq, wk, dims, base, q_mult, sink, cuts, bs=8, window=0):
    """Feed q/k through norm+rotation+store and attention, portion by portion,
    over scattered pages. q [T,H,D], k [T,G,D]; returns [T, H*D]."""
    T, H, D = q.shape
    G = k.shape[1]
    nb = 2 * (-(-T // bs)) + 3
    bt = _paged(T, bs, nb, 5)
    kc = torch.full((nb, G, bs, D), float("nan"))
    vc = torch.full((nb, G, bs, D), float("nan"))
    cos = sin = None
    if dims:
        cos, sin = ref.rope_tables_f64(T + 1, dims, base, "cpu")
    outs = []
    for a, n in portions(T, cuts):
        pos = list(range(a, a + n))
        slots = [int(bt[p // bs]) * bs + p % bs for p in pos]
        wide = torch.zeros(n, H * D + 4)
        qq = q[a : a + n].clone()
        ref.qk_norm_rope_store(qq, k[a : a + n], wq, wk, 1e-5, dims, i32(pos),
                               cos, sin, q_mult, kc, vc, i32(slots))
        ref.sink_attn(qq, kc, vc, bt[None], i32(pos), i32([0] * n),
                      i32([0, n]), sink, window, wide[:, 2 : 2 + H * D], 1.0)
        outs.append(wide[:, 2 : 2 + H * D].clone())
    return torch.cat(outs)


@pytest.mark.parametrize("cuts", [[50], [2, 7, 1, 24], [1] * 50])
@pytest.mark.parametrize("dims", [0, 4, 6])
def test_sink_attention_matches_oracle(cuts, dims):
    torch.manual_seed(6)
    T, H, G, D = 50, 4, 2, 6
    q, k = torch.randn(T, H, D), torch.randn(T, G, D)
    wq, wk = torch.rand(D) + 0.5, torch.rand(D) + 0.5
    temp, sink = torch.rand(H) + 0.5, torch.randn(H) * 2
    scale = 0.4
    qd = O.unit(q.double(), 1e-5) * wq.double()
    kd = O.unit(k.double(), 1e-5) * wk.double()
    if dims:
        qd, kd = O.rotate(qd, dims, 3000.0), O.rotate(kd, dims, 3000.0)
    want = O.softmax_sink_core(qd, kd, k.double(), scale, temp, sink)
    got = _attend(q, k, k, wq, wk, dims, 3000.0, temp * scale, sink, cuts)
    assert torch.allclose(got.double(), want.reshape(T, -1), atol=1e-5)


def test_sink_takes_weight_and_counts_once():
    """With a large sink most of the weight goes to it (the output shrinks);
    a sink of -inf equals plain softmax; the sink is neither scaled nor
    multiplied by the head's score multiplier."""
    torch.manual_seed(7)
    T, H, D = 12, 2, 4
    q, k = torch.randn(T, H, D), torch.randn(T, 1, D)
    one = torch.ones(D)
    big = _attend(q, k, k, one, one, 0, 1.0, torch.tensor([5.0, 0.1]),
                  torch.tensor([6.0, 6.0]), [T])
    none = _attend(q, k, k, one, one, 0, 1.0, torch.tensor([5.0, 0.1]), None,
                   [T])
    # head 1 (small multiplier, scores near 0): weight of the sink is
    # exp(6) / (exp(6) + ~n) however many keys there are
    ratio = big[:, D:].norm(dim=-1) / none[:, D:].norm(dim=-1)
    n = torch.arange(1, T + 1, dtype=torch.float32)
    want = n / (n + torch.exp(torch.tensor(6.0)))
    assert torch.allclose(ratio, want, rtol=0.35)
    assert float(ratio.max()) < 0.05


@pytest.mark.parametrize("decoded", [False, True])
@pytest.mark.parametrize("far", [0, 7, 8, 63, 64, 200])
def test_far_key_among_hundreds(decoded, far):
    """One key far back (first token, page borders) is made to stand out for
    the last query; the output must be that key's value."""
    torch.manual_seed(8)
    T, H, D, bs = 330, 2, 8, 8
    q, k = torch.randn(T, H, D) * 0.1, torch.randn(T, 1, D) * 0.1
    mark = torch.nn.functional.normalize(torch.randn(D), dim=0)
    k[far, 0] = 5.0 * mark
    q[T - 1] = 9.0 * mark
    one = torch.ones(D)
    cuts = [300] + [1] * 30 if decoded else [64, 200, 66]
    # the head norm keeps directions (weights one); a large multiplier
    # lets the marked key win over the hundreds of random ones
    got = _attend(q, k, k, one, one, 0, 1.0, torch.tensor([12.0, 12.0]),
                  torch.zeros(H), cuts, bs=bs)
    last = got[T - 1].view(H, D)
    assert torch.allclose(last, k[far, 0].expand(H, D), atol=2e-3)


@pytest.mark.parametrize("decoded", [False, True])
def test_window_edges(decoded):
    """The op's window parameter: the key just inside is seen, the key just
    outside is not."""
    torch.manual_seed(9)
    T, D, W = 40, 4, 9
    one = torch.ones(D)
    cuts = [30] + [1] * 10 if decoded else [13, 27]
    for dist, seen in ((W - 1, True), (W, False)):
        q, k = torch.randn(T, 1, D) * 0.05, torch.randn(T, 1, D) * 0.05
        mark = torch.tensor([1.0, 0.0, 0.0, 0.0])
        k[T - 1 - dist, 0] = 6.0 * mark
        q[T - 1, 0] = 8.0 * mark
        got = _attend(q, k, k, one, one, 0, 1.0, torch.tensor([3.0]), None,
                      cuts, window=W)[T - 1]
        assert (float(got[0]) > 5.0) == seen


@pytest.mark.parametrize("H,Dv,weighted,act", [(3, 5, True, "silu"),
                                               (1, 8, False, "silu"),
                                               (2, 6, True, "sigmoid")])
def test_head_gated_norm(H, Dv, weighted, act):
    torch.manual_seed(10)
    T = 6
    o, gate = torch.randn(T, H, Dv) * 3, torch.randn(T, H * Dv)
    w = torch.randn(Dv) if weighted else None
    wide = torch.zeros(T, H * Dv + 5)
    ref.head_gated_norm(o, w, gate, act, 1e-5, wide[:, 1 : 1 + H * Dv], 0.6)
    y = O.unit(o.double(), 1e-5)
    if weighted:
        y = y * w.double()
    gd = gate.double().view(T, H, Dv)
    y = y * (torch.sigmoid(gd) if act == "sigmoid" else O.silu(gd)) * 0.6
    assert torch.allclose(wide[:, 1 : 1 + H * Dv].double(),
                          y.reshape(T, -1), atol=1e-5)
    assert float(wide[:, 0].abs().sum() + wide[:, 1 + H * Dv :].abs().sum()) == 0


# ------------------------------------------------------------- config

def test_config_is_read_not_assumed():
    cfg = O.make_config(order=("delta", "parallel", "retention", "parallel"),
                        shared=((3, 1),), heads=6, kv_heads=3, dim=10,
                        rot_dims=4, rot_base=123.0, scale=0.77,
                        left_scale=0.3, right_scale=1.9, r_heads=3,
                        r_kv_heads=3, r_conv=2, ret_heads=2,
                        ret_decay=(0.5, 0.75), ret_rot=2, d_conv=5,
                        emb_scale=1.5, eps=3e-4, ff=24)
    cfg["layers"][2]["mlp"] = None
    shapes = {"l1.mix.right.a1": (7, 40), "l1.mix.right.g1": (9, 40)}
    s = pugozen_spec("x", cfg, shapes)
    d, p, r, p2 = s.layer_specs
    assert s.is_hybrid and s.arch == "pugozen" and s.n_layers == 4
    assert (s.embed_scale, s.rms_eps, s.canon_taps) == (1.5, 3e-4, 0)
    assert all(l.form == "parallel" for l in s.layer_specs)
    assert (d.mixer.taps, d.mixer.channel_decay, d.mixer.gate) == (5, False,
                                                                   "silu")
    a, b = p.mixer.left, p.mixer.right
    assert (a.heads, a.kv_heads, a.dim, a.rope_dims, a.rope_base, a.scale) == (
        6, 3, 10, 4, 123.0, 0.77)
    assert (b.heads, b.kv_heads, b.taps, b.channel_decay, b.gate,
            b.decay_rank, b.gate_rank) == (3, 3, 2, True, "sigmoid", 7, 9)
    assert (p.mixer.left_scale, p.mixer.right_scale) == (0.3, 1.9)
    assert r.mixer.decay == (0.5, 0.75) and r.mixer.rope_dims == 2
    assert r.ffn is None and p.ffn.ff == 24
    assert p2.weights_of == 1 and p.weights_of is None
    # the shared layer takes its low-rank widths from the owner's tensors
    assert (p2.mixer.right.decay_rank, p2.mixer.right.gate_rank) == (7, 9)


# ------------------------------------------------------------ served model

VARIANTS = {
    "base": dict(order=("parallel", "retention", "delta", "parallel",
                        "retention"), shared=((3, 0), (4, 1))),
    "ones": dict(order=("delta", "parallel", "retention"), heads=1,
                 kv_heads=1, dim=2, rot_dims=2, r_heads=1, r_kv_heads=1,
                 r_dim=1, r_vdim=1, r_conv=1, ret_heads=1, ret_dim=2,
                 ret_vdim=1, ret_rot=2, ret_decay=(1.0,), d_heads=1,
                 d_kv_heads=1, d_dim=1, d_vdim=1, d_conv=1, emb_scale=1.0,
                 left_scale=1.0, right_scale=1.0, scale=1.0),
    "equal-sizes": dict(order=("retention", "parallel", "delta"), heads=2,
                        kv_heads=2, dim=8, rot_dims=8, r_heads=2, r_kv_heads=2,
                        r_dim=8, r_vdim=8, r_conv=2, ret_heads=2, ret_dim=8,
                        ret_vdim=8, ret_rot=8, ret_decay=(0.9, 0.9), d_heads=2,
                        d_kv_heads=2, d_dim=8, d_vdim=8, d_conv=2, ff=40,
                        width=40),
    "shared-chain": dict(order=("delta", "delta", "delta", "parallel"),
                         shared=((1, 0), (2, 0)), width=24, vocab=33, ff=17),
    "wide-heads": dict(order=("parallel", "delta"), heads=6, kv_heads=1,
                       dim=20, rot_dims=10, d_heads=6, d_kv_heads=3, d_dim=9,
                       d_vdim=3, r_heads=4, r_kv_heads=2, r_dim=3, r_vdim=9,
                       r_conv=5),
}


def _cfg(name):
    cfg = O.make_config(**VARIANTS[name])
    if name == "wide-heads":
        cfg["layers"][1]["mlp"] = None      # a layer without feed-forward
    return cfg


@pytest.mark.parametrize("name", list(VARIANTS))
def test_served_model_matches_oracle(tmp_path, name):
    cfg = _cfg(name)
    W = O.random_weights(cfg, seed=11)
    eng = make_engine(tmp_path, cfg, W)
    toks = random_tokens(45, cfg["vocab"], 1)
    want = oracle_logits(cfg, W, toks)
    schedules = {
        "whole": [[("a", 45)]],
        "decode": [[("a", 9)]] + [[("a", 1)]] * 36,
        "portions": chunk_schedule("a", 45, [2, 5, 1, 16, 3]),
        "twos": chunk_schedule("a", 45, [2]),
        "token-by-token": [[("a", 1)]] * 45,
    }
    for what, sched in schedules.items():
        got = replay(eng, {"a": toks}, sched)["a"]
        assert_logits(got, want, F32, what)
    assert eng.kv.free_blocks == eng.kv.n_blocks - 1     # scratch page only


def test_layer_residuals_match_oracle(tmp_path):
    cfg = _cfg("base")
    W = O.random_weights(cfg, seed=12)
    eng = make_engine(tmp_path, cfg, W)
    toks = random_tokens(19, cfg["vocab"], 2)
    layers = []
    O.forward(toks, cfg, W, layers)
    seen = []
    eng.runner.layer_tap = lambda i, x: seen.append(x.clone())
    eng.feed([("a", toks, [])], ["a"])
    assert len(seen) == len(layers) == 5
    for i, x in enumerate(seen):
        assert torch.allclose(x.double(), layers[i], atol=1e-3), i


def test_shared_layers_keep_their_own_state(tmp_path):
    """Layers that run the same tensors have their own pages and state: the
    logits differ from a model in which the copy is left out, and decoding
    equals the whole prompt."""
    cfg = _cfg("shared-chain")
    W = O.random_weights(cfg, seed=19)
    eng = make_engine(tmp_path, cfg, W)
    assert eng.weights.layers[1] is eng.weights.layers[0]
    assert eng.kv.rec_state[1] is not eng.kv.rec_state[0]
    toks = random_tokens(30, cfg["vocab"], 7)
    got = replay(eng, {"a": toks}, [[("a", 4)]] + [[("a", 1)]] * 26)["a"]
    assert_logits(got, oracle_logits(cfg, W, toks), F32)


def test_mixed_batches_and_reuse(tmp_path):
    """Unequal requests side by side (portions next to single tokens, a
    request sitting out a step) equal each request alone; the pool is far
    smaller than the sum of the requests, so pages and slots come back."""
    cfg = _cfg("base")
    W = O.random_weights(cfg, seed=13)
    eng = make_engine(tmp_path, cfg, W, kv_blocks=7, block_size=8,
                      max_batch=3)
    lens = [21, 6, 30, 11, 17, 2, 26]
    reqs = {f"r{i}": random_tokens(n, cfg["vocab"], 20 + i)
            for i, n in enumerate(lens)}
    sched = [
        [("r0", 9), ("r1", 2)],
        [("r0", 1), ("r1", 3), ("r2", 5)],
        [("r0", 11), ("r2", 1)],                    # r1 sits out; r0 ends
        [("r1", 1), ("r2", 2), ("r3", 11)],         # r1, r3 end
        [("r2", 22), ("r4", 2)],                    # r2 ends
        [("r4", 15), ("r5", 2), ("r6", 3)],         # r4, r5 end
        [("r6", 1)], [("r6", 22)],
    ]
    got = replay(eng, reqs, sched)
    for rid, toks in reqs.items():
        assert_logits(got[rid], oracle_logits(cfg, W, toks), F32, rid)
    assert eng.kv.free_blocks == eng.kv.n_blocks - 1
    assert eng.kv.free_state_slots == eng.kv.n_state_slots - 1


def test_long_decode_crosses_pages(tmp_path):
    cfg = _cfg("base")
    W = O.random_weights(cfg, seed=14)
    eng = make_engine(tmp_path, cfg, W, block_size=4, kv_blocks=50)
    toks = random_tokens(140, cfg["vocab"], 3)
    got = replay(eng, {"a": toks}, [[("a", 3)]] + [[("a", 1)]] * 137)["a"]
    assert_logits(got, oracle_logits(cfg, W, toks), F32)


def test_first_tokens_after_slot_reuse(tmp_path):
    """A request that takes over a slot and pages another one just left must
    not see anything of it in its first tokens."""
    cfg = _cfg("base")
    W = O.random_weights(cfg, seed=15)
    eng = make_engine(tmp_path, cfg, W, max_batch=1, kv_blocks=3, block_size=16)
    a, b = random_tokens(40, cfg["vocab"], 4), random_tokens(6, cfg["vocab"], 5)
    replay(eng, {"a": a}, [[("a", 40)]])
    for sched in ([[("b", 6)]], [[("b", 1)]] * 6, [[("b", 2)], [("b", 4)]]):
        got = replay(eng, {"b": b}, sched)["b"]
        assert_logits(got, oracle_logits(cfg, W, b), F32)


def test_greedy_generation_through_scheduler(tmp_path):
    """submit()/generate(): admission, chunked prompt prefill (budget of 7
    tokens a step), batched decode of concurrent requests, retirement."""
    cfg = _cfg("base")
    W = O.random_weights(cfg, seed=16)
    eng = make_engine(tmp_path, cfg, W, max_prefill_tokens=7)
    try:
        from bee2bee_amd.engine.engine import GenerationRequest
        from bee2bee_amd.engine.sampler import SamplingParams

        prompts = [random_tokens(n, cfg["vocab"], 30 + n) for n in (17, 3, 9)]
        reqs = [eng.submit(GenerationRequest(
            prompt_ids=list(p), max_new_tokens=10,
            sampling=SamplingParams(greedy=True))) for p in prompts]
        for r in reqs:
            while r.done_ts is None:
                r.out_queue.get(timeout=60)
        for p, r in zip(prompts, reqs):
            assert len(r.output_ids) == 10 and r.error is None
            seq = list(p)
            for tok in r.output_ids:
                logits = oracle_logits(cfg, W, seq)[-1]
                top2 = torch.topk(logits, 2).values
                if float(top2[0] - top2[1]) > 1e-3:
                    assert int(logits.argmax()) == tok
                seq.append(tok)
    finally:
        eng.shutdown()


def test_trace_replay_writes_wanted_logits(tmp_path, monkeypatch, capsys):
    from bee2bee_amd.engine import trace

    cfg = _cfg("wide-heads")
    W = O.random_weights(cfg, seed=17)
    O.save_checkpoint(str(tmp_path / "m"), cfg, W)
    toks = random_tokens(12, cfg["vocab"], 6)
    steps = [
        {"step": 0, "entries": [{"id": "q", "tokens": toks[:7], "want": [0, 6]}],
         "end": []},
        {"step": 1, "entries": [{"id": "q", "tokens": toks[7:8], "want": []}],
         "end": []},
        {"step": 2, "entries": [{"id": "q", "tokens": toks[8:], "want": [3]}],
         "end": ["q"]},
    ]
    monkeypatch.setattr(sys, "stdin", io.StringIO(
        "\n".join(json.dumps(s) for s in steps) + "\n"))
    out = tmp_path / "out"
    assert trace.main(["--model", str(tmp_path / "m"), "--dtype", "float32",
                       "--out", str(out), "--max-tokens", "64"]) == 0
    assert capsys.readouterr().out.split() == ["done", "0", "done", "1",
                                               "done", "2"]
    import numpy as np

    want = oracle_logits(cfg, W, toks)
    a = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1))
    c = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4").reshape(1, -1))
    assert not (out / "1.f32").exists()
    assert rel_err(a, want[[0, 6]]) < 2e-4 and rel_err(c, want[[11]]) < 2e-4


def test_checkpoint_roundtrip(tmp_path):
    """load -> save_hf -> load: the same tensors under the same names, the
    same config, the same logits."""
    from safetensors.torch import load_file

    from bee2bee_amd.models.weights import safetensors_shapes, save_hf

    cfg = _cfg("base")
    W = O.random_weights(cfg, seed=18)
    eng = make_engine(tmp_path, cfg, W)
    out = tmp_path / "resaved"
    save_hf(eng.weights, str(out))
    W2 = load_file(str(out / "model.safetensors"))
    assert set(W2) == set(W)
    for k in W2:
        assert torch.allclose(W2[k].float(), W[k].float(), rtol=1e-2), k
        if not k.endswith("A_log"):          # stored as exp(), logged back
            assert torch.equal(W2[k].float(), W[k].float()), k
    cfg2 = json.load(open(out / "config.json"))
    a = pugozen_spec("a", cfg, safetensors_shapes(str(tmp_path / "ckpt")))
    b = pugozen_spec("b", cfg2, safetensors_shapes(str(out)))
    assert a.layer_specs == b.layer_specs
    assert (a.vocab_size, a.hidden_size, a.embed_scale, a.rms_eps) == (
        b.vocab_size, b.hidden_size, b.embed_scale, b.rms_eps)
