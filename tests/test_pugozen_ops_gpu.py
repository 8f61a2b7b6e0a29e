"""HIP kernels of the parallel-form stacks (weighted fp32 norms, relu^2,
short conv, delta-rule gates and recurrence, per-head gated norm, q/k norm +
rotation + page store, sink attention, retention) against the fp32 torch
reference of the same op (ops/reference.py), in bf16 and fp32, at sizes that
are neither powers of two nor multiples of the wave size, on column slices
of wider buffers as the runner passes them."""
import pytest
import torch

from bee2bee_amd import ops
from bee2bee_amd.ops import reference as ref

pytestmark = pytest.mark.gpu

if not torch.cuda.is_available():
    pytest.skip("needs a GPU", allow_module_level=True)

from tests.test_hybrid_ops_gpu import DEV, DTYPES, batch_meta, tol  # noqa: E402


def sliced(T, n, dtype, pad=8, scale=1.0):
    """A [T, n] column slice in the middle of a wider buffer."""
    buf = (torch.randn(T, n + 2 * pad, device=DEV) * scale).to(dtype)
    return buf[:, pad : pad + n]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W", [37, 48, 200, 1024])
def test_weighted_norms(dtype, W):
    torch.manual_seed(0)
    x = torch.randn(6, W, device=DEV) * 3
    w = torch.randn(W, device=DEV)
    y = ops.rmsnorm_f32(x, w, 1e-5, dtype)
    torch.testing.assert_close(
        y.float(), ref.rmsnorm_f32(x, w, 1e-5, dtype).float(), **tol(dtype))
    add = torch.randn(6, W, device=DEV).to(dtype)
    r1, r2 = x.clone(), x.clone()
    a = ops.add_rmsnorm_f32(r1, add, w, 1e-5, dtype)
    b = ref.add_rmsnorm_f32(r2, add, w, 1e-5, dtype)
    torch.testing.assert_close(r1, r2, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(a.float(), b.float(), **tol(dtype))
    assert ops.add_rmsnorm_f32(r1, add, None, 1e-5, dtype) is None
    ref.add_rmsnorm_f32(r2, add, None, 1e-5, dtype)
    torch.testing.assert_close(r1, r2, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n,pad", [(40, 8), (37, 3), (512, 8)])
def test_relu2(dtype, n, pad):
    torch.manual_seed(1)
    x = sliced(9, n, dtype, pad)
    o1 = sliced(9, n, dtype, pad)
    o2 = o1.clone()
    ops.relu2(x, o1)
    ref.relu2(x, o2)
    torch.testing.assert_close(o1.float(), o2.float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C,taps,pad", [(40, 4, 8), (37, 3, 3), (300, 2, 8),
                                        (24, 1, 8)])
def test_short_conv(dtype, C, taps, pad):
    torch.manual_seed(2)
    m = batch_meta([5, 1, 2, 9], [0, 7, 1, 3], 16, 8)
    x = sliced(m["T"], C, dtype, pad)
    w = torch.randn(taps, C, device=DEV) * 0.5
    st1 = torch.randn(6, max(taps - 1, 0), C, device=DEV).to(dtype)
    st1[m["state_slots"].long()[0]] = float("nan")   # starts at position 0
    st2 = st1.clone()
    for silu in (True, False):
        a = ops.short_conv(x, w, st1, m["state_slots"], m["cu"], m["seq"],
                           m["pos"], silu)
        b = ref.short_conv(x, w, st2, m["state_slots"], m["cu"], m["seq"],
                           m["pos"], silu)
        assert a.dtype == torch.float32
        torch.testing.assert_close(a, b, **tol(torch.float32))
        live = m["state_slots"].long()
        torch.testing.assert_close(st1[live].float(), st2[live].float(),
                                   rtol=0, atol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("G,H,D,chan", [(2, 4, 24, False), (3, 3, 40, True),
                                        (1, 2, 64, True)])
def test_delta_gates(dtype, G, H, D, chan):
    torch.manual_seed(3)
    T = 11
    qk1 = torch.randn(T, 2 * G * D + 5, device=DEV)
    qk2 = qk1.clone()
    per = D if chan else 1
    b = sliced(T, H, dtype, 3)
    a = sliced(T, H * per, dtype, 8, scale=3.0)
    dt_bias = torch.randn(H * per, device=DEV)
    rate = torch.rand(H, device=DEV) + 0.2
    beta1, g1 = ops.delta_gates(qk1, G, D, b, a, dt_bias, rate, chan)
    beta2, g2 = ref.delta_gates(qk2, G, D, b, a, dt_bias, rate, chan)
    torch.testing.assert_close(qk1, qk2, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(beta1, beta2, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(g1, g2, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("G,H,D,Dv,chan", [
    (2, 4, 24, 40, False), (3, 3, 40, 24, True), (1, 2, 64, 64, True),
    (2, 2, 128, 128, False), (1, 1, 7, 5, True), (2, 4, 200, 20, False),
    # enough (sequence, head, column) work for 8 and for 4 row groups
    (8, 32, 16, 128, True), (64, 64, 12, 128, False)])
def test_delta_rule(G, H, D, Dv, chan):
    torch.manual_seed(4)
    m = batch_meta([19, 1, 2, 33], [0, 7, 1, 3], 16, 8)
    T = m["T"]
    C = 2 * G * D + H * Dv
    buf = torch.randn(T, C, device=DEV)
    nq = G * D
    q = buf[:, :nq].view(T, G, D)
    k = buf[:, nq : 2 * nq].view(T, G, D)
    v = buf[:, 2 * nq :].view(T, H, Dv)
    q.mul_(torch.rsqrt(q.pow(2).sum(-1, keepdim=True)) * D ** -0.5)
    k.mul_(torch.rsqrt(k.pow(2).sum(-1, keepdim=True)))
    beta = torch.rand(T, H, device=DEV)
    g = torch.rand(T, H * (D if chan else 1), device=DEV) * 0.5 + 0.5
    st1 = torch.randn(6, H, D, Dv, device=DEV)
    st1[m["state_slots"].long()[0]] = float("nan")
    st2 = st1.clone()
    a = ops.delta_rule(q, k, v, beta, g, st1, m["state_slots"], m["cu"],
                       m["pos"])
    b = ref.delta_rule(q, k, v, beta, g, st2, m["state_slots"], m["cu"],
                       m["pos"])
    torch.testing.assert_close(a, b, rtol=2e-4, atol=2e-5)
    live = m["state_slots"].long()
    torch.testing.assert_close(st1[live], st2[live], rtol=2e-4, atol=2e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,Dv,weighted,act", [(3, 40, True, "silu"),
                                               (2, 64, False, "silu"),
                                               (5, 129, True, "sigmoid")])
def test_head_gated_norm(dtype, H, Dv, weighted, act):
    torch.manual_seed(5)
    T = 7
    o = torch.randn(T, H, Dv, device=DEV) * 4
    w = torch.randn(Dv, device=DEV) if weighted else None
    gate = sliced(T, H * Dv, dtype, 8)
    o1 = sliced(T, H * Dv, dtype, 8)
    o2 = o1.clone()
    ops.head_gated_norm(o, w, gate, act, 1e-5, o1, 0.7)
    ref.head_gated_norm(o, w, gate, act, 1e-5, o2, 0.7)
    torch.testing.assert_close(o1.float(), o2.float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,dims,window", [
    (6, 3, 64, 16, 0), (4, 1, 40, 40, 0), (2, 2, 24, 0, 0), (8, 2, 128, 64, 0),
    (4, 2, 72, 8, 5), (3, 3, 200, 100, 0), (2, 1, 20, 4, 0), (6, 1, 12, 12, 3), (2, 1, 21, 0, 0), (4, 4, 160, 32, 0)])
def test_sink_attention(dtype, H, G, D, dims, window):
    torch.manual_seed(6)
    bs, nb = 16, 24
    m = batch_meta([21, 1, 2, 40, 1], [0, 70, 15, 3, 0], bs, nb)
    T = m["T"]
    qbuf = (torch.randn(T, H * D + G * D + 16, device=DEV)).to(dtype)
    q1 = qbuf[:, 8 : 8 + H * D].view(T, H, D)
    k = qbuf[:, 8 + H * D : 8 + H * D + G * D].view(T, G, D)
    q2 = q1.clone()
    wq = torch.randn(D, device=DEV)
    wk = torch.randn(D, device=DEV)
    q_mult = torch.rand(H, device=DEV) * 0.3 + 0.05
    cos = sin = None
    if dims:
        cos, sin = ops.rope_tables_f64(128, dims, 5e4, DEV)
    kc1 = torch.randn(nb, G, bs, D, device=DEV).to(dtype)
    vc1 = torch.randn(nb, G, bs, D, device=DEV).to(dtype)
    # history of the chunks that do not start at position 0
    kc2, vc2 = kc1.clone(), vc1.clone()
    ops.qk_norm_rope_store(q1, k, wq, wk, 1e-5, dims, m["pos"], cos, sin,
                           q_mult, kc1, vc1, m["slot_map"])
    ref.qk_norm_rope_store(q2, k, wq, wk, 1e-5, dims, m["pos"], cos, sin,
                           q_mult, kc2, vc2, m["slot_map"])
    torch.testing.assert_close(q1.float(), q2.float(), **tol(dtype))
    torch.testing.assert_close(kc1.float(), kc2.float(), **tol(dtype))
    torch.testing.assert_close(vc1.float(), vc2.float(), rtol=0, atol=0)
    sink = torch.randn(H, device=DEV)
    for sk in (sink, None):
        for max_q in (40, 1):
            o1 = sliced(T, H * D, dtype)
            o2 = o1.clone()
            ops.sink_attn(q2, kc2, vc2, m["bt"], m["pos"], m["seq"], m["cu"],
                          sk, window, o1, 0.8, max_q)
            ref.sink_attn(q2, kc2, vc2, m["bt"], m["pos"], m["seq"], m["cu"],
                          sk, window, o2, 0.8)
            torch.testing.assert_close(o1.float(), o2.float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_sink_attention_decode_split(dtype):
    """Few rows over long contexts: the key-split path and its merge."""
    torch.manual_seed(7)
    H, G, D, bs, nb = 4, 2, 64, 16, 80
    m = batch_meta([1, 1, 1], [700, 0, 255], bs, nb)
    T = m["T"]
    q = torch.randn(T, H, D, device=DEV).to(dtype) * 0.3
    kc = torch.randn(nb, G, bs, D, device=DEV).to(dtype)
    vc = torch.randn(nb, G, bs, D, device=DEV).to(dtype)
    sink = torch.randn(H, device=DEV)
    o1 = sliced(T, H * D, dtype)
    o2 = o1.clone()
    ops.sink_attn(q, kc, vc, m["bt"], m["pos"], m["seq"], m["cu"], sink, 0,
                  o1, 1.0, 1)
    ref.sink_attn(q, kc, vc, m["bt"], m["pos"], m["seq"], m["cu"], sink, 0,
                  o2, 1.0)
    torch.testing.assert_close(o1.float(), o2.float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,D,Dv,dims,lens", [
    (3, 24, 40, 24, [19, 1, 2, 33]), (2, 64, 64, 32, [5, 1, 1, 300]),
    (2, 32, 72, 0, [600, 1, 2, 7])])
def test_retention(dtype, H, D, Dv, dims, lens):
    torch.manual_seed(8)
    m = batch_meta(lens, [0, 7, 1, 3], 16, 64)
    T = m["T"]
    buf = (torch.randn(T, 2 * H * D + H * Dv, device=DEV)).to(dtype)
    q = buf[:, : H * D].view(T, H, D)
    k = buf[:, H * D : 2 * H * D].view(T, H, D)
    v = buf[:, 2 * H * D :].view(T, H, Dv)
    decay = torch.tensor([1 - 2.0 ** -(3 + h) for h in range(H)], device=DEV)
    cos = sin = None
    if dims:
        cos, sin = ops.rope_tables_f64(1024, dims, 1e4, DEV)
    st1 = torch.randn(6, H, D, Dv, device=DEV)
    st1[m["state_slots"].long()[0]] = float("nan")
    st2 = st1.clone()
    a = ops.retention_attn(q, k, v, decay, dims, cos, sin, D ** -0.5, st1,
                           m["state_slots"], m["cu"], m["pos"], max(lens))
    b = ref.retention_attn(q, k, v, decay, dims, cos, sin, D ** -0.5, st2,
                           m["state_slots"], m["cu"], m["pos"])
    torch.testing.assert_close(a, b, rtol=3e-4, atol=3e-4)
    live = m["state_slots"].long()
    torch.testing.assert_close(st1[live], st2[live], rtol=3e-4, atol=3e-4)
