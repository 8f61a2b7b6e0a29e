"""HIP kernels of the hybrid stacks against the fp32 torch reference of the
same op (ops/reference.py), in bf16 and fp32, at sizes that are neither
powers of two nor multiples of the wave size."""
import pytest
import torch

from bee2bee_amd import ops
from bee2bee_amd.ops import reference as ref

pytestmark = pytest.mark.gpu

if not torch.cuda.is_available():
    pytest.skip("needs a GPU", allow_module_level=True)

DEV = torch.device("cuda:0")
DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype):
    return dict(rtol=2e-5, atol=2e-5) if dtype is torch.float32 else dict(
        rtol=2e-2, atol=2e-2)


def batch_meta(lens, starts, block_size, n_blocks, seed=0):
    """Packed-chunk metadata with scattered pages and shuffled slots."""
    g = torch.Generator().manual_seed(seed)
    B = len(lens)
    cu = [0]
    pos, seq = [], []
    for b, (L, s) in enumerate(zip(lens, starts)):
        cu.append(cu[-1] + L)
        pos += list(range(s, s + L))
        seq += [b] * L
    need = [-(-(s + L) // block_size) for L, s in zip(lens, starts)]
    perm = torch.randperm(n_blocks, generator=g).tolist()
    bt = torch.zeros(B, max(need), dtype=torch.int32)
    k = 0
    for b in range(B):
        for j in range(need[b]):
            bt[b, j] = perm[k]
            k += 1
    slot_map = [int(bt[b, p // block_size]) * block_size + p % block_size
                for b, p in zip(seq, pos)]
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)  # noqa: E731
    state_slots = torch.randperm(B + 2, generator=g)[:B].to(torch.int32).to(DEV)
    return dict(cu=i32(cu), pos=i32(pos), seq=i32(seq), bt=bt.to(DEV),
                slot_map=i32(slot_map), state_slots=state_slots, T=cu[-1])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W", [37, 48, 200, 1024, 4096])
def test_scalar_norms(dtype, W):
    torch.manual_seed(0)
    x = torch.randn(7, W, device=DEV) * 3
    y = ops.scalar_rmsnorm(x, 1.3, 1e-5, dtype)
    torch.testing.assert_close(y.float(), ref.scalar_rmsnorm(
        x, 1.3, 1e-5, dtype).float(), **tol(dtype))
    for y_dtype in {dtype, torch.float32}:
        a = (torch.randn(7, W, device=DEV) * 2).to(y_dtype)
        b = (torch.randn(7, W, device=DEV)).to(y_dtype)
        for pre, y2 in ((0.7, None), (None, None), (1.1, b)):
            r1, r2 = x.clone(), x.clone()
            o1 = ops.add_scalar_rmsnorm(r1, a, 0.9, pre, 1e-5, dtype, y2=y2)
            o2 = ref.add_scalar_rmsnorm(r2, a, 0.9, pre, 1e-5, dtype, y2=y2)
            torch.testing.assert_close(r1, r2, rtol=1e-5, atol=1e-5)
            assert (o1 is None) == (o2 is None)
            if o1 is not None:
                torch.testing.assert_close(o1.float(), o2.float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_gated_norm_and_glu(dtype):
    torch.manual_seed(1)
    x = torch.randn(9, 168, device=DEV)
    w = torch.rand(168, device=DEV) + 0.5
    big = torch.randn(9, 400, device=DEV).to(dtype)
    gate = big[:, 100:268]                      # strided view, odd offset
    y = ops.gated_rmsnorm(x, w, gate, 1e-6, dtype)
    torch.testing.assert_close(
        y.float(), ref.gated_rmsnorm(x, w, gate, 1e-6, dtype).float(),
        **tol(dtype))
    gu = (torch.randn(3, 11, 2 * 37, device=DEV) * 3).to(dtype)
    torch.testing.assert_close(
        ops.clamped_glu(gu, 1.5, 1.702).float(),
        ref.clamped_glu(gu, 1.5, 1.702).float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("taps", [1, 2, 4])
@pytest.mark.parametrize("C", [72, 73, 1024])
def test_canon_conv_chunks_and_state(dtype, taps, C):
    torch.manual_seed(2)
    m = batch_meta([5, 1, 2, 9], [0, 7, 1, 30], 16, 16)
    h = torch.randn(m["T"], C, device=DEV).to(dtype)
    w = torch.randn(taps, C, device=DEV) * 0.3
    st = torch.randn(6, max(taps - 1, 0), C, device=DEV).to(dtype)
    st1, st2 = st.clone(), st.clone()
    o1 = ops.canon_conv(h, w, st1, m["state_slots"], m["cu"], m["seq"], m["pos"])
    o2 = ref.canon_conv(h, w, st2, m["state_slots"], m["cu"], m["seq"], m["pos"])
    torch.testing.assert_close(o1.float(), o2.float(), **tol(dtype))
    torch.testing.assert_close(st1.float(), st2.float(), rtol=0, atol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,C,R,dims,window", [
    (3, 20, 4, 4, 7), (7, 88, 24, 16, 37), (5, 130, 24, 16, 1),
    (2, 512, 64, 64, 300)])
def test_latent_store_and_attention(dtype, H, C, R, dims, window):
    torch.manual_seed(3)
    bs = 16
    lens, starts = [33, 1, 2, 1], [0, 47, 15, 0]
    m = batch_meta(lens, starts, bs, 16)
    T = m["T"]
    cache = (torch.randn(16, bs, C + R, device=DEV)).to(dtype)
    # history rows of the sequences that do not start at 0
    proj = (torch.randn(T, H * R + C + R + H + 3, device=DEV)).to(dtype)
    q_rot = proj[:, : H * R].view(T, H, R)
    kv = proj[:, H * R + 1 : H * R + 1 + C + R]
    gate = proj[:, H * R + 1 + C + R :][:, :H]
    norm_w = torch.rand(C, device=DEV) + 0.5
    cos, sin = ops.rope_tables(128, dims, 10000.0, DEV)
    c1, c2 = cache.clone(), cache.clone()
    p1, p2 = proj.clone(), proj.clone()

    def views(p):
        return (p[:, : H * R].view(T, H, R),
                p[:, H * R + 1 : H * R + 1 + C + R],
                p[:, H * R + 1 + C + R :][:, :H])

    q1, kv1, g1 = views(p1)
    q2, kv2, g2 = views(p2)
    ops.latent_rope_store(q1, kv1, norm_w, 1e-5, C, dims, m["pos"], cos, sin,
                          c1, m["slot_map"])
    ref.latent_rope_store(q2, kv2, norm_w, 1e-5, C, dims, m["pos"], cos, sin,
                          c2, m["slot_map"])
    torch.testing.assert_close(c1.float(), c2.float(), **tol(dtype))
    torch.testing.assert_close(p1.float(), p2.float(), **tol(dtype))
    q_abs = (torch.randn(H, T, C, device=DEV) * C ** -0.5).to(dtype)
    o1 = ops.latent_attn(q_abs, q2, g2, c2, m["bt"], m["pos"], m["seq"],
                         m["cu"], window, 0.3, max(lens))
    o2 = ref.latent_attn(q_abs, q2, g2, c2, m["bt"], m["pos"], m["seq"],
                         m["cu"], window, 0.3)
    torch.testing.assert_close(o1.float(), o2.float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,D,Dv", [(2, 8, 12), (4, 48, 64), (3, 128, 80),
                                    (1, 40, 16)])
@pytest.mark.parametrize("lens,starts", [
    ([70, 1, 2, 5], [0, 9, 0, 130]),
    # chunks above one segment: the segment-parallel passes and their scan
    ([600, 1, 300, 257], [0, 9, 130, 0]),
    ([1, 512], [77, 3])])
def test_lightning_chunks_and_state(dtype, H, D, Dv, lens, starts):
    torch.manual_seed(4)
    m = batch_meta(lens, starts, 64, 32)
    T = m["T"]
    proj = (torch.randn(T, 2 * H * D + H * Dv + 5, device=DEV)).to(dtype)
    q = proj[:, : H * D].view(T, H, D)
    k = proj[:, H * D : 2 * H * D].view(T, H, D)
    v = proj[:, 2 * H * D : 2 * H * D + H * Dv].view(T, H, Dv)
    decay = torch.tensor([0.5, 0.9, 0.99, 0.999][:H], device=DEV)
    st = torch.randn(6, H, D, Dv, device=DEV)
    s1, s2 = st.clone(), st.clone()
    o1 = ops.lightning_attn(q, k, v, decay, s1, m["state_slots"], m["cu"],
                            m["pos"], max(lens))
    o2 = ref.lightning_attn(q, k, v, decay, s2, m["state_slots"], m["cu"],
                            m["pos"])
    scale = float(o2.abs().max())
    torch.testing.assert_close(o1 / scale, o2 / scale, rtol=1e-4, atol=2e-5)
    torch.testing.assert_close(s1, s2, rtol=1e-4, atol=1e-4 * float(
        s2.abs().max()))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,C,R,window", [(3, 20, 4, 7), (6, 72, 8, 50),
                                          (16, 512, 64, 300), (20, 130, 24, 90)])
def test_latent_attention_decode_step(dtype, H, C, R, window):
    """A step of single tokens (one row per sequence) at scattered
    positions: the key-split decode kernels and their merge."""
    torch.manual_seed(5)
    bs = 16
    lens, starts = [1, 1, 1, 1, 1], [0, 47, 15, 200, 95]
    m = batch_meta(lens, starts, bs, 32)
    T = m["T"]
    cache = torch.randn(32, bs, C + R, device=DEV).to(dtype)
    q_abs = (torch.randn(H, T, C, device=DEV) * C ** -0.5).to(dtype)
    q_rot = torch.randn(T, H, R, device=DEV).to(dtype)
    gate = torch.randn(T, H, device=DEV).to(dtype)
    o1 = ops.latent_attn(q_abs, q_rot, gate, cache, m["bt"], m["pos"],
                         m["seq"], m["cu"], window, 0.3, 1)
    o2 = ref.latent_attn(q_abs, q_rot, gate, cache, m["bt"], m["pos"],
                         m["seq"], m["cu"], window, 0.3)
    torch.testing.assert_close(o1.float(), o2.float(), **tol(dtype))
