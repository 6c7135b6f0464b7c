"""HIP sequence-mixer kernels (kllms_amd._C_seq) against the plain PyTorch
fp32 reference of the same op (ops/torch_ref.py), in bf16 and fp32, on sizes
that are not multiples of the tile / wave sizes."""

import math

import pytest
import torch

from kllms_amd import ops
from kllms_amd.ops import torch_ref

pytestmark = pytest.mark.gpu

DEV = "cuda"
DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype):
    return (2e-5, 2e-5) if dtype == torch.float32 else (2e-2, 2e-2)


def close(a, b, dtype, scale=1.0):
    rt, at = tol(dtype)
    torch.testing.assert_close(a.float(), b.float(), rtol=rt * scale, atol=at * scale)


def rnd(*shape, dtype=torch.float32, std=1.0, seed=0):
    g = torch.Generator(device="cpu").manual_seed(seed + sum(shape))
    return (torch.randn(*shape, generator=g) * std).to(DEV).to(dtype)


def segments(lens, starts):
    cu = [0]
    tseg = []
    for b, n in enumerate(lens):
        cu.append(cu[-1] + n)
        tseg += [b] * n
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    return i32(cu), i32(starts), i32(tseg)


def test_extension_loaded():
    x = torch.zeros(2, 8, device=DEV)
    ops.rmsnorm_cast(x, torch.ones(8, device=DEV), 1e-6, torch.float32)
    assert ops.seq_hip_loaded()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W", [40, 320, 1000])
def test_embed_and_norms(dtype, W):
    table = rnd(97, W, dtype=dtype)
    w = rnd(W, seed=1) * 0.1 + 1
    ids = torch.randint(0, 97, (13,), device=DEV)
    x = ops.embed_rmsnorm(ids, table, w, 1e-6)
    close(x, torch_ref.embed_rmsnorm(ids, table, w, 1e-6), torch.float32)
    h = ops.rmsnorm_cast(x, w, 1e-6, dtype)
    close(h, torch_ref.rmsnorm_cast(x, w, 1e-6, dtype), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dual", [False, True])
@pytest.mark.parametrize("nxt", [False, True])
@pytest.mark.parametrize("W", [328, 36])      # 8-wide path / scalar path
def test_sandwich_residual(dtype, dual, nxt, W):
    T = 9
    x = rnd(T, W, std=3.0)
    a, b = rnd(T, W, dtype=dtype, seed=1), rnd(T, W, dtype=dtype, seed=2)
    wa, wb, wp, wn = (rnd(W, seed=s) * 0.2 + 1 for s in (3, 4, 5, 6))
    kw = dict(b=b, wa=wa, wb=wb) if dual else {}
    x1, x2 = x.clone(), x.clone()
    h1 = ops.sandwich_residual(x1, a, wp, 1e-6, w_next=wn if nxt else None, out_dtype=dtype, **kw)
    h2 = torch_ref.sandwich_residual(x2, a, wp, 1e-6, w_next=wn if nxt else None, out_dtype=dtype,
                                     **{"b": None, "wa": None, "wb": None, **kw})
    close(x1, x2, torch.float32)
    assert (h1 is None) == (not nxt)
    if nxt:
        close(h1, h2, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("S,off,ff", [(72, 8, 104), (70, 3, 101), (128, 16, 96), (4096, 0, 64)])   # 8-wide / scalar / short-row / long-row
def test_gated_rmsnorm_and_glu(dtype, S, off, ff):
    T, G = 7, 3
    o = rnd(T, G, S, std=2.0)
    w = rnd(S) * 0.1 + 1
    fused = rnd(T, G * S + 24, dtype=dtype, seed=3)
    gate = fused[:, off:off + G * S]
    close(ops.gated_rmsnorm(o, w, gate, 1e-6, dtype), torch_ref.gated_rmsnorm(o, w, gate, 1e-6, dtype), dtype)
    gu = rnd(T, 2 * ff, dtype=dtype, std=2.0, seed=5)
    close(ops.clamped_glu(gu[:, :ff], gu[:, ff:], 1.5, 1.702),
          torch_ref.clamped_glu(gu[:, :ff], gu[:, ff:], 1.5, 1.702), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("D,R,mask,pad", [(64, 32, 24, 8), (40, 10, 0, 6), (128, 64, 100, 8), (64, 8, 24, 6),
                                          (16, 8, 0, 8)])      # pad 8: aligned rows (8-wide kernel); 6: scalar kernel
def test_rope_store_and_blocklocal_attention(dtype, D, R, mask, pad):
    H, G, BS, NB = 6, 2, 16, 40
    lens, starts = [50, 1, 7, 1], [0, 130, 37, 24]
    T = sum(lens)
    cu, st, tseg = segments(lens, starts)
    pos = torch.tensor([s + i for n, s in zip(lens, starts) for i in range(n)], device=DEV)
    # distinct, shuffled blocks per segment
    perm = torch.randperm(NB, generator=torch.Generator().manual_seed(1)).tolist()
    need = [(s + n + BS - 1) // BS for n, s in zip(lens, starts)]
    bt = torch.zeros(len(lens), max(need), dtype=torch.int32)
    off = 0
    for b, nb in enumerate(need):
        bt[b, :nb] = torch.tensor(perm[off:off + nb], dtype=torch.int32)
        off += nb
    bt = bt.to(DEV)
    slots = torch.stack([bt[int(tseg[t]), int(pos[t]) // BS].long() * BS + int(pos[t]) % BS for t in range(T)])
    inv_freq = (10000.0 ** (-torch.arange(R, dtype=torch.float64) * 2 / (2 * R))).float().to(DEV)
    kc = rnd(NB, G, BS, D, dtype=dtype, seed=7)    # stands for keys stored by earlier steps
    vc = rnd(NB, G, BS, D, dtype=dtype, seed=8)
    fused = rnd(T, H * D + G * D + pad, dtype=dtype, seed=9)
    res = []
    for impl in (ops, torch_ref):
        f = fused.clone()
        q = f[:, :H * D].unflatten(1, (H, D))
        k = f[:, H * D:H * D + G * D].unflatten(1, (G, D))
        gate = f[:, H * D + G * D:H * D + G * D + H]
        k1, v1 = kc.clone(), vc.clone()
        impl.rope_pairs_store(q, k, None, pos, inv_freq, k1, v1, slots)
        out = impl.attn_blocklocal_paged(q, k1, v1, bt, tseg, pos, 0.17, mask, gate)
        res.append((q.clone(), k1, v1, out))
    for a, b in zip(*res):
        close(a, b, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,D,V", [(3, 24, 40), (2, 64, 130), (1, 128, 64), (3, 20, 33)])
def test_linear_attn_decay(dtype, H, D, V):
    lens, starts = [33, 1, 5], [0, 9, 2]
    T = sum(lens)
    cu, st, _ = segments(lens, starts)
    slots = torch.tensor([4, 0, 2], dtype=torch.int32, device=DEV)
    q, k, v = rnd(T, H, D, dtype=dtype, seed=1), rnd(T, H, D, dtype=dtype, seed=2), rnd(T, H, V, dtype=dtype, seed=3)
    decay = torch.tensor([0.6, 0.9, 0.999][:H], device=DEV)
    state = rnd(5, H, D, V, seed=4)
    s1, s2 = state.clone(), state.clone()
    o1 = ops.linear_attn_decay(q, k, v, decay, s1, slots, cu, st)
    o2 = torch_ref.linear_attn_decay(q, k, v, decay, s2, slots, cu, st)
    close(o1, o2, torch.float32, scale=20)
    close(s1, s2, torch.float32, scale=20)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("K", [1, 2, 4, 7])
@pytest.mark.parametrize("C,off", [(88, 8), (84, 5)])      # 8-wide path / scalar path
def test_causal_conv_silu(dtype, K, C, off):
    lens, starts = [20, 1, 2, 3], [0, 5, 1, 0]
    T = sum(lens)
    cu, st, tseg = segments(lens, starts)
    slots = torch.tensor([3, 1, 0, 2], dtype=torch.int32, device=DEV)
    fused = rnd(T, C + 16, dtype=dtype, seed=1)
    x = fused[:, off:off + C]
    w = rnd(K, C, seed=2) * 0.5
    hist = rnd(4, K - 1, C, dtype=dtype, seed=3)
    h1, h2 = hist.clone(), hist.clone()
    y1 = ops.causal_conv_silu(x, w, h1, slots, cu, st, tseg)
    y2 = torch_ref.causal_conv_silu(x, w, h2, slots, cu, st)
    close(y1, y2, dtype)
    close(h1, h2, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,V", [(4, 2, 24, 40), (2, 2, 64, 72), (2, 1, 128, 128)])
def test_gated_delta_rule(dtype, H, G, D, V):
    lens, starts = [40, 1, 3], [0, 11, 4]
    T = sum(lens)
    cu, st, _ = segments(lens, starts)
    slots = torch.tensor([1, 3, 0], dtype=torch.int32, device=DEV)
    q, k = rnd(T, G, D, dtype=dtype, seed=1), rnd(T, G, D, dtype=dtype, seed=2)
    v = rnd(T, H, V, dtype=dtype, seed=3)
    beta, a = rnd(T, H, dtype=dtype, seed=4), rnd(T, H * D, dtype=dtype, seed=5)
    dt, alog = rnd(H * D, seed=6) * 0.5, rnd(H, seed=7) * 0.5
    state = rnd(4, H, D, V, seed=8)
    s1, s2 = state.clone(), state.clone()
    o1 = ops.gated_delta_rule(q, k, v, beta, a, dt, alog, s1, slots, cu, st)
    o2 = torch_ref.gated_delta_rule(q, k, v, beta, a, dt, alog, s2, slots, cu, st)
    close(o1, o2, torch.float32, scale=10)
    close(s1, s2, torch.float32, scale=10)
