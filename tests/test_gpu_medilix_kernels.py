"""HIP kernels of the parallel-layer family (kllms_amd._C_seq) against the
plain PyTorch reference of the same op (ops/torch_ref.py), in fp32 and bf16,
on sizes that are not multiples of the wave or vector sizes."""

import pytest
import torch

from kllms_amd import ops
from kllms_amd.ops import torch_ref

pytestmark = pytest.mark.gpu

DEV = "cuda"
DTYPES = [torch.float32, torch.bfloat16]


def close(a, b, dtype, scale=1.0):
    rt, at = (2e-5, 2e-5) if dtype == torch.float32 else (2e-2, 2e-2)
    torch.testing.assert_close(a.float(), b.float(), rtol=rt * scale, atol=at * scale)


def rnd(*shape, dtype=torch.float32, std=1.0, seed=0):
    g = torch.Generator(device="cpu").manual_seed(seed + sum(shape))
    return (torch.randn(*shape, generator=g) * std).to(DEV).to(dtype)


def segments(lens, starts):
    cu, tseg = [0], []
    for b, n in enumerate(lens):
        cu.append(cu[-1] + n)
        tseg += [b] * n
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    return i32(cu), i32(starts), i32(tseg)


@pytest.mark.parametrize("dtype", DTYPES)
def test_embed_bigram(dtype):
    W, V, buckets = 72, 50, 13
    table, big = rnd(V, W, dtype=dtype), rnd(buckets + 1, W, dtype=dtype, seed=1)
    cu, st, tseg = segments([5, 1, 3], [0, 7, 2])
    slots = torch.tensor([2, 0, 3], dtype=torch.int32, device=DEV)
    ids = torch.randint(0, V, (9,), device=DEV)
    s1 = torch.tensor([4, 5, 6, 7], dtype=torch.int32, device=DEV)
    s2 = s1.clone()
    x = ops.embed_bigram(ids, table, big, 3.0, 11, 5, buckets, s1, slots, cu, st, tseg)
    ref = torch_ref.embed_bigram(ids, table, big, 3.0, 11, 5, buckets, s2, slots, cu, st)
    close(x, ref, torch.float32)
    assert torch.equal(s1, s2)
    x = ops.embed_bigram(ids, table, None, 3.0, 0, 0, 1, None, slots, cu, st, tseg)
    close(x, table[ids].float() * 3.0, torch.float32)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W,groups", [(48, 3), (320, 1), (1000, 4), (2048, 2), (4096, 8), (36, 2)])
def test_group_norm_pair_and_concat(dtype, W, groups):
    T = 7
    x = rnd(T, W, std=3.0)
    a, b = rnd(T, W, dtype=dtype, seed=1), rnd(T, W, dtype=dtype, seed=2)
    w1, w2 = rnd(W, seed=3) * 0.1 + 1, rnd(W, seed=4) * 0.1 + 1
    for aa, bb, ww2 in [(None, None, w2), (a, b, w2), (a, None, None)]:
        x1, x2 = x.clone(), x.clone()
        h1, h2 = ops.group_norm_pair(x1, aa, bb, w1, ww2, groups, 1e-5, dtype)
        r1, r2 = torch_ref.group_norm_pair(x2, aa, bb, w1, ww2, groups, 1e-5, dtype)
        close(x1, x2, torch.float32)
        close(h1, r1, dtype)
        if ww2 is not None:
            close(h2, r2, dtype)
    x0 = rnd(T, W, seed=9)
    x1, x2 = x.clone(), x.clone()
    close(ops.cast_concat(x1, x0, a, b, dtype), torch_ref.cast_concat(x2, x0, a, b, dtype), dtype)
    close(x1, x2, torch.float32)
    close(ops.cast_concat(x1, x0, None, None, dtype), torch_ref.cast_concat(x2, x0, None, None, dtype), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("D,Dv", [(64, 64), (24, 40), (128, 128), (20, 12)])
@pytest.mark.parametrize("mask", [(1, 9, 3, True), (1, 40, 0, True), (1, 0, 0, True), (1, 6, 8, False), (0, 16, 0, True)])
def test_qk_norm_and_masked_attention(dtype, D, Dv, mask):
    kind, size, keep, sink = mask
    H, G, BS, NB = 4, 2, 16, 24
    lens, starts = [37, 1, 5], [0, 90, 61]
    cu, st, tseg = segments(lens, starts)
    T = sum(lens)
    kc = rnd(NB, G, BS, D, dtype=dtype, std=0.5)
    vc = rnd(NB, G, BS, Dv, dtype=dtype, seed=1)
    kc2, vc2 = kc.clone(), vc.clone()
    perm = torch.randperm(NB)[:21].to(torch.int32)
    bt = torch.stack([perm[:7], perm[7:14], perm[14:21]]).to(DEV).contiguous()
    pos, slot = [], []
    for b, (n, s) in enumerate(zip(lens, starts)):
        for p in range(s, s + n):
            pos.append(p)
            slot.append(int(bt[b, p // BS]) * BS + p % BS)
    pos = torch.tensor(pos, device=DEV)
    slot = torch.tensor(slot, device=DEV)
    y = rnd(T, H * D + G * D + G * Dv + H * Dv + 8, dtype=dtype, seed=2)
    y2 = y.clone()

    def parts(t):
        o = 0
        q = t[:, o:o + H * D].unflatten(1, (H, D)); o += H * D
        k = t[:, o:o + G * D].unflatten(1, (G, D)); o += G * D
        v = t[:, o:o + G * Dv].unflatten(1, (G, Dv)); o += G * Dv
        return q, k, v, t[:, o:o + H * Dv]

    wq, wk = rnd(D, seed=5) * 0.2 + 1, rnd(D, seed=6) * 0.2 + 1
    q, k, v, g = parts(y)
    q2, k2, v2, g2 = parts(y2)
    ops.qk_norm_store(q, k, v, wq, wk, 1e-5, kc, vc, slot)
    torch_ref.qk_norm_store(q2, k2, v2, wq, wk, 1e-5, kc2, vc2, slot)
    close(q, q2, dtype)
    close(kc, kc2, dtype)
    close(vc, vc2, dtype)
    for gate in (g, None, g[:, :H]):
        o = ops.attn_masked_paged(q2, kc2, vc2, bt, tseg, pos, 0.3, kind, size, keep, sink, gate)
        r = torch_ref.attn_masked_paged(q2, kc2, vc2, bt, tseg, pos, 0.3, kind, size, keep, sink, gate)
        close(o, r, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("D,Dv", [(64, 64), (128, 128), (24, 40)])
@pytest.mark.parametrize("mask", [(1, 300, 5, True), (1, 0, 0, True), (0, 512, 0, False), (1, 1024, 4, True)])
def test_masked_attention_long_context(dtype, D, Dv, mask):
    """More visible keys than one pass of the kernel's waves covers (256):
    a window of 300 with kept tokens, plain causal over 1100, a block of 512,
    and a window of 1024 that positions beyond it slide out of."""
    kind, size, keep, sink = mask
    H, G, BS = 4, 2, 16
    lens, starts = [3, 2, 1], [298, 700, 1100]
    cu, st, tseg = segments(lens, starts)
    NB = 3 * 70 + 2
    kc = rnd(NB, G, BS, D, dtype=dtype, std=0.5)
    vc = rnd(NB, G, BS, Dv, dtype=dtype, seed=1)
    bt = (torch.randperm(NB)[:210].to(torch.int32).view(3, 70)).to(DEV).contiguous()
    pos = torch.tensor([p for n, s in zip(lens, starts) for p in range(s, s + n)], device=DEV)
    q = rnd(sum(lens), H, D, dtype=dtype, seed=2)
    gate = rnd(sum(lens), H * Dv, dtype=dtype, seed=3)
    o = ops.attn_masked_paged(q, kc, vc, bt, tseg, pos, 0.2, kind, size, keep, sink, gate)
    r = torch_ref.attn_masked_paged(q, kc, vc, bt, tseg, pos, 0.2, kind, size, keep, sink, gate)
    close(o, r, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W", [200, 2048, 36])
def test_token_shift(dtype, W):
    cu, st, tseg = segments([4, 1, 6], [0, 3, 9])
    slots = torch.tensor([1, 3, 0], dtype=torch.int32, device=DEV)
    h = rnd(11, W, dtype=dtype)
    mu = torch.rand(5, W, device=DEV)
    s1 = rnd(4, W, dtype=dtype, seed=3)
    s2 = s1.clone()
    a, f = ops.token_shift_mix(h, mu, s1, slots, cu, st, tseg, 4)
    ra, rf = torch_ref.token_shift_mix(h, mu, s2, slots, cu, st, 4, dtype)
    close(a, ra, dtype)
    close(f, rf, torch.float32)
    close(s1, s2, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,D,V", [(3, 48, 48), (2, 64, 64), (1, 20, 20), (2, 128, 128)])
def test_wkv_recurrence(dtype, H, D, V):
    lens, starts = [45, 1, 6, 2], [0, 5, 77, 0]
    cu, st, _ = segments(lens, starts)
    T = sum(lens)
    slots = torch.tensor([3, 1, 0, 4], dtype=torch.int32, device=DEV)
    r, k, v = (rnd(T, H, D, dtype=dtype, std=0.5, seed=s) for s in (1, 2, 3))
    d = rnd(T, H * D, std=0.7, seed=4) - 1.0
    w0, u = rnd(H * D, seed=5) * 0.3, rnd(H, D, seed=6) * 0.3
    s1 = rnd(5, H, D, V, seed=7)
    s2 = s1.clone()
    o = ops.wkv_recurrence(r, k, v, d, w0, u, s1, slots, cu, st)
    ref = torch_ref.wkv_recurrence(r, k, v, d, w0, u, s2, slots, cu, st)
    close(o, ref, torch.float32, scale=5)
    close(s1, s2, torch.float32, scale=5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,D,V", [(2, 48, 64), (3, 16, 24), (1, 64, 128), (2, 128, 63)])
def test_mlstm_recurrence(dtype, H, D, V):
    lens, starts = [45, 1, 6, 2], [0, 5, 77, 0]
    cu, st, _ = segments(lens, starts)
    T = sum(lens)
    slots = torch.tensor([3, 1, 0, 4], dtype=torch.int32, device=DEV)
    q, k, v = (rnd(T, H, D if s < 3 else V, dtype=dtype, std=0.7, seed=s) for s in (1, 2, 3))
    z = rnd(T, 2 * H, std=3.0, seed=4)
    zb = rnd(2 * H, seed=5)
    # carried state as a kernel leaves it: matrix, normaliser column, maximum row
    s1 = rnd(5, H, D + 1, V + 1, seed=7) * 0.3
    s1[:, :, D, :] = torch.rand(5, H, 1, device=DEV) * 3
    s2 = s1.clone()
    o = ops.mlstm_recurrence(q, k, v, z, zb, 15.0, s1, slots, cu, st)
    ref = torch_ref.mlstm_recurrence(q, k, v, z, zb, 15.0, s2, slots, cu, st)
    close(o, ref, torch.float32, scale=5)
    close(s1, s2, torch.float32, scale=5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("act", ["sigmoid", "silu"])
def test_head_norm_gate_and_act(dtype, act):
    T, H, S = 9, 3, 40
    o = rnd(T, H, S, std=2.0)
    w = rnd(H * S, seed=1) * 0.1 + 1
    gate = rnd(T, H * S + 8, dtype=dtype, seed=2)[:, :H * S]
    close(ops.head_rmsnorm_gate(o, w, gate, 1e-5, act, dtype),
          torch_ref.head_rmsnorm_gate(o, w, gate, 1e-5, act, dtype), dtype)
    gu = rnd(T, 2 * 56, dtype=dtype, std=2.0, seed=3)
    close(ops.silu_glu(gu[:, :56], gu[:, 56:]), torch_ref.gated_act(gu[:, :56], gu[:, 56:], float("inf"), 1.0, 0.0),
          dtype)
    close(ops.clamped_glu(gu[:, :56], gu[:, 56:], 1.5, 1.702), torch_ref.clamped_glu(gu[:, :56], gu[:, 56:], 1.5, 1.702),
          dtype)


@pytest.mark.parametrize("N,top,gc,gk", [(12, 3, 2, 1), (8, 2, 1, 1), (16, 4, 4, 2), (130, 5, 2, 2), (6, 1, 3, 1)])
def test_router(N, top, gc, gk):
    T = 50
    z = rnd(T, N, std=2.0)
    corr = rnd(N, seed=1) * 0.05
    idx, w = ops.moe_route(z, corr, top, gc, gk)
    ridx, rw = torch_ref.moe_route(z, corr, top, gc, gk)
    assert torch.equal(idx, ridx)
    close(w, rw, torch.float32)


@pytest.mark.parametrize("dtype", DTYPES)
def test_combine(dtype):
    T, W, top, R = 10, 88, 3, 17
    rows, h = rnd(R, W, dtype=dtype), rnd(T, W, dtype=dtype, seed=1)
    rowidx = torch.randint(-1, R, (T, top), device=DEV, dtype=torch.int32)
    w = torch.rand(T, top, device=DEV)
    close(ops.moe_combine(rows, h, rowidx, w, dtype), torch_ref.moe_combine(rows, h, rowidx, w, dtype), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N,E,top,gc,gk", [(12, 8, 3, 2, 1), (8, 8, 2, 1, 1), (9, 6, 2, 3, 2)])
def test_router_with_its_projection(dtype, N, E, top, gc, gk):
    """Router logits computed inside the routing kernel, and the row indices of
    the all-experts form."""
    T, W = 40, 200
    h = rnd(T, W, dtype=dtype)
    router = rnd(N, W, std=0.3, seed=1)
    corr = rnd(N, seed=2) * 0.05
    idx, w, rowidx = ops.moe_route_rows(h, router, corr, top, gc, gk, E, True)
    z = torch.nn.functional.linear(h.float(), router)
    ridx, rw = torch_ref.moe_route(z, corr, top, gc, gk)
    assert torch.equal(idx, ridx)
    close(w, rw, torch.float32, scale=5)
    t_idx = torch.arange(T, dtype=torch.int32, device=DEV).unsqueeze(1)
    assert torch.equal(rowidx, torch.where(ridx < E, ridx * T + t_idx, torch.full_like(ridx, -1)))
    assert ops.moe_route_rows(h, router, corr, top, gc, gk, E, False)[2] is None


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,D,V", [(2, 48, 64), (3, 16, 24)])
def test_mlstm_with_fused_read_out(dtype, H, D, V):
    lens, starts = [45, 1, 6], [0, 5, 77]
    cu, st, _ = segments(lens, starts)
    T = sum(lens)
    slots = torch.tensor([3, 1, 0], dtype=torch.int32, device=DEV)
    q, k, v = (rnd(T, H, D if s < 3 else V, dtype=dtype, std=0.7, seed=s) for s in (1, 2, 3))
    z, zb = rnd(T, 2 * H, std=3.0, seed=4), rnd(2 * H, seed=5)
    s1 = rnd(4, H, D + 1, V + 1, seed=7) * 0.3
    s1[:, :, D, :] = torch.rand(4, H, 1, device=DEV) * 3
    s2 = s1.clone()
    wt = rnd(H * V, seed=8) * 0.1 + 1
    gate = rnd(T, H * V, dtype=dtype, seed=9)
    got = ops.mlstm_mix_out(q, k, v, z, zb, 15.0, s1, slots, cu, st, wt, gate, 1e-5, dtype)
    o = torch_ref.mlstm_recurrence(q, k, v, z, zb, 15.0, s2, slots, cu, st)
    close(got, torch_ref.head_rmsnorm_gate(o, wt, gate, 1e-5, "sigmoid", dtype), dtype)
    close(s1, s2, torch.float32, scale=5)
