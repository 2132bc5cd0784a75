"""The entry points under HIP graph capture: a captured decode step, a captured paged decode
step and a captured training step (forward + backward) are replayed several times over inputs
rewritten in place, with eager work and synchronisations between the replays, and every replay
is compared with the eager result on the same inputs (bit-exact: the kernels are deterministic)
and with the fp32 oracle.  The library records only kernel launches on the caller's stream: no
allocation, no synchronisation and no memset node."""
import math

import pytest
import torch

from dkernel_amd import LocalStrideSparseAttention
from oracle import attention as OA
from oracle import layout as OL
from helpers import LSE_TOL, TOL, assert_close, expand_heads, make_qkv, oracle_fwd

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _capture(fn):
    """Warm up on a side stream (first calls set kernel attributes), then capture fn()."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        res = fn()
    return graph, res


def _seq_oracle(q, k, v, bm, bs, sm):
    mask = OA.sequence_token_mask(bm, bs, q.shape[0], k.shape[0], causal=True)
    o, lse = OA.dense_attention(q[None], k[None], v[None], torch.from_numpy(mask), sm, seq_dim=1)
    return o[0], lse[0]


@pytest.mark.parametrize("Hkv,D", [(2, 128), (8, 64)])
def test_captured_decode_step(Hkv, D):
    B, Hq, Lmax, bs = 4, 8, 2048, 64
    sm = 1 / math.sqrt(D)
    mod = LocalStrideSparseAttention(Hq, Lmax, bs, 2, 4, num_kv_heads=Hkv).to(DEV)
    bm = expand_heads(OL.block_mask(Hq, Lmax, bs, 2, 4, num_kv_heads=Hkv), Hq)
    q = torch.zeros(B, 1, Hq, D, dtype=torch.bfloat16, device=DEV)
    k = torch.zeros(B, Lmax, Hkv, D, dtype=torch.bfloat16, device=DEV)
    v = torch.zeros_like(k)
    pads = torch.zeros(B, dtype=torch.int32, device=DEV)
    graph, (out, lse) = _capture(lambda: mod(q, k, v, sm, return_lse=True, left_paddings=pads))
    for step, lens in enumerate([[2048, 1, 777, 64 * 5], [64 * 21 + 12, 300, 2048, 65], [5, 1999, 64, 1024]]):
        print(f"decode replay {step} lens={lens}", flush=True)
        hq, hk, hv = make_qkv(B, 1, Lmax, Hq, Hkv, D, torch.bfloat16, 1, seed=20 + step)
        kp, vp = torch.zeros_like(hk), torch.zeros_like(hv)
        for i, l in enumerate(lens):
            kp[i, Lmax - l:], vp[i, Lmax - l:] = hk[i, :l], hv[i, :l]
        q.copy_(hq)
        k.copy_(kp)
        v.copy_(vp)
        pads.copy_(torch.tensor([Lmax - l for l in lens], dtype=torch.int32))
        graph.replay()
        torch.cuda.synchronize()
        got_o, got_lse = out.clone(), lse.clone()
        eager_o, eager_lse = mod(q, k, v, sm, return_lse=True, left_paddings=pads)
        torch.cuda.synchronize()
        assert torch.equal(got_o, eager_o) and torch.equal(got_lse, eager_lse), f"replay {step} differs from eager"
        for i, l in enumerate(lens):
            ro, rl = _seq_oracle(hq[i], hk[i, :l], hv[i, :l], bm, bs, sm)
            assert_close(f"O[{i}]", got_o[i], ro, **TOL)
            assert_close(f"LSE[{i}]", got_lse[i], rl, atol=LSE_TOL, rtol=0)


def test_captured_paged_decode_step():
    """Serving loop: the pools, the page table and the lengths are rewritten in place between replays."""
    B, Hq, Hkv, D, Lmax, bs, page = 3, 8, 2, 128, 1024, 64, 16
    sm = 1 / math.sqrt(D)
    mod = LocalStrideSparseAttention(Hq, Lmax, bs, 2, 4, num_kv_heads=Hkv).to(DEV)
    bm = expand_heads(OL.block_mask(Hq, Lmax, bs, 2, 4, num_kv_heads=Hkv), Hq)
    num_pages = B * Lmax // page + 5
    q = torch.zeros(B, Hq, D, dtype=torch.bfloat16, device=DEV)
    k_pool = torch.zeros(num_pages, page, Hkv, D, dtype=torch.bfloat16, device=DEV)
    v_pool = torch.zeros_like(k_pool)
    table = torch.zeros((B, Lmax // page), dtype=torch.int32, device=DEV)  # warm-up and capture read page 0
    ctx = torch.ones(B, dtype=torch.int32, device=DEV)
    graph, (out, lse) = _capture(lambda: mod.paged_decode(q, k_pool, v_pool, table, ctx, sm, return_lse=True))
    g = torch.Generator().manual_seed(20)
    for step, lens in enumerate([[1024, 1, 333], [17, 640, 1000], [64, 65, 1023]]):
        print(f"paged replay {step} lens={lens}", flush=True)
        hq = torch.randn(B, Hq, D, generator=g).to(torch.bfloat16)
        ks = [torch.randn(l, Hkv, D, generator=g).to(torch.bfloat16) for l in lens]
        vs = [torch.randn(l, Hkv, D, generator=g).to(torch.bfloat16) for l in lens]
        perm = torch.randperm(num_pages, generator=g).tolist()
        hk, hv = torch.randn(k_pool.shape, generator=g).to(torch.bfloat16), torch.randn(k_pool.shape, generator=g).to(torch.bfloat16)
        ht = torch.full(table.shape, -1, dtype=torch.int32)
        nxt = 0
        for i, l in enumerate(lens):
            for pi in range(-(-l // page)):
                pg, n = perm[nxt], min(page, l - pi * page)
                nxt += 1
                ht[i, pi] = pg
                hk[pg, :n], hv[pg, :n] = ks[i][pi * page: pi * page + n], vs[i][pi * page: pi * page + n]
        q.copy_(hq)
        k_pool.copy_(hk)
        v_pool.copy_(hv)
        table.copy_(ht)
        ctx.copy_(torch.tensor(lens, dtype=torch.int32))
        graph.replay()
        torch.cuda.synchronize()
        got_o, got_lse = out.clone(), lse.clone()
        eager_o, eager_lse = mod.paged_decode(q, k_pool, v_pool, table, ctx, sm, return_lse=True)
        torch.cuda.synchronize()
        assert torch.equal(got_o, eager_o) and torch.equal(got_lse, eager_lse), f"replay {step} differs from eager"
        for i, l in enumerate(lens):
            ro, rl = _seq_oracle(hq[i:i + 1], ks[i], vs[i], bm, bs, sm)
            assert_close(f"O[{i}]", got_o[i:i + 1], ro, **TOL)
            assert_close(f"LSE[{i}]", got_lse[i], rl, atol=LSE_TOL, rtol=0)


@pytest.mark.parametrize("Hkv", [4, 2])
def test_captured_training_step(Hkv):
    """Forward + backward through autograd inside one graph (Hkv < Hq: the dK/dV pass with its scratch)."""
    B, Hq, L, D, bs = 2, 4, 640, 128, 64
    sm = 1 / math.sqrt(D)
    mod = LocalStrideSparseAttention(Hq, L, bs, 2, 3, num_kv_heads=Hkv).to(DEV)
    bm = expand_heads(OL.block_mask(Hq, L, bs, 2, 3, num_kv_heads=Hkv), Hq)
    q = torch.zeros(B, L, Hq, D, dtype=torch.bfloat16, device=DEV, requires_grad=True)
    k = torch.zeros(B, L, Hkv, D, dtype=torch.bfloat16, device=DEV, requires_grad=True)
    v = torch.zeros(B, L, Hkv, D, dtype=torch.bfloat16, device=DEV, requires_grad=True)
    do = torch.zeros(B, L, Hq, D, dtype=torch.bfloat16, device=DEV)

    def step():
        out = mod(q, k, v, sm)
        dq, dk, dv = torch.autograd.grad(out, (q, k, v), do)
        return out, dq, dk, dv

    graph, res = _capture(step)
    for it in range(3):
        print(f"training replay {it}", flush=True)
        hq, hk, hv, hdo = make_qkv(B, L, L, Hq, Hkv, D, torch.bfloat16, 1, seed=30 + it, with_do=True)
        with torch.no_grad():
            q.copy_(hq)
            k.copy_(hk)
            v.copy_(hv)
            do.copy_(hdo)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in res]
        eager = step()
        torch.cuda.synchronize()
        for name, a, b in zip(("O", "dQ", "dK", "dV"), got, eager):
            assert torch.equal(a, b), f"replay {it}: {name} differs from eager"
        qo, ko, vo = (x.clone().float().requires_grad_(True) for x in (hq, hk, hv))
        ro, _ = oracle_fwd(qo, ko, vo, bm, bs, sm)
        ro.backward(hdo.float())
        for name, a, b in zip(("O", "dQ", "dK", "dV"), got, (ro, qo.grad, ko.grad, vo.grad)):
            assert_close(name, a, b, **TOL)
