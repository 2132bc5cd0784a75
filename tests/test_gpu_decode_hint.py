"""Split-KV decode with a max_row_entries hint that understates the real rows: the grid and the
workspace are sized from the hint, the kernel cuts each row into no more units than that and
lets every unit take a larger share, so the result is still the full row's."""
from __future__ import annotations

import math

import pytest
import torch

from dkernel_amd import LocalStrideSparseAttention
from helpers import LSE_TOL, TOL, assert_close
from oracle import attention as OA
from oracle import layout as OL

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _oracle(q1, k, v, bm, l, sm):
    mask = OA.sequence_token_mask(bm, 64, 1, l)
    return OA.dense_attention(q1[None], k[None], v[None], torch.from_numpy(mask), sm)


@pytest.mark.parametrize("hint", [1, 2, 5])
def test_padded_and_packed_decode_with_understated_hint(hint):
    B, Hq, Hkv, D, Lmax = 3, 8, 2, 128, 4096
    sm = 1 / math.sqrt(D)
    g = torch.Generator().manual_seed(hint)
    lens = [4096, 64 * 40 + 3, 777]
    q = torch.randn(B, 1, Hq, D, generator=g).to(torch.bfloat16)
    ks = [torch.randn(l, Hkv, D, generator=g).to(torch.bfloat16) for l in lens]
    vs = [torch.randn(l, Hkv, D, generator=g).to(torch.bfloat16) for l in lens]
    # an instance of its own (the class is cached by constructor arguments): its hint is changed below
    mod = LocalStrideSparseAttention.__wrapped__(Hq, Lmax, 64, 4, 2, num_kv_heads=Hkv).to(DEV)   # rows of up to 34 entries
    assert mod.lut_max_row > 32
    mod.lut_max_row = hint
    mod.kwargs["lut_max_row"] = hint
    bm = OL.block_mask(Hq, Lmax, 64, 4, 2, num_kv_heads=Hkv)
    kp = torch.zeros(B, Lmax, Hkv, D, dtype=torch.bfloat16)
    vp = torch.zeros_like(kp)
    for i, l in enumerate(lens):
        kp[i, Lmax - l:], vp[i, Lmax - l:] = ks[i], vs[i]
    out, lse = mod(q.to(DEV), kp.to(DEV), vp.to(DEV), sm, return_lse=True,
                   left_paddings=torch.tensor([Lmax - l for l in lens]))
    # packed, one query token per sequence
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    outp = mod(q[:, 0].to(DEV), torch.cat(ks).to(DEV), torch.cat(vs).to(DEV), sm, cu_seqlen_k=cu.to(DEV))
    for i, l in enumerate(lens):
        ro, rl = _oracle(q[i], ks[i], vs[i], bm, l, sm)
        assert_close(f"O[{i}]", out[i:i + 1], ro, **TOL)
        assert_close(f"LSE[{i}]", lse[i:i + 1], rl, atol=LSE_TOL, rtol=0)
        assert_close(f"O packed[{i}]", outp[i:i + 1, None], ro, **TOL)


@pytest.mark.parametrize("page_size", [16, 128])
def test_paged_decode_with_units_of_more_than_16_entries(page_size):
    """A hint of 1 leaves one unit per row: 34 entries in one wave, whose page numbers are
    fetched 16 entries at a time."""
    B, Hq, Hkv, D, Lmax = 2, 8, 2, 128, 4096
    sm = 1 / math.sqrt(D)
    g = torch.Generator().manual_seed(7)
    lens = [4096, 64 * 37 + 9]
    q = torch.randn(B, Hq, D, generator=g).to(torch.bfloat16)
    ks = [torch.randn(l, Hkv, D, generator=g).to(torch.bfloat16) for l in lens]
    vs = [torch.randn(l, Hkv, D, generator=g).to(torch.bfloat16) for l in lens]
    pages = [-(-l // page_size) for l in lens]
    num_pages = sum(pages) + 3
    perm = torch.randperm(num_pages, generator=g).tolist()
    k_pool = torch.randn(num_pages, page_size, Hkv, D, generator=g).to(torch.bfloat16)
    v_pool = torch.randn(num_pages, page_size, Hkv, D, generator=g).to(torch.bfloat16)
    table = torch.full((B, Lmax // page_size), -1, dtype=torch.int32)
    nxt = 0
    for i, l in enumerate(lens):
        for pi in range(pages[i]):
            pg = perm[nxt]
            nxt += 1
            table[i, pi] = pg
            n = min(page_size, l - pi * page_size)
            k_pool[pg, :n] = ks[i][pi * page_size: pi * page_size + n]
            v_pool[pg, :n] = vs[i][pi * page_size: pi * page_size + n]
    mod = LocalStrideSparseAttention.__wrapped__(Hq, Lmax, 64, 4, 2, num_kv_heads=Hkv).to(DEV)
    mod.lut_max_row = 1
    bm = OL.block_mask(Hq, Lmax, 64, 4, 2, num_kv_heads=Hkv)
    out, lse = mod.paged_decode(q.to(DEV), k_pool.to(DEV), v_pool.to(DEV), table.to(DEV),
                                torch.tensor(lens, dtype=torch.int32).to(DEV), sm, return_lse=True)
    for i, l in enumerate(lens):
        ro, rl = _oracle(q[i:i + 1], ks[i], vs[i], bm, l, sm)
        assert_close(f"O[{i}]", out[i:i + 1, None], ro, **TOL)
        assert_close(f"LSE[{i}]", lse[i:i + 1], rl, atol=LSE_TOL, rtol=0)


def test_debug_mode_rejects_page_numbers_outside_the_pools(monkeypatch):
    """DKERNEL_DEBUG=1: a table entry inside a sequence that names no page of the pools is refused
    on the host, before anything is launched (the kernel itself cannot check the upper bound)."""
    B, Hq, Hkv, D, Lmax, ps = 2, 8, 2, 128, 1024, 64
    g = torch.Generator().manual_seed(3)
    q = torch.randn(B, Hq, D, generator=g).to(torch.bfloat16).to(DEV)
    k_pool = torch.randn(40, ps, Hkv, D, generator=g).to(torch.bfloat16).to(DEV)
    v_pool = torch.randn(40, ps, Hkv, D, generator=g).to(torch.bfloat16).to(DEV)
    table = torch.arange(B * (Lmax // ps), dtype=torch.int32).view(B, -1)
    lens = torch.tensor([1000, 300], dtype=torch.int32)
    mod = LocalStrideSparseAttention.__wrapped__(Hq, Lmax, 64, 4, 2, num_kv_heads=Hkv).to(DEV)
    monkeypatch.setenv("DKERNEL_DEBUG", "1")
    good = mod.paged_decode(q, k_pool, v_pool, table.to(DEV), lens.to(DEV), 1 / math.sqrt(D))
    assert torch.isfinite(good.float()).all()
    bad = table.clone()
    bad[1, 4] = 40        # tokens 256..319 of sequence 1 (300 keys): inside the sequence, beyond the pools
    with pytest.raises(AssertionError, match="outside the pools"):
        mod.paged_decode(q, k_pool, v_pool, bad.to(DEV), lens.to(DEV), 1 / math.sqrt(D))
    bad = table.clone()
    bad[1, 5] = 4000      # tokens 320..: beyond sequence 1's keys, never read, so not an error
    mod.paged_decode(q, k_pool, v_pool, bad.to(DEV), lens.to(DEV), 1 / math.sqrt(D))
