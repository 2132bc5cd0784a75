"""Patterns whose long rows are not their last ones (global rows at the start of a non-causal
pattern, random patterns): the forward and dQ kernels take the rows in the table's own order,
longest first (dk_lut.row_order / pair_order), instead of starting from the last row.  The order
only decides which workgroup computes which row: results must match the oracle and be bit-identical
to the default hand-out."""
from __future__ import annotations

import math

import numpy as np
import pytest
import torch

from dkernel_amd import SparseAttention, ops
from helpers import F32_TOL, LSE_TOL, TOL, assert_close, make_qkv, oracle_fwd

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _global_rows_pattern(heads, n, causal, seed=3):
    """Window of 2 blocks either side, two global rows and columns, a few random blocks; per-head
    variations so that the heads' orders differ."""
    rng = np.random.default_rng(seed)
    i = np.arange(n)
    pat = np.zeros((heads, n, n), dtype=bool)
    for h in range(heads):
        pat[h] = np.abs(i[:, None] - i[None, :]) <= 2
        pat[h, :2, :] = True
        pat[h, :, :2] = True
        pat[h, (3 * h + 9) % n, :] = True  # one more long row, at another place in every head
        pat[h] |= rng.random((n, n)) < 1.5 / n
        if causal:
            pat[h] &= i[:, None] >= i[None, :]
            pat[h, i, i] = True
    return pat


# (q heads, kv heads, head dim, dtype, causal, tokens, keys before the first query)
CASES = [
    (4, 4, 128, torch.bfloat16, False, 1024, 0),   # two rows per workgroup
    (8, 2, 128, torch.bfloat16, False, 1024, 0),   # a GQA group per workgroup, one row each
    (4, 4, 64, torch.float16, False, 960, 0),      # the last table rows hold no query
    (2, 2, 192, torch.bfloat16, False, 768, 0),    # 256-wide tiles: dQ one row per workgroup
    (4, 4, 96, torch.bfloat16, True, 1024, 0),     # causal, with long rows in the middle
    (4, 4, 128, torch.bfloat16, True, 640, 384),   # queries are the last 640 of 1024 positions
    (3, 3, 64, torch.float32, False, 768, 0),      # fp32 on the matrix cores
]


@pytest.mark.parametrize("Hq,Hkv,D,dtype,causal,L,past", CASES)
def test_forward_and_backward_in_the_tables_own_order(Hq, Hkv, D, dtype, causal, L, past):
    print(f"case Hq={Hq} Hkv={Hkv} D={D} {dtype} causal={causal} L={L} past={past}", flush=True)
    n = 16
    Lk = L + past
    sm = 1 / math.sqrt(D)
    pat = _global_rows_pattern(Hkv, n, causal)
    mod = SparseAttention(64, torch.from_numpy(pat), causal=causal).to(DEV)
    assert mod.kwargs["unsorted_rows"]
    nb = (Lk + 63) // 64
    bm = np.repeat(pat, Hq // Hkv, axis=0)[:, :nb, :nb]
    q, k, v, do = make_qkv(1, L, Lk, Hq, Hkv, D, dtype, 1, with_do=True)
    qo, ko, vo = (x.clone().float().requires_grad_() for x in (q, k, v))
    ro, rlse = oracle_fwd(qo, ko, vo, bm, 64, sm, causal=causal)
    ro.backward(do.float())
    results = []
    for own_order in (True, False):
        mod.kwargs["unsorted_rows"] = own_order
        qd, kd, vd = (x.to(DEV).requires_grad_() for x in (q, k, v))
        out, lse = mod(qd, kd, vd, sm, return_lse=True)
        out.backward(do.to(DEV))
        results.append((out, lse, qd.grad, kd.grad, vd.grad))
    tol = F32_TOL if dtype == torch.float32 else TOL
    out, lse, dq, dk, dv = results[0]
    assert_close("O", out, ro, **tol)
    assert_close("LSE", lse, rlse, atol=1e-4 if dtype == torch.float32 else LSE_TOL, rtol=0)
    assert_close("dQ", dq, qo.grad, **tol)
    assert_close("dK", dk, ko.grad, **tol)
    assert_close("dV", dv, vo.grad, **tol)
    for a, b in zip(*results):
        assert torch.equal(a, b)


@pytest.mark.parametrize("Hq,Hkv,D", [(4, 4, 128), (8, 2, 64)])
def test_padded_prefill_in_the_tables_own_order(Hq, Hkv, D):
    """Left- and right-padded batches: rows of the table before / beyond a sequence's queries
    are skipped, the padding rows come back cleared either way."""
    print(f"case Hq={Hq} Hkv={Hkv} D={D}", flush=True)
    L, B, n = 1024, 3, 16
    sm = 1 / math.sqrt(D)
    mod = SparseAttention(64, torch.from_numpy(_global_rows_pattern(Hkv, n, True)), causal=True).to(DEV)
    assert mod.kwargs["unsorted_rows"]
    q, k, v = (x.to(DEV) for x in make_qkv(B, L, L, Hq, Hkv, D, torch.bfloat16, 1))
    lens = torch.tensor([1000, 130, 577], dtype=torch.int32, device=DEV)
    results = []
    for own_order in (True, False):
        mod.kwargs["unsorted_rows"] = own_order
        got = list(mod(q, k, v, sm, left_paddings=L - lens, return_lse=True))
        got += list(mod(q, k, v, sm, seqlens=lens, return_lse=True))
        results.append(got)
    for a, b in zip(*results):
        assert torch.equal(a, b)
    # against the unpadded call, sequence by sequence (right-padded)
    mod.kwargs["unsorted_rows"] = True
    out = mod(q, k, v, sm, seqlens=lens)
    for b in range(B):
        n_b = int(lens[b])
        alone = mod(q[b:b + 1, :n_b], k[b:b + 1, :n_b], v[b:b + 1, :n_b], sm)
        assert torch.equal(out[b, :n_b], alone[0])
        assert (out[b, n_b:] == 0).all()
