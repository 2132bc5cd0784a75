"""Padded prefill: the kernels themselves clear the output rows that hold no query of their
sequence (o = 0, lse = -inf; bit 2 of dk_seqs.packed) -- the reference clears the whole output
with torch.zeros before its launch (dkernel/ops/sparse_attn_inference.py:67).  Outputs start
poisoned here (freed blocks of NaNs that the next allocations of the same sizes receive; the test
checks that they did), so a row that no workgroup clears fails the test.  Every
kernel family that takes padded inputs, lengths that leave no spare q tile, empty and full
sequences, both paddings, both tensor orders."""
from __future__ import annotations

import math

import pytest
import torch

from dkernel_amd import LocalStrideSparseAttention, _lib, ops
from helpers import LSE_TOL, TOL, F32_TOL, assert_close, expand_heads, oracle_fwd
from oracle import attention as OA
from oracle import layout as OL

pytestmark = pytest.mark.gpu
DEV = "cuda"
New = LocalStrideSparseAttention.__wrapped__


def _poisoned_like(shape, dtype):
    x = torch.full(shape, float("nan"), dtype=dtype, device=DEV)
    return x


@pytest.mark.parametrize("impl,Hq,Hkv,D,dtype,bs", [
    ("auto", 8, 2, 128, torch.bfloat16, 64),     # several heads per workgroup
    ("auto", 4, 4, 128, torch.float16, 64),      # two q tiles of a head per workgroup
    ("auto", 4, 2, 192, torch.bfloat16, 64),     # 256-wide tiles
    ("auto", 4, 4, 64, torch.float32, 64),       # fp32 matrix-core kernel
    ("auto", 6, 2, 128, torch.bfloat16, 16),     # sub-block tables
    ("generic", 4, 2, 72, torch.bfloat16, 64),   # generic kernel
    ("generic", 2, 2, 36, torch.float16, 32),    # generic kernel, rows without 16-byte alignment
])
@pytest.mark.parametrize("seq_dim", [1, 2])
def test_rows_without_queries_are_cleared(impl, Hq, Hkv, D, dtype, bs, seq_dim):
    ops.set_impl(impl)
    try:
        L = 320
        lens = [320, 319, 0, 1, 130, 257]      # full, one short (no spare q tile), empty, one token, ...
        B = len(lens)
        sm = 1 / math.sqrt(D)
        g = torch.Generator().manual_seed(7)
        bm = OL.block_mask(Hq, L, bs, 2, 3, num_kv_heads=Hkv)
        tol = F32_TOL if dtype == torch.float32 else TOL
        for left in (True, False):
            q, k, v = (torch.randn(B, L, h, D, generator=g).to(dtype) for h in (Hq, Hkv, Hkv))
            if seq_dim == 2:
                qd, kd, vd = (x.transpose(1, 2).contiguous().to(DEV) for x in (q, k, v))
            else:
                qd, kd, vd = (x.to(DEV) for x in (q, k, v))
            lens_t = torch.tensor(lens, dtype=torch.int32)
            kw = dict(left_paddings=(L - lens_t).to(DEV)) if left else dict(seqlens=lens_t.to(DEV))
            mod = New(Hq, L, bs, 2, 3, num_kv_heads=Hkv, seq_dim=seq_dim).to(DEV)
            torch.cuda.synchronize()
            poison_o = _poisoned_like(qd.shape, dtype)
            poison_l = torch.full((B, Hq, L), float("nan"), dtype=torch.float32, device=DEV)
            addr_o, addr_l = poison_o.data_ptr(), poison_l.data_ptr()
            del poison_o, poison_l  # the blocks go back to the allocator and come out again as the outputs
            got, lse = mod(qd, kd, vd, sm, return_lse=True, **kw)
            assert got.data_ptr() == addr_o and lse.data_ptr() == addr_l, "the outputs did not start poisoned"
            if seq_dim == 2:
                got = got.transpose(1, 2)
            got, lse = got.cpu(), lse.cpu()
            assert not torch.isnan(got).any(), "rows that no workgroup wrote"
            assert not torch.isnan(lse).any(), "log-sum-exps that no workgroup wrote"
            for i, l in enumerate(lens):
                rows = slice(L - l, L) if left else slice(0, l)
                pad = torch.ones(L, dtype=torch.bool)
                pad[rows] = False
                assert (got[i, pad] == 0).all() and torch.isinf(lse[i][:, pad]).all() and (lse[i][:, pad] < 0).all()
                if l == 0:
                    continue
                mask = OA.sequence_token_mask(bm, bs, l, l)
                ro, rl = OA.dense_attention(q[i:i + 1, rows].float(), k[i:i + 1, rows].float(), v[i:i + 1, rows].float(),
                                            torch.from_numpy(mask), sm)
                assert_close(f"O[{i}]", got[i, rows], ro[0], **tol)
                assert_close(f"LSE[{i}]", lse[i][:, rows], rl[0], atol=1e-4 if dtype == torch.float32 else LSE_TOL, rtol=0)
    finally:
        ops.set_impl("auto")
