"""Shared by the tests: seeded inputs (one CPU generator, seed 20, draw order
q, k, v, dO, fp32 N(0,1) cast to the test dtype -- so oracle and kernel see the
same bits), oracle calls and the tolerances of the parity bar."""
from __future__ import annotations

import numpy as np
import torch

from oracle import attention as OA
from oracle import layout as OL

# parity bar: O and grads within 2e-2 abs/rel of the fp32 oracle, LSE within 1e-3
TOL = dict(atol=2e-2, rtol=2e-2)
LSE_TOL = 1e-3
F32_TOL = dict(atol=2e-4, rtol=2e-4)


def make_qkv(B, Lq, Lk, Hq, Hkv, D, dtype, seq_dim=1, seed=20, with_do=False):
    g = torch.Generator().manual_seed(seed)

    def draw(L, H):
        shape = (B, L, H, D) if seq_dim == 1 else (B, H, L, D)
        return torch.randn(shape, generator=g, dtype=torch.float32).to(dtype)
    q, k, v = draw(Lq, Hq), draw(Lk, Hkv), draw(Lk, Hkv)
    if with_do:
        return q, k, v, draw(Lq, Hq)
    return q, k, v


def expand_heads(block_mask, Hq):
    """(1 | Hkv | Hq, nb, nb) block mask -> (Hq, nb, nb)."""
    bm = np.asarray(block_mask)
    if bm.shape[0] == Hq:
        return bm
    return np.repeat(bm, Hq // bm.shape[0], axis=0)


def oracle_fwd(q, k, v, block_mask, block_size, sm_scale, seq_dim=1, causal=True):
    """Dense fp32 oracle for unpadded 4-D inputs; queries are the last Lq
    positions of the Lk keys when causal."""
    Lq, Lk = q.shape[seq_dim], k.shape[seq_dim]
    Hq = q.shape[3 - seq_dim]
    bm = expand_heads(block_mask, Hq)
    mask = OA.sequence_token_mask(bm, block_size, Lq, Lk, causal=causal)
    return OA.dense_attention(q, k, v, torch.from_numpy(mask), sm_scale, seq_dim=seq_dim)


def assert_close(name, got, want, atol, rtol):
    got, want = got.detach().float().cpu(), want.detach().float().cpu()
    assert got.shape == want.shape, f"{name}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    finite = torch.isfinite(want)
    assert torch.equal(torch.isfinite(got), finite), f"{name}: finiteness differs"
    assert torch.equal(got[~finite], want[~finite]), f"{name}: non-finite entries differ"
    err = (got[finite] - want[finite]).abs()
    bound = atol + rtol * want[finite].abs()
    bad = err > bound
    assert not bad.any(), (f"{name}: {int(bad.sum())} of {bad.numel()} beyond atol={atol} rtol={rtol}; "
                           f"max abs err {err.max().item():.4g}")
