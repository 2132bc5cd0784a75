"""Explicit block_m > block_size over user patterns that merging widens (reference:
dkernel/utils.py:299-308 builds the merged table, dkernel/ops/sparse_attn_fwd.py:113-134 applies
its micro_M row limit): every pattern row of a merged tile up to the last holder of a column
attends that column.  The expected mask is expanded by brute force from the merged table itself
(the `layout_csr_*` buffers, pinned by the golden fixtures); forward and backward are checked
against the dense oracle over that mask, on the generic and on the matrix-core kernels."""
from __future__ import annotations

import math
import warnings

import numpy as np
import pytest
import torch

from dkernel_amd import SparseAttention, ops
from helpers import LSE_TOL, TOL, assert_close, oracle_fwd

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(params=["generic", "auto"])
def impl(request):
    ops.set_impl(request.param)
    yield request.param
    ops.set_impl("auto")


def _attended_blocks(mod, H, n, bs):
    """(H, n, n) block mask that the module's merged table attends: rows below micro_M of each
    listed (merged tile, column), lower triangle."""
    mm = mod.block_m // bs
    crow = mod.layout_csr_crow.cpu().numpy()
    col = mod.layout_csr_col.cpu().numpy()
    assert col.ndim == 3, "a merged table carries (column, micro_M)"
    eff = np.zeros((H, n, n), dtype=np.uint8)
    for h in range(H):
        hh = h if crow.shape[0] > 1 else 0
        for i in range(crow.shape[1] - 1):
            for c, micro in col[hh, crow[hh, i]:crow[hh, i + 1]]:
                for s in range(mm):
                    if i * mm + s < n and s * bs < micro:
                        eff[h, i * mm + s, c] = 1
    return np.tril(eff)


@pytest.mark.parametrize("bs,block_m,D,dtype", [(64, 128, 128, torch.bfloat16), (32, 128, 64, torch.float16),
                                                 (16, 64, 128, torch.bfloat16), (128, 256, 96, torch.bfloat16)])
def test_merged_rows_that_widen_the_pattern(impl, bs, block_m, D, dtype):
    H, n = 3, 16
    L = n * bs
    g = torch.Generator().manual_seed(bs + block_m)
    pat = torch.rand(H, n, n, generator=g) < 0.3
    pat |= torch.eye(n, dtype=torch.bool)[None]
    pat = torch.tril(pat.to(torch.uint8))
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        mod = SparseAttention(bs, pat, block_m=block_m).to(DEV)
    want = _attended_blocks(mod, H, n, bs)
    assert (want >= pat.numpy()).all() and (want != pat.numpy()).any(), "the case must widen the pattern"
    if impl == "auto":  # the matrix-core kernels run their own tiles over the widened pattern
        assert mod.exact_tile is not None or mod.kernel_tile is not None or mod.mask_tile is not None
    sm = 1 / math.sqrt(D)
    q, k, v, do = (torch.randn(2, L, H, D, generator=g).to(dtype) for _ in range(4))
    qo, ko, vo = (x.float().requires_grad_() for x in (q, k, v))
    ro, rl = oracle_fwd(qo, ko, vo, want, bs, sm)
    ro.backward(do.float())
    qd, kd, vd = (x.to(DEV).requires_grad_() for x in (q, k, v))
    out, lse = mod(qd, kd, vd, sm, return_lse=True)
    out.backward(do.to(DEV))
    assert_close("O", out, ro, **TOL)
    assert_close("LSE", lse, rl, atol=LSE_TOL, rtol=0)
    assert_close("dQ", qd.grad, qo.grad, **TOL)
    assert_close("dK", kd.grad, ko.grad, **TOL)
    assert_close("dV", vd.grad, vo.grad, **TOL)
