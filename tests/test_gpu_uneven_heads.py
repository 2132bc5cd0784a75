"""Patterns whose heads hold clearly different numbers of blocks (num_dense_heads beside sparse
heads): the matrix-core kernels deal such heads to the hardware's workgroup queues in rotation
(dk_lut.uneven_heads).  Every (head, work item) pair is still computed exactly once, so the results
must match the fp32 oracle like any other and be bit-identical to the unrotated launch."""
from __future__ import annotations

import math

import pytest
import torch

from dkernel_amd import LocalStrideSparseAttention, ops
from helpers import F32_TOL, LSE_TOL, TOL, assert_close, expand_heads, make_qkv, oracle_fwd
from oracle import layout as OL

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
New = LocalStrideSparseAttention.__wrapped__  # a module of the test's own (the class is lru_cached)


def _last_fwd() -> bytes:
    from dkernel_amd import _lib
    return _lib.lib().dk_last_kernels()


# (q heads, kv heads, dense heads, tokens, head dim, dtype): 32 and 16 heads sit on fixed queues
# without the rotation; 2 heads over 16 row pairs move on every second / fourth step; a GQA group
# per workgroup; head dims of the padded and of the 256-wide kernels; fp32 on the matrix cores
CASES = [
    (32, 32, 4, 1024, 128, torch.bfloat16),
    (16, 16, 2, 1024, 64, torch.float16),
    (2, 2, 1, 2048, 128, torch.bfloat16),
    (8, 2, 1, 1024, 128, torch.bfloat16),
    (6, 6, 2, 640, 96, torch.bfloat16),
    (4, 4, 1, 512, 192, torch.bfloat16),
    (4, 4, 1, 768, 64, torch.float32),
]


@pytest.mark.parametrize("Hq,Hkv,dense,L,D,dtype", CASES)
def test_forward_and_backward_match_the_oracle(Hq, Hkv, dense, L, D, dtype):
    print(f"case Hq={Hq} Hkv={Hkv} dense={dense} L={L} D={D} {dtype}", flush=True)
    sm = 1 / math.sqrt(D)
    kw = {"num_dense_heads": dense}
    if Hkv != Hq:
        kw["num_kv_heads"] = Hkv
    mod = New(Hq, L, 64, 2, 4, **kw).to(DEV)
    assert mod.kwargs["uneven_heads"]
    bm = expand_heads(OL.block_mask(Hq, L, 64, 2, 4, **kw), Hq)
    q, k, v, do = make_qkv(1, L, L, Hq, Hkv, D, dtype, 1, with_do=True)
    qo, ko, vo = (x.clone().float().requires_grad_() for x in (q, k, v))
    ro, rlse = oracle_fwd(qo, ko, vo, bm, 64, sm)
    ro.backward(do.float())
    qd, kd, vd = (x.to(DEV).requires_grad_() for x in (q, k, v))
    out, lse = mod(qd, kd, vd, sm, return_lse=True)
    assert b"heads in rotation" in _last_fwd(), _last_fwd()
    out.backward(do.to(DEV))
    assert ops.last_bwd_kernels.count(b"heads in rotation") == 2, ops.last_bwd_kernels  # dQ and dK/dV
    tol = F32_TOL if dtype == torch.float32 else TOL
    assert_close("O", out, ro, **tol)
    assert_close("LSE", lse, rlse, atol=1e-4 if dtype == torch.float32 else LSE_TOL, rtol=0)
    assert_close("dQ", qd.grad, qo.grad, **tol)
    assert_close("dK", kd.grad, ko.grad, **tol)
    assert_close("dV", vd.grad, vo.grad, **tol)

    # the same launches with every head on its own queues: the same bits
    mod.kwargs["uneven_heads"] = False
    q2, k2, v2 = (x.to(DEV).requires_grad_() for x in (q, k, v))
    out2, lse2 = mod(q2, k2, v2, sm, return_lse=True)
    assert b"heads in rotation" not in _last_fwd()
    out2.backward(do.to(DEV))
    assert b"heads in rotation" not in ops.last_bwd_kernels
    assert torch.equal(out, out2) and torch.equal(lse, lse2)
    assert torch.equal(qd.grad, q2.grad) and torch.equal(kd.grad, k2.grad) and torch.equal(vd.grad, v2.grad)


@pytest.mark.parametrize("Hq,Hkv,D", [(16, 16, 128), (8, 2, 64), (2, 2, 128)])
def test_padded_and_packed_prefill_do_not_depend_on_the_rotation(Hq, Hkv, D):
    print(f"case Hq={Hq} Hkv={Hkv} D={D}", flush=True)
    L, B = 1024, 3
    sm = 1 / math.sqrt(D)
    kw = {"num_dense_heads": max(1, Hkv // 4)}
    if Hkv != Hq:
        kw["num_kv_heads"] = Hkv
    mod = New(Hq, L, 64, 2, 4, **kw).to(DEV)
    assert mod.kwargs["uneven_heads"]
    q, k, v = (x.to(DEV) for x in make_qkv(B, L, L, Hq, Hkv, D, torch.bfloat16, 1))
    lens = torch.tensor([1000, 130, 577], dtype=torch.int32, device=DEV)
    results = []
    for uneven in (True, False):
        mod.kwargs["uneven_heads"] = uneven
        got = []
        # left-padded and right-padded batches (the padding rows come back cleared)
        got += list(mod(q, k, v, sm, left_paddings=L - lens, return_lse=True))
        assert (b"heads in rotation" in _last_fwd()) == uneven, _last_fwd()
        got += list(mod(q, k, v, sm, seqlens=lens, return_lse=True))
        assert (b"heads in rotation" in _last_fwd()) == uneven
        # the same sequences packed along one token dimension
        cu = torch.zeros(B + 1, dtype=torch.int32, device=DEV)
        cu[1:] = lens.cumsum(0)
        pack = lambda x: torch.cat([x[b, :int(lens[b])] for b in range(B)])  # noqa: E731
        got += list(mod(pack(q), pack(k), pack(v), sm, cu_seqlen_k=cu, return_lse=True))
        assert (b"heads in rotation" in _last_fwd()) == uneven
        # a decode step never rotates (one work item per head)
        got += [mod(q[:, -1:], k, v, sm, seqlens=lens)]
        assert b"heads in rotation" not in _last_fwd()
        results.append(got)
    for a, b in zip(*results):
        assert torch.equal(a, b)


@pytest.mark.parametrize("H,L", [(32, 16384), (16, 8192)])
def test_long_contexts_do_not_depend_on_the_rotation(H, L):
    """At the lengths where the rotation pays (and where the dK/dV grid is long enough for steps of
    two): forward and backward are bit-identical with and without it."""
    print(f"case H={H} L={L}", flush=True)
    D = 128
    sm = 1 / math.sqrt(D)
    mod = New(H, L, 64, 8, 8, num_dense_heads=H // 8).to(DEV)
    assert mod.kwargs["uneven_heads"]
    g = torch.Generator(device=DEV).manual_seed(20)
    q, k, v, do = (torch.randn(1, L, H, D, generator=g, device=DEV).to(torch.bfloat16) for _ in range(4))
    results = []
    for uneven in (True, False):
        mod.kwargs["uneven_heads"] = uneven
        qd, kd, vd = (x.clone().requires_grad_() for x in (q, k, v))
        out, lse = mod(qd, kd, vd, sm, return_lse=True)
        assert (b"heads in rotation" in _last_fwd()) == uneven
        out.backward(do)
        assert ops.last_bwd_kernels.count(b"heads in rotation") == (2 if uneven else 0)
        results.append((out, lse, qd.grad, kd.grad, vd.grad))
    assert torch.isfinite(results[0][0].float()).all() and torch.isfinite(results[0][2].float()).all()
    for a, b in zip(*results):
        assert torch.equal(a, b)
