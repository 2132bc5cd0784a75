"""Constructor kwargs the reference documents as kernel args (dkernel/interface.py:31-34:
`out`, `inference`, `d_splits`), a non-positive softmax scale, and the backward pass with more
keys than queries (past > 0), all against the fp32 oracle."""
from __future__ import annotations

import math

import numpy as np
import pytest
import torch

from dkernel_amd import LocalStrideSparseAttention, ops
from helpers import LSE_TOL, TOL, assert_close, expand_heads, make_qkv, oracle_fwd
from oracle import attention as OA
from oracle import layout as OL

pytestmark = pytest.mark.gpu
DEV = "cuda"
New = LocalStrideSparseAttention.__wrapped__   # uncached instances: the kwargs under test hold tensors


@pytest.fixture(params=["generic", "auto"])
def impl(request):
    ops.set_impl(request.param)
    yield request.param
    ops.set_impl("auto")


def _bm(Hq, L, local, vert, Hkv):
    return expand_heads(OL.block_mask(Hq, L, 64, local, vert, num_kv_heads=Hkv), Hq)


def test_out_kwarg_unpadded(impl):
    B, Hq, Hkv, L, D = 2, 4, 2, 300, 128
    sm = 1 / math.sqrt(D)
    q, k, v = make_qkv(B, L, L, Hq, Hkv, D, torch.bfloat16)
    # a view with non-dense token / head strides: the kernels write through its strides
    big = torch.full((B, L + 5, Hq + 1, D), float("nan"), dtype=torch.bfloat16, device=DEV)
    out = big[:, 5:, :Hq]
    mod = New(Hq, 512, 64, 2, 3, num_kv_heads=Hkv, out=out).to(DEV)
    res, lse = mod(q.to(DEV), k.to(DEV), v.to(DEV), sm, return_lse=True)
    assert res.data_ptr() == out.data_ptr() and res.stride() == out.stride()
    ro, rl = oracle_fwd(q, k, v, _bm(Hq, 512, 2, 3, Hkv), 64, sm)
    assert_close("O", out, ro, **TOL)
    assert_close("LSE", lse, rl, atol=LSE_TOL, rtol=0)
    assert torch.isnan(big[:, :5]).all() and torch.isnan(big[:, :, Hq]).all()   # nothing else was written


@pytest.mark.parametrize("D", [64, 128])
def test_out_rows_not_cache_line_aligned(D):
    """Output rows that start 16 bytes into a 128-byte line and are 16 bytes longer than the
    head dim apart: the whole-row stores must write exactly the rows' bytes."""
    B, Hq, Hkv, L = 1, 4, 2, 200
    sm = 1 / math.sqrt(D)
    q, k, v = make_qkv(B, L, L, Hq, Hkv, D, torch.bfloat16)
    big = torch.full((B, L, Hq, D + 8), float("nan"), dtype=torch.bfloat16, device=DEV)
    out = big[..., 8:]
    assert out.data_ptr() % 128 == 16 and (out.stride(2) * 2) % 128 != 0
    mod = New(Hq, 256, 64, 2, 3, num_kv_heads=Hkv, out=out).to(DEV)
    res = mod(q.to(DEV), k.to(DEV), v.to(DEV), sm)
    assert res.data_ptr() == out.data_ptr()
    ro, _ = oracle_fwd(q, k, v, _bm(Hq, 256, 2, 3, Hkv), 64, sm)
    assert_close("O", out, ro, **TOL)
    assert torch.isnan(big[..., :8]).all()   # the gaps between the rows were not written


def test_out_kwarg_is_checked():
    q = torch.zeros(1, 128, 2, 64, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(AssertionError, match="out has shape"):
        New(2, 128, 64, 1, 2, out=torch.zeros(1, 128, 2, 32, dtype=torch.bfloat16, device=DEV)).to(DEV)(q, q, q)
    with pytest.raises(AssertionError, match="dtype and device"):
        New(2, 128, 64, 1, 2, out=torch.zeros(1, 128, 2, 64, dtype=torch.float16, device=DEV)).to(DEV)(q, q, q)
    with pytest.raises(AssertionError, match="unit stride"):
        New(2, 128, 64, 1, 2, out=torch.zeros(1, 128, 2, 128, dtype=torch.bfloat16, device=DEV)[..., ::2]).to(DEV)(q, q, q)


def test_out_kwarg_padded_and_packed(impl):
    B, Hq, Hkv, Lmax, D = 3, 4, 2, 512, 64
    sm = 1 / math.sqrt(D)
    lens = [512, 130, 65]
    g = torch.Generator().manual_seed(5)
    ks = [torch.randn(l, Hkv, D, generator=g).to(torch.bfloat16) for l in lens]
    vs = [torch.randn(l, Hkv, D, generator=g).to(torch.bfloat16) for l in lens]
    qs = [torch.randn(l, Hq, D, generator=g).to(torch.bfloat16) for l in lens]
    bm = _bm(Hq, Lmax, 2, 3, Hkv)
    refs = []
    for q1, k1, v1, l in zip(qs, ks, vs, lens):
        mask = OA.sequence_token_mask(bm, 64, l, l)
        refs.append(OA.dense_attention(q1[None], k1[None], v1[None], torch.from_numpy(mask), sm)[0][0])
    # left-padded 4-D input: padding rows of the caller's tensor stay as they were
    qp, kp, vp = (torch.zeros(B, Lmax, h, D, dtype=torch.bfloat16) for h in (Hq, Hkv, Hkv))
    for i, l in enumerate(lens):
        qp[i, Lmax - l:], kp[i, Lmax - l:], vp[i, Lmax - l:] = qs[i], ks[i], vs[i]
    out = torch.full((B, Lmax, Hq, D), 7.0, dtype=torch.bfloat16, device=DEV)
    mod = New(Hq, Lmax, 64, 2, 3, num_kv_heads=Hkv, out=out).to(DEV)
    res = mod(qp.to(DEV), kp.to(DEV), vp.to(DEV), sm, left_paddings=torch.tensor([Lmax - l for l in lens]))
    assert res.data_ptr() == out.data_ptr()
    for i, l in enumerate(lens):
        assert_close(f"O padded[{i}]", out[i, Lmax - l:], refs[i], **TOL)
        assert (out[i, :Lmax - l] == 7.0).all()
    # packed 3-D input
    T = sum(lens)
    outp = torch.full((T, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
    modp = New(Hq, Lmax, 64, 2, 3, num_kv_heads=Hkv, out=outp).to(DEV)
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32, device=DEV)
    resp = modp(torch.cat(qs).to(DEV), torch.cat(ks).to(DEV), torch.cat(vs).to(DEV), sm, cu_seqlen_k=cu)
    assert resp.data_ptr() == outp.data_ptr()
    assert_close("O packed", outp, torch.cat(refs), **TOL)


def test_inference_and_d_splits_kwargs(impl):
    B, Hq, Hkv, L, D = 1, 4, 4, 256, 128
    sm = 1 / math.sqrt(D)
    q, k, v, do = make_qkv(B, L, L, Hq, Hkv, D, torch.bfloat16, with_do=True)
    ro, rl = oracle_fwd(q, k, v, _bm(Hq, L, 2, 3, Hkv), 64, sm)
    base = New(Hq, L, 64, 2, 3).to(DEV)(q.to(DEV), k.to(DEV), v.to(DEV), sm)
    # d_splits is a Triton shared-memory knob: accepted, no effect
    for d_splits in (None, 1, 2):
        got = New(Hq, L, 64, 2, 3, d_splits=d_splits).to(DEV)(q.to(DEV), k.to(DEV), v.to(DEV), sm)
        assert torch.equal(got, base)
    assert_close("O", base, ro, **TOL)
    # inference=True with inputs that require grad: no LSE is kept, backward is refused
    qd, kd, vd = (x.to(DEV).requires_grad_() for x in (q, k, v))
    out = New(Hq, L, 64, 2, 3, inference=True).to(DEV)(qd, kd, vd, sm)
    assert torch.equal(out.detach(), base)
    with pytest.raises(AssertionError, match="inference mode"):
        out.backward(do.to(DEV))
    # ... but LSE is still returned when asked for (the reference fails there)
    out, lse = New(Hq, L, 64, 2, 3, inference=True).to(DEV)(q.to(DEV), k.to(DEV), v.to(DEV), sm, return_lse=True)
    assert_close("LSE", lse, rl, atol=LSE_TOL, rtol=0)
    # inference=False without grads: same output
    got = New(Hq, L, 64, 2, 3, inference=False).to(DEV)(q.to(DEV), k.to(DEV), v.to(DEV), sm)
    assert torch.equal(got, base)


@pytest.mark.parametrize("D", [128, 64])
def test_negative_softmax_scale(D):
    """The matrix-core forward takes the row maximum before scaling (scale > 0); other scales run
    on the generic kernels with the same result as the dense definition."""
    B, H, L = 1, 2, 200
    q, k, v = make_qkv(B, L, L, H, H, D, torch.bfloat16)
    ro, rl = oracle_fwd(q, k, v, _bm(H, 256, 2, 3, H), 64, -0.05)
    out, lse = New(H, 256, 64, 2, 3).to(DEV)(q.to(DEV), k.to(DEV), v.to(DEV), -0.05, return_lse=True)
    assert_close("O", out, ro, **TOL)
    assert_close("LSE", lse, rl, atol=LSE_TOL, rtol=0)


@pytest.mark.parametrize("bs", [16, 32])
def test_negative_softmax_scale_small_blocks(bs):
    """Pattern blocks below the kernel tile normally run on masked 64 x 64 tiles, which only the
    matrix-core kernels read; with a scale <= 0 forward and backward take the unmasked tables."""
    B, H, L, D = 1, 2, 200, 64
    q, k, v, do = make_qkv(B, L, L, H, H, D, torch.bfloat16, with_do=True)
    bm = expand_heads(OL.block_mask(H, 256, bs, 3, 4), H)
    qo, ko, vo = (x.float().requires_grad_() for x in (q, k, v))
    ro, rl = oracle_fwd(qo, ko, vo, bm, bs, -0.05)
    ro.backward(do.float())
    mod = New(H, 256, bs, 3, 4).to(DEV)
    assert mod.mask_tile == 64
    qd, kd, vd = (x.to(DEV).requires_grad_() for x in (q, k, v))
    out, lse = mod(qd, kd, vd, -0.05, return_lse=True)
    out.backward(do.to(DEV))
    assert_close("O", out, ro, **TOL)
    assert_close("LSE", lse, rl, atol=LSE_TOL, rtol=0)
    assert_close("dQ", qd.grad, qo.grad, **TOL)
    assert_close("dK", kd.grad, ko.grad, **TOL)
    assert_close("dV", vd.grad, vo.grad, **TOL)


@pytest.mark.parametrize("past", [37, 64, 200])
@pytest.mark.parametrize("Hq,Hkv,D,dtype", [(4, 4, 128, torch.bfloat16), (4, 2, 64, torch.float16), (2, 2, 96, torch.bfloat16)])
def test_backward_with_more_keys_than_queries(impl, past, Hq, Hkv, D, dtype):
    """Queries are the last Lq positions of Lk = Lq + past keys: dQ, dK, dV (keys before the first
    query included) against autograd through the oracle."""
    B, Lq = 2, 300
    Lk = Lq + past
    sm = 1 / math.sqrt(D)
    g = torch.Generator().manual_seed(past)
    q = torch.randn(B, Lq, Hq, D, generator=g).to(dtype)
    k = torch.randn(B, Lk, Hkv, D, generator=g).to(dtype)
    v = torch.randn(B, Lk, Hkv, D, generator=g).to(dtype)
    do = torch.randn(B, Lq, Hq, D, generator=g).to(dtype)
    dlse = torch.randn(B, Hq, Lq, generator=g)
    bm = _bm(Hq, 512, 2, 3, Hkv)
    qo, ko, vo = (x.float().requires_grad_() for x in (q, k, v))
    ro, rl = oracle_fwd(qo, ko, vo, bm, 64, sm)
    ((ro * do.float()).sum() + (rl * dlse).sum()).backward()
    mod = LocalStrideSparseAttention(Hq, 512, 64, 2, 3, num_kv_heads=Hkv).to(DEV)
    qd, kd, vd = (x.to(DEV).requires_grad_() for x in (q, k, v))
    out, lse = mod(qd, kd, vd, sm, return_lse=True)
    ((out.float() * do.to(DEV).float()).sum() + (lse * dlse.to(DEV)).sum()).backward()
    assert_close("O", out, ro, **TOL)
    assert_close("LSE", lse, rl, atol=LSE_TOL, rtol=0)
    assert_close("dV", vd.grad, vo.grad, **TOL)
    assert_close("dK", kd.grad, ko.grad, **TOL)
    assert_close("dQ", qd.grad, qo.grad, **TOL)


@pytest.mark.parametrize("D,bs,Hq,Hkv,dtype", [(256, 32, 4, 4, torch.bfloat16), (160, 64, 2, 2, torch.bfloat16),
                                               (192, 64, 4, 2, torch.float16), (256, 64, 4, 1, torch.bfloat16),
                                               (200, 16, 2, 2, torch.bfloat16), (136, 128, 2, 2, torch.float16)])
def test_head_dims_above_128_on_the_matrix_cores(D, bs, Hq, Hkv, dtype):
    """Head dims 136 ... 256 run at the 256-wide tile of the matrix-core kernels (forward, dQ,
    dK/dV), with plain, split (blocks of 128) and sub-block-masked (blocks of 16 / 32) tables;
    `mfma` makes the library fail instead of falling back to the generic kernels."""
    B, L = 2, 333
    sm = 1 / math.sqrt(D)
    q, k, v, do = make_qkv(B, L, L, Hq, Hkv, D, dtype, with_do=True)
    Lr = ((L + max(bs, 64) - 1) // max(bs, 64)) * max(bs, 64)
    bm = expand_heads(OL.block_mask(Hq, Lr, bs, 2, 3, num_kv_heads=Hkv), Hq)
    qo, ko, vo = (x.float().requires_grad_() for x in (q, k, v))
    ro, rl = oracle_fwd(qo, ko, vo, bm, bs, sm)
    ro.backward(do.float())
    ops.set_impl("mfma")
    try:
        mod = LocalStrideSparseAttention(Hq, L, bs, 2, 3, num_kv_heads=Hkv).to(DEV)
        qd, kd, vd = (x.to(DEV).requires_grad_() for x in (q, k, v))
        out, lse = mod(qd, kd, vd, sm, return_lse=True)
        out.backward(do.to(DEV))
    finally:
        ops.set_impl("auto")
    assert_close("O", out, ro, **TOL)
    assert_close("LSE", lse, rl, atol=LSE_TOL, rtol=0)
    assert_close("dV", vd.grad, vo.grad, **TOL)
    assert_close("dK", kd.grad, ko.grad, **TOL)
    assert_close("dQ", qd.grad, qo.grad, **TOL)


def test_last_kernels_names_the_path_taken():
    """dk_last_kernels(): which kernels the latest call launched (what bench.py's traffic guard and
    this test read)."""
    lib = ops._lib.lib()
    L, D = 256, 128
    sm = 1 / math.sqrt(D)
    try:
        for Hq, Hkv, impl, want in ((8, 2, "auto", "mfma_fwd_kernel [T = dk::bf16_t, D = 128, G = 4, PAD = false]; "),
                                    (2, 2, "auto", "mfma_fwd_kernel [T = dk::bf16_t, D = 128, PAD = false]; "),
                                    (2, 2, "generic", "generic_fwd_kernel<128> [T = dk::bf16_t]; ")):
            ops.set_impl(impl)
            q, k, v = (x.to(DEV) for x in make_qkv(1, L, L, Hq, Hkv, D, torch.bfloat16))
            New(Hq, L, 64, 2, 3, num_kv_heads=Hkv).to(DEV)(q, k, v, sm)
            assert lib.dk_last_kernels().decode() == want
        q.requires_grad_()
        New(2, L, 64, 2, 3).to(DEV)(q, k, v, sm).sum().backward()
        assert ops.last_bwd_kernels.decode().startswith("generic_delta_kernel")
    finally:
        ops.set_impl("auto")


@pytest.mark.parametrize("H", [3, 32])
def test_backward_with_a_table_longer_than_the_keys(H):
    """The dK/dV pass hands its columns out longest first when the heads do not line up with the
    hardware's 32 workgroup queues (H = 3; with H = 32 in ascending order): its grid then covers
    every column of the table, also those beyond the keys of a sequence shorter than max_seqlen."""
    B, L, D, Lmax = 2, 320, 64, 2048
    sm = 1 / math.sqrt(D)
    q, k, v, do = make_qkv(B, L, L, H, H, D, torch.bfloat16, 1, with_do=True)
    bm = OL.block_mask(H, Lmax, 64, 2, 3)[:, :L // 64, :L // 64]
    qo, ko, vo = (x.float().requires_grad_() for x in (q, k, v))
    ro, _ = oracle_fwd(qo, ko, vo, bm, 64, sm)
    ro.backward(do.float())
    mod = New(H, Lmax, 64, 2, 3).to(DEV)
    qd, kd, vd = (x.to(DEV).requires_grad_() for x in (q, k, v))
    out = mod(qd, kd, vd, sm)
    out.backward(do.to(DEV))
    assert b"mfma_dkdv_kernel" in ops.last_bwd_kernels
    assert_close("O", out, ro, **TOL)
    assert_close("dQ", qd.grad, qo.grad, **TOL)
    assert_close("dK", kd.grad, ko.grad, **TOL)
    assert_close("dV", vd.grad, vo.grad, **TOL)
