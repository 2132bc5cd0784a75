"""fp32 inputs on the matrix cores (v_mfma_f32_32x32x2_f32; head dims up to 64): forward and
backward forced onto them with set_impl("mfma") and checked against the fp32 oracle within 2e-4
(LSE 1e-4), for the reference's fp32 shapes (tests/test_sparse_attn.py:56-67: d = 64 and below),
the CPU-plumbing configuration (B1 L1024 H8 d64, block 64, local 4, vert 4), grouped heads, ragged
lengths, more keys than queries, gradients through the LSE, padded / packed / single-token inputs.
dk_last_kernels() proves which kernels ran."""
from __future__ import annotations

import math

import pytest
import torch

from dkernel_amd import LocalStrideSparseAttention, _lib, ops
from helpers import F32_TOL, assert_close, expand_heads, make_qkv, oracle_fwd
from oracle import attention as OA
from oracle import layout as OL

pytestmark = pytest.mark.gpu
DEV = "cuda"
New = LocalStrideSparseAttention.__wrapped__


@pytest.fixture(autouse=True)
def matrix_cores_only():
    ops.set_impl("mfma")   # anything the matrix-core kernels do not take fails loudly
    yield
    ops.set_impl("auto")


def _ran(kind):
    return (_lib.lib().dk_last_kernels() if kind == "fwd" else ops.last_bwd_kernels).decode()


@pytest.mark.parametrize("B,Hq,Hkv,L,D,bs,local,vert", [
    (1, 8, 8, 1024, 64, 64, 4, 4),      # the CPU-plumbing configuration
    (2, 4, 4, 512, 64, 64, 2, 4),
    (2, 8, 2, 500, 64, 64, 2, 3),       # grouped heads, ragged length
    (1, 2, 2, 384, 48, 64, 2, 3),       # head dims below the tile width (zero-padded on chip)
    (1, 4, 1, 333, 32, 64, 3, 2),
    (1, 2, 2, 200, 4, 64, 1, 2),
    (1, 2, 2, 1024, 64, 128, 1, 2),     # blocks of 128 on split tiles
])
def test_forward_backward(B, Hq, Hkv, L, D, bs, local, vert):
    sm = 1 / math.sqrt(D)
    q, k, v, do = make_qkv(B, L, L, Hq, Hkv, D, torch.float32, with_do=True)
    Lr = (L + max(bs, 64) - 1) // max(bs, 64) * max(bs, 64)
    bm = expand_heads(OL.block_mask(Hq, Lr, bs, local, vert, num_kv_heads=Hkv), Hq)
    dlse = torch.randn(B, Hq, L, generator=torch.Generator().manual_seed(3))
    qo, ko, vo = (x.clone().requires_grad_() for x in (q, k, v))
    ro, rl = oracle_fwd(qo, ko, vo, bm, bs, sm)
    ((ro * do).sum() + (rl * dlse).sum()).backward()
    mod = New(Hq, Lr, bs, local, vert, num_kv_heads=Hkv).to(DEV)
    qd, kd, vd = (x.to(DEV).requires_grad_() for x in (q, k, v))
    out, lse = mod(qd, kd, vd, sm, return_lse=True)
    assert _ran("fwd") == "f32::fwd_kernel; "
    ((out * do.to(DEV)).sum() + (lse * dlse.to(DEV)).sum()).backward()
    assert _ran("bwd") == "f32::delta_kernel; f32::dq_kernel; f32::dkdv_kernel; "
    assert_close("O", out, ro, **F32_TOL)
    assert_close("LSE", lse, rl, atol=1e-4, rtol=0)
    assert_close("dQ", qd.grad, qo.grad, **F32_TOL)
    assert_close("dK", kd.grad, ko.grad, **F32_TOL)
    assert_close("dV", vd.grad, vo.grad, **F32_TOL)


@pytest.mark.parametrize("past", [37, 64, 200])
def test_more_keys_than_queries_and_noncausal(past):
    B, Hq, Hkv, Lq, D = 2, 4, 2, 300, 64
    Lk = Lq + past
    sm = 1 / math.sqrt(D)
    g = torch.Generator().manual_seed(past)
    q, do = (torch.randn(B, Lq, Hq, D, generator=g) for _ in range(2))
    k, v = (torch.randn(B, Lk, Hkv, D, generator=g) for _ in range(2))
    bm = expand_heads(OL.block_mask(Hq, 512, 64, 2, 3, num_kv_heads=Hkv), Hq)
    qo, ko, vo = (x.clone().requires_grad_() for x in (q, k, v))
    ro, _ = oracle_fwd(qo, ko, vo, bm, 64, sm)
    ro.backward(do)
    mod = New(Hq, 512, 64, 2, 3, num_kv_heads=Hkv).to(DEV)
    qd, kd, vd = (x.to(DEV).requires_grad_() for x in (q, k, v))
    out = mod(qd, kd, vd, sm)
    out.backward(do.to(DEV))
    assert "f32::dkdv_kernel" in _ran("bwd")
    for name, got, want in (("O", out, ro), ("dQ", qd.grad, qo.grad), ("dK", kd.grad, ko.grad), ("dV", vd.grad, vo.grad)):
        assert_close(name, got, want, **F32_TOL)
    if past == 64:  # bidirectional pattern, relative vertical positions
        bmn = expand_heads(OL.block_mask(Hq, 512, 64, 2, 3, num_kv_heads=Hkv, causal=False), Hq)
        modn = New(Hq, 512, 64, 2, 3, num_kv_heads=Hkv, causal=False).to(DEV)
        q2, k2, v2 = (torch.randn(1, 512, h, D, generator=g) for h in (Hq, Hkv, Hkv))
        ron, rln = oracle_fwd(q2, k2, v2, bmn, 64, sm, causal=False)
        outn, lsen = modn(q2.to(DEV), k2.to(DEV), v2.to(DEV), sm, return_lse=True)
        assert _ran("fwd") == "f32::fwd_kernel; "
        assert_close("O noncausal", outn, ron, **F32_TOL)
        assert_close("LSE noncausal", lsen, rln, atol=1e-4, rtol=0)


def test_padded_packed_and_single_token():
    Hq, Hkv, D, Lmax = 4, 2, 64, 512
    sm = 1 / math.sqrt(D)
    g = torch.Generator().manual_seed(5)
    lens = [512, 1, 130, 333]
    bm = OL.block_mask(Hq, Lmax, 64, 2, 3, num_kv_heads=Hkv)
    mod = New(Hq, Lmax, 64, 2, 3, num_kv_heads=Hkv).to(DEV)
    qs = [torch.randn(l, Hq, D, generator=g) for l in lens]
    ks = [torch.randn(l, Hkv, D, generator=g) for l in lens]
    vs = [torch.randn(l, Hkv, D, generator=g) for l in lens]

    def want(i, q_rows=None):
        l = lens[i]
        nq = l if q_rows is None else q_rows
        mask = OA.sequence_token_mask(bm, 64, nq, l)
        return OA.dense_attention(qs[i][None, l - nq:], ks[i][None], vs[i][None], torch.from_numpy(mask), sm)

    # left-padded prefill
    qp, kp, vp = (torch.zeros(len(lens), Lmax, h, D) for h in (Hq, Hkv, Hkv))
    for i, l in enumerate(lens):
        qp[i, Lmax - l:], kp[i, Lmax - l:], vp[i, Lmax - l:] = qs[i], ks[i], vs[i]
    left = torch.tensor([Lmax - l for l in lens])
    out, lse = mod(qp.to(DEV), kp.to(DEV), vp.to(DEV), sm, left_paddings=left, return_lse=True)
    assert _ran("fwd") == "f32::fwd_kernel; "
    for i, l in enumerate(lens):
        ro, rl = want(i)
        assert_close(f"O padded[{i}]", out[i, Lmax - l:], ro[0], **F32_TOL)
        assert_close(f"LSE padded[{i}]", lse[i, :, Lmax - l:], rl[0], atol=1e-4, rtol=0)
    # single-token decode over the same left-padded keys
    qd = torch.stack([qs[i][-1:] for i in range(len(lens))])
    outd = mod(qd.to(DEV), kp.to(DEV), vp.to(DEV), sm, left_paddings=left)
    assert _ran("fwd") == "f32::fwd_kernel; "
    for i in range(len(lens)):
        assert_close(f"O decode[{i}]", outd[i], want(i, 1)[0][0], **F32_TOL)
    # packed prefill
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    outp, lsep = mod(torch.cat(qs).to(DEV), torch.cat(ks).to(DEV), torch.cat(vs).to(DEV), sm, cu_seqlen_k=cu.to(DEV),
                     return_lse=True)
    assert _ran("fwd") == "f32::fwd_kernel; "
    for i, l in enumerate(lens):
        s = int(cu[i])
        ro, rl = want(i)
        assert_close(f"O packed[{i}]", outp[s:s + l], ro[0], **F32_TOL)
        assert_close(f"LSE packed[{i}]", lsep[:, s:s + l], rl[0], atol=1e-4, rtol=0)


def test_what_the_fp32_matrix_core_kernels_do_not_take_is_refused():
    """Head dims above 64 and sub-block tables stay on the generic kernels: forced onto the matrix
    cores they fail loudly instead of running something else."""
    q, k, v = (x.to(DEV) for x in make_qkv(1, 256, 256, 2, 2, 128, torch.float32))
    with pytest.raises(Exception, match="no MFMA forward kernel"):
        New(2, 256, 64, 2, 3).to(DEV)(q, k, v, 0.1)
