"""combine_attn_partitions on the device (dk_combine / dk_combine_bwd) against the reference's
torch expression (dkernel/interface.py:303-324: softmax over the stacked log-sum-exps, weighted sum
in fp32, one cast) evaluated on the host with autograd: every layout the module returns --
(batch, heads, tokens, dim), (batch, tokens, heads, dim) with hdim=2, packed (tokens, heads, dim)
with (heads, tokens) log-sum-exps --, 2 to 8 partitions, rows that saw no key in one or in every
partition, head dims with and without 16-byte rows, views with strides."""
from __future__ import annotations

import pytest
import torch

from dkernel_amd import _lib, combine_attn_partitions, ops

pytestmark = pytest.mark.gpu
DEV = "cuda"


def reference(pairs, transposed):
    outs = torch.stack([o.float() for o, _ in pairs])
    w = torch.stack([l.float() for _, l in pairs])
    if transposed:
        w = w.transpose(-1, -2)
    w = w.softmax(0)
    w = torch.where(torch.isnan(w), torch.zeros_like(w), w)
    return (outs * w.unsqueeze(-1)).sum(0)


def make(shape_o, shape_l, parts, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    pairs = []
    for _ in range(parts):
        o = torch.randn(shape_o, generator=g).to(dtype)
        l = torch.randn(shape_l, generator=g) * 3
        pairs.append((o, l))
    # rows without keys: in one partition, and in all of them
    flat = [l.view(-1) for _, l in pairs]
    flat[0][::7] = float("-inf")
    for f in flat:
        f[3::11] = float("-inf")
    for (o, l) in pairs:
        mask = torch.isinf(l)
        if l.shape != o.shape[:-1]:
            mask = mask.transpose(-1, -2)
        o[mask] = 0
    return pairs


CASES = [
    # outputs, lse, hdim, transposed
    ((2, 4, 50, 128), (2, 4, 50), 1, False),
    ((2, 50, 4, 128), (2, 4, 50), 2, True),
    ((333, 4, 128), (4, 333), 1, True),
    ((2, 3, 17, 96), (2, 3, 17), 1, False),
    ((65, 2, 36), (2, 65), 1, True),      # rows of 72 bytes: element-wise accesses
    ((1, 2, 9, 256), (1, 2, 9), 1, False),
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape_o,shape_l,hdim,transposed", CASES)
@pytest.mark.parametrize("parts", [2, 3, 8])
def test_forward_and_backward(shape_o, shape_l, hdim, transposed, parts, dtype):
    pairs = make(shape_o, shape_l, parts, dtype, seed=parts + len(shape_o))
    g = torch.Generator().manual_seed(1)
    dout = torch.randn(shape_o, generator=g).to(dtype)
    host = [(o.clone().float().requires_grad_(), l.clone().requires_grad_()) for o, l in pairs]
    want = reference(host, transposed)
    want.backward(dout.float())
    dev = [(o.to(DEV).requires_grad_(), l.to(DEV).requires_grad_()) for o, l in pairs]
    got = combine_attn_partitions(*dev, hdim=hdim)
    assert _lib.lib().dk_last_kernels() == b"combine_kernel [T = %s, BWD = false]; " % (
        {torch.bfloat16: b"dk::bf16_t", torch.float16: b"_Float16", torch.float32: b"float"}[dtype])
    assert got.dtype == dtype and got.shape == torch.Size(shape_o)
    got.backward(dout.to(DEV))
    assert ops.last_bwd_kernels.startswith(b"combine_bwd_kernel")
    tol = dict(atol=1e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=1e-2)
    torch.testing.assert_close(got.float().cpu(), want, **tol)
    assert not torch.isnan(got).any()
    # rows that saw no key in any partition: autograd through the torch expression gives NaN
    # log-sum-exp gradients there (softmax of all -inf); the kernel gives 0
    dead = torch.stack([torch.isinf(l) for _, l in pairs]).all(0)
    assert dead.any()
    for (od, ld), (oh, lh) in zip(dev, host):
        torch.testing.assert_close(od.grad.float().cpu(), oh.grad, **tol)
        assert not torch.isnan(ld.grad).any() and (ld.grad.cpu()[dead] == 0).all()
        # the log-sum-exp gradients are sums over head_dim of products of rounded values
        torch.testing.assert_close(ld.grad.cpu()[~dead], lh.grad[~dead], atol=1e-4 if dtype == torch.float32 else 5e-2,
                                   rtol=2e-2)


def test_strided_views_and_no_grad():
    """Partition outputs that are views (a slice of a wider buffer, a transposed tensor): strides are
    passed through; without grad nothing is saved."""
    g = torch.Generator().manual_seed(5)
    wide = torch.randn(2, 40, 4, 256, generator=g).to(torch.bfloat16).to(DEV)
    a = wide[..., :128]                         # token stride 1024, rows of 128
    b = wide[..., 128:]
    la, lb = (torch.randn(2, 4, 40, generator=g).to(DEV) for _ in range(2))
    with torch.no_grad():
        got = combine_attn_partitions((a, la), (b, lb), hdim=2)
    want = reference([(a.cpu(), la.cpu()), (b.cpu(), lb.cpu())], True)
    torch.testing.assert_close(got.float().cpu(), want, atol=2e-2, rtol=1e-2)
    at, bt = a.transpose(1, 2), b.transpose(1, 2)   # (batch, heads, tokens, dim) views of the same memory
    got2 = combine_attn_partitions((at, la), (bt, lb))
    torch.testing.assert_close(got2.transpose(1, 2).float().cpu(), want, atol=2e-2, rtol=1e-2)


def test_argument_errors():
    o = torch.zeros(2, 3, 4, 8, device=DEV, dtype=torch.bfloat16)
    l = torch.zeros(2, 3, 4, device=DEV)
    with pytest.raises(AssertionError, match="differ in shape"):
        combine_attn_partitions((o, l), (o[:, :2], l[:, :2]))
    args = _lib.CombineArgs()
    args.num_partitions = 1
    assert _lib.lib().dk_combine(args) == _lib.DK_ERR_INVALID
    assert b"2 to 8 partitions" in _lib.lib().dk_last_error()
