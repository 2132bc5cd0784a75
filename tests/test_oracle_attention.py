"""Pins oracle/attention.py (CPU only) independently of its own formulae.

Softmax attention is a textbook function, so every check below reduces the
oracle to a library routine, a closed form or an invariant:

* dense_attention      vs torch.nn.functional.scaled_dot_product_attention with
                       a boolean mask (MHA, and GQA through repeat_interleave),
                       LSE vs torch.logsumexp of independently built logits,
                       fully masked rows, autograd gradients vs float64 finite
                       differences (torch.autograd.gradcheck) and vs autograd
                       through SDPA.
* sequence_token_mask  vs kron(block mask, ones) & tril cut to the last q_len
                       rows, the construction of the reference's checker
                       (tests/test_sparse_attn.py:333-339, 486-537).
* combine_partitions   vs the softmax closed form of
                       dkernel/interface.py:319-324 and vs unpartitioned
                       attention (tests/test_seq_partition.py:178).
* reference_style_attention vs dense_attention (same function, reference's
                       order of casts).
"""
from __future__ import annotations

import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import attention as OA
from oracle import layout as OL


def _rand(shape, seed, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g, dtype=torch.float32).to(dtype)


def _random_mask(B, H, Lq, Lk, seed, p=0.5, keep_diag=True):
    g = torch.Generator().manual_seed(seed)
    m = torch.rand((B, H, Lq, Lk), generator=g) < p
    if keep_diag:       # every row sees at least one key
        idx = torch.arange(Lq) % Lk
        m[:, :, torch.arange(Lq), idx] = True
    return m


@pytest.mark.parametrize("seq_dim", [1, 2])
@pytest.mark.parametrize("Hq,Hkv", [(4, 4), (8, 2), (6, 1)])
def test_dense_attention_matches_sdpa(seq_dim, Hq, Hkv):
    B, Lq, Lk, D = 2, 37, 53, 16
    shape = (lambda L, H: (B, L, H, D) if seq_dim == 1 else (B, H, L, D))
    q, k, v = _rand(shape(Lq, Hq), 1), _rand(shape(Lk, Hkv), 2), _rand(shape(Lk, Hkv), 3)
    mask = _random_mask(B, Hq, Lq, Lk, 4)
    scale = 0.37
    out, lse = OA.dense_attention(q, k, v, mask, scale, seq_dim=seq_dim)

    tq, tk, tv = (x.transpose(1, 2) if seq_dim == 1 else x for x in (q, k, v))
    g = Hq // Hkv
    tk, tv = tk.repeat_interleave(g, dim=1), tv.repeat_interleave(g, dim=1)
    want = F.scaled_dot_product_attention(tq, tk, tv, attn_mask=mask, scale=scale)
    want = want.transpose(1, 2) if seq_dim == 1 else want
    assert out.shape == q.shape and out.dtype == torch.float32
    torch.testing.assert_close(out, want, atol=2e-6, rtol=1e-5)

    # LSE: logsumexp of logits built without the oracle (matmul, additive mask)
    logits = torch.matmul(tq, tk.transpose(-1, -2)) * scale
    logits = logits + torch.where(mask, 0.0, float("-inf"))
    assert lse.shape == (B, Hq, Lq) and lse.dtype == torch.float32
    torch.testing.assert_close(lse, torch.logsumexp(logits, -1), atol=2e-6, rtol=1e-6)


def test_gqa_head_mapping_is_consecutive_groups():
    # kv head of q head h is h // group: q heads 0..g-1 share kv head 0
    B, L, Hq, Hkv, D = 1, 9, 6, 3, 8
    q, k, v = _rand((B, L, Hq, D), 5), _rand((B, L, Hkv, D), 6), _rand((B, L, Hkv, D), 7)
    mask = torch.ones(L, L, dtype=torch.bool).tril()
    out, lse = OA.dense_attention(q, k, v, mask, None, seq_dim=1)
    for h in range(Hq):
        o1, l1 = OA.dense_attention(q[:, :, h:h + 1], k[:, :, h // 2:h // 2 + 1],
                                    v[:, :, h // 2:h // 2 + 1], mask, None, seq_dim=1)
        torch.testing.assert_close(out[:, :, h:h + 1], o1, atol=1e-6, rtol=1e-6)
        torch.testing.assert_close(lse[:, h:h + 1], l1, atol=1e-6, rtol=1e-6)


def test_default_scale_is_inverse_sqrt_head_dim():
    q, k, v = _rand((1, 5, 2, 32), 8), _rand((1, 5, 2, 32), 9), _rand((1, 5, 2, 32), 10)
    mask = torch.ones(5, 5, dtype=torch.bool)
    a, la = OA.dense_attention(q, k, v, mask, None)
    b, lb = OA.dense_attention(q, k, v, mask, 1.0 / math.sqrt(32))
    assert torch.equal(a, b) and torch.equal(la, lb)


def test_fully_masked_rows_give_zero_and_minus_inf():
    B, H, Lq, Lk, D = 1, 2, 6, 7, 8
    q, k, v = _rand((B, Lq, H, D), 11), _rand((B, Lk, H, D), 12), _rand((B, Lk, H, D), 13)
    mask = _random_mask(B, H, Lq, Lk, 14)
    mask[:, 0, 2] = False
    mask[:, 1, 5] = False
    out, lse = OA.dense_attention(q, k, v, mask, 0.5)
    assert torch.equal(out[:, 2, 0], torch.zeros(B, D))
    assert torch.equal(out[:, 5, 1], torch.zeros(B, D))
    assert torch.isneginf(lse[:, 0, 2]).all() and torch.isneginf(lse[:, 1, 5]).all()
    assert torch.isfinite(out).all()
    fin = torch.ones(B, H, Lq, dtype=torch.bool)
    fin[:, 0, 2] = fin[:, 1, 5] = False
    assert torch.isfinite(lse[fin]).all()


def test_single_key_rows_return_that_value():
    # a row that sees exactly one key returns its v and lse = the logit
    B, H, L, D = 1, 1, 4, 8
    q, k, v = _rand((B, L, H, D), 15), _rand((B, L, H, D), 16), _rand((B, L, H, D), 17)
    mask = torch.eye(L, dtype=torch.bool).roll(1, 1)       # row i sees key (i+1) % L
    out, lse = OA.dense_attention(q, k, v, mask, 0.25)
    for i in range(L):
        j = (i + 1) % L
        torch.testing.assert_close(out[0, i, 0], v[0, j, 0], atol=1e-6, rtol=1e-6)
        torch.testing.assert_close(lse[0, 0, i], (q[0, i, 0] * k[0, j, 0]).sum() * 0.25,
                                   atol=1e-5, rtol=1e-5)


def test_gradients_match_finite_differences_and_sdpa():
    B, Lq, Lk, Hq, Hkv, D = 1, 5, 7, 4, 2, 4
    mask = _random_mask(B, Hq, Lq, Lk, 18)
    q = _rand((B, Lq, Hq, D), 19).double().requires_grad_()
    k = _rand((B, Lk, Hkv, D), 20).double().requires_grad_()
    v = _rand((B, Lk, Hkv, D), 21).double().requires_grad_()

    # the oracle computes in fp32, too coarse for finite differences: float64
    # SDPA (+ logsumexp) is checked against finite differences, and the oracle's
    # fp32 autograd gradients (through O and through LSE) against float64
    # autograd of that function.
    def sdpa64(q, k, v):
        tq, tk, tv = (x.transpose(1, 2) for x in (q, k, v))
        tk, tv = tk.repeat_interleave(2, 1), tv.repeat_interleave(2, 1)
        o = F.scaled_dot_product_attention(tq, tk, tv, attn_mask=mask, scale=0.6)
        logits = torch.matmul(tq, tk.transpose(-1, -2)) * 0.6
        logits = logits.masked_fill(~mask, float("-inf"))
        return o.transpose(1, 2), torch.logsumexp(logits, -1)

    assert torch.autograd.gradcheck(sdpa64, (q, k, v), eps=1e-6, atol=1e-5, rtol=1e-4)

    do = _rand((B, Lq, Hq, D), 22)
    dlse = _rand((B, Hq, Lq), 23)
    o64, l64 = sdpa64(q, k, v)
    want = torch.autograd.grad((o64 * do.double()).sum() + (l64 * dlse.double()).sum(), (q, k, v))

    q32, k32, v32 = (x.detach().float().requires_grad_() for x in (q, k, v))
    o32, l32 = OA.dense_attention(q32, k32, v32, mask, 0.6)
    got = torch.autograd.grad((o32 * do).sum() + (l32 * dlse).sum(), (q32, k32, v32))
    for name, g, w in zip("qkv", got, want):
        torch.testing.assert_close(g.double(), w, atol=2e-5, rtol=1e-4, msg=lambda m: f"d{name}: {m}")


def test_gradients_with_fully_masked_row_are_finite_and_zero_there():
    B, L, H, D = 1, 6, 2, 4
    mask = _random_mask(B, H, L, L, 24)
    mask[:, 1, 3] = False
    q, k, v = (_rand((B, L, H, D), s).requires_grad_() for s in (25, 26, 27))
    out, _ = OA.dense_attention(q, k, v, mask, 0.5)
    dq, dk, dv = torch.autograd.grad(out.sum(), (q, k, v))
    assert all(torch.isfinite(g).all() for g in (dq, dk, dv))
    assert torch.equal(dq[:, 3, 1], torch.zeros(B, D))


@pytest.mark.parametrize("bs,q_len,k_len", [
    (16, 64, 64),     # square, whole blocks
    (16, 1, 50),      # decode row, ragged k_len
    (16, 20, 57),     # chunk with past > 0 starting inside a block
    (8, 33, 33),      # ragged square
    (32, 7, 64),
])
def test_sequence_token_mask_is_kron_and_tril(bs, q_len, k_len):
    H, nb = 3, 8
    rng = np.random.default_rng(bs * 1000 + q_len)
    bm = np.tril(rng.random((H, nb, nb)) < 0.5).astype(np.uint8)
    bm[:, np.arange(nb), np.arange(nb)] = 1
    got = OA.sequence_token_mask(bm, bs, q_len, k_len, causal=True)

    # the reference checker's construction: kron with a block of ones, token
    # tril, keep the k_len x k_len corner, then the last q_len rows
    full = torch.kron(torch.from_numpy(bm).float(), torch.ones(bs, bs))
    full = full[:, :k_len, :k_len] * torch.ones(k_len, k_len).tril()
    want = full[:, k_len - q_len:, :].bool().numpy()
    assert got.shape == (H, q_len, k_len) and got.dtype == np.bool_
    assert np.array_equal(got, want)


def test_sequence_token_mask_non_causal():
    H, nb, bs = 2, 4, 16
    rng = np.random.default_rng(7)
    bm = (rng.random((H, nb, nb)) < 0.5).astype(np.uint8)
    got = OA.sequence_token_mask(bm, bs, 50, 61, causal=False)
    want = np.kron(bm, np.ones((bs, bs), dtype=np.uint8))[:, :50, :61] != 0
    assert np.array_equal(got, want)


def test_token_mask_agrees_with_layout_dense_mask():
    # the layout oracle's dense mask (pinned by the reference's fixtures) and
    # the token mask of a full-length sequence are the same object
    H, bs, L = 4, 16, 128
    bm = OL.block_mask(H, L, block_size=bs, local_blocks=2, vert_stride=3, homo_head=False)
    for q_len in (L, 37, 1):
        dense = OL.token_mask(bm, bs, L, past_len=L - q_len)
        got = OA.sequence_token_mask(bm, bs, q_len, L, causal=True)
        assert np.array_equal(got, dense != 0)


def test_combine_partitions_closed_form():
    # dkernel/interface.py:319-324: weights = softmax over partitions of lse
    shape = (2, 3, 11)
    o = [_rand(shape + (8,), 30 + i) for i in range(3)]
    l = [_rand(shape, 40 + i) * 3 for i in range(3)]
    got = OA.combine_partitions(list(zip(o, l)))
    w = torch.stack(l).softmax(0)
    want = (torch.stack(o) * w.unsqueeze(-1)).sum(0)
    torch.testing.assert_close(got, want, atol=1e-6, rtol=1e-6)


def test_combine_partitions_minus_inf_gets_weight_zero():
    shape = (1, 2, 5)
    oa, ob = _rand(shape + (4,), 50), _rand(shape + (4,), 51)
    la, lb = _rand(shape, 52), _rand(shape, 53)
    lb[0, 0, 1] = float("-inf")
    la[0, 1, 2] = float("-inf")
    lb[0, 1, 2] = float("-inf")
    got = OA.combine_partitions([(oa, la), (ob, lb)])
    assert torch.isfinite(got).all()
    torch.testing.assert_close(got[0, 0, 1], oa[0, 0, 1])
    assert torch.equal(got[0, 1, 2], torch.zeros(4))


@pytest.mark.parametrize("cut", [0, 16, 23, 48])
def test_combine_of_kv_partitions_equals_unpartitioned(cut):
    # tests/test_seq_partition.py:178 -- attention over KV chunks merged by LSE
    B, H, L, D = 2, 3, 48, 8
    q, k, v = _rand((B, H, L, D), 60), _rand((B, H, L, D), 61), _rand((B, H, L, D), 62)
    mask = _random_mask(B, H, L, L, 63, p=0.4).tril()
    mask[..., torch.arange(L), torch.arange(L)] = True
    full, lse_full = OA.dense_attention(q, k, v, mask, None, seq_dim=2)
    parts = []
    for lo, hi in ((0, cut), (cut, L)):
        if hi == lo:
            parts.append((torch.zeros_like(full), torch.full_like(lse_full, float("-inf"))))
            continue
        parts.append(OA.dense_attention(q, k[:, :, lo:hi], v[:, :, lo:hi], mask[..., lo:hi], None, seq_dim=2))
    got = OA.combine_partitions(parts)
    torch.testing.assert_close(got, full, atol=2e-6, rtol=1e-5)
    merged_lse = torch.logsumexp(torch.stack([p[1] for p in parts]), 0)
    torch.testing.assert_close(merged_lse, lse_full, atol=2e-6, rtol=1e-6)


@pytest.mark.parametrize("seq_dim", [1, 2])
def test_reference_style_attention_is_dense_attention(seq_dim):
    B, H, L, D = 2, 3, 40, 16
    shape = (B, L, H, D) if seq_dim == 1 else (B, H, L, D)
    q, k, v = _rand(shape, 70), _rand(shape, 71), _rand(shape, 72)
    mask = torch.ones(L, L, dtype=torch.bool).tril()[None, None].expand(B, H, L, L)
    scale = 1 / math.sqrt(D)
    got = OA.reference_style_attention(q, k, v, mask, scale, seq_dim=seq_dim)
    want, _ = OA.dense_attention(q, k, v, mask, scale, seq_dim=seq_dim)
    torch.testing.assert_close(got, want, atol=2e-6, rtol=1e-5)
    # in bf16 (the reference's test dtype) within its own tolerance
    gb = OA.reference_style_attention(q.bfloat16(), k.bfloat16(), v.bfloat16(), mask, scale, seq_dim=seq_dim)
    wb, _ = OA.dense_attention(q.bfloat16(), k.bfloat16(), v.bfloat16(), mask, scale, seq_dim=seq_dim)
    torch.testing.assert_close(gb.float(), wb, atol=1e-2, rtol=1e-2)


def test_blockwise_reference_branch_equals_token_mask_path():
    # the reference's block_attn_mask branch (tests/test_sparse_attn.py:508-523)
    # restated from the block mask alone must equal dense attention under
    # sequence_token_mask: per q block, keys [0, e), kron mask, token tril
    B, H, bs, nb, D = 1, 2, 8, 6, 8
    L = bs * nb
    rng = np.random.default_rng(3)
    bm = np.tril(rng.random((H, nb, nb)) < 0.5).astype(np.float32)
    bm[:, np.arange(nb), np.arange(nb)] = 1
    q, k, v = _rand((B, H, L, D), 80), _rand((B, H, L, D), 81), _rand((B, H, L, D), 82)
    outs = []
    for s in range(0, L, bs):
        e = s + bs
        attn = torch.einsum("bhmd,bhnd->bhmn", q[:, :, s:e], k[:, :, :e]) * 0.3
        m = torch.kron(torch.from_numpy(bm[:, s // bs:s // bs + 1, :s // bs + 1]), torch.ones(1, bs, bs))
        m[:, :, s:] *= torch.ones(bs, bs).tril()
        attn = attn.masked_fill(~(m[None] != 0), float("-inf")).softmax(-1)
        outs.append(torch.einsum("bhmn,bhnd->bhmd", attn, v[:, :, :e]))
    want = torch.cat(outs, 2)
    tok = OA.sequence_token_mask(bm, bs, L, L, causal=True)
    got, _ = OA.dense_attention(q, k, v, torch.from_numpy(tok), 0.3, seq_dim=2)
    torch.testing.assert_close(got, want, atol=2e-6, rtol=1e-5)
