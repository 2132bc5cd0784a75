"""Oracle (test infrastructure, never shipped): dense masked softmax attention
in fp32 on the CPU, its log-sum-exp, gradients (torch autograd through the
same function) and the LSE merge of KV partitions.

Follows the reference's own checker, tests/test_sparse_attn.py:486-537
(einsum QK^T -> fp32 * sm_scale -> masked_fill(-inf) with the token mask ->
softmax -> einsum PV), upcasting inputs to fp32 first so that the result is
the exact-arithmetic target the bf16 kernels are held to.

Pinning (tests/test_oracle_attention.py): softmax attention is the textbook
definition, so the checks are library identities rather than a retyped
formula -- torch.nn.functional.scaled_dot_product_attention with a boolean
mask on the same inputs, torch.logsumexp of the masked logits, the
partition invariant combine(A, B) == unpartitioned of
tests/test_seq_partition.py:178, and finite differences for the gradients.
GQA results (kv head = q head // group) and LSE from padded / packed inputs
have no counterpart in the reference's tests: parity for those rests on
this dense definition only.
"""
from __future__ import annotations

import math

import numpy as np
import torch


def _to_bhld(x, seq_dim):
    return x.transpose(1, 2) if seq_dim == 1 else x


def dense_attention(q, k, v, mask, sm_scale=None, seq_dim=1):
    """q (B, Lq, Hq, D) [seq_dim=1] or (B, Hq, Lq, D) [seq_dim=2]; k, v with
    Hkv heads (Hq % Hkv == 0, kv head = q head // (Hq // Hkv)); mask
    broadcastable to (B, Hq, Lq, Lk), non-zero = attend.

    Returns (out fp32 in q's layout, lse fp32 (B, Hq, Lq), natural log).  Rows
    with no allowed key give out = 0 and lse = -inf.
    """
    q, k, v = (_to_bhld(x.float(), seq_dim) for x in (q, k, v))
    B, Hq, Lq, D = q.shape
    Hkv = k.shape[1]
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    if Hkv != Hq:
        k = k.repeat_interleave(Hq // Hkv, dim=1)
        v = v.repeat_interleave(Hq // Hkv, dim=1)
    mask = torch.as_tensor(np.asarray(mask) if not torch.is_tensor(mask) else mask)
    while mask.dim() < 4:
        mask = mask[None]
    mask = (mask != 0).expand(B, Hq, Lq, k.shape[2])
    outs, lses = [], []
    for h in range(Hq):                       # one head at a time bounds memory
        s = torch.einsum("bmd,bnd->bmn", q[:, h], k[:, h]) * sm_scale
        s = s.masked_fill(~mask[:, h], float("-inf"))
        lse = torch.logsumexp(s, dim=-1)
        p = torch.exp(s - torch.where(torch.isinf(lse), torch.zeros_like(lse), lse)[..., None])
        p = torch.where(torch.isinf(lse)[..., None], torch.zeros_like(p), p)
        outs.append(torch.einsum("bmn,bnd->bmd", p, v[:, h]))
        lses.append(lse)
    out = torch.stack(outs, dim=1)
    lse = torch.stack(lses, dim=1)
    return _to_bhld(out, seq_dim) if seq_dim == 1 else out, lse


def reference_style_attention(q, k, v, mask, sm_scale, seq_dim=1):
    """The reference checker's arithmetic as written (einsum in the input
    dtype, fp32 scale + softmax, probabilities cast back to v's dtype);
    tests/test_sparse_attn.py:525-537.  MHA only, fully masked rows give NaN
    exactly as there.  Used as the timed CPU baseline."""
    if seq_dim == 1:
        q, k, v = (x.transpose(1, 2) for x in (q, k, v))
    attn = torch.einsum("bhmd,bhnd->bhmn", q, k).float() * sm_scale
    attn = attn.masked_fill(~(mask != 0), float("-inf"))
    attn = attn.softmax(-1)
    out = torch.einsum("bhmn,bhnd->bhmd", attn.type_as(v), v)
    return out.transpose(1, 2) if seq_dim == 1 else out


def combine_partitions(parts):
    """[(out_p, lse_p)] -> merged out.  out_p (..., L, D) with lse_p (..., L);
    dkernel/interface.py:319-324.  -inf partitions get weight 0."""
    outs = torch.stack([o.float() for o, _ in parts])
    lses = torch.stack([l.float() for _, l in parts])
    mx = lses.max(0).values
    mx = torch.where(torch.isinf(mx), torch.zeros_like(mx), mx)
    w = torch.exp(lses - mx)
    den = w.sum(0)
    w = torch.where(den > 0, w / den.clamp_min(1e-38), torch.zeros_like(w))
    return (outs * w[..., None]).sum(0)


def sequence_token_mask(block_mask_full, block_size, q_len, k_len, causal=True):
    """Token mask (H, q_len, k_len) of one sequence whose q_len query tokens are
    the LAST q_len positions of its k_len keys, positions counted from the
    sequence's first real token (the reference's padding semantics,
    tests/test_sparse_attn.py:333-339 and dkernel/ops/sparse_attn_inference.py:503-514).
    block_mask_full is the untrimmed (H, nb, nb) block mask."""
    bm = np.asarray(block_mask_full)
    past = k_len - q_len if causal else 0
    rows = np.arange(past, past + q_len)
    cols = np.arange(k_len)
    m = bm[:, rows[:, None] // block_size, cols[None, :] // block_size] != 0
    if causal:
        m = m & (rows[:, None] >= cols[None, :])[None]
    return m
