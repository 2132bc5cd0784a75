"""Oracle (test infrastructure, never shipped): numpy restatement of the
reference's host-side layout code, dkernel/utils.py.

Each function cites the reference lines it follows.  Pinning, i.e. what fixes
the result independently of the formulae typed here (checked in
tests/test_oracle_layout.py):

* block_mask          -- the two literal 8x8 masks of the reference's own
                         tests/test_utils.py:24-34 and :55-64; invariants
                         (vert_stride=1 => dense causal, GQA groups share a
                         pattern, dense heads are the last kv heads, row chunks
                         of partition masks concatenate to the full mask as in
                         tests/test_seq_partition.py:161-169); golden fixtures
                         tests/golden/lut_*.npz.
* csr_from_dense      -- scipy.sparse.csr_matrix indptr/indices + "right pad
                         with -1"; brute force; golden fixtures.
* merge_split_blocks  -- brute-force reconstruction of the token mask on tiny
                         inputs; golden fixtures (value column, pad width).
* kv_cache_efficient  -- brute force over all row pairs on tiny inputs.
"""
from __future__ import annotations

import numpy as np


def cdiv(a: int, b: int) -> int:
    return -(-a // b)


def block_mask(num_heads, seqlen, block_size=64, local_blocks=4, vert_stride=4,
               homo_head=False, num_kv_heads=None, past_len=None,
               head_sliding_step=None, head_sliding_offset=0, num_dense_heads=0,
               kv_seqlen=None, q_start_position=None, kv_start_position=None,
               vert_position_type=None, causal=True):
    """Block mask of the local + vertical-stride pattern, uint8 (H or 1, nbq, nbk),
    rows before ceil(past_len / block_size) trimmed.  dkernel/utils.py:143-220.
    """
    past_len = past_len or 0
    kv_seqlen = kv_seqlen or seqlen
    if homo_head:                                   # utils.py:147-150
        num_heads = 1
        assert num_dense_heads == 0
    if vert_position_type is None:                  # utils.py:152-155
        vert_position_type = "absolute" if causal else "relative"
    assert vert_position_type in ("absolute", "relative")
    num_kv_heads = num_kv_heads or num_heads        # utils.py:157-159
    num_sparse = num_kv_heads - num_dense_heads
    q_per_kv = num_heads // num_kv_heads
    q_start_block = kv_start_block = 0              # utils.py:161-169
    if q_start_position is not None:
        assert q_start_position % block_size == 0
        assert past_len == 0
        q_start_block = q_start_position // block_size
    if kv_start_position is not None:
        assert kv_start_position % block_size == 0
        kv_start_block = kv_start_position // block_size
    if causal:                                      # utils.py:171-180
        assert local_blocks >= 1
        left, right = local_blocks, 1
    elif isinstance(local_blocks, int):
        assert local_blocks >= 0
        left = right = local_blocks
    else:
        left, right = local_blocks
        assert left > 0 and right > 0

    nbq, nbk = cdiv(seqlen, block_size), cdiv(kv_seqlen, block_size)
    q_pos = (q_start_block + np.arange(nbq))[:, None]
    k_pos = (kv_start_block + np.arange(nbk))[None, :]
    if head_sliding_step is None:                   # utils.py:187-188
        head_sliding_step = max(1, int(vert_stride / num_heads))

    heads = [h for h in range(num_kv_heads) for _ in range(q_per_kv)]
    if vert_position_type == "absolute":            # utils.py:189-196
        local = ((q_pos - k_pos) < left) & ((k_pos - q_pos) < right)
        out = np.empty((len(heads), nbq, nbk), dtype=bool)
        for i, h in enumerate(heads):
            if h < num_sparse:
                vert = (k_pos + h * head_sliding_step + head_sliding_offset) % vert_stride == 0
            else:
                vert = np.ones_like(k_pos, dtype=bool)
            out[i] = vert | local
    else:                                           # utils.py:197-211
        lm = (q_pos - k_pos) - left + 1
        lm = lm * (lm > 0)
        rm = (k_pos - q_pos) - right + 1
        rm = rm * (rm > 0)
        rel = (lm + rm) % vert_stride == 0
        if num_sparse == num_kv_heads:
            out = rel[None]
        elif num_sparse == 0:
            out = np.ones_like(rel)[None]
        else:
            # utils.py:208-211 vstacks 2-D masks, which cannot broadcast against
            # (1, nbq, nbk) afterwards; the evident intent is one mask per head.
            out = np.stack([rel if h < num_sparse else np.ones_like(rel) for h in heads])
    if causal:                                      # utils.py:213-215
        out = out & (q_pos >= k_pos)[None]
    out = out.astype(np.uint8)
    return out[:, cdiv(past_len, block_size):]      # utils.py:219-220


def token_mask(blk_mask, block_size, seqlen, kv_seqlen=None, past_len=0, causal=True):
    """Token-level dense mask from an *untrimmed* block mask.  utils.py:222-227."""
    kv_seqlen = kv_seqlen or seqlen
    dense = np.kron(blk_mask, np.ones((block_size, block_size), dtype=blk_mask.dtype))
    dense = dense[..., :seqlen, :kv_seqlen]
    if causal:
        tril = np.tril(np.ones((seqlen, kv_seqlen), dtype=blk_mask.dtype))[past_len:]
        dense = dense[..., past_len:, :] * tril[None]
    return dense


def csr_from_dense(x, include_values=False, pad=-1):
    """CSR (crow, col) per head, col right-padded with -1 to the max nnz over
    heads; with include_values col becomes (H, nnz, 2) = [col, value], value
    padded with 0.  dkernel/utils.py:19-24 and :27-65."""
    x = np.asarray(x)
    squeeze = x.ndim == 2
    if squeeze:
        x = x[None]
    assert x.ndim == 3
    crows, cols, vals = [], [], []
    for xi in x:
        nz = xi != 0
        crows.append(np.concatenate([[0], np.cumsum(nz.sum(-1))]).astype(np.int32))
        r, c = np.nonzero(nz)                       # row-major order: ascending col within a row
        cols.append(c.astype(np.int32))
        vals.append(xi[nz].astype(np.int32))
    width = max(len(c) for c in cols)
    col = np.full((len(cols), width), pad, dtype=np.int32)
    val = np.zeros((len(cols), width), dtype=np.int32)
    for i, (c, v) in enumerate(zip(cols, vals)):
        col[i, :len(c)] = c
        val[i, :len(v)] = v
    crow = np.stack(crows)
    if include_values:
        col = np.stack([col, val], axis=-1)
    if squeeze:
        crow, col = crow[0], col[0]
    return crow, col


def csc_from_dense(x, **kw):
    """CSC = CSR of the transpose.  dkernel/utils.py:91-95."""
    return csr_from_dense(np.swapaxes(np.asarray(x), -2, -1), **kw)


def merge_split_blocks(block_size, pattern, block_m, block_n):
    """LUT at kernel-tile granularity.  dkernel/utils.py:262-310.

    identity when block_m == block_n == block_size; split (kron + drop of
    sub-blocks strictly above the token diagonal) when a kernel tile is
    smaller than the sparse block; merge of block_m // block_size row blocks,
    recording micro_M = (index of last non-empty sub-row + 1) * block_size.
    """
    pattern = np.asarray(pattern)
    if block_size == block_m and block_size == block_n:
        return csr_from_dense(pattern)
    assert (block_m % block_size == 0) or (block_size % block_n == 0)
    assert block_size % block_n == 0
    m_mult = block_size // block_m if block_size > block_m else 1
    kf = np.ones((m_mult, block_size // block_n), dtype=pattern.dtype)
    if kf.size > 1:                                 # utils.py:290-297
        bm, bn = block_size // kf.shape[0], block_size // kf.shape[1]
        pattern = np.kron(pattern, kf)
        keep = (np.arange(1, pattern.shape[1] + 1)[:, None] * bm
                > np.arange(0, pattern.shape[2])[None, :] * bn)
        pattern = pattern * keep.astype(pattern.dtype)
    if block_size < block_m:                        # utils.py:299-308
        H, M, N = pattern.shape
        mm = block_m // block_size
        assert M % mm == 0
        p = pattern.astype(np.int32).reshape(H, M // mm, mm, N)
        p = (np.cumsum(p[:, :, ::-1], axis=2) > 0).sum(2) * block_size
        return csr_from_dense(p, include_values=True)
    return csr_from_dense(pattern)


def kv_cache_efficient(pattern, block_m, block_n):
    """True when, strictly below the diagonal, no column switches 0 -> 1 going
    down the rows.  dkernel/utils.py:232-245."""
    p = np.asarray(pattern).astype(np.int8)
    non_diag = (np.arange(p.shape[1])[:, None] * block_m
                >= np.arange(1, p.shape[2] + 1)[None, :] * block_n)
    return bool((((p[:, 1:] - p[:, :-1]) <= 0) | ~non_diag[1:]).all())


def lut_to_block_mask(crow, col, ncols):
    """Inverse of csr_from_dense (entries only, values ignored).  Mirrors the
    purpose of dkernel/utils.py:68-88."""
    crow, col = np.asarray(crow), np.asarray(col)
    if crow.ndim == 1:
        crow, col = crow[None], col[None]
    if col.ndim == 3:
        col = col[..., 0]
    out = np.zeros((crow.shape[0], crow.shape[1] - 1, ncols), dtype=np.uint8)
    for h in range(crow.shape[0]):
        for r in range(crow.shape[1] - 1):
            out[h, r, col[h, crow[h, r]:crow[h, r + 1]]] = 1
    return out
