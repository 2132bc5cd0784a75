"""Host-side helpers for 2-D / 3-D block-sparse patterns, same names and
argument meaning as the reference's dkernel/utils.py.  The integer work (block
mask, CSR / CSC look-up tables, kernel-tile merge / split, KV-cache check) is
done by the C++ builder inside libdkernel_hip.so in one pass per table; these
functions only marshal torch tensors across the C ABI.  They run on the CPU
and need no GPU.
"""
from __future__ import annotations

import ctypes as C
from collections import namedtuple
from typing import Optional, Tuple, Union

import numpy as np
import torch
from torch import Tensor

from . import _lib

__all__ = [
    "get_sparse_attn_mask", "dense_to_crow_col", "dense_to_ccol_row", "crow_col_to_dense",
    "ccol_row_to_dense", "merge_split_fwd_kernel_blocks", "is_kv_cache_efficient",
    "verify_sparse_pattern", "is_causal", "zero_stride", "multiple_of", "get_q_block_ids", "cdiv",
    "to_csr", "is_hip", "split_tile_tables", "masked_tile_tables",
]


def cdiv(a: int, b: int) -> int:
    return -(-a // b)


def _ptr(t: Tensor):
    return C.c_void_p(t.data_ptr())


_CsrMatrix = namedtuple("csr_matrix", ("indptr", "indices", "data"))


def to_csr(mat: np.ndarray) -> _CsrMatrix:
    """CSR triple (indptr, indices, data) of one 2-D numpy matrix, int32
    indices.  Reference: dkernel/utils.py:19-24."""
    mat = np.asarray(mat)
    nz = mat != 0
    rows, cols = np.nonzero(nz)
    indptr = np.zeros(mat.shape[0] + 1, dtype=np.int32)
    np.cumsum(np.bincount(rows, minlength=mat.shape[0]), out=indptr[1:])
    return _CsrMatrix(indptr, cols.astype(np.int32), mat[nz])


def is_hip() -> bool:
    """The reference asks Triton for its backend (dkernel/utils.py:327-331) to
    pick tuning configurations; this build runs on ROCm only."""
    return True


def dense_to_crow_col(x: Tensor, include_values: bool = False) -> Tuple[Tensor, Tensor]:
    """2-D / 3-D tensor -> CSR (crow, col) int32 on x's device; col is
    right-padded with -1 to the largest nnz over heads, and carries the
    non-zero values on a trailing dim of 2 when include_values.
    Reference: dkernel/utils.py:27-65."""
    assert x.dim() in (2, 3)
    device = x.device
    squeeze = x.dim() == 2
    pat = (x[None] if squeeze else x).to("cpu", torch.int32)
    H, M, N = pat.shape
    lib = _lib.lib()
    crow = torch.empty((H, M + 1), dtype=torch.int32)
    width = C.c_int32(0)
    sh, sm, sn = pat.stride()
    _lib.check(lib.dk_csr_count(_ptr(pat), H, M, N, sh, sm, sn, _ptr(crow), C.byref(width)))
    w = width.value
    col = torch.empty((H, w), dtype=torch.int32)
    val = torch.empty((H, w), dtype=torch.int32) if include_values else None
    _lib.check(lib.dk_csr_fill(_ptr(pat), H, M, N, sh, sm, sn, w, _ptr(col),
                               _ptr(val) if include_values else None))
    if include_values:
        col = torch.stack([col, val], dim=-1)
    if squeeze:
        crow, col = crow[0], col[0]
    return crow.to(device), col.to(device)


def dense_to_ccol_row(x: Tensor, **kwargs) -> Tuple[Tensor, Tensor]:
    """CSC = CSR of the transpose (strides swapped, no copy).
    Reference: dkernel/utils.py:91-95."""
    return dense_to_crow_col(x.transpose(-2, -1), **kwargs)


def crow_col_to_dense(crows: Tensor, cols: Tensor, dtype: torch.dtype = torch.float16) -> Tensor:
    """Inverse of dense_to_crow_col.  Reference: dkernel/utils.py:68-88."""
    dim = crows.dim()
    if dim == 1:
        crows, cols = crows[None], cols[None]
    device = crows.device
    crows, cols = crows.cpu(), cols.cpu()
    shape = (crows.shape[0], crows.shape[1] - 1, int(cols.max()) + 1)
    x = torch.zeros(shape, dtype=dtype)
    for i in range(shape[0]):
        for j in range(shape[1]):
            s, e = int(crows[i, j]), int(crows[i, j + 1])
            if cols.dim() == 2:
                x[i, j, cols[i, s:e].long()] = 1
            else:
                x[i, j, cols[i, s:e, 0].long()] = cols[i, s:e, 1].to(dtype)
    if dim == 1:
        x = x[0]
    return x.to(device)


def ccol_row_to_dense(ccol: Tensor, rows: Tensor, dtype: torch.dtype = torch.float16) -> Tensor:
    return crow_col_to_dense(ccol, rows, dtype).permute(0, 2, 1).contiguous()


def get_sparse_attn_mask(num_heads: int,
                         seqlen: int,
                         block_size: int = 64,
                         local_blocks: Union[int, Tuple[int, int]] = 4,
                         vert_stride: int = 4,
                         homo_head=False,
                         num_kv_heads=None,
                         past_len=None,
                         dtype=torch.bfloat16,
                         device=None,
                         return_dense=False,
                         head_sliding_step=None,
                         head_sliding_offset=0,
                         num_dense_heads=0,
                         kv_seqlen: int = None,
                         q_start_position=None,
                         kv_start_position=None,
                         vert_position_type=None,
                         causal=True):
    """Block mask of the local + vertical-stride pattern; returns
    ((crow, col), block_mask, dense_token_mask or None) like the reference
    (dkernel/utils.py:105-229): results live on the current ROCm device when
    there is one, else on the CPU (the `device` argument is ignored there too).
    """
    device = torch.cuda.current_device() if torch.cuda.is_available() else "cpu"
    past_len = past_len or 0
    kv_seqlen = kv_seqlen or seqlen
    if homo_head:
        num_heads = 1
        assert num_dense_heads == 0, "Cannot have dense head if stride pattern for heads is homogeneous."
    if vert_position_type is None:
        vert_position_type = "absolute" if causal else "relative"
    else:
        assert vert_position_type in ("absolute", "relative")
    # With one shared pattern the kv-head grouping has no effect on the mask.
    num_kv_heads = (num_kv_heads or num_heads) if not homo_head else 1
    assert num_heads % num_kv_heads == 0, f"{num_heads=} must be a multiple of {num_kv_heads=}"

    q_start_block = kv_start_block = 0
    if q_start_position is not None:
        assert q_start_position % block_size == 0, "Sequence chunking must be at the block boundary"
        q_start_block = q_start_position // block_size
        assert past_len in [0, None], "Cannot specify both past_len and q_start_position"
    if kv_start_position is not None:
        assert kv_start_position % block_size == 0, "Sequence chunking must be at the block boundary"
        kv_start_block = kv_start_position // block_size

    if causal:
        assert local_blocks >= 1
        local = (local_blocks, 1)
    elif isinstance(local_blocks, int):
        assert local_blocks >= 0
        local = (local_blocks, local_blocks)
    else:
        assert isinstance(local_blocks, tuple) and len(local_blocks) == 2
        assert all(x > 0 for x in local_blocks)
        local = local_blocks

    nb_q, nb_k = cdiv(seqlen, block_size), cdiv(kv_seqlen, block_size)
    if head_sliding_step is None:
        head_sliding_step = max(1, int(vert_stride / num_heads))
    relative = vert_position_type == "relative"
    # relative positions with every kv head sparse (or every one dense) share one pattern
    n_out = num_heads
    if relative and num_dense_heads in (0, num_kv_heads):
        n_out, kvh, dense = 1, 1, (1 if num_dense_heads == num_kv_heads and num_dense_heads > 0 else 0)
    else:
        kvh, dense = num_kv_heads, num_dense_heads
    mask = torch.empty((n_out, nb_q, nb_k), dtype=torch.uint8)
    _lib.check(_lib.lib().dk_local_stride_mask(
        n_out, kvh, nb_q, nb_k, local[0], local[1], vert_stride, dense, head_sliding_step,
        head_sliding_offset, q_start_block, kv_start_block, int(bool(causal)), int(relative), _ptr(mask)))

    block_mask = mask.to(dtype).to(device)
    trimmed = block_mask[:, cdiv(past_len, block_size):]
    mask_dense = None
    if return_dense:
        mask_dense = torch.kron(block_mask, block_mask.new_ones((block_size, block_size)))[..., :seqlen, :kv_seqlen]
        if causal:
            causal_mask = torch.tril(torch.ones(seqlen, kv_seqlen)).type_as(mask_dense)[past_len:]
            mask_dense = mask_dense[..., past_len:, :] * causal_mask[None].to(mask_dense.device)
    return dense_to_crow_col(trimmed), trimmed, mask_dense


def is_kv_cache_efficient(sparse_pattern: Tensor, block_m: int, block_n: int) -> bool:
    """A pattern is KV-cache friendly when the non-local KV used by later
    tokens is also used by earlier ones.  Reference: dkernel/utils.py:232-245."""
    p = (sparse_pattern != 0).to("cpu", torch.uint8).contiguous()
    if p.dim() == 2:
        p = p[None]
    H, M, N = p.shape
    rc = _lib.lib().dk_kv_cache_efficient(_ptr(p), H, M, N, block_m, block_n)
    if rc < 0:
        _lib.check(rc)
    return bool(rc)


def verify_sparse_pattern(sparse_pattern: Tensor) -> None:
    assert sparse_pattern.dim() in (2, 3)


def is_causal(sparse_pattern: Tensor) -> bool:
    sparse_pattern = sparse_pattern.to(torch.int8)
    assert sparse_pattern.size(-2) == sparse_pattern.size(-1)
    upper = sparse_pattern * (1 - torch.tril(torch.ones_like(sparse_pattern[0])))
    return not upper.any()


def _tile_pattern(block_size: int, sparse_pattern: Tensor, block_m: int, block_n: int,
                  causal: bool) -> Tuple[Tensor, bool]:
    """Block pattern re-expressed in block_m x block_n kernel tiles (int32, on
    the CPU) and whether rows were merged (entries then hold micro_M)."""
    assert (block_m % block_size == 0) or (block_size % block_n == 0), \
        "block_m must be mutliple or a factor of sparse block size for merging on Q blocks"
    assert block_size % block_n == 0, \
        "block_n must be a factor of sparse block size for splitting on K blocks"
    p = (sparse_pattern != 0).to("cpu", torch.uint8).contiguous()
    H, M, N = p.shape
    lib = _lib.lib()
    om, on, merged = C.c_int32(), C.c_int32(), C.c_int32()
    _lib.check(lib.dk_tile_pattern_shape(M, N, block_size, block_m, block_n,
                                         C.byref(om), C.byref(on), C.byref(merged)))
    out = torch.empty((H, om.value, on.value), dtype=torch.int32)
    _lib.check(lib.dk_tile_pattern(_ptr(p), H, M, N, block_size, block_m, block_n, int(bool(causal)), _ptr(out)))
    return out, bool(merged.value)


def merge_split_fwd_kernel_blocks(block_size: int, sparse_pattern: Tensor, block_m: int, block_n: int,
                                  causal: bool = True) -> Tuple[Tensor, Tensor]:
    """Look-up table at kernel-tile granularity (reference:
    dkernel/utils.py:262-310).  `causal=False` keeps the sub-blocks above the
    token diagonal, which the reference would drop even for bidirectional
    patterns."""
    if block_size == block_m and block_size == block_n:
        return dense_to_crow_col(sparse_pattern)
    out, merged = _tile_pattern(block_size, sparse_pattern, block_m, block_n, causal)
    return dense_to_crow_col(out.to(sparse_pattern.device), include_values=merged)


def tile_sizes_keep_pattern(block_size: int, sparse_pattern: Tensor, block_m: int, block_n: int,
                            causal: bool = True) -> bool:
    """Whether a table of block_m x block_n kernel tiles attends exactly the pattern's own
    blocks.  Splitting never changes what is attended; merging q rows does when a column is
    held only by a later pattern row of a merged tile, because every row of the tile up to
    the last holder then attends it (dkernel/utils.py:299-308).  Blocks entirely above the
    token diagonal do not count (the kernels mask them)."""
    out, merged = _tile_pattern(block_size, sparse_pattern, block_m, block_n, causal)
    if not merged:
        return True
    p = (sparse_pattern != 0).to("cpu")
    H, M, N = p.shape
    mm, split_n = block_m // block_size, block_size // block_n
    om, on = out.shape[1:]
    # rows s of merged tile i attend column j iff s * block_size < out[i, j]
    sub = torch.arange(mm)[None, None, :, None] * block_size
    eff = (out[:, :, None, :] > sub).reshape(H, om * mm, on)[:, :M]
    own = p.repeat_interleave(split_n, dim=2)[:, :, :on]
    rows = torch.arange(M)[:, None]
    cols = torch.arange(on)[None, :]
    visible = cols * block_n < (rows + 1) * block_size if causal else torch.ones(M, on, dtype=torch.bool)
    return bool(((eff == own) | ~visible[None]).all())


def merged_rows_pattern(block_size: int, sparse_pattern: Tensor, block_m: int, block_n: int,
                        causal: bool = True) -> Tensor:
    """The block pattern that a table of block_m x block_n kernel tiles attends, at the pattern's
    own granularity: with merged q rows (block_m > block_size) every pattern row of a merged tile
    up to the last one that holds a column attends that column (rows at or beyond micro_M are
    excluded, dkernel/utils.py:299-308; dkernel/ops/sparse_attn_fwd.py:113-134), so a column held
    only by a later row widens the rows before it.  Blocks entirely above the token diagonal stay
    out when causal.  Without merging this is the pattern itself."""
    p = (sparse_pattern != 0).to("cpu")
    out, merged = _tile_pattern(block_size, sparse_pattern, block_m, block_n, causal)
    if not merged:
        return p.to(torch.uint8)
    H, M, N = p.shape
    mm, split_n = block_m // block_size, block_size // block_n
    om, on = out.shape[1:]
    sub = torch.arange(mm)[None, None, :, None] * block_size
    eff = (out[:, :, None, :] > sub).reshape(H, om * mm, on)[:, :M]   # (H, M, column tiles)
    wide = eff[:, :, ::split_n][:, :, :N]                              # first column tile of each block
    if causal:
        wide = wide & (torch.arange(N)[None, :] <= torch.arange(M)[:, None])[None]
    return wide.to(torch.uint8)


def split_tile_tables(block_size: int, sparse_pattern: Tensor, tile: int,
                      causal: bool = True) -> Tuple[Tuple[Tensor, Tensor], Tuple[Tensor, Tensor]]:
    """CSR and CSC tables of a pattern whose blocks are split into tile x tile
    kernel tiles (tile divides block_size).  With `causal`, tiles that lie
    entirely above the token diagonal are dropped, as in
    `merge_split_fwd_kernel_blocks`.  The reference has no counterpart: its
    dK/dV pass always walks columns of block_size (dkernel/interface.py:134)."""
    assert block_size % tile == 0 and block_size > tile
    out, merged = _tile_pattern(block_size, sparse_pattern, tile, tile, causal)
    assert not merged
    out = out.to(sparse_pattern.device)
    return dense_to_crow_col(out), dense_to_ccol_row(out)


def masked_tile_tables(block_size: int, sparse_pattern: Tensor, tile: int
                       ) -> Tuple[Tuple[Tensor, Tensor], Tuple[Tensor, Tensor]]:
    """CSR and CSC tables of a pattern whose blocks are smaller than the kernel
    tile: one entry per tile x tile tile that holds any active block, with a
    bit mask over the f x f pattern blocks inside it on the trailing dim
    (bit i * f + j: row part i, column part j; f = tile // block_size).  The
    pattern is zero-padded to whole tiles.  The reference has no counterpart
    (its kernels take tiles of the block size)."""
    assert tile % block_size == 0 and tile > block_size
    f = tile // block_size
    assert f * f <= 16
    p = (sparse_pattern != 0).to("cpu", torch.int32)
    H, M, N = p.shape
    Mp, Np = cdiv(M, f) * f, cdiv(N, f) * f
    padded = torch.zeros((H, Mp, Np), dtype=torch.int32)
    padded[:, :M, :N] = p
    weight = (1 << (torch.arange(f)[:, None] * f + torch.arange(f)[None, :])).to(torch.int32)
    bits = (padded.view(H, Mp // f, f, Np // f, f) * weight[None, None, :, None, :]).sum(dim=(2, 4)).to(torch.int32)
    bits = bits.to(sparse_pattern.device)
    return dense_to_crow_col(bits, include_values=True), dense_to_ccol_row(bits, include_values=True)


def zero_stride(x: Tensor, dim=0) -> Tensor:
    """Stride 0 on a broadcastable dim of size <= 1.  Reference: dkernel/utils.py:313-320."""
    assert x.size(dim) <= 1, f"Cannot set stride at {dim=} to 0 as the size is {x.size(dim)}."
    strides = list(x.stride())
    strides[dim] = 0
    return x.as_strided(x.shape, tuple(strides))


def multiple_of(x: int, y: int) -> int:
    return ((x + y - 1) // y) * y


def get_q_block_ids(past_len, q_len, block_size):
    return range(past_len // block_size, cdiv(past_len + q_len, block_size))
