"""Module API: `SparseAttention`, `LocalStrideSparseAttention` and
`combine_attn_partitions`, with the constructor / forward signatures, buffer
names, defaults and error behaviour of the reference's dkernel/interface.py, so
that a model written against `dkernel` runs unchanged.
"""
from __future__ import annotations

import copy
import math
import warnings
from functools import lru_cache
from typing import Optional, Tuple

import torch
from torch import Tensor

from . import _lib, ops
from .ops import _sparse_attention
from .utils import (dense_to_ccol_row, dense_to_crow_col, get_sparse_attn_mask, is_kv_cache_efficient,
                    masked_tile_tables, merge_split_fwd_kernel_blocks, multiple_of, split_tile_tables,
                    merged_rows_pattern, tile_sizes_keep_pattern,
                    verify_sparse_pattern, zero_stride)

_KERNEL_TILE = 64  # q and k tile of the matrix-core kernels


class _NoGradContext:
    """Stands in for the autograd context when no input requires grad."""

    def save_for_backward(self, *tensors):
        pass


def _identical_head_run(pattern: Tensor) -> int:
    """Largest g dividing the number of pattern heads such that every run of g
    consecutive heads holds one and the same pattern."""
    H = pattern.size(0)
    p = pattern.cpu()
    for g in (8, 4, 2):
        if H % g == 0 and H >= g:
            grouped = p.reshape(H // g, g, *p.shape[1:])
            if bool((grouped == grouped[:, :1]).all()):
                return g
    return 1


def _uneven_heads(pattern: Tensor) -> bool:
    """True when some head of the pattern holds clearly more blocks than the average head (a
    fifth more: below that, keeping each head on its own workgroup queues shares more tiles
    through the caches than spreading the heads would gain)."""
    if pattern.size(0) < 2 or pattern.stride(0) == 0:
        return False
    counts = pattern.reshape(pattern.size(0), -1).sum(1, dtype=torch.int64).cpu()
    return bool(counts.max() * counts.numel() > 1.2 * counts.sum())


def _unsorted_rows(pattern: Tensor) -> bool:
    """True when some row of some head holds clearly more blocks (a quarter more, and at least
    two) than every row after it: starting from the last row is then not longest first."""
    lens = pattern.sum(2, dtype=torch.int64).cpu()
    if lens.size(1) < 2:
        return False
    later = torch.flip(torch.cummax(torch.flip(lens, (1,)), dim=1).values, (1,))[:, 1:]  # longest later row
    return bool((4 * lens[:, :-1] > 5 * later + 8).any())


class SparseAttention(torch.nn.Module):
    """Block-sparse attention over a user-given block pattern.

    Arguments
    =========
    block_size: sparse block size, a power of 2, at least 16.
    sparse_pattern: 2-D or 3-D (per head) bool / uint8 tensor, 1 = attend.
    causal: default True.
    seq_dim: None / 1 -> (batch, seq, heads, dim); 2 -> (batch, heads, seq, dim).
        Ignored for packed variable-length (3-D) inputs.
    block_m, block_n: kernel tile sizes on q and k (powers of 2, >= 16).
        Default block_m = max(block_size, 64) if causal else block_size,
        block_n = block_size; the attributes and the `layout_*` buffers follow
        these values as in the reference.  The kernels themselves read extra
        tables built for their 64 x 64 tiles (`kernel_*`: larger blocks split;
        `masked_*`: smaller blocks as tiles with a bit mask; `exact_*`:
        unmerged tiles), which follow the pattern exactly.  When block_m is
        given and merging q rows widens the pattern (a later pattern row of a
        merged tile holds a column an earlier one lacks, and the reference's
        merged table lets the earlier rows attend it too), those tables are
        built from the widened pattern: the result is that of the merged table.
    kwargs: "out" (output tensor), "d_splits" (accepted, unused), "inference"
        (skip saving the log-sum-exp for backward; default: no input needs grad).

    forward(q, k, v, sm_scale=None, *, cu_seqlen_k, cu_seqlen_q, left_paddings,
            seqlens, return_lse, split_qkv): see the method.

    Reference: dkernel/interface.py:18-215.
    """

    def __init__(self,
                 block_size: int,
                 sparse_pattern: Tensor,
                 *,
                 causal: bool = True,
                 seq_dim: Optional[int] = None,
                 block_m: Optional[int] = None,
                 block_n: Optional[int] = None,
                 **kwargs):
        super().__init__()

        def _check_block_size(block_size: int, name: str):
            if block_size is not None:
                assert block_size >= 16 and math.log2(block_size) % 1 == 0, \
                    f"{name} must be power of 2 and at least 16, but {block_size} is given."

        _check_block_size(block_size, "block_size")
        _check_block_size(block_m, "block_m")
        _check_block_size(block_n, "block_n")

        explicit_tiles = block_m is not None or block_n is not None
        if block_m is None:
            block_m = max(block_size, 64) if causal else block_size
        if block_n is None:
            block_n = block_size

        sparse_pattern = sparse_pattern.to(torch.uint8)
        if sparse_pattern.dim() == 2:
            sparse_pattern = zero_stride(sparse_pattern[None])
        verify_sparse_pattern(sparse_pattern)
        if causal and not is_kv_cache_efficient(sparse_pattern, block_size, block_size):
            warnings.warn("The provided sparse_pattern is not efficient for KV cache, "
                          "i.e., KV cache needed for later tokens are not used in "
                          "earlier tokens. This may result in unexpected larger KV cache.")

        self.block_size = block_size
        self.block_m = block_m
        self.block_n = block_n
        self.seq_dim = seq_dim
        self.max_seqlen = max(sparse_pattern.shape[1:]) * block_size
        self.kwargs = copy.copy(kwargs)
        self.kwargs["max_seqlen"] = self.max_seqlen
        self.kwargs['causal'] = causal
        # q heads whose patterns are identical (a GQA group) can share K/V tiles on chip
        self.lut_group = _identical_head_run(sparse_pattern)
        self.kwargs['lut_group'] = self.lut_group
        # heads that hold clearly different numbers of blocks (dense heads beside sparse ones): the
        # prefill and backward kernels then deal the heads to the hardware's workgroup queues in
        # rotation, so that no part of the chip is left with the dense heads alone
        self.kwargs['uneven_heads'] = _uneven_heads(sparse_pattern)
        # rows that are clearly longer than every row after them (global rows at the start of a
        # non-causal pattern): the forward and dQ kernels, which otherwise start from the last row
        # - the longest of a causal pattern -, then take the rows in the table's own order, longest
        # first, instead of starting the long ones when the rest of the chip has run out of work
        self.kwargs['unsorted_rows'] = _unsorted_rows(sparse_pattern)

        if not causal:
            # merged q tiles are a causal-only optimisation
            assert self.block_m <= block_size
            assert self.block_n <= block_size

        # Tile sizes given by the caller are honoured in the layout_* buffers.  The kernels run
        # 64 x 64 tiles of their own (below), which attend the same blocks.
        # (a merged-row table over a pattern that it widens: the kernels' own tiles then follow
        # the widened pattern, block by block what the merged table attends)
        kernel_pattern = sparse_pattern
        if explicit_tiles and not tile_sizes_keep_pattern(block_size, sparse_pattern, self.block_m, self.block_n,
                                                          causal):
            kernel_pattern = merged_rows_pattern(block_size, sparse_pattern, self.block_m, self.block_n,
                                                 causal).to(sparse_pattern.device)
            if kernel_pattern.size(0) == 1:
                kernel_pattern = zero_stride(kernel_pattern)
        widened = kernel_pattern is not sparse_pattern
        own_tiles = True
        # patterns with blocks larger than the 64 x 64 tile of the matrix-core kernels run on
        # tables split to that tile
        split_for_kernels = own_tiles and block_size > _KERNEL_TILE
        # ... and patterns with smaller blocks on tile tables whose entries carry a bit mask over
        # the pattern blocks inside the tile
        mask_for_kernels = own_tiles and block_size < _KERNEL_TILE

        layout_csr = list(merge_split_fwd_kernel_blocks(block_size, sparse_pattern,
                                                        self.block_m, self.block_n, causal=causal))
        # the dK/dV pass always walks columns at the sparse block size
        self.block_m2, self.block_n2 = self.block_size, self.block_size
        layout_csc = list(dense_to_ccol_row(sparse_pattern, include_values=False))

        if layout_csr[0].dim() == 1:
            layout_csr = [x[None] for x in layout_csr]
            layout_csc = [x[None] for x in layout_csc]
        if layout_csr[0].size(0) == 1:
            layout_csr = [zero_stride(x) for x in layout_csr]
            layout_csc = [zero_stride(x) for x in layout_csc]

        # longest row of the table: sizes the split-KV decode grid
        crow = layout_csr[0]
        self.lut_max_row = int((crow[:, 1:] - crow[:, :-1]).max()) if crow.size(1) > 1 else 0
        self.kwargs['lut_max_row'] = self.lut_max_row

        self.register_buffer("layout_csr_crow", layout_csr[0].to(torch.int32), persistent=False)
        self.register_buffer("layout_csr_col", layout_csr[1].to(torch.int32), persistent=False)
        self.register_buffer("layout_csc_ccol", layout_csc[0].to(torch.int32), persistent=False)
        self.register_buffer("layout_csc_row", layout_csc[1].to(torch.int32), persistent=False)

        # The layout_* buffers keep the reference's shapes; the kernels read these when present.
        self.kernel_tile = None
        if split_for_kernels:
            tile_csr, tile_csc = split_tile_tables(block_size, kernel_pattern, _KERNEL_TILE, causal=causal)
            tile_csr, tile_csc = list(tile_csr), list(tile_csc)
            if tile_csr[0].size(0) == 1:
                tile_csr = [zero_stride(x) for x in tile_csr]
                tile_csc = [zero_stride(x) for x in tile_csc]
            crow = tile_csr[0]
            self.lut_max_row = int((crow[:, 1:] - crow[:, :-1]).max()) if crow.size(1) > 1 else 0
            self.kwargs['lut_max_row'] = self.lut_max_row
            self.kernel_tile = _KERNEL_TILE
            self.register_buffer("kernel_csr_crow", tile_csr[0].to(torch.int32), persistent=False)
            self.register_buffer("kernel_csr_col", tile_csr[1].to(torch.int32), persistent=False)
            self.register_buffer("kernel_csc_ccol", tile_csc[0].to(torch.int32), persistent=False)
            self.register_buffer("kernel_csc_row", tile_csc[1].to(torch.int32), persistent=False)

        # The reference's default for blocks below 64 is a merged-row table (block_m = 64), in which
        # a column held only by a later part of the 64 rows is attended by the earlier parts too
        # (dkernel/utils.py:299-308): exact for local-stride patterns, not for arbitrary ones.  The
        # layout_csr_* buffers keep that table; the kernels follow the pattern itself: unmerged
        # tiles for the generic kernels, masked 64 x 64 tiles for the matrix-core kernels.
        self.exact_tile = None
        self.exact_csc = False
        if own_tiles and not split_for_kernels and (self.block_m != block_size or self.block_n != block_size):
            exact = list(dense_to_crow_col(kernel_pattern))
            if exact[0].dim() == 1:
                exact = [x[None] for x in exact]
            if exact[0].size(0) == 1:
                exact = [zero_stride(x) for x in exact]
            self.exact_tile = block_size
            crow = exact[0]
            self.lut_max_row = int((crow[:, 1:] - crow[:, :-1]).max()) if crow.size(1) > 1 else 0
            self.kwargs['lut_max_row'] = self.lut_max_row
            self.register_buffer("exact_csr_crow", exact[0].to(torch.int32), persistent=False)
            self.register_buffer("exact_csr_col", exact[1].to(torch.int32), persistent=False)
            if widened:  # the column walk of the backward follows the widened pattern as well
                exact_c = list(dense_to_ccol_row(kernel_pattern, include_values=False))
                if exact_c[0].dim() == 1:
                    exact_c = [x[None] for x in exact_c]
                if exact_c[0].size(0) == 1:
                    exact_c = [zero_stride(x) for x in exact_c]
                self.exact_csc = True
                self.register_buffer("exact_csc_ccol", exact_c[0].to(torch.int32), persistent=False)
                self.register_buffer("exact_csc_row", exact_c[1].to(torch.int32), persistent=False)

        self.mask_tile = None
        if mask_for_kernels:
            m_csr, m_csc = masked_tile_tables(block_size, kernel_pattern, _KERNEL_TILE)
            m_csr, m_csc = list(m_csr), list(m_csc)
            if m_csr[0].size(0) == 1:
                m_csr = [zero_stride(x) for x in m_csr]
                m_csc = [zero_stride(x) for x in m_csc]
            crow = m_csr[0]
            self.mask_tile = _KERNEL_TILE
            self.mask_lut_max_row = int((crow[:, 1:] - crow[:, :-1]).max()) if crow.size(1) > 1 else 0
            self.register_buffer("masked_csr_crow", m_csr[0].to(torch.int32), persistent=False)
            self.register_buffer("masked_csr_col", m_csr[1].to(torch.int32), persistent=False)
            self.register_buffer("masked_csc_ccol", m_csc[0].to(torch.int32), persistent=False)
            self.register_buffer("masked_csc_row", m_csc[1].to(torch.int32), persistent=False)

    def forward(self,
                q: Tensor,
                k: Optional[Tensor] = None,
                v: Optional[Tensor] = None,
                sm_scale: Optional[float] = None,
                *,
                cu_seqlen_k: Optional[Tensor] = None,
                cu_seqlen_q: Optional[Tensor] = None,
                left_paddings: Optional[Tensor] = None,
                seqlens: Optional[Tensor] = None,
                return_lse: bool = False,
                split_qkv: Optional[callable] = None):
        """
        q, k, v:
            packing: with k and v None, `q` holds qkv and `split_qkv(q)` gives
            (q, k, v); with only v None, `k` holds kv and `split_qkv(k)` gives (k, v).
            shapes: (batch, seq, heads, dim) [seq_dim 1 / None] or
            (batch, heads, seq, dim) [seq_dim 2]; for inference also 4-D with
            `left_paddings` / `seqlens`, or packed 3-D (total_tokens, heads, dim)
            with `cu_seqlen_k` (and `cu_seqlen_q`).
        sm_scale: softmax scale, default 1 / sqrt(dim).
        return_lse: also return the natural-log softmax normaliser, (batch,
            heads, seq) for 4-D inputs and (heads, total_tokens) for packed ones.
        """
        inf_kwargs = {"cu_seqlen_k": cu_seqlen_k,
                      "cu_seqlen_q": cu_seqlen_q,
                      "left_paddings": left_paddings,
                      "seqlens": seqlens}
        kwargs = copy.copy(self.kwargs)
        kwargs["return_lse"] = return_lse
        kwargs['split_qkv'] = split_qkv
        if self.kernel_tile is not None:
            layout_csr = (self.kernel_csr_crow, self.kernel_csr_col, self.kernel_tile, self.kernel_tile)
            layout_csc = (self.kernel_csc_ccol, self.kernel_csc_row, self.kernel_tile, self.kernel_tile)
        else:
            layout_csr = (self.layout_csr_crow, self.layout_csr_col, self.block_m, self.block_n)
            layout_csc = (self.layout_csc_ccol, self.layout_csc_row, self.block_m2, self.block_n2)
            if self.exact_tile is not None:
                layout_csr = (self.exact_csr_crow, self.exact_csr_col, self.exact_tile, self.exact_tile)
                if self.exact_csc:
                    layout_csc = (self.exact_csc_ccol, self.exact_csc_row, self.exact_tile, self.exact_tile)
        if self.mask_tile is not None:
            # (crow, (col, mask), tile rows, tile cols, pattern block size), longest row
            kwargs["masked_layouts"] = ((self.masked_csr_crow, self.masked_csr_col, self.mask_tile,
                                         self.mask_tile, self.block_size),
                                        (self.masked_csc_ccol, self.masked_csc_row, self.mask_tile,
                                         self.mask_tile, self.block_size), self.mask_lut_max_row)
        needs_grad = torch.is_grad_enabled() and any(
            x is not None and x.requires_grad for x in (q, k, v))
        if needs_grad:
            output, lse = _sparse_attention.apply(
                q, k, v, sm_scale, layout_csr, layout_csc,
                self.seq_dim, inf_kwargs, kwargs)
        else:
            # nothing to differentiate: the same forward without the autograd bookkeeping (several
            # microseconds of a decode step's host time)
            output, lse = _sparse_attention.forward(
                _NoGradContext(), q, k, v, sm_scale, layout_csr, layout_csc,
                self.seq_dim, inf_kwargs, kwargs)
        if return_lse:
            return output, lse
        return output


    def paged_decode(self, q: Tensor, k_pool: Tensor, v_pool: Tensor, block_table: Tensor,
                     context_lens: Tensor, sm_scale: Optional[float] = None, *,
                     return_lse: bool = False, out: Optional[Tensor] = None,
                     k_scale: float = 1.0, v_scale: float = 1.0):
        """One new token per sequence over a paged K/V cache (serving).

        q: (batch, heads, dim) or (batch, 1, heads, dim); k_pool / v_pool: (pages, page_size,
        kv heads, dim), page_size a power of two >= 16; block_table: int32 (batch, pages per
        sequence); context_lens: int32 (batch,) keys per sequence including the new token's.
        Pools of dtype torch.float8_e4m3fn hold K / k_scale and V / v_scale (head_dim 64 / 128,
        blocks of at least 64).  Needs the matrix-core decode kernels (bf16 / fp16, head_dim a multiple
        of 8 up to 256).  No counterpart in the reference."""
        from .ops import paged_decode_attn
        assert self.kwargs.get('causal', True), "paged decode is causal"
        if self.kernel_tile is not None:
            layout = (self.kernel_csr_crow, self.kernel_csr_col, self.kernel_tile, self.kernel_tile)
            max_row = self.lut_max_row
        elif self.mask_tile is not None:
            layout = (self.masked_csr_crow, self.masked_csr_col, self.mask_tile, self.mask_tile, self.block_size)
            max_row = self.mask_lut_max_row
        elif self.exact_tile is not None:
            layout = (self.exact_csr_crow, self.exact_csr_col, self.exact_tile, self.exact_tile)
            max_row = self.lut_max_row
        else:
            layout = (self.layout_csr_crow, self.layout_csr_col, self.block_m, self.block_n)
            max_row = self.lut_max_row
        sm_scale = sm_scale or 1. / math.sqrt(float(q.size(-1)))
        return paged_decode_attn(q, k_pool, v_pool, block_table, context_lens, sm_scale, layout,
                                 max_seqlen=self.max_seqlen, out=out, return_lse=return_lse,
                                 lut_group=self.lut_group, lut_max_row=max_row,
                                 k_scale=k_scale, v_scale=v_scale)


@lru_cache(maxsize=8)
class LocalStrideSparseAttention(SparseAttention):
    """Local window + vertical stride pattern with per-head shifted columns
    (the Phi-3-small pattern).  As in the reference the class is wrapped in
    `functools.lru_cache(maxsize=8)`: identical constructor arguments return the
    same cached module.

    num_heads: number of q heads.
    max_seq_len: longest sequence the module will see (rounded up to a multiple
        of max(block_size, block_m, block_n, 64)).
    block_size / local_blocks / vert_stride: sparse block size, number of local
        blocks (including the diagonal one), and 1-in-`vert_stride` vertical columns.
    homo_head: one pattern for every head.
    num_dense_heads: the last `num_dense_heads` kv heads attend densely.
    num_kv_heads: grouped-query attention; q heads of a group share a pattern.
    active_head_range: (start, end) q heads handled by this rank (head /
        tensor parallelism).
    head_sliding_offset: shifts which head owns vertical column 0.

    Reference: dkernel/interface.py:218-300.
    """

    def __init__(self,
                 num_heads: int,
                 max_seq_len: int,
                 block_size: int,
                 local_blocks: int,
                 vert_stride: int,
                 *,
                 homo_head: bool = False,
                 num_dense_heads: int = 0,
                 num_kv_heads: Optional[int] = None,
                 active_head_range: Optional[Tuple[int, int]] = None,
                 head_sliding_offset: int = 0,
                 block_m: Optional[int] = None,
                 block_n: Optional[int] = None,
                 causal: bool = True,
                 **kwargs):
        assert vert_stride >= 1, "Vertical stride should be position integer. Value 1 will collapse to dense attention."
        if vert_stride > 1:
            assert local_blocks >= 1, "Token in the first block will attend to nothing in some blocks."
        self.max_seq_len = multiple_of(max_seq_len, max([block_size, block_m or 1, block_n or 1, 64]))
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.local_blocks = local_blocks
        self.vert_stride = vert_stride
        self.homo_head = homo_head
        self.num_dense_heads = num_dense_heads
        sparse_pattern = get_sparse_attn_mask(num_heads, self.max_seq_len,
                                              block_size=block_size,
                                              local_blocks=local_blocks,
                                              vert_stride=vert_stride,
                                              homo_head=homo_head,
                                              dtype=torch.uint8,
                                              num_kv_heads=num_kv_heads,
                                              head_sliding_offset=head_sliding_offset,
                                              num_dense_heads=num_dense_heads,
                                              causal=causal)[1]
        # homogeneous heads share one pattern, nothing to slice
        if (not homo_head) and (active_head_range is not None) and sparse_pattern.size(0) > 1:
            assert isinstance(active_head_range, tuple)
            assert len(active_head_range) == 2, '"active_head_range" should be a tuple of start/end index of the heads.'
            h_start, h_end = active_head_range
            sparse_pattern = sparse_pattern[h_start:h_end]
        super().__init__(block_size, sparse_pattern, block_m=block_m, block_n=block_n, causal=causal, **kwargs)


def combine_attn_partitions(*x: Tuple[Tensor, Tensor], hdim=1):
    """Merge attention results computed over disjoint K/V partitions:
    out = sum_p softmax_p(lse_p) * out_p.  Each argument is (out_p, lse_p).

    `hdim` is the head dimension of the outputs: with the default 1 the
    outputs are (batch, heads, seq, dim) and line up with the (batch, heads,
    seq) log-sum-exps as in the reference (dkernel/interface.py:303-324); when
    the head dimension comes right before `dim` -- (batch, seq, heads, dim) with
    hdim=2, or packed (tokens, heads, dim) -- the (.., heads, seq) log-sum-exps
    are transposed to match.  Partitions in which a row saw no key (lse = -inf)
    get weight 0.  Device tensors go through one fused kernel (and one for the backward);
    host tensors through the reference's torch expression.
    """
    assert len(x) >= 2 and len(x[0]) == 2
    outputs, weights = list(zip(*x))
    o0, w0 = outputs[0], weights[0]
    head_before_dim = (hdim % o0.dim()) == o0.dim() - 2
    straight = w0.shape == o0.shape[:-1]
    swapped = w0.dim() >= 2 and w0.transpose(-1, -2).shape == o0.shape[:-1]
    transposed = swapped and (not straight or (head_before_dim and w0.dim() >= 2))
    if o0.is_cuda and 2 <= o0.dim() <= 4 and len(x) <= _lib.MAX_PARTITIONS and (straight or swapped):
        # one fused kernel each way (dk_combine, dk_combine_bwd)
        return ops.combine_partitions(list(outputs), list(weights), transposed)
    # host tensors, more than three dims in front of head_dim or more partitions than the
    # kernel takes: the reference's torch expression
    weights = torch.stack(weights, dim=0)
    outputs = torch.stack(outputs, dim=0)
    if transposed:
        weights = weights.transpose(-1, -2)
    weights = weights.softmax(dim=0)
    weights = torch.where(torch.isnan(weights), torch.zeros_like(weights), weights)
    output = (outputs * weights.unsqueeze(-1)).sum(0).type_as(outputs)
    return output


__all__ = [
    "SparseAttention",
    "LocalStrideSparseAttention",
    "combine_attn_partitions",
]
