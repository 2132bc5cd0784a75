"""autograd Function and host launchers, mirroring the reference's
dkernel/ops/__init__.py (dispatch, packing, error behaviour) and the host
halves of sparse_attn_fwd.py / sparse_attn_bwd.py / sparse_attn_inference.py.
The device work goes through the C ABI of libdkernel_hip.so; there is no
other execution path (CPU tensors are refused).

Differences from the reference, all supersets: grouped-query attention works
on every path (kv head = q head // group), LSE is returned whenever asked
(also from padded and packed inputs, and without grad), and no launcher
synchronises with the host.
"""
from __future__ import annotations

import ctypes as C
import os
import math
from typing import Dict, Optional, Tuple, Union

import torch
from torch import Tensor

from . import _lib

_DTYPES = {torch.bfloat16: _lib.DK_BF16, torch.float16: _lib.DK_F16, torch.float32: _lib.DK_F32}

# Kernel selection for tests and benchmarks: "auto", "generic" or "mfma".
_IMPL = {"auto": _lib.DK_IMPL_AUTO, "generic": _lib.DK_IMPL_GENERIC, "mfma": _lib.DK_IMPL_MFMA}
_impl = _lib.DK_IMPL_AUTO


_bwd_workspace = True  # hand dk_bwd the scratch it asks for (off: tests of the path without it)
_fwd_workspace = True  # the same for dk_fwd


def set_impl(name: str) -> None:
    global _impl
    _impl = _IMPL[name]


def _matrix_core_applies(*xs: Optional[Tensor]) -> bool:
    """Whether dk_fwd / dk_bwd will run these tensors on the matrix-core kernels with a masked tile table:
    16-bit floats, head_dim a multiple of 8 up to 256, 16-byte aligned rows (the library's own
    conditions; it fails loudly if they were judged wrong here)."""
    q = xs[0]
    if _impl == _lib.DK_IMPL_GENERIC or q.dtype not in (torch.bfloat16, torch.float16):
        return False
    if q.size(-1) % 8 or not 8 <= q.size(-1) <= 256:
        return False
    for x in xs:
        if x is None:
            continue
        if x.stride(-1) != 1 or x.data_ptr() % 16 or any(st % 8 for st in x.stride()[:-1]):
            return False
    return True


def _require_gpu(*xs: Tensor) -> None:
    for x in xs:
        if not x.is_cuda:
            raise RuntimeError(
                "dkernel_amd runs on ROCm (MI355X) tensors only; got a tensor on "
                f"{x.device}. There is no CPU execution path.")
    if xs[0].dtype not in _DTYPES:
        raise TypeError(f"unsupported dtype {xs[0].dtype}; use bfloat16, float16 or float32")
    assert all(x.dtype == xs[0].dtype for x in xs), "q, k, v must share a dtype"


def _unit_last(x: Tensor) -> Tensor:
    return x if x.stride(-1) == 1 else x.contiguous()


def _tensor4(x: Tensor, hdim: int, seq_dim: int) -> _lib.Tensor:
    return _lib.Tensor(x.data_ptr(), x.stride(0), x.stride(hdim), x.stride(seq_dim))


def _tensor3(x: Tensor) -> _lib.Tensor:  # packed (tokens, heads, dim)
    return _lib.Tensor(x.data_ptr(), 0, x.stride(1), x.stride(0))


def _rowvec(x: Optional[Tensor], strides=None) -> _lib.RowVec:
    if x is None:
        return _lib.RowVec(None, 0, 0, 0)
    sb, sh, st = strides if strides is not None else x.stride()
    return _lib.RowVec(x.data_ptr(), sb, sh, st)


_LUT_CACHE = {}


def _lut(layout: Tuple[Tensor, Tensor, int, int], device, group: int = 1, max_row: int = 0,
         longest_first: bool = False, uneven: bool = False) -> _lib.Lut:
    """dk_lut of a layout tuple.  The descriptor of a module's tables never changes, so it is
    built (and checked) once per (tables, hints) and copied from then on (a decode step's host
    time counts).  An entry keeps its two tensors alive, so their addresses cannot be handed to
    other tensors while the entry exists; the caller gets a copy of its own."""
    key = (layout[0].data_ptr(), layout[1].data_ptr(), layout[0].dtype, layout[1].dtype, layout[0].shape,
           layout[1].shape, layout[0].stride(), layout[1].stride(), tuple(int(x) for x in layout[2:]), device, group,
           max_row, longest_first, uneven)
    hit = _LUT_CACHE.get(key)
    if hit is None:
        if len(_LUT_CACHE) > 256:
            _LUT_CACHE.clear()
        lut = _make_lut(layout, device, group, max_row)
        lut.uneven_heads = int(bool(uneven))
        order = None
        if longest_first:
            # rows of every head by descending length (stable: equal lengths stay in index order),
            # computed on the device once per table: the dK/dV pass hands its columns out in this
            # order, the forward and dQ kernels the rows of a pattern whose long rows are not its last
            ptr = layout[0] if layout[0].dim() == 2 else layout[0][None]
            lens = ptr[:, 1:] - ptr[:, :-1]
            rows = lens.size(1)
            # ... followed by the pairs of rows (2u, 2u + 1) by descending length of the pair
            pair_lens = torch.nn.functional.pad(lens, (0, rows % 2)).view(lens.size(0), -1, 2).sum(2)
            order = torch.cat([torch.argsort(x, dim=1, descending=True, stable=True) for x in (lens, pair_lens)],
                              dim=1).to(torch.int32).contiguous()
            lut.row_order, lut.row_order_stride_h = order.data_ptr(), order.stride(0)
            lut.pair_order = order.data_ptr() + 4 * rows
        hit = _LUT_CACHE[key] = (lut, layout[0], layout[1], order)
    return _lib.Lut.from_buffer_copy(hit[0])


def _make_lut(layout: Tuple[Tensor, Tensor, int, int], device, group: int = 1, max_row: int = 0) -> _lib.Lut:
    ptr, idx, block_rows, block_cols = layout[:4]
    sub_block = int(layout[4]) if len(layout) > 4 else 0  # entries carry a bit mask over pattern blocks
    assert ptr.dtype == torch.int32 and idx.dtype == torch.int32
    assert ptr.device == device and idx.device == device, \
        "sparse layout is on another device than q; move the module with .to(device)"
    if ptr.dim() == 1:
        ptr, idx = ptr[None], idx[None]
    assert ptr.stride(-1) == 1
    width = 1
    if idx.dim() == 3:
        assert idx.size(2) == 2 and idx.stride(2) == 1 and idx.stride(1) == 2
        width = 2
    else:
        assert idx.stride(-1) == 1 or idx.size(-1) <= 1
    return _lib.Lut(ptr.data_ptr(), idx.data_ptr(), ptr.stride(0), idx.stride(0), width,
                    ptr.size(0), ptr.size(1) - 1, int(block_rows), int(block_cols), int(group), int(max_row),
                    sub_block)


_CONST_I32 = {}


def _const_i32(device, n: int, value: int) -> Tensor:
    """Cached constant int32 vector (sequence starts / ends that do not depend
    on the data), so that a decode step launches no fill kernels."""
    key = (device, n, value)
    t = _CONST_I32.get(key)
    if t is None:
        if len(_CONST_I32) > 64:
            _CONST_I32.clear()
        t = _CONST_I32[key] = torch.full((n,), value, dtype=torch.int32, device=device)
    return t


def _check_out(out: Optional[Tensor], q: Tensor) -> None:
    """A caller's output tensor is written in place by the kernels: it must look like q."""
    if out is None:
        return
    assert out.shape == q.shape, f"out has shape {tuple(out.shape)}, q has {tuple(q.shape)}"
    assert out.dtype == q.dtype and out.device == q.device, "out must have q's dtype and device"
    assert out.stride(-1) == 1, "out must have unit stride on head_dim"


def _stream() -> C.c_void_p:
    # the raw handle of torch's current stream (building a torch.cuda.Stream object for it costs
    # several microseconds per call, a fifth of a decode step's host time)
    return C.c_void_p(torch._C._cuda_getCurrentRawStream(torch.cuda.current_device()))


def _as_i32(x: Tensor, device) -> Tensor:
    """int32, contiguous, on `device` -- without a dispatcher round trip when it already is."""
    if x.dtype == torch.int32 and x.device == device and x.is_contiguous():
        return x
    return x.to(device, dtype=torch.int32).contiguous()


last_fwd_workspace_bytes = 0  # scratch the library asked for in the latest forward (non-zero: split-KV decode)
last_bwd_kernels = b""        # dk_last_kernels() after the latest backward


def _run_fwd(args: _lib.FwdArgs, device) -> None:
    global last_fwd_workspace_bytes
    lib = _lib.lib()
    need = lib.dk_fwd_workspace_bytes(C.byref(args)) if _fwd_workspace else 0
    last_fwd_workspace_bytes = need
    ws = None
    if need:
        ws = torch.empty(need, dtype=torch.uint8, device=device)
        args.workspace, args.workspace_bytes = ws.data_ptr(), need
    _lib.check(lib.dk_fwd(C.byref(args)))


def _forward(ctx, q: Tensor, k: Tensor, v: Tensor, sm_scale: float,
             layout_csr: Tuple[Tensor, Tensor, int, int],
             seq_dim: int = 1,
             inference: Optional[bool] = None,
             out: Optional[Tensor] = None,
             d_splits: Optional[int] = None,
             max_seqlen: Optional[int] = None,
             return_lse: bool = False,
             causal=True,
             split_qkv=None,
             lut_group: int = 1,
             lut_max_row: int = 0,
             uneven_heads: bool = False,
             unsorted_rows: bool = False) -> Tuple[Tensor, Optional[Tensor]]:
    """Unpadded 4-D forward (training, prefill, single-token decode).
    Reference: dkernel/ops/sparse_attn_fwd.py:383-567.  `d_splits` is accepted
    and ignored (a Triton shared-memory workaround)."""
    assert seq_dim in [2, 1]
    hdim = 3 - seq_dim
    assert q.shape[-1] == k.shape[-1] == v.shape[-1]
    assert k.shape[seq_dim] == v.shape[seq_dim]
    qlen, klen = q.size(seq_dim), k.size(seq_dim)
    num_heads, num_kv_heads = q.size(hdim), k.size(hdim)
    if max_seqlen is not None:
        assert klen <= max_seqlen
    num_head_patterns = layout_csr[0].size(0) if layout_csr[0].dim() == 2 else 1
    if num_head_patterns > 1:
        assert num_head_patterns in [num_heads, num_kv_heads]

    q, k, v = _unit_last(q), _unit_last(k), _unit_last(v)
    _check_out(out, q)
    o = out if out is not None else q.new_empty(q.shape).contiguous()
    if inference is None:
        inference = (not q.requires_grad) and (not k.requires_grad) and (not v.requires_grad)
    need_lse = return_lse or not inference
    lse = torch.empty((q.size(0), num_heads, qlen), dtype=torch.float32, device=q.device) if need_lse else None

    args = _lib.FwdArgs()
    args.q, args.k, args.v, args.o = (_tensor4(x, hdim, seq_dim) for x in (q, k, v, o))
    args.lse = _rowvec(lse)
    args.csr = _lut(layout_csr, q.device, lut_group, lut_max_row, uneven=uneven_heads,
                    longest_first=unsorted_rows and qlen > 1)
    args.seqs = _lib.Seqs(q.size(0), qlen, klen, 0, None, None, None, None)
    args.num_q_heads, args.num_kv_heads, args.head_dim = num_heads, num_kv_heads, q.size(-1)
    args.dtype, args.causal, args.impl = _DTYPES[q.dtype], int(bool(causal)), _impl
    args.sm_scale = float(sm_scale)
    args.stream = _stream()
    _run_fwd(args, q.device)

    ctx.save_for_backward(q, k, v, o, lse)
    ctx.sm_scale = sm_scale
    ctx.seq_dim = seq_dim
    ctx.hdim = hdim
    ctx.causal = causal
    ctx.lut_group = lut_group
    ctx.uneven_heads = uneven_heads
    ctx.unsorted_rows = unsorted_rows
    return o, (lse if return_lse else None)


def _backward(ctx, do: Tensor, dlse: Optional[Tensor],
              dq: Optional[Tensor] = None, dk: Optional[Tensor] = None, dv: Optional[Tensor] = None
              ) -> Tuple[Tensor, Tensor, Tensor]:
    """dQ, dK, dV.  Reference: dkernel/ops/sparse_attn_bwd.py:724-852."""
    q, k, v, o, lse = ctx.saved_tensors
    hdim, seq_dim = ctx.hdim, ctx.seq_dim
    assert lse is not None, "forward ran in inference mode; backward needs the saved log-sum-exp"
    do = _unit_last(do)

    def _check_or_new(x, like):
        if x is not None:
            assert x.shape == like.shape
            assert x.stride(-1) == 1
            return x
        return like.new_empty(like.shape)

    dq, dk, dv = _check_or_new(dq, q), _check_or_new(dk, k), _check_or_new(dv, v)
    B, Hq, Lq = q.size(0), q.size(hdim), q.size(seq_dim)
    delta = torch.empty((B, Hq, Lq), dtype=torch.float32, device=q.device)

    args = _lib.BwdArgs()
    for name, x in (("q", q), ("k", k), ("v", v), ("o", o), ("dout", do), ("dq", dq), ("dk", dk), ("dv", dv)):
        setattr(args, name, _tensor4(x, hdim, seq_dim))
    args.lse = _rowvec(lse)
    if dlse is not None:
        assert dlse.shape == lse.shape
        args.dlse = _rowvec(dlse.float() if dlse.dtype != torch.float32 else dlse)
    else:
        args.dlse = _rowvec(None)
    args.delta = delta.data_ptr()
    layout_csr, layout_csc = ctx.layout_csr, ctx.layout_csc
    masked = getattr(ctx, "masked_layouts", None)
    if masked is not None and _matrix_core_applies(q, k, v, o, do, dq, dk, dv):
        layout_csr, layout_csc = masked[0], masked[1]
    uneven = getattr(ctx, "uneven_heads", False)
    args.csr = _lut(layout_csr, q.device, ctx.lut_group, uneven=uneven,
                    longest_first=getattr(ctx, "unsorted_rows", False))
    args.csc = _lut(layout_csc, q.device, ctx.lut_group, longest_first=True, uneven=uneven)
    args.seqs = _lib.Seqs(B, Lq, k.size(seq_dim), 0, None, None, None, None)
    args.num_q_heads, args.num_kv_heads, args.head_dim = Hq, k.size(hdim), q.size(-1)
    args.dtype, args.causal, args.impl = _DTYPES[q.dtype], int(bool(ctx.causal)), _impl
    args.sm_scale = float(ctx.sm_scale)
    args.stream = _stream()
    lib = _lib.lib()
    need = lib.dk_bwd_workspace_bytes(C.byref(args)) if _bwd_workspace else 0
    if need:  # per-q-head dK/dV partials of the head-split pass (several q heads per kv head)
        ws = torch.empty(need, dtype=torch.uint8, device=q.device)
        args.workspace, args.workspace_bytes = ws.data_ptr(), need
    _lib.check(lib.dk_bwd(C.byref(args)))
    global last_bwd_kernels
    last_bwd_kernels = lib.dk_last_kernels()  # (backward runs on an autograd thread; the list is per thread)
    return dq, dk, dv


def padded_sparse_attn(q: Tensor, k: Tensor, v: Tensor, sm_scale: float,
                       sparse_layout: Tuple[Tensor, Tensor, int, int], *,
                       left_paddings: Optional[Tensor] = None,
                       seqlens: Optional[Tensor] = None,
                       max_seqlen: Optional[int] = None,
                       seq_dim: int = 1,
                       d_splits: Optional[int] = None,
                       out: Optional[Tensor] = None,
                       inference: bool = True,
                       causal: bool = True,
                       return_lse: bool = False,
                       lut_group: int = 1,
                       lut_max_row: int = 0,
                       uneven_heads: bool = False,
                       unsorted_rows: bool = False):
    """4-D inputs with left paddings and / or explicit sequence lengths; q has
    either one token per sequence (decode) or the same padded length as k.
    Reference: dkernel/ops/sparse_attn_inference.py:10-147.  Padding rows of
    the output are zero.  Nothing here reads device memory on the host."""
    assert seq_dim in (1, 2)
    hdim = 3 - seq_dim
    batches, head_size = q.size(0), q.size(3)
    q_len, k_len = q.size(seq_dim), k.size(seq_dim)
    num_heads, num_kv_heads = q.size(hdim), k.size(hdim)
    assert q.dim() == k.dim() == v.dim() == 4
    assert num_heads % num_kv_heads == 0
    assert q.size(0) == k.size(0) and q.size(3) == k.size(3)
    assert k.shape == v.shape
    assert q_len == 1 or q_len == k_len, \
        (f'q length can only 1 for decoding or the same as k length for prefilling, '
         f'but got {q_len=}, {k_len=}.')
    if max_seqlen:
        assert k_len <= max_seqlen, \
            f'k has seqlen {k_len} while max sequence length is set to {max_seqlen}.'
    q, k, v = _unit_last(q), _unit_last(k), _unit_last(v)
    dev = q.device
    _check_out(out, q)
    # decode writes every row; in padded prefill the kernel clears the padding rows of an output
    # allocated here itself (bit 2 of dk_seqs.packed), so nothing is filled.  The padding rows of
    # a caller's `out` stay as they were.
    clear_padding = out is None and q_len > 1
    if out is None:
        out = q.new_empty(q.shape)

    if left_paddings is not None:
        assert left_paddings.shape == (batches,)
        k_starts = _as_i32(left_paddings, dev)
    else:
        k_starts = _const_i32(dev, batches, 0)
    if seqlens is not None:
        # ends beyond the padded length are clamped on the device
        k_ends = k_starts + _as_i32(seqlens, dev)
    else:
        k_ends = _const_i32(dev, batches, k_len)
    if q_len == 1:
        q_starts, q_ends = _const_i32(dev, batches, 0), _const_i32(dev, batches, 1)
    else:
        q_starts, q_ends = k_starts, k_ends

    lse = None
    if return_lse:
        lse = (torch.empty((batches, num_heads, q_len), dtype=torch.float32, device=dev) if clear_padding or q_len == 1
               else torch.full((batches, num_heads, q_len), float("-inf"), dtype=torch.float32, device=dev))
    args = _lib.FwdArgs()
    args.q, args.k, args.v, args.o = (_tensor4(x, hdim, seq_dim) for x in (q, k, v, out))
    args.lse = _rowvec(lse)
    args.csr = _lut(sparse_layout, dev, lut_group, lut_max_row, uneven=uneven_heads and q_len > 1,
                    longest_first=unsorted_rows and q_len > 1)
    args.seqs = _lib.Seqs(batches, q_len, k_len, 4 if clear_padding else 0, q_starts.data_ptr(), q_ends.data_ptr(),
                          k_starts.data_ptr(), k_ends.data_ptr())
    args.num_q_heads, args.num_kv_heads, args.head_dim = num_heads, num_kv_heads, head_size
    args.dtype, args.causal, args.impl = _DTYPES[q.dtype], int(bool(causal)), _impl
    args.sm_scale = float(sm_scale)
    args.stream = _stream()
    _run_fwd(args, dev)
    return (out, lse) if return_lse else out


def paged_decode_attn(q: Tensor, k_pool: Tensor, v_pool: Tensor, block_table: Tensor, context_lens: Tensor,
                      sm_scale: float, sparse_layout: Tuple, *, max_seqlen: int, out: Optional[Tensor] = None,
                      return_lse: bool = False, lut_group: int = 1, lut_max_row: int = 0,
                      k_scale: float = 1.0, v_scale: float = 1.0):
    """One new token per sequence over a paged K/V cache.

    q: (batch, heads, dim) or (batch, 1, heads, dim); k_pool, v_pool: (pages, page_size, kv heads,
    dim) with page_size a power of two >= 16; block_table: int32 (batch, pages per sequence),
    entry i = pool page of tokens [i, i + 1) * page_size; context_lens: int32 (batch,), keys per
    sequence including the new token's own (the query sits at position context_len - 1).
    Pools of dtype torch.float8_e4m3fn hold K / k_scale and V / v_scale (per-tensor scales; head_dim
    64 or 128, pattern blocks of at least 64); otherwise the pools have q's dtype.
    Returns O shaped like q (and LSE (batch, heads, 1) when asked).  The reference has no paged
    path (its README lists per-sequence KV-cache sizes as future work); this is the split-KV
    decode kernel reading K/V through the page table."""
    squeeze = q.dim() == 3
    q4 = q[:, None] if squeeze else q
    assert q4.dim() == 4 and q4.size(1) == 1, "paged decode takes one query token per sequence"
    assert k_pool.dim() == 4 and k_pool.shape == v_pool.shape
    _require_gpu(q4)
    assert k_pool.is_cuda and v_pool.is_cuda and k_pool.dtype == v_pool.dtype
    batches, num_heads, head_size = q4.size(0), q4.size(2), q4.size(3)
    page_size, num_kv_heads = k_pool.size(1), k_pool.size(2)
    assert k_pool.size(3) == head_size and num_heads % num_kv_heads == 0
    assert block_table.dim() == 2 and block_table.size(0) == batches and context_lens.shape == (batches,)
    dev = q4.device
    q4, k_pool, v_pool = _unit_last(q4), _unit_last(k_pool), _unit_last(v_pool)
    table = block_table.to(dev, dtype=torch.int32)
    table = table if table.stride(1) == 1 else table.contiguous()
    if os.environ.get("DKERNEL_DEBUG"):
        # The kernel cannot check page numbers against the pools' size.  This check costs a
        # device-to-host synchronisation, so it only runs when asked for: every table entry that
        # a sequence's tokens reach must name a page of the pools.
        used = (torch.arange(table.size(1), device=dev)[None] * page_size) < context_lens.to(dev)[:, None]
        bad = used & ((table < 0) | (table >= k_pool.size(0)))
        assert not bool(bad.any()), (
            f"block_table names pages outside the pools ({k_pool.size(0)} pages) inside a sequence: "
            f"first at (sequence, entry) {tuple(bad.nonzero()[0].tolist())}")
    o4 = (out[:, None] if out.dim() == 3 else out) if out is not None else q4.new_empty(q4.shape)
    lse = torch.full((batches, num_heads, 1), float("-inf"), dtype=torch.float32, device=dev) if return_lse else None
    k_ends = context_lens.to(dev, dtype=torch.int32).contiguous()
    zeros, ones = _const_i32(dev, batches, 0), _const_i32(dev, batches, 1)

    args = _lib.FwdArgs()
    args.q, args.o = _tensor4(q4, 2, 1), _tensor4(o4, 2, 1)
    args.k = _lib.Tensor(k_pool.data_ptr(), 0, k_pool.stride(2), k_pool.stride(1))
    args.v = _lib.Tensor(v_pool.data_ptr(), 0, v_pool.stride(2), v_pool.stride(1))
    args.lse = _rowvec(lse)
    args.csr = _lut(sparse_layout, dev, lut_group, lut_max_row)
    capacity = min(table.size(1) * page_size, int(max_seqlen))
    args.seqs = _lib.Seqs(batches, 1, capacity, 0, zeros.data_ptr(), ones.data_ptr(), zeros.data_ptr(), k_ends.data_ptr())
    args.num_q_heads, args.num_kv_heads, args.head_dim = num_heads, num_kv_heads, head_size
    args.dtype, args.causal, args.impl = _DTYPES[q4.dtype], 1, _impl
    args.sm_scale = float(sm_scale)
    args.stream = _stream()
    fp8 = k_pool.dtype == torch.float8_e4m3fn
    assert fp8 or k_pool.dtype == q4.dtype, f"K/V pools must have q's dtype or float8_e4m3fn, got {k_pool.dtype}"
    pages = _lib.PagedKV(table.data_ptr(), table.stride(0), k_pool.stride(0), v_pool.stride(0), page_size,
                         _lib.DK_FP8_E4M3 if fp8 else _DTYPES[q4.dtype], float(k_scale), float(v_scale))
    lib = _lib.lib()
    need = lib.dk_fwd_workspace_bytes(C.byref(args))
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=dev)
    args.workspace, args.workspace_bytes = ws.data_ptr(), need
    _lib.check(lib.dk_fwd_paged(C.byref(args), C.byref(pages)))
    res = o4[:, 0] if squeeze and out is None else (out if out is not None else o4)
    return (res, lse) if return_lse else res


def varlen_sparse_attn(q: Tensor, k: Tensor, v: Tensor,
                       cu_seqlens_k: Tensor, cu_seqlens_q: Optional[Tensor],
                       sm_scale: float,
                       sparse_layout: Tuple[Tensor, Tensor, int, int], *,
                       max_seqlen: int = None,
                       d_splits: Optional[int] = None,
                       out: Optional[Tensor] = None,
                       inference: bool = True,
                       causal: bool = True,
                       return_lse: bool = False,
                       lut_group: int = 1,
                       lut_max_row: int = 0,
                       uneven_heads: bool = False):
    """Packed variable-length inputs (total_tokens, heads, head_dim) with
    cumulative sequence lengths.  Reference:
    dkernel/ops/sparse_attn_inference.py:150-287.  The query tokens of a
    sequence are the last q_len positions of its keys (q_len == k_len for
    prefill, 1 for decode; anything between is chunked prefill).  LSE, when
    asked for, has shape (heads, total_q_tokens)."""
    assert isinstance(sparse_layout, (list, tuple))
    _, num_heads, head_size = q.shape
    batch_size = cu_seqlens_k.size(0) - 1
    assert q.dim() == k.dim() == v.dim() == 3
    assert q.size(1) % k.size(1) == 0
    assert q.size(2) == k.size(2)
    assert k.shape == v.shape
    assert cu_seqlens_k.dim() == 1
    dev = q.device
    single_query = False
    if cu_seqlens_q is None:
        if q.size(0) == batch_size:  # decoding only
            cu_seqlens_q = torch.arange(0, batch_size + 1, dtype=torch.int32, device=dev)
            single_query = True  # lets the library take the split-KV decode kernel
        elif q.size(0) == k.size(0):
            cu_seqlens_q = cu_seqlens_k
        else:
            raise ValueError("cu_seqlens_q must be specified if it mix of prefilling and decoding.")
    else:
        assert cu_seqlens_k.size(0) == cu_seqlens_q.size(0)
    cu_q = cu_seqlens_q.to(dev, dtype=torch.int32).contiguous()
    cu_k = cu_seqlens_k.to(dev, dtype=torch.int32).contiguous()
    q, k, v = _unit_last(q), _unit_last(k), _unit_last(v)
    _check_out(out, q)
    out = out if out is not None else q.new_empty(q.shape)
    lse = torch.full((num_heads, q.size(0)), float("-inf"), dtype=torch.float32, device=dev) if return_lse else None

    args = _lib.FwdArgs()
    args.q, args.k, args.v, args.o = (_tensor3(x) for x in (q, k, v, out))
    args.lse = _rowvec(lse, (0, lse.stride(0), lse.stride(1))) if lse is not None else _rowvec(None)
    args.csr = _lut(sparse_layout, dev, lut_group, lut_max_row, uneven=uneven_heads and not single_query)
    isz = cu_q.element_size()
    args.seqs = _lib.Seqs(batch_size, q.size(0), k.size(0), 3 if single_query else 1,
                          cu_q.data_ptr(), cu_q.data_ptr() + isz, cu_k.data_ptr(), cu_k.data_ptr() + isz)
    args.num_q_heads, args.num_kv_heads, args.head_dim = num_heads, k.size(1), head_size
    args.dtype, args.causal, args.impl = _DTYPES[q.dtype], int(bool(causal)), _impl
    args.sm_scale = float(sm_scale)
    args.stream = _stream()
    _run_fwd(args, dev)
    return (out, lse) if return_lse else out


def get_qkv_and_pack_mode(q: Tensor, k: Optional[Tensor], v: Optional[Tensor], split_qkv=None):
    """Unpack `qkv` (k, v None) or `kv` (v None) with the user's callable.
    Reference: dkernel/ops/__init__.py:128-149."""
    qkv_pack_mode = 'split_qkv'
    packed_shape = None
    if v is None:
        assert split_qkv is not None, "Callable `split_qkv` must be specified if qkv or kv are packed."
        if k is None:
            packed_shape = q.shape
            q, k, v = split_qkv(q)
            qkv_pack_mode = 'packed_qkv'
        else:
            packed_shape = k.shape
            k, v = split_qkv(k)
            qkv_pack_mode = 'packed_kv'
    return (q, k, v), (packed_shape, qkv_pack_mode, split_qkv)


class _sparse_attention(torch.autograd.Function):
    """Same 9-argument form and dispatch as the reference's
    dkernel/ops/__init__.py:10-125."""

    @staticmethod
    def forward(ctx, q: Tensor, k: Optional[Tensor], v: Optional[Tensor], sm_scale: float,
                layout_csr: Tuple[Tensor, Tensor, int, int],
                layout_csc: Tuple[Tensor, Tensor, int, int],
                seq_dim: Optional[int], inf_kwargs: Dict, kwargs: Dict):
        (q, k, v), (packed_shape, packed_mode, split_qkv) = \
            get_qkv_and_pack_mode(q, k, v, split_qkv=kwargs.get("split_qkv", None))
        _require_gpu(q, k, v)
        ctx.layout_csr = layout_csr
        ctx.layout_csc = layout_csc
        ctx.packed_shape = packed_shape
        ctx.packed_mode = packed_mode
        ctx.split_qkv = split_qkv

        seq_dim = 1 if seq_dim is None else seq_dim
        max_seqlen = kwargs.get("max_seqlen", None)
        causal = kwargs.get("causal", True)
        return_lse = kwargs.get("return_lse", False)
        lut_group = kwargs.get("lut_group", 1)
        lse = None

        assert q.dim() in (3, 4)
        hdim = 3 - (seq_dim or 1) if q.dim() == 4 else 1
        layout_csr_crow = layout_csr[0]
        assert layout_csr_crow.size(0) in [1, k.size(hdim), q.size(hdim)], \
            (f"Input (q, k) have ({q.size(hdim)}, {k.size(hdim)}) heads"
             f"but the number of heads in the sparse pattern is {layout_csr_crow.size(0)}")
        sm_scale = sm_scale or 1. / math.sqrt(float(q.size(-1)))

        # Patterns with blocks below the kernel tile run on the masked tile tables whenever the
        # matrix-core kernels take these inputs (the backward decides again for its own tensors).
        masked = kwargs.get("masked_layouts", None)
        if masked is not None and sm_scale <= 0:
            # the matrix-core forward takes row maxima before scaling (scale > 0) and only it reads
            # masked tiles: other scales run forward and backward on the unmasked tables
            masked = None
        ctx.masked_layouts = masked
        if masked is not None and _matrix_core_applies(q, k, v, kwargs.get("out", None)):
            layout_csr, _, lut_max_row = masked
        else:
            lut_max_row = kwargs.get("lut_max_row", 0)

        if q.dim() == 3:
            assert inf_kwargs.get("cu_seqlen_k", None) is not None
            ctx.support_backward = False
            ctx.message = "Currently does not suppoort variable length inputs. WIP."
            res = varlen_sparse_attn(q, k, v, inf_kwargs["cu_seqlen_k"], inf_kwargs.get("cu_seqlen_q", None),
                                     sm_scale, layout_csr, max_seqlen=max_seqlen, causal=causal,
                                     out=kwargs.get("out", None), return_lse=return_lse, lut_group=lut_group, lut_max_row=lut_max_row,
                                     uneven_heads=kwargs.get("uneven_heads", False))
            output, lse = res if return_lse else (res, None)
        else:
            assert k.size(seq_dim) <= max_seqlen, \
                (f"Input length {k.size(seq_dim)} is larger "
                 f"than the maximum length allowed ({max_seqlen})")
            left_paddings = inf_kwargs.get("left_paddings", None)
            seqlens = inf_kwargs.get("seqlens", None)
            if (left_paddings is not None) or (seqlens is not None):
                ctx.support_backward = False
                ctx.message = "Currently does not support paddings in inputs. WIP."
                res = padded_sparse_attn(q, k, v, sm_scale, layout_csr, left_paddings=left_paddings,
                                         seqlens=seqlens, seq_dim=seq_dim, max_seqlen=max_seqlen,
                                         out=kwargs.get("out", None),
                                         causal=causal, return_lse=return_lse, lut_group=lut_group,
                                         lut_max_row=lut_max_row, uneven_heads=kwargs.get("uneven_heads", False),
                                         unsorted_rows=kwargs.get("unsorted_rows", False))
                output, lse = res if return_lse else (res, None)
            else:
                ctx.support_backward = True
                ctx.message = ""
                fwd_kwargs = {k_: v_ for k_, v_ in kwargs.items()
                              if k_ in ("inference", "out", "d_splits", "max_seqlen", "return_lse",
                                        "causal", "split_qkv", "lut_group", "uneven_heads", "unsorted_rows")}
                fwd_kwargs["lut_max_row"] = lut_max_row
                output, lse = _forward(ctx, q, k, v, sm_scale, layout_csr, seq_dim=seq_dim, **fwd_kwargs)
        return output, lse

    @staticmethod
    def backward(ctx, do: Tensor, dlse: Optional[Tensor]) -> Tuple[Union[Tensor, None], ...]:
        assert ctx.support_backward, ctx.message
        q, k = ctx.saved_tensors[:2]
        dq, dk, dv = None, None, None
        if ctx.packed_mode == 'packed_qkv':
            dqkv = q.new_empty(ctx.packed_shape)
            dq, dk, dv = ctx.split_qkv(dqkv)
        elif ctx.packed_mode == 'packed_kv':
            dkv = k.new_empty(ctx.packed_shape)
            dk, dv = ctx.split_qkv(dkv)
        dq, dk, dv = _backward(ctx, do, dlse, dq=dq, dk=dk, dv=dv)[:3]
        if ctx.packed_mode == 'packed_qkv':
            grads = (dqkv, None, None)
        elif ctx.packed_mode == 'packed_kv':
            grads = (dq, dkv, None)
        else:
            grads = (dq, dk, dv)
        return grads + (None,) * 6


__all__ = ["_sparse_attention", "padded_sparse_attn", "varlen_sparse_attn", "get_qkv_and_pack_mode", "set_impl"]


# ---------------------------------------------------------------------------
# combine_attn_partitions on the device (reference: dkernel/interface.py:303-324)
# ---------------------------------------------------------------------------
def _rows3(x: Tensor) -> Tuple[Tuple[int, int, int], Tuple[int, int, int]]:
    """Extents and element strides of the (at most three) dims in front of head_dim."""
    lead = x.dim() - 1
    shape = (1,) * (3 - lead) + tuple(x.shape[:-1])
    strides = (0,) * (3 - lead) + tuple(x.stride()[:-1])
    return shape, strides


def _fill_combine(args: _lib.CombineArgs, outputs, lses, transposed: bool) -> None:
    o0 = outputs[0]
    shape, _ = _rows3(o0)
    args.num_partitions = len(outputs)
    args.dtype = _DTYPES[o0.dtype]
    args.n0, args.n1, args.n2 = shape
    args.head_dim = o0.size(-1)
    for i, (o, l) in enumerate(zip(outputs, lses)):
        args.parts[i] = _lib.Tensor(o.data_ptr(), *_rows3(o)[1])
        args.lses[i] = _lib.RowVec(l.data_ptr(), *_lse_strides(l, o0.dim() - 1, transposed))
    args.stream = _stream()


def _lse_strides(l: Tensor, lead: int, transposed: bool) -> Tuple[int, int, int]:
    st = list(l.stride())
    if transposed:
        st[-1], st[-2] = st[-2], st[-1]
    return tuple([0] * (3 - lead) + st)


class _CombinePartitions(torch.autograd.Function):
    """out = sum_p softmax_p(lse_p) * out_p through dk_combine / dk_combine_bwd."""

    @staticmethod
    def forward(ctx, transposed: bool, n: int, *tensors: Tensor) -> Tensor:
        outputs = [_unit_last(t) for t in tensors[:n]]
        lses = [t if t.dtype == torch.float32 else t.float() for t in tensors[n:]]
        out = torch.empty(outputs[0].shape, dtype=outputs[0].dtype, device=outputs[0].device)
        args = _lib.CombineArgs()
        with torch.cuda.device(out.device):
            _fill_combine(args, outputs, lses, transposed)
            args.out = _lib.Tensor(out.data_ptr(), *_rows3(out)[1])
            _lib.check(_lib.lib().dk_combine(C.byref(args)))
        ctx.save_for_backward(*outputs, *lses)
        ctx.transposed, ctx.n = transposed, n
        ctx.lse_dtypes = [t.dtype for t in tensors[n:]]
        return out

    @staticmethod
    def backward(ctx, dout: Tensor):
        n, transposed = ctx.n, ctx.transposed
        saved = ctx.saved_tensors
        outputs, lses = saved[:n], saved[n:]
        dout = _unit_last(dout)
        dparts = [torch.empty(o.shape, dtype=o.dtype, device=o.device) for o in outputs]
        dlses = [torch.empty(l.shape, dtype=torch.float32, device=l.device) if ctx.needs_input_grad[2 + n + i] else None
                 for i, l in enumerate(lses)]
        args = _lib.CombineArgs()
        with torch.cuda.device(dout.device):
            _fill_combine(args, outputs, lses, transposed)
            args.dout = _lib.Tensor(dout.data_ptr(), *_rows3(dout)[1])
            for i in range(n):
                args.dparts[i] = _lib.Tensor(dparts[i].data_ptr(), *_rows3(dparts[i])[1])
                if dlses[i] is not None:
                    args.dlses[i] = _lib.RowVec(dlses[i].data_ptr(), *_lse_strides(dlses[i], dout.dim() - 1, transposed))
            _lib.check(_lib.lib().dk_combine_bwd(C.byref(args)))
            global last_bwd_kernels
            last_bwd_kernels = _lib.lib().dk_last_kernels()  # (autograd's thread: the caller's own record is another)
        dlses = [None if d is None else d.to(dt) for d, dt in zip(dlses, ctx.lse_dtypes)]
        return (None, None, *dparts, *dlses)


def combine_partitions(outputs, lses, transposed: bool) -> Tensor:
    """Device path of combine_attn_partitions: `outputs` share one shape (.., head_dim) with at
    most three dims in front of head_dim, `lses` hold one value per row, in the order of the
    outputs' leading dims or (transposed) with the last two swapped."""
    o0, l0 = outputs[0], lses[0]
    assert o0.dtype in _DTYPES, f"unsupported dtype {o0.dtype}"
    for o, l in zip(outputs, lses):
        assert o.shape == o0.shape and o.dtype == o0.dtype and o.device == o0.device, "partition outputs differ in shape, dtype or device"
        assert l.shape == l0.shape and l.device == o0.device, "partition log-sum-exps differ in shape or device"
    want = tuple(o0.shape[:-1])
    have = tuple(l0.shape[:-2] + l0.shape[-2:][::-1]) if transposed else tuple(l0.shape)
    assert have == want, f"log-sum-exps of shape {tuple(l0.shape)} do not line up with outputs of shape {tuple(o0.shape)}"
    return _CombinePartitions.apply(transposed, len(outputs), *outputs, *lses)
