"""ctypes binding of libdkernel_hip.so (the C ABI declared in
include/dkernel_hip.h).  The library is built in-tree by
``make -C dkernel_amd/csrc`` (or ``__graft_entry__.build()``); there is no
fallback: if it is missing, importing the ops raises.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# DKERNEL_AMD_LIB points at another build of the same library (A/B comparisons of kernel variants)
LIB_PATH = os.environ.get("DKERNEL_AMD_LIB") or os.path.join(_HERE, "libdkernel_hip.so")

DK_BF16, DK_F16, DK_F32, DK_FP8_E4M3 = 0, 1, 2, 3
DK_IMPL_AUTO, DK_IMPL_GENERIC, DK_IMPL_MFMA = 0, 1, 2
DK_ERR_INVALID, DK_ERR_UNSUPPORTED, DK_ERR_HIP = -1, -2, -3
DK_NOALLOC_SCRATCH_BYTES = 8 << 20

i32, i64, f32, vp = C.c_int32, C.c_int64, C.c_float, C.c_void_p


class Tensor(C.Structure):
    _fields_ = [("ptr", vp), ("stride_b", i64), ("stride_h", i64), ("stride_t", i64)]


class RowVec(C.Structure):
    _fields_ = [("ptr", vp), ("stride_b", i64), ("stride_h", i64), ("stride_t", i64)]


class Lut(C.Structure):
    _fields_ = [("ptr", vp), ("idx", vp), ("ptr_stride_h", i64), ("idx_stride_h", i64),
                ("entry_width", i32), ("num_heads", i32), ("num_rows", i32),
                ("block_rows", i32), ("block_cols", i32), ("group", i32), ("max_row_entries", i32),
                ("sub_block", i32), ("row_order", vp), ("row_order_stride_h", i64),
                ("uneven_heads", i32), ("reserved", i32), ("pair_order", vp)]


class Seqs(C.Structure):
    _fields_ = [("batch", i32), ("max_q_len", i32), ("max_k_len", i32), ("packed", i32),
                ("q_starts", vp), ("q_ends", vp), ("k_starts", vp), ("k_ends", vp)]


class FwdArgs(C.Structure):
    _fields_ = [("q", Tensor), ("k", Tensor), ("v", Tensor), ("o", Tensor), ("lse", RowVec),
                ("csr", Lut), ("seqs", Seqs),
                ("num_q_heads", i32), ("num_kv_heads", i32), ("head_dim", i32),
                ("dtype", i32), ("causal", i32), ("impl", i32), ("sm_scale", f32),
                ("workspace", vp), ("workspace_bytes", C.c_size_t), ("stream", vp)]


class BwdArgs(C.Structure):
    _fields_ = [("q", Tensor), ("k", Tensor), ("v", Tensor), ("o", Tensor), ("dout", Tensor),
                ("dq", Tensor), ("dk", Tensor), ("dv", Tensor),
                ("lse", RowVec), ("dlse", RowVec), ("delta", vp),
                ("csr", Lut), ("csc", Lut), ("seqs", Seqs),
                ("num_q_heads", i32), ("num_kv_heads", i32), ("head_dim", i32),
                ("dtype", i32), ("causal", i32), ("impl", i32), ("sm_scale", f32),
                ("workspace", vp), ("workspace_bytes", C.c_size_t), ("stream", vp)]


class PagedKV(C.Structure):
    _fields_ = [("block_table", vp), ("table_stride_b", i64), ("page_stride_k", i64), ("page_stride_v", i64),
                ("page_size", i32), ("kv_dtype", i32), ("k_scale", f32), ("v_scale", f32)]


MAX_PARTITIONS = 8  # DK_MAX_PARTITIONS


class CombineArgs(C.Structure):
    _fields_ = [("num_partitions", i32), ("dtype", i32), ("n0", i32), ("n1", i32), ("n2", i32), ("head_dim", i32),
                ("out", Tensor), ("dout", Tensor), ("parts", Tensor * MAX_PARTITIONS), ("lses", RowVec * MAX_PARTITIONS),
                ("dparts", Tensor * MAX_PARTITIONS), ("dlses", RowVec * MAX_PARTITIONS), ("stream", vp)]


# name -> (restype, argtypes); every symbol include/dkernel_hip.h declares
SYMBOLS = {
    "dk_version": (C.c_int, []),
    "dk_last_error": (C.c_char_p, []),
    "dk_last_kernels": (C.c_char_p, []),
    "dk_local_stride_mask": (C.c_int, [i32] * 14 + [vp]),
    "dk_csr_count": (C.c_int, [vp, i32, i32, i32, i64, i64, i64, vp, C.POINTER(i32)]),
    "dk_csr_fill": (C.c_int, [vp, i32, i32, i32, i64, i64, i64, i32, vp, vp]),
    "dk_tile_pattern_shape": (C.c_int, [i32] * 5 + [C.POINTER(i32)] * 3),
    "dk_tile_pattern": (C.c_int, [vp, i32, i32, i32, i32, i32, i32, i32, vp]),
    "dk_kv_cache_efficient": (C.c_int, [vp, i32, i32, i32, i32, i32]),
    "dk_fwd": (C.c_int, [C.POINTER(FwdArgs)]),
    "dk_fwd_workspace_bytes": (C.c_size_t, [C.POINTER(FwdArgs)]),
    "dk_fwd_noalloc": (C.c_int, [C.POINTER(FwdArgs)]),
    "dk_fwd_paged": (C.c_int, [C.POINTER(FwdArgs), C.POINTER(PagedKV)]),
    "dk_bwd": (C.c_int, [C.POINTER(BwdArgs)]),
    "dk_bwd_workspace_bytes": (C.c_size_t, [C.POINTER(BwdArgs)]),
    "dk_combine": (C.c_int, [C.POINTER(CombineArgs)]),
    "dk_combine_bwd": (C.c_int, [C.POINTER(CombineArgs)]),
}

_lib = None


def lib():
    """The loaded library (loads on first use)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `make -C dkernel_amd/csrc` "
                "(hipcc, gfx950). dkernel_amd has no other execution path.")
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = res, args
        _lib = handle
    return _lib


class DKernelError(RuntimeError):
    pass


def check(rc: int):
    """Raise on a non-zero return code: argument errors as AssertionError (the
    reference raises its argument errors with ``assert``), the rest as
    DKernelError."""
    if rc == 0:
        return
    msg = lib().dk_last_error().decode(errors="replace")
    if rc == DK_ERR_INVALID:
        raise AssertionError(msg)
    raise DKernelError(f"libdkernel_hip error {rc}: {msg}")
