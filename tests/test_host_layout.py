"""CPU tests of the product's host side: the C++ look-up-table builder behind
the C ABI against the golden fixtures and the oracle (bit-exact), the module
constructors, and the C-ABI surface (library loads, every declared symbol is
exported).  No compute call is made without a GPU."""
import ctypes
import os
import re
import warnings
import zlib

import numpy as np
import pytest
import torch

import dkernel_amd
from dkernel_amd import _lib, utils as U
from dkernel_amd.interface import (LocalStrideSparseAttention, SparseAttention, _uneven_heads,
                                   combine_attn_partitions)
from oracle import layout as OL
from conftest import ROOT, mask_kwargs


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "dkernel_hip.h")).read()
    declared = set(re.findall(r"\b(dk_[a-z_0-9]+)\s*\(", header))
    assert declared == set(_lib.SYMBOLS), declared ^ set(_lib.SYMBOLS)
    handle = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(handle, name), name
    assert _lib.lib().dk_version() >= 200
    assert _lib.lib().dk_last_error() is not None


def test_struct_sizes_match_header():
    # natural alignment on x86-64: catches a field added on one side only
    assert ctypes.sizeof(_lib.Tensor) == 32 and ctypes.sizeof(_lib.RowVec) == 32
    assert ctypes.sizeof(_lib.Lut) == 96 and ctypes.sizeof(_lib.Seqs) == 48
    assert ctypes.sizeof(_lib.FwdArgs) == 4 * 32 + 32 + 96 + 48 + 7 * 4 + 4 + 3 * 8
    assert ctypes.sizeof(_lib.BwdArgs) == 8 * 32 + 2 * 32 + 8 + 2 * 96 + 48 + 7 * 4 + 4 + 3 * 8
    assert ctypes.sizeof(_lib.CombineArgs) == 6 * 4 + 2 * 32 + 4 * 8 * 32 + 8


def test_mask_and_luts_match_fixtures(lut_fixtures):
    z, meta = lut_fixtures
    for name, kw in meta["mask"].items():
        (crow, col), bm, _ = U.get_sparse_attn_mask(dtype=torch.uint8, **mask_kwargs(kw))
        assert bm.dtype == torch.uint8 and crow.dtype == torch.int32 and col.dtype == torch.int32
        assert np.array_equal(bm.cpu().numpy(), z[f"mask/{name}/block_mask"]), name
        assert np.array_equal(crow.cpu().numpy(), z[f"mask/{name}/crow"]), name
        assert np.array_equal(col.cpu().numpy(), z[f"mask/{name}/col"]), name
        ccol, row = U.dense_to_ccol_row(bm)
        assert np.array_equal(ccol.cpu().numpy(), z[f"mask/{name}/ccol"]), name
        assert np.array_equal(row.cpu().numpy(), z[f"mask/{name}/row"]), name
        assert U.is_kv_cache_efficient(bm, kw["block_size"], kw["block_size"]) == bool(z[f"mask/{name}/kv_eff"])


def test_tile_luts_match_fixtures(lut_fixtures):
    z, meta = lut_fixtures
    for name, t in meta["tile"].items():
        pat = torch.from_numpy(z[f"tile/{name}/pattern"])
        crow, col = U.merge_split_fwd_kernel_blocks(t["block_size"], pat, t["block_m"], t["block_n"])
        assert np.array_equal(crow.cpu().numpy(), z[f"tile/{name}/crow"]), name
        assert np.array_equal(col.cpu().numpy(), z[f"tile/{name}/col"]), name


def test_headline_lut(lut_fixtures):
    z, meta = lut_fixtures
    (crow, col), bm, _ = U.get_sparse_attn_mask(dtype=torch.uint8, **meta["c1"])
    ccol, row = U.dense_to_ccol_row(bm)
    assert np.array_equal(crow.cpu().numpy(), z["c1/crow"]) and np.array_equal(ccol.cpu().numpy(), z["c1/ccol"])
    crc = [zlib.crc32(np.ascontiguousarray(x.cpu().numpy()).tobytes()) for x in (bm, col, row)]
    assert crc == list(z["c1/crc"])


@pytest.mark.parametrize("kw", [
    dict(num_heads=8, seqlen=777, block_size=32, local_blocks=3, vert_stride=5, num_kv_heads=4,
         head_sliding_offset=2, num_dense_heads=1),
    dict(num_heads=6, seqlen=512, block_size=16, local_blocks=1, vert_stride=7, head_sliding_step=2),
    dict(num_heads=4, seqlen=320, block_size=64, local_blocks=2, vert_stride=3, causal=False),
    dict(num_heads=4, seqlen=320, block_size=64, local_blocks=2, vert_stride=3, causal=False,
         num_dense_heads=2),
    dict(num_heads=4, seqlen=256, block_size=32, local_blocks=2, vert_stride=3, past_len=100),
    dict(num_heads=2, seqlen=128, block_size=32, local_blocks=2, vert_stride=3,
         q_start_position=256, kv_start_position=64, kv_seqlen=320),
])
def test_mask_matches_oracle(kw):
    (crow, col), bm, dense = U.get_sparse_attn_mask(dtype=torch.uint8, return_dense=True, **kw)
    want = OL.block_mask(**kw)
    assert np.array_equal(bm.cpu().numpy(), want)
    ocrow, ocol = OL.csr_from_dense(want)
    assert np.array_equal(crow.cpu().numpy(), ocrow) and np.array_equal(col.cpu().numpy(), ocol)
    if "q_start_position" not in kw:
        full = OL.block_mask(**{k: v for k, v in kw.items() if k != "past_len"})
        tok = OL.token_mask(full, kw["block_size"], kw["seqlen"], past_len=kw.get("past_len", 0),
                            causal=kw.get("causal", True))
        assert np.array_equal(dense.cpu().numpy(), np.broadcast_to(tok, dense.shape))


def test_csr_random_and_edge_cases():
    rng = np.random.default_rng(1)
    x = torch.from_numpy((rng.random((3, 7, 11)) < 0.4).astype(np.uint8))
    x[2] = 0
    for t in (x, x[0], x.transpose(1, 2), x.to(torch.bool), x.to(torch.bfloat16)):
        crow, col = U.dense_to_crow_col(t)
        ocrow, ocol = OL.csr_from_dense(t.to(torch.int32).numpy())
        assert np.array_equal(crow.numpy(), ocrow) and np.array_equal(col.numpy(), ocol)
    crow, col = U.dense_to_crow_col(torch.zeros(2, 3, 4))      # all empty: zero-width col
    assert col.shape == (2, 0) and (crow == 0).all()
    vals = torch.from_numpy(rng.integers(0, 4, (2, 5, 6)).astype(np.int32)) * 16
    crow, col = U.dense_to_crow_col(vals, include_values=True)
    ocrow, ocol = OL.csr_from_dense(vals.numpy(), include_values=True)
    assert np.array_equal(crow.numpy(), ocrow) and np.array_equal(col.numpy(), ocol)
    assert np.array_equal(U.crow_col_to_dense(*U.dense_to_crow_col(x), dtype=torch.uint8).numpy()[:2],
                          x.numpy()[:2, :, :U.dense_to_crow_col(x)[1].max() + 1])


def test_to_csr_matches_scipy():
    import scipy.sparse
    rng = np.random.default_rng(3)
    for shape in ((1, 1), (5, 7), (16, 16), (3, 0)):
        mat = (rng.random(shape) < 0.3) * rng.integers(1, 9, size=shape)
        got = U.to_csr(mat)
        want = scipy.sparse.csr_matrix(mat)
        assert got.indptr.dtype == np.int32 and got.indices.dtype == np.int32
        assert np.array_equal(got.indptr, want.indptr) and np.array_equal(got.indices, want.indices)
        assert np.array_equal(got.data, want.data)
    assert U.is_hip() is True


def test_kv_cache_check_and_warning():
    rng = np.random.default_rng(3)
    for _ in range(20):
        p = np.tril((rng.random((2, 6, 6)) < 0.5).astype(np.uint8))
        assert U.is_kv_cache_efficient(torch.from_numpy(p), 4, 4) == OL.kv_cache_efficient(p, 4, 4)
    pat = torch.tril((torch.rand(4, 8, 8, generator=torch.Generator().manual_seed(0)) < 0.3).to(torch.uint8))
    pat[:, torch.arange(8), torch.arange(8)] = 1
    with warnings.catch_warnings(record=True) as w:
        warnings.simplefilter("always")
        SparseAttention(64, pat)
    assert any("not efficient for KV cache" in str(x.message) for x in w)


def test_module_construction_matches_reference_surface():
    assert dkernel_amd.__all__ == ["SparseAttention", "LocalStrideSparseAttention",
                                   "get_sparse_attn_mask", "combine_attn_partitions"]
    m = LocalStrideSparseAttention(32, 8192, 64, 16, 8, num_kv_heads=8)
    assert m is LocalStrideSparseAttention(32, 8192, 64, 16, 8, num_kv_heads=8)     # lru_cache
    assert (m.block_m, m.block_n, m.block_m2, m.block_n2, m.max_seqlen) == (64, 64, 64, 64, 8192)
    assert m.layout_csr_crow.shape == (32, 129) and m.layout_csr_col.shape == (32, 2768)
    assert m.layout_csc_ccol.shape == (32, 129) and m.layout_csc_row.shape == (32, 2768)
    assert all(b.dtype == torch.int32 for b in m.buffers()) and len(m.state_dict()) == 0
    assert int(m.layout_csr_crow[:, -1].sum()) == 87008
    # homogeneous pattern: one head with stride 0
    h = LocalStrideSparseAttention(8, 1000, 64, 4, 4, homo_head=True)
    assert h.max_seq_len == 1024 and h.layout_csr_crow.shape[0] == 1 and h.layout_csr_crow.stride(0) == 0
    # head slicing for head parallelism
    full = LocalStrideSparseAttention(8, 1024, 64, 2, 8)
    part = LocalStrideSparseAttention(8, 1024, 64, 2, 8, active_head_range=(2, 6))
    assert torch.equal(part.layout_csr_crow, full.layout_csr_crow[2:6])
    # merged-q table carries (col, micro_M)
    mq = LocalStrideSparseAttention(2, 512, 16, 2, 4, block_m=128, block_n=16)
    assert mq.layout_csr_col.dim() == 3 and mq.layout_csr_col.shape[-1] == 2
    with pytest.raises(AssertionError):
        SparseAttention(24, torch.ones(4, 4))
    with pytest.raises(AssertionError):
        LocalStrideSparseAttention(8, 1024, 64, 0, 8)


@pytest.mark.parametrize("bs,causal", [(128, True), (256, True), (128, False)])
def test_large_blocks_get_split_kernel_tables(bs, causal):
    """Blocks larger than the 64 x 64 kernel tile: the layout_* buffers keep the
    reference's shapes, the kernel tables are the pattern expanded to 64 x 64
    tiles (tiles above the token diagonal dropped when causal), as CSR and CSC."""
    L, H = 2048, 4
    m = LocalStrideSparseAttention(H, L, bs, 2, 4, causal=causal)
    assert m.kernel_tile == 64 and (m.block_m, m.block_n, m.block_m2, m.block_n2) == (bs, bs, bs, bs)
    pattern = np.asarray(OL.block_mask(H, L, bs, 2, 4, causal=causal)) != 0
    assert m.layout_csr_crow.shape == (pattern.shape[0], L // bs + 1)
    f = bs // 64
    want = np.kron(pattern, np.ones((f, f), dtype=bool))
    if causal:
        want = np.tril(want)
    got_csr = U.crow_col_to_dense(m.kernel_csr_crow, m.kernel_csr_col, torch.uint8).numpy() != 0
    got_csc = U.ccol_row_to_dense(m.kernel_csc_ccol, m.kernel_csc_row, torch.uint8).numpy() != 0
    assert np.array_equal(got_csr, want) and np.array_equal(got_csc, want)
    assert m.lut_max_row == int(want.sum(-1).max())
    # explicit tile sizes shape the layout_* buffers; the kernels still get their own tiles
    e = LocalStrideSparseAttention(H, L, bs, 2, 4, causal=causal, block_m=bs, block_n=64)
    assert e.kernel_tile == 64 and (e.block_m, e.block_n) == (bs, 64)
    assert e.layout_csr_crow.shape[-1] == L // bs + 1 and torch.equal(e.kernel_csr_col, m.kernel_csr_col)
    assert LocalStrideSparseAttention(H, L, 64, 2, 4, causal=causal).kernel_tile is None


@pytest.mark.parametrize("bs,causal", [(16, True), (32, True), (16, False)])
def test_small_blocks_get_masked_tile_tables(bs, causal):
    """Blocks below the 64 x 64 kernel tile: one table entry per tile that holds any active
    block, with a bit mask (bit i * f + j: row part i, column part j) that reconstructs the
    pattern exactly, as CSR and CSC; the layout_* buffers keep the reference's shapes."""
    L, H = 1000, 4
    m = LocalStrideSparseAttention(H, L, bs, 3, 5, causal=causal)
    assert m.mask_tile == 64 and m.kernel_tile is None
    assert (m.block_m, m.block_n) == ((64, bs) if causal else (bs, bs))
    pattern = np.asarray(OL.block_mask(H, 1024, bs, 3, 5, causal=causal)) != 0
    f = 64 // bs

    def rebuild(ptr, idx, transposed):
        ptr, idx = ptr.numpy(), idx.numpy()
        out = np.zeros((ptr.shape[0], 1024 // bs, 1024 // bs), dtype=bool)
        for h in range(ptr.shape[0]):
            for a in range(ptr.shape[1] - 1):
                for e in range(ptr[h, a], ptr[h, a + 1]):
                    b, bits = idx[h, e]
                    r, c = (b, a) if transposed else (a, b)
                    assert bits != 0
                    for i in range(f):
                        for j in range(f):
                            out[h, r * f + i, c * f + j] = (bits >> (i * f + j)) & 1
        return out
    want = np.broadcast_to(pattern, (m.masked_csr_crow.shape[0],) + pattern.shape[1:])
    assert np.array_equal(rebuild(m.masked_csr_crow, m.masked_csr_col, False), want)
    assert np.array_equal(rebuild(m.masked_csc_ccol, m.masked_csc_row, True), want)
    crow = m.masked_csr_crow.numpy()
    assert m.mask_lut_max_row == int((crow[:, 1:] - crow[:, :-1]).max())
    # explicit tile sizes shape the layout_* buffers; the kernels still get their own tiles
    e = LocalStrideSparseAttention(H, L, bs, 3, 5, causal=causal, block_m=bs, block_n=bs)
    assert e.mask_tile == 64 and e.exact_tile is None and e.layout_csr_crow.shape[-1] == e.max_seqlen // bs + 1


def test_tile_sizes_given_by_the_caller_keep_the_pattern_or_not():
    """Explicit block_m / block_n only re-tile a local-stride pattern (the kernels may then run
    their own 64 x 64 tiles); a merged-row table over a pattern whose later row holds a column the
    earlier row lacks attends more than the pattern (checked against a brute-force expansion)."""
    for bs, bm, bn in [(16, 128, 16), (64, 128, 32), (16, 64, 16), (32, 32, 16), (64, 64, 64)]:
        pat = torch.from_numpy(np.asarray(OL.block_mask(4, 1024, bs, 2, 3))).to(torch.uint8)
        assert U.tile_sizes_keep_pattern(bs, pat, bm, bn, True)
        mod = LocalStrideSparseAttention(4, 1024, bs, 2, 3, block_m=bm, block_n=bn)
        assert (mod.block_m, mod.block_n) == (bm, bn)                      # layout_* buffers as asked
        assert mod.layout_csr_crow.shape[-1] == 1024 // bm + 1
        if bs < 64:
            assert mod.mask_tile == 64 and mod.exact_tile == bs
        elif (bm, bn) != (bs, bs):
            assert mod.exact_tile == 64 and mod.exact_csr_crow.shape[-1] == 1024 // 64 + 1
    # row 1 of the merged pair (0, 1) holds column 0... so does row 0: same; row 3 holds column 1, row 2 does not
    pat = torch.tensor([[[1, 0, 0, 0], [1, 1, 0, 0], [0, 0, 1, 0], [0, 1, 1, 1]]], dtype=torch.uint8)
    assert not U.tile_sizes_keep_pattern(64, pat, 128, 64, True)
    assert U.tile_sizes_keep_pattern(64, pat, 64, 32, True)                 # splitting alone never changes it
    with pytest.warns(UserWarning, match="not efficient for KV cache"):
        mod = SparseAttention(64, pat, block_m=128)
    # the kernels' own tiles follow the widened pattern (row 2 attends column 1 as well), rows and columns
    assert mod.exact_tile == 64 and mod.exact_csc and mod.mask_tile is None and mod.kernel_tile is None
    wide = torch.tensor([[1, 0, 0, 0], [1, 1, 0, 0], [0, 1, 1, 0], [0, 1, 1, 1]])
    assert (U.merged_rows_pattern(64, pat, 128, 64, True)[0] == wide).all()
    assert mod.exact_csr_crow.flatten().tolist() == [0, 1, 3, 5, 8]
    assert mod.exact_csc_ccol.flatten().tolist() == [0, 2, 5, 7, 8]
    assert mod.layout_csr_crow.flatten().tolist() == [0, 2, 5]          # the merged table itself, as asked
    # brute force on random causal patterns: expand the merged table and compare
    rng = np.random.default_rng(3)
    for _ in range(40):
        mm = int(rng.choice([2, 4]))
        n = mm * int(rng.integers(1, 5))  # the builder takes whole merged tiles only
        dense = np.tril(rng.random((1, n, n)) < 0.5).astype(np.uint8)
        dense[0, np.arange(n), np.arange(n)] = 1
        crow, col = U.merge_split_fwd_kernel_blocks(16, torch.from_numpy(dense), 16 * mm, 16)
        crow, col = crow.numpy().reshape(1, -1), col.numpy().reshape(1, -1, 2)
        eff = np.zeros_like(dense)
        for i in range(crow.shape[1] - 1):
            for c, micro in col[0, crow[0, i]:crow[0, i + 1]]:
                for s in range(mm):
                    if i * mm + s < n and s * 16 < micro:
                        eff[0, i * mm + s, c] = 1
        same = bool((np.tril(eff) == dense).all())
        assert U.tile_sizes_keep_pattern(16, torch.from_numpy(dense), 16 * mm, 16, True) == same
        # ... and what the merged table attends, block by block
        assert (U.merged_rows_pattern(16, torch.from_numpy(dense), 16 * mm, 16, True).numpy() == np.tril(eff)).all()


def _fake_fwd_args(B=2, Hq=8, Hkv=2, D=128, Lq=1, Lk=2048, dtype=0, max_row=10):
    """dk_fwd_args over made-up (never dereferenced) device addresses: a decode-shaped call."""
    a = _lib.FwdArgs()
    fake = 0x10000

    def tensor(L, H):
        return _lib.Tensor(fake, L * H * D, D, H * D)
    a.q, a.k, a.v, a.o = tensor(Lq, Hq), tensor(Lk, Hkv), tensor(Lk, Hkv), tensor(Lq, Hq)
    a.lse = _lib.RowVec(None, 0, 0, 0)
    a.csr = _lib.Lut(fake, fake, Lk // 64 + 1, 1024, 1, Hkv, Lk // 64, 64, 64, 1, max_row, 0)
    a.seqs = _lib.Seqs(B, Lq, Lk, 0, fake, fake, fake, fake)
    a.num_q_heads, a.num_kv_heads, a.head_dim = Hq, Hkv, D
    a.dtype, a.causal, a.impl, a.sm_scale = dtype, 1, 0, 0.1
    return a


def test_c_abi_argument_checks_fail_before_any_launch():
    """Every entry point validates its arguments on the host and returns a negative code with a
    message before anything touches the GPU; the workspace queries are pure host functions."""
    lib = _lib.lib()
    INVALID = -1

    def refused(rc, text):
        assert rc == INVALID, rc
        assert text in lib.dk_last_error().decode(), lib.dk_last_error().decode()

    refused(lib.dk_fwd(None), "args is NULL")
    a = _fake_fwd_args(Hq=8, Hkv=3)
    refused(lib.dk_fwd(ctypes.byref(a)), "must be a multiple of num_kv_heads")
    a = _fake_fwd_args(D=264)
    refused(lib.dk_fwd(ctypes.byref(a)), "head_dim 264")
    a = _fake_fwd_args(dtype=7)
    refused(lib.dk_fwd(ctypes.byref(a)), "unknown dtype")
    a = _fake_fwd_args()
    a.csr.num_heads = 5
    refused(lib.dk_fwd(ctypes.byref(a)), "number of heads in the sparse pattern is 5")
    a = _fake_fwd_args()
    a.csr.block_cols = 48
    refused(lib.dk_fwd(ctypes.byref(a)), "powers of 2")
    a = _fake_fwd_args()
    a.csr.sub_block = 8
    refused(lib.dk_fwd(ctypes.byref(a)), "sub_block must be 0, or 16 / 32")
    a = _fake_fwd_args()
    a.seqs.max_k_len = 4096
    refused(lib.dk_fwd(ctypes.byref(a)), "larger than the maximum length")
    a = _fake_fwd_args()
    a.seqs.k_ends = None
    refused(lib.dk_fwd(ctypes.byref(a)), "must be given together")
    a = _fake_fwd_args()
    a.q.ptr = None
    refused(lib.dk_fwd(ctypes.byref(a)), "q/k/v/o is NULL")
    # nothing to do is not an error, whatever the pointers are
    a = _fake_fwd_args(B=0)
    a.q.ptr = None
    assert lib.dk_fwd(ctypes.byref(a)) == 0

    # paged decode
    a = _fake_fwd_args()
    pg = _lib.PagedKV(0x10000, 128, 16 * 2 * 128, 16 * 2 * 128, 16, 0, 1.0, 1.0)
    refused(lib.dk_fwd_paged(ctypes.byref(a), None), "page table is NULL")
    pg.page_size = 24
    refused(lib.dk_fwd_paged(ctypes.byref(a), ctypes.byref(pg)), "power of two >= 16, got 24")
    pg.page_size, pg.kv_dtype = 16, 1
    refused(lib.dk_fwd_paged(ctypes.byref(a), ctypes.byref(pg)), "kv_dtype must be the q dtype")
    pg.kv_dtype, pg.k_scale = _lib.DK_FP8_E4M3, 0.0
    refused(lib.dk_fwd_paged(ctypes.byref(a), ctypes.byref(pg)), "scales must be positive")
    pg.kv_dtype, pg.k_scale = 0, 1.0
    refused(lib.dk_fwd_paged(ctypes.byref(a), ctypes.byref(pg)), "decode workspace too small")
    a.seqs.q_starts = a.seqs.q_ends = a.seqs.k_starts = a.seqs.k_ends = None
    a.seqs.max_q_len = a.seqs.max_k_len
    refused(lib.dk_fwd_paged(ctypes.byref(a), ctypes.byref(pg)), "per-sequence lengths")

    # workspace queries: decode-shaped calls ask for [batch][q heads][units][D + 2] floats
    a = _fake_fwd_args(B=2, Hq=8, Hkv=2, D=128, max_row=10)
    need = lib.dk_fwd_workspace_bytes(ctypes.byref(a))
    assert need > 0 and need % (2 * 8 * 130 * 4) == 0 and need // (2 * 8 * 130 * 4) >= 4
    a.seqs.packed = 4                          # rows without a query to be cleared: the prefill kernels' job
    assert lib.dk_fwd_workspace_bytes(ctypes.byref(a)) == 0
    a.seqs.packed = 0
    a.seqs.max_q_len = 7                       # neither decode nor prefill of the same length
    assert lib.dk_fwd_workspace_bytes(ctypes.byref(a)) == 0
    a = _fake_fwd_args(D=160)                  # head dims above 128 decode on 256-wide tiles
    assert lib.dk_fwd_workspace_bytes(ctypes.byref(a)) > 0
    a = _fake_fwd_args(D=164)                  # not a multiple of 8: no matrix-core decode kernel
    assert lib.dk_fwd_workspace_bytes(ctypes.byref(a)) == 0

    # backward: paddings are refused as in the reference; GQA asks for fp32 per-head partials
    b = _lib.BwdArgs()
    t = _lib.Tensor(0x10000, 1024 * 8 * 128, 128, 8 * 128)
    tk = _lib.Tensor(0x10000, 1024 * 2 * 128, 128, 2 * 128)
    b.q, b.o, b.dout, b.dq = t, t, t, t
    b.k, b.v, b.dk, b.dv = tk, tk, tk, tk
    b.lse = _lib.RowVec(0x10000, 8 * 1024, 1024, 1)
    b.dlse = _lib.RowVec(None, 0, 0, 0)
    b.delta = 0x10000
    b.csr = _lib.Lut(0x10000, 0x10000, 17, 1024, 1, 2, 16, 64, 64, 1, 0, 0)
    b.csc = _lib.Lut(0x10000, 0x10000, 17, 1024, 1, 2, 16, 64, 64, 1, 0, 0)
    b.seqs = _lib.Seqs(3, 1024, 1024, 0, None, None, None, None)
    b.num_q_heads, b.num_kv_heads, b.head_dim, b.dtype, b.causal, b.impl, b.sm_scale = 8, 2, 128, 0, 1, 0, 0.1
    assert lib.dk_bwd_workspace_bytes(ctypes.byref(b)) == 2 * 3 * 8 * 1024 * 128 * 4
    b.num_kv_heads = 8
    b.csr.num_heads = b.csc.num_heads = 8
    assert lib.dk_bwd_workspace_bytes(ctypes.byref(b)) == 0
    b.seqs = _lib.Seqs(3, 1024, 1024, 0, 0x10000, 0x10000, 0x10000, 0x10000)
    refused(lib.dk_bwd(ctypes.byref(b)), "does not support paddings")
    b.seqs = _lib.Seqs(3, 1024, 1024, 0, None, None, None, None)
    b.csc.entry_width = 2
    refused(lib.dk_bwd(ctypes.byref(b)), "csc table cannot carry values")
    b.csc.entry_width = 1
    b.delta = None
    refused(lib.dk_bwd(ctypes.byref(b)), "lse / delta is NULL")


def test_cpu_tensors_are_refused_loudly():
    m = LocalStrideSparseAttention(2, 128, 64, 1, 2)
    x = torch.zeros(1, 128, 2, 64)
    with pytest.raises(RuntimeError, match="no CPU execution path"):
        m(x, x, x)


def test_combine_matches_closed_form():
    g = torch.Generator().manual_seed(0)
    o = [torch.randn(2, 3, 5, 4, generator=g) for _ in range(3)]
    l = [torch.randn(2, 3, 5, generator=g) for _ in range(3)]
    l[1][0, 0, 0] = float("-inf")
    got = combine_attn_partitions(*zip(o, l))
    w = torch.softmax(torch.stack(l), 0)
    want = (torch.stack(o) * w[..., None]).sum(0)
    assert torch.allclose(got, want, atol=1e-6)
    # (batch, seq, heads, dim) outputs with (batch, heads, seq) log-sum-exps
    got2 = combine_attn_partitions(*[(x.transpose(1, 2), y) for x, y in zip(o, l)], hdim=2)
    assert torch.allclose(got2, want.transpose(1, 2), atol=1e-6)
    # packed (tokens, heads, dim) outputs with (heads, tokens) log-sum-exps
    got3 = combine_attn_partitions(*[(x[0].transpose(0, 1), y[0]) for x, y in zip(o, l)])
    assert torch.allclose(got3, want[0].transpose(0, 1), atol=1e-6)
    # every partition empty for a row -> 0, not NaN
    l2 = [x.clone() for x in l]
    for x in l2:
        x[1, 2, 3] = float("-inf")
    assert torch.isfinite(combine_attn_partitions(*zip(o, l2))).all()


def test_longest_first_order_of_a_table():
    """ops._lut(longest_first=True): a permutation of the table rows of every head by descending
    length, equal lengths in index order (what the dK/dV pass hands out)."""
    from dkernel_amd import ops
    from dkernel_amd.utils import dense_to_ccol_row, get_sparse_attn_mask
    _, mask, _ = get_sparse_attn_mask(4, 1024, block_size=64, local_blocks=2, vert_stride=4, dtype=torch.uint8)
    ccol, row = dense_to_ccol_row(mask.to(torch.uint8))
    lut = ops._lut((ccol, row, 64, 64), ccol.device, longest_first=True)
    # 16 rows, followed by the 8 pairs of rows (2u, 2u + 1) in the order of the pairs' lengths
    assert lut.row_order and lut.row_order_stride_h == 24 and lut.pair_order == lut.row_order + 4 * 16
    both = np.ctypeslib.as_array(ctypes.cast(lut.row_order, ctypes.POINTER(ctypes.c_int32)), shape=(ccol.size(0), 24))
    lens = (ccol[:, 1:] - ccol[:, :-1]).numpy()
    for order, lens_of in ((both[:, :16], lens), (both[:, 16:], lens[:, 0::2] + lens[:, 1::2])):
        n = order.shape[1]
        for h in range(ccol.size(0)):
            assert sorted(order[h]) == list(range(n))
            got = lens_of[h][order[h]]
            assert (np.diff(got) <= 0).all()
            for a, b in zip(order[h][:-1], order[h][1:]):
                assert lens_of[h][a] > lens_of[h][b] or a < b
    plain = ops._lut((ccol, row, 64, 64), ccol.device)
    assert not plain.row_order and not plain.pair_order


def test_which_patterns_start_their_long_rows_first():
    from dkernel_amd.interface import _unsorted_rows
    for kw in (dict(), dict(homo_head=True), dict(head_sliding_offset=1), dict(num_dense_heads=2), dict(causal=False)):
        for local, vert in ((2, 4), (8, 8), (1, 3), (16, 1)):
            mask = torch.from_numpy(OL.block_mask(8, 4096, 64, local, vert, **kw).astype("uint8"))
            assert not _unsorted_rows(mask), (kw, local, vert)
    i = torch.arange(64)
    window = (i[:, None] - i[None, :]).abs() <= 3
    with_global = window.clone()
    with_global[:2, :] = True
    with_global[:, :2] = True
    assert not _unsorted_rows(window[None].to(torch.uint8))
    assert _unsorted_rows(with_global[None].to(torch.uint8))           # global rows first, the longest by far
    assert not _unsorted_rows((with_global & (i[:, None] >= i[None, :]))[None].to(torch.uint8))  # causal: rows only grow


def test_which_patterns_count_as_uneven():
    mask = lambda **kw: torch.from_numpy(OL.block_mask(8, 2048, 64, 2, 4, **kw).astype("uint8"))  # noqa: E731
    assert not _uneven_heads(mask())
    assert not _uneven_heads(mask(homo_head=True))
    assert not _uneven_heads(mask(head_sliding_offset=1))
    assert _uneven_heads(mask(num_dense_heads=1))
    assert _uneven_heads(mask(num_dense_heads=4))
    assert not _uneven_heads(mask(num_dense_heads=8))  # every head dense: even again
