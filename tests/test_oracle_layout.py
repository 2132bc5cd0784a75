"""Pins oracle/layout.py: reference KATs, golden fixtures, library routines,
brute force and invariants (CPU only)."""
import itertools
import zlib

import numpy as np
import pytest
import scipy.sparse

from oracle import layout as OL
from conftest import mask_kwargs

# literal masks of the reference's tests/test_utils.py:24-34 and :55-64
KAT_CAUSAL = np.array(
    [[1, 0, 0, 0, 0, 0, 0, 0],
     [1, 1, 0, 0, 0, 0, 0, 0],
     [1, 1, 1, 0, 0, 0, 0, 0],
     [1, 0, 1, 1, 0, 0, 0, 0],
     [1, 0, 0, 1, 1, 0, 0, 0],
     [1, 0, 0, 1, 1, 1, 0, 0],
     [1, 0, 0, 1, 0, 1, 1, 0],
     [1, 0, 0, 1, 0, 0, 1, 1]], dtype=np.uint8)
KAT_BIDIR = np.array(
    [[1, 1, 0, 0, 1, 0, 0, 1],
     [1, 1, 1, 0, 0, 1, 0, 0],
     [0, 1, 1, 1, 0, 0, 1, 0],
     [0, 0, 1, 1, 1, 0, 0, 1],
     [1, 0, 0, 1, 1, 1, 0, 0],
     [0, 1, 0, 0, 1, 1, 1, 0],
     [0, 0, 1, 0, 0, 1, 1, 1],
     [1, 0, 0, 1, 0, 0, 1, 1]], dtype=np.uint8)


def test_kat_causal():
    m = OL.block_mask(2, 16, block_size=2, local_blocks=2, vert_stride=3, causal=True, homo_head=True)
    assert m.shape == (1, 8, 8) and (m[0] == KAT_CAUSAL).all()


def test_kat_bidirectional():
    m = OL.block_mask(2, 16, block_size=2, local_blocks=2, vert_stride=3, causal=False, homo_head=True)
    assert m.shape == (1, 8, 8) and (m[0] == KAT_BIDIR).all()


def test_mask_fixtures(lut_fixtures):
    z, meta = lut_fixtures
    for name, kw in meta["mask"].items():
        kw = mask_kwargs(kw)
        bm = OL.block_mask(**kw)
        assert bm.shape == z[f"mask/{name}/block_mask"].shape, name
        assert (bm == z[f"mask/{name}/block_mask"]).all(), name
        crow, col = OL.csr_from_dense(bm)
        assert crow.dtype == np.int32 and col.dtype == np.int32
        assert (crow == z[f"mask/{name}/crow"]).all() and (col == z[f"mask/{name}/col"]).all(), name
        ccol, row = OL.csc_from_dense(bm)
        assert (ccol == z[f"mask/{name}/ccol"]).all() and (row == z[f"mask/{name}/row"]).all(), name
        assert OL.kv_cache_efficient(bm, kw["block_size"], kw["block_size"]) == bool(z[f"mask/{name}/kv_eff"]), name


def test_tile_fixtures(lut_fixtures):
    z, meta = lut_fixtures
    for name, t in meta["tile"].items():
        crow, col = OL.merge_split_blocks(t["block_size"], z[f"tile/{name}/pattern"], t["block_m"], t["block_n"])
        assert crow.shape == z[f"tile/{name}/crow"].shape and col.shape == z[f"tile/{name}/col"].shape, name
        assert (crow == z[f"tile/{name}/crow"]).all(), name
        assert (col == z[f"tile/{name}/col"]).all(), name


def test_headline_lut_crc(lut_fixtures):
    z, meta = lut_fixtures
    bm = OL.block_mask(**meta["c1"])
    crow, col = OL.csr_from_dense(bm)
    ccol, row = OL.csc_from_dense(bm)
    assert (crow == z["c1/crow"]).all() and (ccol == z["c1/ccol"]).all()
    crc = [zlib.crc32(np.ascontiguousarray(x).tobytes()) for x in (bm, col, row)]
    assert crc == list(z["c1/crc"])
    assert list(z["c1/shapes"]) == [*col.shape, *row.shape]
    # 87008 active blocks per batch element, the count the FLOP figure is built on
    assert int(crow[:, -1].sum()) == 87008
    assert col.shape == (32, 2768)


def test_c0_block_counts():
    bm = OL.block_mask(8, 1024, 64, 4, 4)
    assert bm.sum((1, 2)).tolist() == [82, 73, 76, 79, 82, 73, 76, 79]


@pytest.mark.parametrize("seed", range(4))
def test_csr_matches_scipy(seed):
    rng = np.random.default_rng(seed)
    x = (rng.random((3, 9, 13)) < 0.3).astype(np.uint8)
    x[1] = 0                                       # an empty head
    crow, col = OL.csr_from_dense(x)
    width = col.shape[1]
    for h in range(3):
        s = scipy.sparse.csr_matrix(x[h])
        s.sort_indices()
        assert (crow[h] == s.indptr).all()
        assert (col[h, :s.nnz] == s.indices).all() and (col[h, s.nnz:] == -1).all()
    assert width == max(int(x[h].sum()) for h in range(3))
    ccol, row = OL.csc_from_dense(x)
    for h in range(3):
        s = scipy.sparse.csc_matrix(x[h])
        s.sort_indices()
        assert (ccol[h] == s.indptr).all() and (row[h, :s.nnz] == s.indices).all()
    assert (OL.lut_to_block_mask(crow, col, 13) == x).all()


def test_invariants():
    # vert_stride = 1 collapses to dense causal (reference tests/test_sparse_attn.py:137-139)
    m = OL.block_mask(4, 640, 64, 3, 1)
    assert (m == np.tril(np.ones((10, 10), dtype=np.uint8))[None]).all()
    # GQA: q heads of a group share the pattern; dense heads are the last kv heads
    m = OL.block_mask(8, 1024, 64, 2, 4, num_kv_heads=4, num_dense_heads=1)
    for g in range(4):
        assert (m[2 * g] == m[2 * g + 1]).all()
    assert (m[6] == np.tril(np.ones((16, 16), dtype=np.uint8))).all()
    assert not (m[0] == m[6]).all()
    # every causal local-stride mask is KV-cache efficient
    for hs in (0, 1, 5):
        assert OL.kv_cache_efficient(OL.block_mask(8, 2048, 64, 4, 8, head_sliding_offset=hs), 64, 64)
    # head_sliding_offset shifts the vertical columns: offset o at head h == offset 0 at head h+o (step 1)
    a = OL.block_mask(8, 1024, 64, 2, 8, head_sliding_offset=0)
    b = OL.block_mask(8, 1024, 64, 2, 8, head_sliding_offset=3)
    assert (b[:5] == a[3:]).all()


def test_partition_masks_concatenate():
    # reference tests/test_seq_partition.py:161-169
    H, L, bs, parts = 3, 1024, 32, 4
    full = OL.block_mask(H, L, bs, 4, 4)
    chunk = L // parts
    for qc in range(parts):
        pieces = [OL.block_mask(H, chunk, bs, 4, 4, q_start_position=qc * chunk,
                                kv_start_position=kc * chunk, kv_seqlen=chunk) for kc in range(qc + 1)]
        cat = np.concatenate(pieces, -1)
        rows = full[:, qc * (chunk // bs):(qc + 1) * (chunk // bs), :cat.shape[-1]]
        assert (cat == rows).all()


@pytest.mark.parametrize("bs,bm,bn", [(16, 64, 16), (32, 64, 16), (32, 16, 16), (16, 16, 8), (32, 128, 32)])
def test_merge_split_brute_force(bs, bm, bn):
    """Expand the tile LUT back to tokens and compare with the token mask of the
    block pattern: every token pair allowed by the pattern (and causal) must be
    covered by a listed tile within its micro_M rows, and no listed tile may lie
    wholly above the diagonal."""
    H, L = 2, 256
    pattern = OL.block_mask(H, L, bs, 2, 3)
    tok = OL.token_mask(pattern, bs, L)
    crow, col = OL.merge_split_blocks(bs, pattern, bm, bn)
    merged = col.ndim == 3
    cover = np.zeros_like(tok)
    for h in range(H):
        for r in range(crow.shape[1] - 1):
            for e in range(crow[h, r], crow[h, r + 1]):
                c = col[h, e, 0] if merged else col[h, e]
                micro = col[h, e, 1] if merged else bm
                assert c >= 0 and 0 < micro <= bm
                assert (r + 1) * bm > c * bn                      # not wholly above the diagonal
                cover[h, r * bm:r * bm + micro, c * bn:(c + 1) * bn] = 1
    cover *= np.tril(np.ones((L, L), dtype=cover.dtype))[None]
    # tiles listed may include token pairs outside the block pattern only when merging rows
    assert (cover >= tok).all()
    if not merged:
        assert (cover == tok).all()
    else:
        # rows beyond micro_M of a merged tile are excluded; within them the block pattern decides
        sub = np.kron(pattern, np.ones((bs, bs), dtype=np.uint8)) * np.tril(np.ones((L, L), dtype=np.uint8))[None]
        assert (sub == tok).all()


def test_kv_cache_efficient_brute_force():
    rng = np.random.default_rng(0)
    for _ in range(50):
        p = np.tril((rng.random((1, 6, 6)) < 0.5).astype(np.uint8))
        want = True
        for i, j in itertools.product(range(1, 6), range(6)):
            if i * 4 >= (j + 1) * 4 and p[0, i, j] > p[0, i - 1, j]:
                want = False
        assert OL.kv_cache_efficient(p, 4, 4) == want
