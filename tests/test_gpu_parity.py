"""GPU parity tests: the HIP path (through the module API and the C ABI)
against the fp32 dense oracle on identical seeded inputs.  Bar: O and
dQ/dK/dV within 2e-2 abs/rel, LSE within 1e-3 (fp32 inputs: 2e-4)."""
import math

import numpy as np
import pytest
import torch

from dkernel_amd import LocalStrideSparseAttention, SparseAttention, combine_attn_partitions, get_sparse_attn_mask
from dkernel_amd import _lib, ops
from oracle import attention as OA
from oracle import layout as OL
from helpers import F32_TOL, LSE_TOL, TOL, assert_close, expand_heads, make_qkv, oracle_fwd

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(params=["generic", "auto"])
def impl(request):
    ops.set_impl(request.param)
    yield request.param
    ops.set_impl("auto")


def _tol(dtype):
    return F32_TOL if dtype == torch.float32 else TOL


def _module(Hq, L, bs, local, vert, **kw):
    # the class is lru_cached on its constructor arguments
    return LocalStrideSparseAttention(Hq, L, bs, local, vert, **kw).to(DEV)


def _block_mask(Hq, L, bs, local, vert, **kw):
    kw = {k: v for k, v in kw.items() if k in ("homo_head", "num_kv_heads", "num_dense_heads",
                                                "head_sliding_offset", "causal")}
    L = ((L + max(bs, 64) - 1) // max(bs, 64)) * max(bs, 64)
    return expand_heads(OL.block_mask(Hq, L, bs, local, vert, **kw), Hq)


def run_fwd_bwd(B, Hq, Hkv, L, D, dtype, bs=64, local=4, vert=4, seq_dim=1, backward=True,
                non_contiguous=False, with_dlse=False, **mkw):
    print(f"case B={B} Hq={Hq} Hkv={Hkv} L={L} D={D} {dtype} bs={bs} local={local} vert={vert} "
          f"seq_dim={seq_dim} nc={non_contiguous} {mkw}", flush=True)
    sm_scale = 1.0 / math.sqrt(D)
    if non_contiguous:
        q, k, v, do = make_qkv(B, L + 19, L + 19, Hq + 3, Hkv + 3, D, dtype, seq_dim, with_do=True)
        sl = (slice(None), slice(0, L), slice(0, Hq)) if seq_dim == 1 else (slice(None), slice(0, Hq), slice(0, L))
        slk = (slice(None), slice(0, L), slice(0, Hkv)) if seq_dim == 1 else (slice(None), slice(0, Hkv), slice(0, L))
        q, k, v, do = q[sl], k[slk], v[slk], do[sl]
    else:
        q, k, v, do = make_qkv(B, L, L, Hq, Hkv, D, dtype, seq_dim, with_do=True)
    kw = dict(mkw)
    if Hkv != Hq:
        kw["num_kv_heads"] = Hkv
    mod = _module(Hq, L, bs, local, vert, seq_dim=seq_dim, **kw)
    bm = _block_mask(Hq, L, bs, local, vert, **kw)
    causal = kw.get("causal", True)

    qo, ko, vo = (x.clone().float().requires_grad_(backward) for x in (q, k, v))
    ref_o, ref_lse = oracle_fwd(qo, ko, vo, bm, bs, sm_scale, seq_dim, causal=causal)

    qd, kd, vd = (x.to(DEV).requires_grad_(backward) for x in (q, k, v))
    out, lse = mod(qd, kd, vd, sm_scale, return_lse=True)
    tol = _tol(dtype)
    assert out.shape == q.shape and out.dtype == dtype
    assert_close("O", out, ref_o, **tol)
    assert_close("LSE", lse, ref_lse, atol=LSE_TOL if dtype != torch.float32 else 1e-4, rtol=0)
    if not backward:
        return
    dlse = None
    if with_dlse:
        dlse = torch.randn(ref_lse.shape, generator=torch.Generator().manual_seed(7))
        (ref_o * do.float()).sum().add((ref_lse * dlse).sum()).backward()
        (out.float() * do.to(DEV).float()).sum().add((lse * dlse.to(DEV)).sum()).backward()
    else:
        ref_o.backward(do.float())
        out.backward(do.to(DEV))
    assert_close("dV", vd.grad, vo.grad, **tol)
    assert_close("dK", kd.grad, ko.grad, **tol)
    assert_close("dQ", qd.grad, qo.grad, **tol)


def test_c0_fp32_plumbing(impl):
    """B1 L1024 H8 d64 fp32, bs64 local4 vert4, heterogeneous heads, LSE."""
    run_fwd_bwd(1, 8, 8, 1024, 64, torch.float32, 64, 4, 4, backward=False)


@pytest.mark.parametrize("dtype,D,bs", [
    (torch.bfloat16, 128, 64), (torch.float16, 64, 64), (torch.float32, 64, 64),
    (torch.bfloat16, 256, 32), (torch.bfloat16, 128, 16), (torch.bfloat16, 64, 128),
])
def test_dims_dtypes_block_sizes(impl, dtype, D, bs):
    run_fwd_bwd(2, 4, 4, 512, D, dtype, bs, 2, 4)


@pytest.mark.parametrize("D,dtype", [(48, torch.float32), (96, torch.bfloat16), (160, torch.bfloat16),
                                     (192, torch.float16)])
def test_dims_not_power_of_two(impl, D, dtype):
    run_fwd_bwd(1, 2, 2, 384, D, dtype, 64, 2, 3, homo_head=(D < 100))


@pytest.mark.parametrize("D,dtype", [(96, torch.bfloat16), (48, torch.float16), (80, torch.bfloat16),
                                     (8, torch.float16), (120, torch.bfloat16)])
def test_head_dims_below_tile_width(impl, D, dtype):
    """Head dims that are multiples of 8 below 64 / 128 run the matrix-core kernels zero-padded
    on chip: GQA group of 4 (shared K/V tiles), MHA (software-pipelined forward), ragged length,
    blocks of 128 on split tiles, non-causal."""
    run_fwd_bwd(2, 8, 2, 512, D, dtype, 64, 2, 4)
    run_fwd_bwd(1, 4, 4, 1000, D, dtype, 64, 3, 3)
    run_fwd_bwd(1, 4, 2, 777, D, dtype, 128, 1, 2, non_contiguous=True)
    run_fwd_bwd(1, 2, 2, 512, D, dtype, 64, 2, 4, causal=False)


def test_matrix_core_kernels_take_padded_dims_and_split_blocks():
    """With the implementation forced to the matrix-core kernels (no generic fallback), padded
    head dims and 128-blocks must run, and a head dim they do not cover must be refused."""
    ops.set_impl("mfma")
    try:
        run_fwd_bwd(1, 8, 2, 512, 96, torch.bfloat16, 64, 2, 4)
        run_fwd_bwd(1, 4, 4, 512, 48, torch.float16, 128, 1, 2)
        # blocks of 16 / 32: tile tables with a bit mask per entry, forward and backward
        run_fwd_bwd(2, 8, 2, 1000, 128, torch.bfloat16, 16, 5, 7)
        run_fwd_bwd(1, 4, 4, 777, 64, torch.float16, 32, 3, 3)
        run_fwd_bwd(1, 2, 2, 512, 128, torch.bfloat16, 16, 3, 9, causal=False)
        # ... together with head dims below the tile width
        run_fwd_bwd(2, 8, 2, 1000, 96, torch.bfloat16, 16, 5, 7)
        run_fwd_bwd(1, 4, 4, 777, 40, torch.float16, 32, 3, 3)
        run_fwd_bwd(1, 4, 1, 640, 120, torch.bfloat16, 32, 2, 5)
        run_fwd_bwd(1, 2, 2, 512, 80, torch.float16, 16, 3, 9, causal=False)
        # head dims above 128 run at the 256-wide tile
        run_fwd_bwd(1, 2, 2, 256, 160, torch.bfloat16, 64, 2, 4)
        with pytest.raises(Exception, match="no MFMA"):
            run_fwd_bwd(1, 2, 2, 256, 100, torch.bfloat16, 64, 2, 4)   # not a multiple of 8
    finally:
        ops.set_impl("auto")


@pytest.mark.parametrize("L", [15, 100, 1028, 777])
def test_ragged_lengths(impl, L):
    run_fwd_bwd(2, 4, 4, L, 128, torch.bfloat16, 64 if L != 1028 else 32, 2, 4)


def test_gqa(impl):
    run_fwd_bwd(2, 8, 2, 512, 128, torch.bfloat16, 64, 3, 4)


def test_gqa_backward_with_and_without_scratch(monkeypatch):
    """dk_bwd sums dK/dV over a kv group either inside one workgroup (no scratch) or from
    per-q-head partials (scratch given): both must meet the oracle, for plain and padded dims."""
    for use in (True, False):
        monkeypatch.setattr(ops, "_bwd_workspace", use)
        run_fwd_bwd(2, 8, 2, 1024, 128, torch.bfloat16, 64, 3, 4)
        run_fwd_bwd(1, 6, 2, 777, 96, torch.float16, 64, 2, 3)
        run_fwd_bwd(1, 8, 1, 512, 64, torch.bfloat16, 64, 2, 4, seq_dim=2, non_contiguous=True)


def test_patterns(impl):
    run_fwd_bwd(1, 8, 8, 1024, 128, torch.bfloat16, 64, 10, 3)
    run_fwd_bwd(1, 8, 8, 1024, 128, torch.bfloat16, 64, 1, 8)
    run_fwd_bwd(1, 8, 8, 1024, 128, torch.bfloat16, 64, 8, 1)
    run_fwd_bwd(1, 8, 8, 1024, 128, torch.bfloat16, 64, 4, 4, num_dense_heads=2)
    run_fwd_bwd(1, 8, 8, 1024, 128, torch.bfloat16, 64, 4, 4, homo_head=True)
    run_fwd_bwd(1, 8, 8, 1024, 128, torch.bfloat16, 64, 2, 8, head_sliding_offset=3)


def test_seq_dim_and_non_contiguous(impl):
    run_fwd_bwd(2, 4, 4, 512, 128, torch.bfloat16, 64, seq_dim=2)
    run_fwd_bwd(2, 4, 4, 512, 128, torch.bfloat16, 64, seq_dim=1, non_contiguous=True)
    run_fwd_bwd(2, 4, 4, 512, 128, torch.bfloat16, 64, seq_dim=2, non_contiguous=True)


def test_keys_broadcast_along_tokens(impl):
    """K and V expanded along the token dim (token stride 0): every row of a K/V tile is the
    same memory, which the tile copies' 32-bit row offsets must handle like any other stride."""
    B, H, L, D = 1, 2, 256, 128
    sm_scale = 1.0 / math.sqrt(D)
    q, k, v = make_qkv(B, L, L, H, H, D, torch.bfloat16)
    k1, v1 = k[:, :1], v[:, :1]
    mod = _module(H, L, 64, 2, 2)
    ref_o, ref_lse = oracle_fwd(q.float(), k1.expand(-1, L, -1, -1).float(), v1.expand(-1, L, -1, -1).float(),
                                _block_mask(H, L, 64, 2, 2), 64, sm_scale)
    kd, vd = k1.to(DEV).expand(-1, L, -1, -1), v1.to(DEV).expand(-1, L, -1, -1)
    assert kd.stride(1) == 0
    out, lse = mod(q.to(DEV), kd, vd, sm_scale, return_lse=True)
    assert_close("O", out, ref_o, **TOL)
    assert_close("LSE", lse, ref_lse, atol=LSE_TOL, rtol=0)


def test_noncausal(impl):
    run_fwd_bwd(1, 2, 2, 1024, 64, torch.float16, 64, 4, 8, causal=False)
    run_fwd_bwd(1, 1, 1, 1024, 64, torch.float16, 32, 4, 10000, causal=False)


@pytest.mark.parametrize("bs,bm,bn", [(16, 16, 16), (16, 128, 16), (64, 128, 32), (16, 64, 16)])
def test_kernel_tile_sizes(impl, bs, bm, bn):
    run_fwd_bwd(1, 2, 2, 1024, 128, torch.bfloat16, bs, 2, 4, block_m=bm, block_n=bn)
    run_fwd_bwd(1, 2, 2, 1024, 128, torch.bfloat16, bs, 1, 4, block_m=bm, block_n=bn)


@pytest.mark.parametrize("bs,bm,bn", [(16, 128, 16), (64, 128, 32), (32, 64, 32), (128, 128, 64)])
def test_kernel_tile_sizes_on_the_matrix_cores(bs, bm, bn):
    """Tile sizes given by the caller do not keep a local-stride pattern off the matrix-core
    kernels (forced here): they run their own 64 x 64 tiles over the same blocks."""
    ops.set_impl("mfma")
    try:
        run_fwd_bwd(1, 4, 2, 1024, 128, torch.bfloat16, bs, 2, 4, block_m=bm, block_n=bn)
        run_fwd_bwd(1, 2, 2, 1000, 96, torch.float16, bs, 1, 3, block_m=bm, block_n=bn)
    finally:
        ops.set_impl("auto")


@pytest.mark.parametrize("bs,D,dtype", [(128, 128, torch.bfloat16), (256, 128, torch.bfloat16),
                                        (128, 64, torch.float16)])
def test_large_blocks_run_on_split_tiles(impl, bs, D, dtype):
    """Pattern blocks of 128 / 256 are split into the 64 x 64 tiles of the
    matrix-core kernels (forward CSR and backward CSC); results must equal the
    dense oracle of the unsplit pattern."""
    mod = _module(8, 1024, bs, 2, 4, num_kv_heads=2)
    assert mod.kernel_tile == 64 and mod.block_m == bs and mod.block_n == bs
    assert mod.kernel_csr_crow.shape[-1] == 1024 // 64 + 1
    run_fwd_bwd(2, 8, 2, 1024, D, dtype, bs, 2, 4)
    run_fwd_bwd(1, 4, 4, 1000, D, dtype, bs, 1, 3, num_dense_heads=1)
    run_fwd_bwd(1, 2, 2, 1024, D, dtype, bs, 2, 4, causal=False)


def test_grad_through_lse(impl):
    run_fwd_bwd(1, 4, 4, 512, 64, torch.float32, 64, 2, 4, with_dlse=True)
    run_fwd_bwd(1, 4, 2, 512, 128, torch.bfloat16, 64, 2, 4, with_dlse=True)


def test_packed_qkv_and_kv(impl):
    B, H, L, D = 2, 4, 512, 128
    q, k, v, do = make_qkv(B, L, L, H, H, D, torch.bfloat16, 1, with_do=True)
    mod = _module(H, L, 64, 2, 4)
    qd, kd, vd = (x.to(DEV).requires_grad_() for x in (q, k, v))
    mod(qd, kd, vd).backward(do.to(DEV))
    qkv = torch.cat([q, k, v], dim=2).to(DEV).requires_grad_()
    out = mod(qkv, split_qkv=lambda x: x.chunk(3, dim=2))
    out.backward(do.to(DEV))
    dq, dk, dv = qkv.grad.chunk(3, dim=2)
    assert torch.equal(dq, qd.grad) and torch.equal(dk, kd.grad) and torch.equal(dv, vd.grad)
    kv = torch.cat([k, v], dim=2).to(DEV).requires_grad_()
    q2 = q.to(DEV).requires_grad_()
    mod(q2, kv, split_qkv=lambda x: x.chunk(2, dim=2)).backward(do.to(DEV))
    dk, dv = kv.grad.chunk(2, dim=2)
    assert torch.equal(q2.grad, qd.grad) and torch.equal(dk, kd.grad) and torch.equal(dv, vd.grad)


# ----------------------------------------------------------------------------
# inference: paddings, packed variable length, decode
# ----------------------------------------------------------------------------

def _seq_oracle(q, k, v, bm, bs, sm_scale, causal=True):
    """One sequence, (L, H, D) tensors, queries = last positions of the keys."""
    mask = OA.sequence_token_mask(bm, bs, q.shape[0], k.shape[0], causal=causal)
    o, lse = OA.dense_attention(q[None], k[None], v[None], torch.from_numpy(mask), sm_scale, seq_dim=1)
    return o[0], lse[0]


@pytest.mark.parametrize("seq_dim,bs,dtype,homo", [(1, 64, torch.bfloat16, False), (2, 16, torch.float16, True)])
def test_left_padded_prefill(impl, seq_dim, bs, dtype, homo):
    B, Hq, Hkv, L, D = 3, 4, 2, 640, 128
    sm = 1 / math.sqrt(D)
    q, k, v = make_qkv(B, L, L, Hq, Hkv, D, dtype, 1)
    lens = [640, 333, 1]
    mod = _module(Hq, 1024, bs, 2, 4, num_kv_heads=None if homo else Hkv, homo_head=homo, seq_dim=seq_dim)
    bm = _block_mask(Hq, 1024, bs, 2, 4, num_kv_heads=None if homo else Hkv, homo_head=homo)
    qp, kp, vp = (torch.zeros_like(x) for x in (q, k, v))
    for i, l in enumerate(lens):
        qp[i, L - l:], kp[i, L - l:], vp[i, L - l:] = q[i, :l], k[i, :l], v[i, :l]
    tr = (lambda x: x.transpose(1, 2)) if seq_dim == 2 else (lambda x: x)
    out, lse = mod(tr(qp).to(DEV), tr(kp).to(DEV), tr(vp).to(DEV), sm,
                   left_paddings=torch.tensor([L - l for l in lens]), return_lse=True)
    out = tr(out)
    for i, l in enumerate(lens):
        ro, rl = _seq_oracle(q[i, :l], k[i, :l], v[i, :l], bm, bs, sm)
        assert_close(f"O[{i}]", out[i, L - l:], ro, **TOL)
        assert_close(f"LSE[{i}]", lse[i, :, L - l:], rl, atol=LSE_TOL, rtol=0)
        assert (out[i, :L - l] == 0).all() and torch.isinf(lse[i, :, :L - l]).all()


def test_right_padded_prefill(impl):
    B, H, L, D, bs = 2, 4, 512, 128, 64
    sm = 1 / math.sqrt(D)
    q, k, v = make_qkv(B, L, L, H, H, D, torch.bfloat16, 2)
    lens = [421, 77]
    mod = _module(H, 1024, bs, 2, 4, seq_dim=2)
    bm = _block_mask(H, 1024, bs, 2, 4)
    out = mod(q.to(DEV), k.to(DEV), v.to(DEV), sm, seqlens=torch.tensor(lens))
    for i, l in enumerate(lens):
        ro, _ = _seq_oracle(q[i, :, :l].transpose(0, 1), k[i, :, :l].transpose(0, 1),
                            v[i, :, :l].transpose(0, 1), bm, bs, sm)
        assert_close(f"O[{i}]", out[i, :, :l].transpose(0, 1), ro, **TOL)
        assert (out[i, :, l:] == 0).all()


@pytest.mark.parametrize("bs,block_m,left", [(64, None, True), (32, None, True), (16, 128, False), (64, None, False),
                                             (128, None, True)])
def test_decode(impl, bs, block_m, left):
    """One new token per sequence over left-padded / right-padded / unpadded KV, GQA."""
    _decode_case(bs, block_m, left, 128)


@pytest.mark.parametrize("D,left", [(96, True), (48, False), (120, True)])
def test_decode_head_dims_below_tile_width(impl, D, left):
    _decode_case(64, None, left, D)


@pytest.mark.parametrize("D,bs,left", [(256, 64, True), (192, 64, False), (160, 32, True), (136, 128, False)])
def test_decode_head_dims_above_128(D, bs, left):
    """Head dims above 128 take the split-KV decode kernels too (256-wide tiles)."""
    _decode_case(bs, None, left, D)
    assert _lib.lib().dk_last_kernels().decode().startswith("decode_partial_kernel [T = dk::bf16_t, D = 256")


@pytest.mark.parametrize("bs,D,left", [(16, 96, True), (32, 40, False)])
def test_decode_small_blocks_with_padded_head_dims(bs, D, left):
    """Blocks of 16 / 32 (masked tiles) and a head dim below the tile width, matrix-core kernels forced."""
    ops.set_impl("mfma")
    try:
        _decode_case(bs, None, left, D)
    finally:
        ops.set_impl("auto")


@pytest.mark.parametrize("page_size,bs,D,head_major", [(16, 64, 128, False), (32, 64, 128, True), (64, 64, 96, False),
                                                        (128, 64, 128, False), (16, 16, 128, False),
                                                        (32, 128, 64, True), (256, 32, 128, False),
                                                        (16, 16, 96, False), (64, 32, 40, True),
                                                        (16, 64, 256, False), (64, 32, 192, True)])
def test_paged_decode(page_size, bs, D, head_major):
    """Single-token decode over a paged K/V cache: pages scattered in the pools, table rows padded
    with -1 past each sequence, pools token-major or head-major inside a page; against the oracle
    on the gathered keys and against padded decode."""
    B, Hq, Hkv, Lmax = 5, 8, 2, 2048
    sm = 1 / math.sqrt(D)
    g = torch.Generator().manual_seed(20)
    lens = [64 * 21 + 12, 2048, 1, 64 * 5, 777]
    q = torch.randn(B, Hq, D, generator=g).to(torch.bfloat16)
    ks = [torch.randn(l, Hkv, D, generator=g).to(torch.bfloat16) for l in lens]
    vs = [torch.randn(l, Hkv, D, generator=g).to(torch.bfloat16) for l in lens]
    pages_per_seq = [-(-l // page_size) for l in lens]
    num_pages = sum(pages_per_seq) + 7
    perm = torch.randperm(num_pages, generator=g).tolist()
    pool_shape = (num_pages, Hkv, page_size, D) if head_major else (num_pages, page_size, Hkv, D)
    k_pool = torch.randn(pool_shape, generator=g).to(torch.bfloat16)   # stale data in unused slots
    v_pool = torch.randn(pool_shape, generator=g).to(torch.bfloat16)
    if head_major:
        k_pool, v_pool = k_pool.transpose(1, 2), v_pool.transpose(1, 2)  # views: (pages, page_size, heads, dim)
    table = torch.full((B, Lmax // page_size + 1), -1, dtype=torch.int32)
    nxt = 0
    for i, l in enumerate(lens):
        for pi in range(pages_per_seq[i]):
            pg = perm[nxt]
            nxt += 1
            table[i, pi] = pg
            n = min(page_size, l - pi * page_size)
            k_pool[pg, :n] = ks[i][pi * page_size: pi * page_size + n]
            v_pool[pg, :n] = vs[i][pi * page_size: pi * page_size + n]
    mod = _module(Hq, Lmax, bs, 2, 4, num_kv_heads=Hkv)
    bm = _block_mask(Hq, Lmax, bs, 2, 4, num_kv_heads=Hkv)
    out, lse = mod.paged_decode(q.to(DEV), k_pool.to(DEV), v_pool.to(DEV), table.to(DEV),
                                torch.tensor(lens, dtype=torch.int32).to(DEV), sm, return_lse=True)
    assert out.shape == (B, Hq, D) and lse.shape == (B, Hq, 1)
    for i, l in enumerate(lens):
        ro, rl = _seq_oracle(q[i:i + 1], ks[i], vs[i], bm, bs, sm)
        assert_close(f"O[{i}]", out[i:i + 1], ro, **TOL)
        assert_close(f"LSE[{i}]", lse[i], rl, atol=LSE_TOL, rtol=0)


def test_paged_decode_empty_context_gives_zero_output():
    """A sequence without any key (context length 0, e.g. a free slot of a serving batch): O = 0,
    LSE = -inf, and its page-table row is not read."""
    B, Hq, Hkv, D, Lmax, page = 3, 8, 2, 128, 256, 16
    g = torch.Generator().manual_seed(20)
    q = torch.randn(B, Hq, D, generator=g).to(torch.bfloat16).to(DEV)
    k_pool = torch.randn(4, page, Hkv, D, generator=g).to(torch.bfloat16).to(DEV)
    v_pool = torch.randn(4, page, Hkv, D, generator=g).to(torch.bfloat16).to(DEV)
    table = torch.full((B, Lmax // page), -1, dtype=torch.int32, device=DEV)
    table[1, 0] = 2
    lens = torch.tensor([0, 5, 0], dtype=torch.int32, device=DEV)
    mod = _module(Hq, Lmax, 64, 2, 4, num_kv_heads=Hkv)
    out, lse = mod.paged_decode(q, k_pool, v_pool, table, lens, 0.1, return_lse=True)
    assert torch.count_nonzero(out[0]) == 0 and torch.count_nonzero(out[2]) == 0
    assert torch.isneginf(lse[0]).all() and torch.isneginf(lse[2]).all()
    ro, rl = _seq_oracle(q[1:2].cpu(), k_pool[2, :5].cpu(), v_pool[2, :5].cpu(),
                         _block_mask(Hq, Lmax, 64, 2, 4, num_kv_heads=Hkv), 64, 0.1)
    assert_close("O[1]", out[1:2], ro, **TOL)
    assert_close("LSE[1]", lse[1], rl, atol=LSE_TOL, rtol=0)


def test_paged_decode_negative_table_entry_reads_page_zero():
    """A page-table slot marked unused (-1) inside a sequence is a caller's mistake; the kernel
    reads page 0 for it instead of an address before the pools."""
    B, Hq, Hkv, D, Lmax, page = 2, 8, 2, 128, 256, 16
    g = torch.Generator().manual_seed(20)
    q = torch.randn(B, Hq, D, generator=g).to(torch.bfloat16).to(DEV)
    k_pool = torch.randn(4, page, Hkv, D, generator=g).to(torch.bfloat16).to(DEV)
    v_pool = torch.randn(4, page, Hkv, D, generator=g).to(torch.bfloat16).to(DEV)
    table = torch.full((B, Lmax // page), -1, dtype=torch.int32, device=DEV)
    mod = _module(Hq, Lmax, 64, 2, 4, num_kv_heads=Hkv)
    out = mod.paged_decode(q, k_pool, v_pool, table, torch.ones(B, dtype=torch.int32, device=DEV), 0.1)
    # one key per sequence: O = V of token 0 of page 0
    want = v_pool[0, 0].repeat_interleave(Hq // Hkv, dim=0)[None].expand(B, Hq, D)
    assert torch.equal(out, want)


@pytest.mark.parametrize("page_size,bs,D,dtype", [(16, 64, 128, torch.bfloat16), (64, 128, 64, torch.float16)])
def test_paged_decode_fp8_cache(page_size, bs, D, dtype):
    """Paged decode over OCP e4m3 K/V pools with per-tensor scales: the oracle attends to the
    dequantised keys and values (byte as e4m3 times the scale), which the kernel reproduces
    exactly before its 16-bit products."""
    B, Hq, Hkv, Lmax = 4, 8, 2, 1024
    sm = 1 / math.sqrt(D)
    g = torch.Generator().manual_seed(20)
    lens = [1000, 65, 1, 513]
    k_scale, v_scale = 0.05, 0.125
    q = torch.randn(B, Hq, D, generator=g).to(dtype)
    ks8 = [(torch.randn(l, Hkv, D, generator=g) / k_scale).to(torch.float8_e4m3fn) for l in lens]
    vs8 = [(torch.randn(l, Hkv, D, generator=g) / v_scale).to(torch.float8_e4m3fn) for l in lens]
    pages_per_seq = [-(-l // page_size) for l in lens]
    num_pages = sum(pages_per_seq) + 3
    perm = torch.randperm(num_pages, generator=g).tolist()
    k_pool = torch.zeros(num_pages, page_size, Hkv, D, dtype=torch.uint8)
    v_pool = torch.zeros_like(k_pool)
    table = torch.full((B, Lmax // page_size), -1, dtype=torch.int32)
    nxt = 0
    for i, l in enumerate(lens):
        for pi in range(pages_per_seq[i]):
            pg = perm[nxt]
            nxt += 1
            table[i, pi] = pg
            n = min(page_size, l - pi * page_size)
            k_pool[pg, :n] = ks8[i][pi * page_size: pi * page_size + n].view(torch.uint8)
            v_pool[pg, :n] = vs8[i][pi * page_size: pi * page_size + n].view(torch.uint8)
    mod = _module(Hq, Lmax, bs, 2, 4, num_kv_heads=Hkv)
    bm = _block_mask(Hq, Lmax, bs, 2, 4, num_kv_heads=Hkv)
    out, lse = mod.paged_decode(q.to(DEV), k_pool.to(DEV).view(torch.float8_e4m3fn),
                                v_pool.to(DEV).view(torch.float8_e4m3fn), table.to(DEV),
                                torch.tensor(lens, dtype=torch.int32).to(DEV), sm, return_lse=True,
                                k_scale=k_scale, v_scale=v_scale)
    for i, l in enumerate(lens):
        kd, vd = ks8[i].float() * k_scale, vs8[i].float() * v_scale
        ro, rl = _seq_oracle(q[i:i + 1].float(), kd, vd, bm, bs, sm)
        assert_close(f"O[{i}]", out[i:i + 1], ro, **TOL)
        assert_close(f"LSE[{i}]", lse[i], rl, atol=LSE_TOL, rtol=0)


def _decode_case(bs, block_m, left, D):
    B, Hq, Hkv, Lmax = 4, 8, 2, 2048
    sm = 1 / math.sqrt(D)
    q, k, v = make_qkv(B, 1, Lmax, Hq, Hkv, D, torch.bfloat16, 1)
    lens = [64 * 21 + 12, 2048, 1, 64 * 5]
    kw = dict(num_kv_heads=Hkv)
    if block_m:
        kw["block_m"] = block_m
    mod = _module(Hq, Lmax, bs, 2, 4, **kw)
    bm = _block_mask(Hq, Lmax, bs, 2, 4, num_kv_heads=Hkv)
    kp, vp = torch.zeros_like(k), torch.zeros_like(v)
    for i, l in enumerate(lens):
        if left:
            kp[i, Lmax - l:], vp[i, Lmax - l:] = k[i, :l], v[i, :l]
        else:
            kp[i, :l], vp[i, :l] = k[i, :l], v[i, :l]
    extra = dict(left_paddings=torch.tensor([Lmax - l for l in lens])) if left else dict(seqlens=torch.tensor(lens))
    out, lse = mod(q.to(DEV), kp.to(DEV), vp.to(DEV), sm, return_lse=True, **extra)
    for i, l in enumerate(lens):
        ro, rl = _seq_oracle(q[i], k[i, :l], v[i, :l], bm, bs, sm)
        assert_close(f"O[{i}]", out[i], ro, **TOL)
        assert_close(f"LSE[{i}]", lse[i], rl, atol=LSE_TOL, rtol=0)
    # unpadded decode through the training entry (q_len 1 < k_len)
    l = lens[0]
    out2 = mod(q[:1].to(DEV), k[:1, :l].to(DEV).contiguous(), v[:1, :l].to(DEV).contiguous(), sm)
    ro, _ = _seq_oracle(q[0], k[0, :l], v[0, :l], bm, bs, sm)
    assert_close("O unpadded", out2[0], ro, **TOL)


@pytest.mark.parametrize("D,bs", [(128, 32), (96, 64), (128, 128)])
def test_packed_varlen_prefill_and_decode(impl, D, bs):
    Hq, Hkv = 4, 2
    sm = 1 / math.sqrt(D)
    lens = [300, 1, 64, 517, 129]
    T = sum(lens)
    g = torch.Generator().manual_seed(20)
    q, k, v = (torch.randn(T, h, D, generator=g).to(torch.bfloat16) for h in (Hq, Hkv, Hkv))
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)
    mod = _module(Hq, 1024, bs, 2, 4, num_kv_heads=Hkv)
    bm = _block_mask(Hq, 1024, bs, 2, 4, num_kv_heads=Hkv)
    out, lse = mod(q.to(DEV), k.to(DEV), v.to(DEV), sm, cu_seqlen_k=cu.to(DEV), return_lse=True)
    assert lse.shape == (Hq, T)
    for i, l in enumerate(lens):
        s, e = int(cu[i]), int(cu[i + 1])
        ro, rl = _seq_oracle(q[s:e], k[s:e], v[s:e], bm, bs, sm)
        assert_close(f"O[{i}]", out[s:e], ro, **TOL)
        assert_close(f"LSE[{i}]", lse[:, s:e], rl, atol=LSE_TOL, rtol=0)
    # decode: one query token per sequence (cu_seqlen_q defaults to arange)
    qd = torch.randn(len(lens), Hq, D, generator=g).to(torch.bfloat16)
    outd = mod(qd.to(DEV), k.to(DEV), v.to(DEV), sm, cu_seqlen_k=cu.to(DEV))
    # one query token per packed sequence takes the split-KV decode kernel whenever 64-tiles apply
    assert (ops.last_fwd_workspace_bytes > 0) == (impl == "auto")
    for i, l in enumerate(lens):
        s, e = int(cu[i]), int(cu[i + 1])
        ro, _ = _seq_oracle(qd[i:i + 1], k[s:e], v[s:e], bm, bs, sm)
        assert_close(f"Od[{i}]", outd[i:i + 1], ro, **TOL)
    # chunked prefill: the last q_len tokens of each sequence
    qlens = [100, 1, 64, 17, 129]
    cuq = torch.tensor([0] + list(np.cumsum(qlens)), dtype=torch.int32)
    qc = torch.cat([q[int(cu[i + 1]) - ql:int(cu[i + 1])] for i, ql in enumerate(qlens)])
    outc = mod(qc.to(DEV), k.to(DEV), v.to(DEV), sm, cu_seqlen_k=cu.to(DEV), cu_seqlen_q=cuq.to(DEV))
    for i, ql in enumerate(qlens):
        assert_close(f"Oc[{i}]", outc[int(cuq[i]):int(cuq[i + 1])], out[int(cu[i + 1]) - ql:int(cu[i + 1])].cpu(),
                     atol=1e-2, rtol=1e-2)


@pytest.mark.parametrize("Hq,Hkv,nseq", [(4, 2, 200), (2, 2, 700)])
def test_packed_prefill_with_hundreds_of_sequences(monkeypatch, Hq, Hkv, nseq):
    """A workgroup finds its sequence by bisecting running tile counts that a small kernel wrote
    into the scratch, or, without scratch, by a wave-wide scan of the lengths: both must place
    every tile (sequences of 0 to 150 tokens, several lanes' worth of them), agree bit for bit,
    and match the generic kernels and the oracle."""
    D, bs = 64, 64
    sm = 1 / math.sqrt(D)
    rng = np.random.default_rng(nseq)
    lens = [int(x) for x in rng.integers(0, 151, nseq)]
    lens[3] = lens[nseq // 2] = lens[-1] = 0
    T = sum(lens)
    g = torch.Generator().manual_seed(20)
    q, k, v = (torch.randn(T, h, D, generator=g).to(torch.bfloat16) for h in (Hq, Hkv, Hkv))
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)
    mod = _module(Hq, 256, bs, 2, 2, num_kv_heads=Hkv)
    bm = _block_mask(Hq, 256, bs, 2, 2, num_kv_heads=Hkv)
    res = {}
    for name, impl_name, ws in (("bisect", "mfma", True), ("scan", "mfma", False), ("generic", "generic", True)):
        ops.set_impl(impl_name)
        monkeypatch.setattr(ops, "_fwd_workspace", ws)
        try:
            res[name] = mod(q.to(DEV), k.to(DEV), v.to(DEV), sm, cu_seqlen_k=cu.to(DEV), return_lse=True)
            assert (ops.last_fwd_workspace_bytes > 0) == (name == "bisect")
        finally:
            ops.set_impl("auto")
    assert torch.equal(res["bisect"][0], res["scan"][0]) and torch.equal(res["bisect"][1], res["scan"][1])
    assert_close("O vs generic", res["bisect"][0], res["generic"][0], **TOL)
    assert_close("LSE vs generic", res["bisect"][1], res["generic"][1], atol=LSE_TOL, rtol=0)
    for i in list(range(0, nseq, 37)) + [nseq - 2]:
        s, e = int(cu[i]), int(cu[i + 1])
        if e > s:
            ro, rl = _seq_oracle(q[s:e], k[s:e], v[s:e], bm, bs, sm)
            assert_close(f"O[{i}]", res["bisect"][0][s:e], ro, **TOL)
            assert_close(f"LSE[{i}]", res["bisect"][1][:, s:e], rl, atol=LSE_TOL, rtol=0)


def test_packed_chunked_prefill_every_sequence_starts_inside_a_block(impl):
    """Packed chunked prefill where every sequence's queries start inside a row block and end
    in another: each touches ceil(q_len / 64) + 1 row blocks, the most the launch has to cover."""
    Hq, Hkv, D, bs = 2, 1, 64, 64
    sm = 1 / math.sqrt(D)
    lens = [273, 961, 142, 434, 130, 200]
    qlens = [252, 396, 15, 77, 66, 129]
    g = torch.Generator().manual_seed(20)
    ks = [torch.randn(l, Hkv, D, generator=g).to(torch.bfloat16) for l in lens]
    vs = [torch.randn(l, Hkv, D, generator=g).to(torch.bfloat16) for l in lens]
    qs = [torch.randn(l, Hq, D, generator=g).to(torch.bfloat16) for l in qlens]
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32).to(DEV)
    cuq = torch.tensor([0] + list(np.cumsum(qlens)), dtype=torch.int32).to(DEV)
    mod = _module(Hq, 1024, bs, 3, 4, num_kv_heads=Hkv)
    bm = _block_mask(Hq, 1024, bs, 3, 4, num_kv_heads=Hkv)
    out, lse = mod(torch.cat(qs).to(DEV), torch.cat(ks).to(DEV), torch.cat(vs).to(DEV), sm,
                   cu_seqlen_k=cu, cu_seqlen_q=cuq, return_lse=True)
    offs = np.cumsum([0] + qlens)
    for i in range(len(lens)):
        ro, rl = _seq_oracle(qs[i], ks[i], vs[i], bm, bs, sm)
        assert_close(f"O[{i}]", out[offs[i]:offs[i + 1]], ro, **TOL)
        assert_close(f"LSE[{i}]", lse[:, offs[i]:offs[i + 1]], rl, atol=LSE_TOL, rtol=0)


def test_c4_user_pattern_varlen_partitions(impl):
    """A reduced copy of the user-pattern configuration: per-head Bernoulli
    block pattern (diagonal forced, lower triangular), packed sequences, LSE,
    K/V columns split in 2 partitions merged with combine_attn_partitions."""
    H, D, bs, nb = 4, 128, 64, 32
    sm = 1 / math.sqrt(D)
    g = torch.Generator().manual_seed(20)
    pat = (torch.rand(H, nb, nb, generator=g) < 0.2)
    pat |= torch.eye(nb, dtype=torch.bool)[None]
    pat = torch.tril(pat.to(torch.uint8))
    lens = [512, 700, 64, 333]
    T = sum(lens)
    q, k, v = (torch.randn(T, H, D, generator=g).to(torch.bfloat16) for _ in range(3))
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32).to(DEV)
    full = SparseAttention(bs, pat).to(DEV)
    c = 6
    pa, pb = pat.clone(), pat.clone()
    pa[:, :, c:] = 0
    pb[:, :, :c] = 0
    import warnings
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        part_a, part_b = SparseAttention(bs, pa).to(DEV), SparseAttention(bs, pb).to(DEV)
    args = (q.to(DEV), k.to(DEV), v.to(DEV), sm)
    o_full, lse_full = full(*args, cu_seqlen_k=cu, return_lse=True)
    ra = part_a(*args, cu_seqlen_k=cu, return_lse=True)
    rb = part_b(*args, cu_seqlen_k=cu, return_lse=True)
    assert torch.isinf(rb[1]).any() and (rb[0][torch.isinf(rb[1]).transpose(0, 1)] == 0).all()
    merged = combine_attn_partitions(ra, rb)
    assert_close("combine vs unpartitioned", merged, o_full.cpu(), atol=1e-2, rtol=1e-2)
    lse_merged = torch.logaddexp(ra[1], rb[1])
    assert_close("lse merge", lse_merged, lse_full.cpu(), atol=LSE_TOL, rtol=0)
    s = 0
    for l in lens:
        ro, rl = _seq_oracle(q[s:s + l], k[s:s + l], v[s:s + l], pat.numpy(), bs, sm)
        assert_close("O vs oracle", merged[s:s + l], ro, **TOL)
        assert_close("LSE vs oracle", lse_full[:, s:s + l], rl, atol=LSE_TOL, rtol=0)
        s += l


@pytest.mark.parametrize("D,dtype", [(128, torch.bfloat16), (64, torch.float16), (96, torch.bfloat16)])
def test_row_pairs_user_pattern_and_offsets(D, dtype):
    """One head per workgroup and unpacked inputs: two adjacent q tiles share a workgroup and
    merge their table rows on the fly.  A random per-head pattern (rows that share few columns,
    rows with one entry, empty partitions), odd numbers of row blocks, k longer than q (the first
    row block is the odd half of a pair) and left / right padding exercise that merge."""
    H, bs, nb = 3, 64, 24
    sm = 1 / math.sqrt(D)
    g = torch.Generator().manual_seed(7)
    pat = (torch.rand(H, nb, nb, generator=g) < 0.25)
    pat |= torch.eye(nb, dtype=torch.bool)[None]
    pat[:, 5, :5] = False            # a row with its diagonal block only
    pat = torch.tril(pat.to(torch.uint8))
    import warnings
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        mod = SparseAttention(bs, pat).to(DEV)
    bm = pat.numpy()
    for Lq, Lk in ((nb * 64, nb * 64), (700, 700), (64, 64), (65, 65), (300, 1000), (1, 129), (200, 264)):
        print(f"row pairs: D={D} Lq={Lq} Lk={Lk}", flush=True)
        q = torch.randn(2, Lq, H, D, generator=g).to(dtype)
        k, v = (torch.randn(2, Lk, H, D, generator=g).to(dtype) for _ in range(2))
        out, lse = mod(q.to(DEV), k.to(DEV), v.to(DEV), sm, return_lse=True)
        for b in range(2):
            ro, rl = _seq_oracle(q[b], k[b], v[b], bm, bs, sm)
            assert_close(f"O[{b}]", out[b], ro, **TOL)
            assert_close(f"LSE[{b}]", lse[b], rl.transpose(0, 1) if rl.shape != lse[b].shape else rl, atol=LSE_TOL, rtol=0)
    # left-padded and right-padded prefill (per-sequence offsets, unpacked)
    Lmax, lens = 1024, [1024, 1, 333, 640]
    q, k, v = (torch.randn(len(lens), Lmax, H, D, generator=g).to(dtype) for _ in range(3))
    for left in (True, False):
        qp, kp, vp = torch.zeros_like(q), torch.zeros_like(k), torch.zeros_like(v)
        for i, l in enumerate(lens):
            sl = slice(Lmax - l, Lmax) if left else slice(0, l)
            qp[i, sl], kp[i, sl], vp[i, sl] = q[i, :l], k[i, :l], v[i, :l]
        extra = dict(left_paddings=torch.tensor([Lmax - l for l in lens])) if left else dict(seqlens=torch.tensor(lens))
        out = mod(qp.to(DEV), kp.to(DEV), vp.to(DEV), sm, **extra)
        for i, l in enumerate(lens):
            sl = slice(Lmax - l, Lmax) if left else slice(0, l)
            ro, _ = _seq_oracle(q[i, :l], k[i, :l], v[i, :l], bm, bs, sm)
            assert_close(f"O padded[{i}] left={left}", out[i, sl], ro, **TOL)


def test_seq_partition_with_backward(impl):
    """Context-parallel emulation in one process (reference:
    tests/test_seq_partition.py): q chunks x kv partitions, non-square masks,
    merge with combine_attn_partitions, gradients through the LSE."""
    B, H, L, D, bs, parts = 1, 3, 1024, 64, 32, 4
    dtype = torch.float16
    q, k, v, do = make_qkv(B, L, L, H, H, D, dtype, 2, with_do=True)
    qd, kd, vd = (x.to(DEV).requires_grad_() for x in (q, k, v))
    chunk = L // parts
    outs = []
    for qc in range(parts):
        pieces = []
        for kc in range(qc + 1):
            _, bmask, _ = get_sparse_attn_mask(H, chunk, bs, 4, 4, dtype=dtype, q_start_position=qc * chunk,
                                               kv_start_position=kc * chunk, kv_seqlen=chunk)
            layer = SparseAttention(bs, bmask, seq_dim=2, causal=(kc == qc)).to(DEV)
            pieces.append(layer(qd[:, :, qc * chunk:(qc + 1) * chunk], kd[:, :, kc * chunk:(kc + 1) * chunk],
                                vd[:, :, kc * chunk:(kc + 1) * chunk], return_lse=True))
        outs.append(pieces[0][0] if len(pieces) == 1 else combine_attn_partitions(*pieces, hdim=1))
    out = torch.cat(outs, dim=2)
    out.backward(do.to(DEV))
    bm = OL.block_mask(H, L, bs, 4, 4)
    qo, ko, vo = (x.clone().float().requires_grad_() for x in (q, k, v))
    ref, _ = oracle_fwd(qo, ko, vo, bm, bs, 1 / math.sqrt(D), seq_dim=2)
    ref.backward(do.float())
    assert_close("O", out, ref, **TOL)
    assert_close("dQ", qd.grad, qo.grad, **TOL)
    assert_close("dK", kd.grad, ko.grad, **TOL)
    assert_close("dV", vd.grad, vo.grad, **TOL)


def test_error_paths(impl):
    mod = _module(4, 512, 64, 2, 4)
    x = torch.zeros(1, 1024, 4, 128, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(AssertionError, match="larger than the maximum length"):
        mod(x, x, x)
    y = torch.zeros(1, 256, 4, 128, dtype=torch.bfloat16, device=DEV, requires_grad=True)
    out = mod(y, y, y, left_paddings=torch.zeros(1, dtype=torch.int32))
    with pytest.raises(AssertionError, match="does not support paddings"):
        out.sum().backward()
    z = torch.zeros(1, 256, 3, 128, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(AssertionError, match="number of heads in the sparse pattern"):
        mod(z, z, z)
    with pytest.raises(AssertionError, match="q length can only 1"):
        mod(y[:, :7], y, y, seqlens=torch.tensor([5]))
    # empty batch is a no-op
    e = torch.zeros(0, 256, 4, 128, dtype=torch.bfloat16, device=DEV)
    assert mod(e, e, e).shape == e.shape
