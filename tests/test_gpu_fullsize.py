"""GPU tests at the full sizes of the benchmark configurations.  The dense
oracle cannot cover 64 (batch, head) pairs at L=8192 in seconds, so each case
checks (a) the whole result against the independent generic kernel on the GPU
and (b) sampled heads / sequences against the fp32 oracle, plus
size-independent properties (LSE merge of partitions equals the unpartitioned
result, padded rows untouched)."""
import math
import warnings

import numpy as np
import pytest
import torch

from dkernel_amd import LocalStrideSparseAttention, SparseAttention, combine_attn_partitions, ops
from oracle import attention as OA
from oracle import layout as OL
from helpers import LSE_TOL, TOL, assert_close

pytestmark = pytest.mark.gpu
DEV = "cuda"
BS, LOCAL, VERT, D = 64, 16, 8, 128
SM = 1.0 / math.sqrt(D)


def gen(shape, g, dtype=torch.bfloat16):
    return torch.randn(shape, generator=g, dtype=torch.float32).to(dtype)


def with_impl(name, fn):
    ops.set_impl(name)
    try:
        return fn()
    finally:
        ops.set_impl("auto")


def head_oracle(q, k, v, bm_head, requires_grad=False):
    """One (batch, head): q (L, D), k, v (L, D) fp32 oracle."""
    L = q.shape[0]
    mask = OA.sequence_token_mask(bm_head[None], BS, L, k.shape[0])
    qq, kk, vv = (x.float()[None, :, None].requires_grad_(requires_grad) for x in (q, k, v))
    o, lse = OA.dense_attention(qq, kk, vv, torch.from_numpy(mask), SM, seq_dim=1)
    return o, lse, (qq, kk, vv)


def test_c1_prefill_forward_full_size():
    """B=2 L=8192 Hq=32 Hkv=8 d=128 bf16, block 64, local 16, vert 8, LSE."""
    B, L, Hq, Hkv = 2, 8192, 32, 8
    g = torch.Generator().manual_seed(20)
    q, k, v = gen((B, L, Hq, D), g), gen((B, L, Hkv, D), g), gen((B, L, Hkv, D), g)
    mod = LocalStrideSparseAttention(Hq, L, BS, LOCAL, VERT, num_kv_heads=Hkv).to(DEV)
    assert mod.lut_group == 4
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    with torch.no_grad():
        o_m, lse_m = with_impl("mfma", lambda: mod(qd, kd, vd, SM, return_lse=True))
        o_g, lse_g = with_impl("generic", lambda: mod(qd, kd, vd, SM, return_lse=True))
    assert_close("O mfma vs generic", o_m, o_g.cpu(), atol=1e-2, rtol=1e-2)
    assert_close("LSE mfma vs generic", lse_m, lse_g.cpu(), atol=LSE_TOL, rtol=0)
    bm = OL.block_mask(Hq, L, BS, LOCAL, VERT, num_kv_heads=Hkv)
    for b, h in [(0, 0), (1, 13), (1, 31)]:
        print(f"oracle head b={b} h={h}", flush=True)
        o, lse, _ = head_oracle(q[b, :, h], k[b, :, h // 4], v[b, :, h // 4], bm[h])
        assert_close(f"O[{b},{h}]", o_m[b, :, h], o[0, :, 0], **TOL)
        assert_close(f"LSE[{b},{h}]", lse_m[b, h], lse[0, 0], atol=LSE_TOL, rtol=0)


def test_c2_backward_full_size():
    """B=1 L=8192 H=32 (MHA) d=128 bf16, same pattern, dQ/dK/dV through autograd."""
    L, H = 8192, 32
    g = torch.Generator().manual_seed(20)
    q, k, v, do = (gen((1, L, H, D), g) for _ in range(4))
    mod = LocalStrideSparseAttention(H, L, BS, LOCAL, VERT).to(DEV)

    def run():
        qd, kd, vd = (x.to(DEV).requires_grad_() for x in (q, k, v))
        out = mod(qd, kd, vd, SM)
        out.backward(do.to(DEV))
        return out.detach(), qd.grad, kd.grad, vd.grad
    res_m = with_impl("mfma", run)
    res_g = with_impl("generic", run)
    for name, a, b in zip(("O", "dQ", "dK", "dV"), res_m, res_g):
        assert_close(f"{name} mfma vs generic", a, b.cpu(), atol=1e-2, rtol=1e-2)
    bm = OL.block_mask(H, L, BS, LOCAL, VERT)
    for h in (5, 30):
        print(f"oracle head h={h}", flush=True)
        o, _, (qq, kk, vv) = head_oracle(q[0, :, h], k[0, :, h], v[0, :, h], bm[h], requires_grad=True)
        o.backward(do[0, :, h].float()[None, :, None])
        assert_close(f"dQ[{h}]", res_m[1][0, :, h], qq.grad[0, :, 0], **TOL)
        assert_close(f"dK[{h}]", res_m[2][0, :, h], kk.grad[0, :, 0], **TOL)
        assert_close(f"dV[{h}]", res_m[3][0, :, h], vv.grad[0, :, 0], **TOL)


def test_c3_batched_decode_full_size():
    """32 sequences x 1 token, Hq=32 Hkv=8, KV lengths U[1024, 8192] left-padded to 8192."""
    nseq, Lmax, Hq, Hkv = 32, 8192, 32, 8
    g = torch.Generator().manual_seed(20)
    lens = torch.randint(1024, 8193, (nseq,), generator=g)
    lens[0], lens[1] = 1024, 8192
    q = gen((nseq, 1, Hq, D), g)
    ks = [gen((int(l), Hkv, D), g) for l in lens]
    vs = [gen((int(l), Hkv, D), g) for l in lens]
    kp = torch.full((nseq, Lmax, Hkv, D), 7.0, dtype=torch.bfloat16)   # padding holds garbage
    vp = torch.full((nseq, Lmax, Hkv, D), -3.0, dtype=torch.bfloat16)
    for i, l in enumerate(lens.tolist()):
        kp[i, Lmax - l:], vp[i, Lmax - l:] = ks[i], vs[i]
    mod = LocalStrideSparseAttention(Hq, Lmax, BS, LOCAL, VERT, num_kv_heads=Hkv).to(DEV)
    left = (Lmax - lens).to(torch.int32)
    qd, kd, vd = q.to(DEV), kp.to(DEV), vp.to(DEV)
    with torch.no_grad():
        out, lse = mod(qd, kd, vd, SM, left_paddings=left, return_lse=True)
        out_g = with_impl("generic", lambda: mod(qd, kd, vd, SM, left_paddings=left))
    assert_close("decode auto vs generic", out, out_g.cpu(), atol=1e-2, rtol=1e-2)
    bm = OL.block_mask(Hq, Lmax, BS, LOCAL, VERT, num_kv_heads=Hkv)
    for i in range(nseq):
        mask = OA.sequence_token_mask(bm, BS, 1, int(lens[i]))
        o, l = OA.dense_attention(q[i][None], ks[i][None], vs[i][None], torch.from_numpy(mask), SM, seq_dim=1)
        assert_close(f"O[{i}]", out[i], o[0], **TOL)
        assert_close(f"LSE[{i}]", lse[i], l[0], atol=LSE_TOL, rtol=0)


def test_c4_user_pattern_packed_partitions_full_size():
    """16 heads, 256 x 256 Bernoulli(0.2) lower-triangular pattern with the
    diagonal forced, 8 packed sequences with lengths U[512, 4096] (sum <= 16384),
    LSE, 2 KV partitions merged with combine_attn_partitions."""
    H, nb = 16, 256
    g = torch.Generator().manual_seed(20)
    pat = torch.rand(H, nb, nb, generator=g) < 0.2
    pat |= torch.eye(nb, dtype=torch.bool)[None]
    pat = torch.tril(pat.to(torch.uint8))
    lens = torch.randint(512, 4097, (8,), generator=g)
    while int(lens.sum()) > 16384:
        lens = (lens * 0.9).long().clamp_min(512)
    T = int(lens.sum())
    q, k, v = (gen((T, H, D), g) for _ in range(3))
    cu = torch.cat([torch.zeros(1, dtype=torch.long), lens.cumsum(0)]).to(torch.int32)
    c = 32
    pa, pb = pat.clone(), pat.clone()
    pa[:, :, c:] = 0
    pb[:, :, :c] = 0
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        full, part_a, part_b = (SparseAttention(BS, x).to(DEV) for x in (pat, pa, pb))
    args = (q.to(DEV), k.to(DEV), v.to(DEV), SM)
    cud = cu.to(DEV)
    with torch.no_grad():
        o_full, lse_full = full(*args, cu_seqlen_k=cud, return_lse=True)
        ra = part_a(*args, cu_seqlen_k=cud, return_lse=True)
        rb = part_b(*args, cu_seqlen_k=cud, return_lse=True)
        o_gen = with_impl("generic", lambda: full(*args, cu_seqlen_k=cud))
    merged = combine_attn_partitions(ra, rb)
    assert_close("combine(A, B) vs unpartitioned", merged, o_full.cpu(), atol=1e-2, rtol=1e-2)
    assert_close("LSE merge", torch.logaddexp(ra[1], rb[1]), lse_full.cpu(), atol=LSE_TOL, rtol=0)
    assert_close("auto vs generic", o_full, o_gen.cpu(), atol=1e-2, rtol=1e-2)
    # oracle on the shortest and one more sequence, 4 heads each
    order = np.argsort(lens.numpy())
    for si in (int(order[0]), int(order[3])):
        s, e = int(cu[si]), int(cu[si + 1])
        print(f"oracle sequence {si} len {e - s}", flush=True)
        hs = [0, 5, 10, 15]
        mask = OA.sequence_token_mask(pat.numpy()[hs], BS, e - s, e - s)
        o, l = OA.dense_attention(q[s:e, hs][None], k[s:e, hs][None], v[s:e, hs][None],
                                  torch.from_numpy(mask), SM, seq_dim=1)
        assert_close("O vs oracle", merged[s:e][:, hs], o[0], **TOL)
        assert_close("LSE vs oracle", lse_full[hs][:, s:e], l[0], atol=LSE_TOL, rtol=0)
