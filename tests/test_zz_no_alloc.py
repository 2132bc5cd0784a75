"""dk_fwd_noalloc (scratch inside the library image, no allocation) against dk_fwd with a caller
workspace, through the C ABI: same kernels, so every output bit must agree.  Two calls in a row
per case, the second on a smaller input, so that what the first call left in the shared scratch
is there when the second one runs."""
from __future__ import annotations

import ctypes as C
import math

import pytest
import torch

from dkernel_amd import LocalStrideSparseAttention, _lib, ops
from helpers import LSE_TOL, TOL, assert_close
from oracle import attention as OA
from oracle import layout as OL

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _decode_args(mod, q, k, v, o, lse, left, lens):
    """Padded single-token decode (left-padded K/V) as dk_fwd_args."""
    B, Lmax = k.size(0), k.size(1)
    a = _lib.FwdArgs()
    a.q, a.k, a.v, a.o = (ops._tensor4(x, 2, 1) for x in (q, k, v, o))
    a.lse = ops._rowvec(lse)
    a.csr = ops._lut((mod.layout_csr_crow, mod.layout_csr_col, 64, 64), q.device, mod.lut_group, mod.lut_max_row)
    zeros = torch.zeros(B, dtype=torch.int32, device=DEV)
    keep = [zeros, zeros + 1, left, left + lens]
    a.seqs = _lib.Seqs(B, 1, Lmax, 0, *(t.data_ptr() for t in keep))
    a.num_q_heads, a.num_kv_heads, a.head_dim = q.size(2), k.size(2), q.size(3)
    a.dtype, a.causal, a.impl = _lib.DK_BF16, 1, _lib.DK_IMPL_AUTO
    a.sm_scale = 1 / math.sqrt(q.size(3))
    a.stream = None
    return a, keep


def _run_both(a):
    """(need, rc) after running dk_fwd with a torch workspace; the caller then runs dk_fwd_noalloc."""
    lib = _lib.lib()
    need = lib.dk_fwd_workspace_bytes(C.byref(a))
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=DEV)
    a.workspace, a.workspace_bytes = ws.data_ptr(), need
    _lib.check(lib.dk_fwd(C.byref(a)))
    torch.cuda.synchronize()
    return need


def _decode_case(B, Hq, Hkv, Lmax, lens, seed):
    D = 128
    g = torch.Generator().manual_seed(seed)
    mod = LocalStrideSparseAttention(Hq, Lmax, 64, 4, 4, num_kv_heads=Hkv).to(DEV)
    q = torch.randn(B, 1, Hq, D, generator=g).to(torch.bfloat16).to(DEV)
    k = torch.randn(B, Lmax, Hkv, D, generator=g).to(torch.bfloat16).to(DEV)
    v = torch.randn(B, Lmax, Hkv, D, generator=g).to(torch.bfloat16).to(DEV)
    lens_t = torch.tensor(lens, dtype=torch.int32, device=DEV)
    left = Lmax - lens_t
    outs = []
    for entry in ("dk_fwd", "dk_fwd_noalloc"):
        o = torch.full_like(q, float("nan"))
        lse = torch.full((B, Hq, 1), float("nan"), dtype=torch.float32, device=DEV)
        a, keep = _decode_args(mod, q, k, v, o, lse, left, lens_t)
        if entry == "dk_fwd":
            need = _run_both(a)
            # the case must really go through the scratch: rows longer than one workgroup's units
            assert need > 0
        else:
            a.workspace, a.workspace_bytes = None, 0
            _lib.check(_lib.lib().dk_fwd_noalloc(C.byref(a)))
            torch.cuda.synchronize()
        outs.append((o, lse))
    (o_ref, lse_ref), (o_new, lse_new) = outs
    assert torch.equal(o_ref, o_new), "O differs between dk_fwd and dk_fwd_noalloc"
    assert torch.equal(lse_ref, lse_new), "LSE differs between dk_fwd and dk_fwd_noalloc"
    # and both are right: the oracle on sequence 0
    bm = OL.block_mask(Hq, Lmax, 64, 4, 4, num_kv_heads=Hkv)
    l0 = lens[0]
    mask = OA.sequence_token_mask(bm, 64, 1, l0)
    want, want_lse = OA.dense_attention(q[:1].cpu(), k[:1, Lmax - l0:].cpu(), v[:1, Lmax - l0:].cpu(),
                                        torch.from_numpy(mask), 1 / math.sqrt(D))
    assert_close("O", o_new[:1], want, **TOL)
    assert_close("LSE", lse_new[:1], want_lse, atol=LSE_TOL, rtol=0)
    return need


def test_decode_through_static_scratch_twice():
    # few rows with long contexts: every row is cut into several workgroups of units, whose
    # partials meet in the scratch and are merged by the second kernel
    need1 = _decode_case(B=3, Hq=8, Hkv=2, Lmax=4096, lens=[4096, 3000, 2049], seed=1)
    need2 = _decode_case(B=2, Hq=8, Hkv=2, Lmax=2048, lens=[1500, 2048], seed=2)   # smaller, same scratch
    assert need2 < need1 <= _lib.DK_NOALLOC_SCRATCH_BYTES


def _packed_case(lens, seed):
    """Packed prefill: the running tile counts of the sequences live in the scratch."""
    Hq, Hkv, D, Lmax = 4, 2, 64, 1024
    g = torch.Generator().manual_seed(seed)
    T = sum(lens)
    mod = LocalStrideSparseAttention(Hq, Lmax, 64, 2, 3, num_kv_heads=Hkv).to(DEV)
    q = torch.randn(T, Hq, D, generator=g).to(torch.bfloat16).to(DEV)
    k = torch.randn(T, Hkv, D, generator=g).to(torch.bfloat16).to(DEV)
    v = torch.randn(T, Hkv, D, generator=g).to(torch.bfloat16).to(DEV)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32, device=DEV)
    outs = []
    for entry in ("dk_fwd", "dk_fwd_noalloc"):
        o = torch.full_like(q, float("nan"))
        lse = torch.full((Hq, T), float("nan"), dtype=torch.float32, device=DEV)
        a = _lib.FwdArgs()
        a.q, a.k, a.v, a.o = (ops._tensor3(x) for x in (q, k, v, o))
        a.lse = ops._rowvec(lse, (0, lse.stride(0), lse.stride(1)))
        a.csr = ops._lut((mod.layout_csr_crow, mod.layout_csr_col, 64, 64), q.device, mod.lut_group)
        a.seqs = _lib.Seqs(len(lens), T, T, 1, cu.data_ptr(), cu.data_ptr() + 4, cu.data_ptr(), cu.data_ptr() + 4)
        a.num_q_heads, a.num_kv_heads, a.head_dim = Hq, Hkv, D
        a.dtype, a.causal, a.impl = _lib.DK_BF16, 1, _lib.DK_IMPL_AUTO
        a.sm_scale = 1 / math.sqrt(D)
        a.stream = None
        if entry == "dk_fwd":
            assert _run_both(a) > 0
        else:
            a.workspace, a.workspace_bytes = None, 0
            _lib.check(_lib.lib().dk_fwd_noalloc(C.byref(a)))
            torch.cuda.synchronize()
        outs.append((o, lse))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
    assert torch.isfinite(outs[1][0]).all()


def test_packed_prefill_through_static_scratch_twice():
    _packed_case([300, 64, 1, 513, 129, 70], seed=3)
    _packed_case([65, 200], seed=4)


def test_too_much_scratch_is_refused_before_any_launch():
    # 64 sequences x 32 q heads with long rows ask for more than the static scratch holds
    B, Hq, Hkv, Lmax, D = 64, 32, 8, 8192, 128
    mod = LocalStrideSparseAttention(Hq, Lmax, 64, 16, 8, num_kv_heads=Hkv).to(DEV)
    q = torch.zeros(B, 1, Hq, D, dtype=torch.bfloat16, device=DEV)
    k = torch.zeros(B, 1, Hkv, D, dtype=torch.bfloat16, device=DEV).expand(B, Lmax, Hkv, D)  # never read
    lens = torch.full((B,), 1, dtype=torch.int32, device=DEV)
    o = torch.zeros_like(q)
    a, keep = _decode_args(mod, q, k, k, o, None, Lmax - lens, lens)
    a.csr.max_row_entries = 128 * 8     # a hint that makes every row many units long
    lib = _lib.lib()
    assert lib.dk_fwd_workspace_bytes(C.byref(a)) > _lib.DK_NOALLOC_SCRATCH_BYTES
    assert lib.dk_fwd_noalloc(C.byref(a)) == _lib.DK_ERR_INVALID
    assert "bytes of scratch" in lib.dk_last_error().decode()


def test_recorded_into_a_graph_after_a_warm_up_call():
    """The entry point under stream capture (one of the callers it exists for): after one ordinary
    call, a decode step is recorded into a graph and every replay, with K/V and q rewritten in
    place between them, must give dk_fwd's bits."""
    B, Hq, Hkv, Lmax, D = 3, 8, 2, 4096, 128
    lens = [4096, 3000, 2049]
    g = torch.Generator().manual_seed(11)
    mod = LocalStrideSparseAttention(Hq, Lmax, 64, 4, 4, num_kv_heads=Hkv).to(DEV)
    q = torch.randn(B, 1, Hq, D, generator=g).to(torch.bfloat16).to(DEV)
    k = torch.randn(B, Lmax, Hkv, D, generator=g).to(torch.bfloat16).to(DEV)
    v = torch.randn(B, Lmax, Hkv, D, generator=g).to(torch.bfloat16).to(DEV)
    lens_t = torch.tensor(lens, dtype=torch.int32, device=DEV)
    left = Lmax - lens_t
    o = torch.zeros_like(q)
    lse = torch.zeros((B, Hq, 1), dtype=torch.float32, device=DEV)
    lib = _lib.lib()
    a, keep = _decode_args(mod, q, k, v, o, lse, left, lens_t)
    a.workspace, a.workspace_bytes = None, 0
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):   # the warm-up call, on the stream that will capture
        a.stream = ops._stream()
        _lib.check(lib.dk_fwd_noalloc(C.byref(a)))
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        a.stream = ops._stream()
        _lib.check(lib.dk_fwd_noalloc(C.byref(a)))
    for rep in range(3):
        q.copy_(torch.randn(B, 1, Hq, D, generator=g).to(torch.bfloat16))
        k.copy_(torch.randn(B, Lmax, Hkv, D, generator=g).to(torch.bfloat16))
        o.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        o_graph, lse_graph = o.clone(), lse.clone()
        o2 = torch.full_like(q, float("nan"))
        lse2 = torch.full_like(lse, float("nan"))
        b, keep2 = _decode_args(mod, q, k, v, o2, lse2, left, lens_t)
        assert _run_both(b) > 0
        assert torch.equal(o_graph, o2) and torch.equal(lse_graph, lse2), f"replay {rep} differs from dk_fwd"
