"""Latency sweep of the block-sparse attention over sequence length and vertical stride.

    python benchmark/benchmark_sparse_attn.py [--mode fwd|bwd|both] [--max-log2 16] [--csv out.csv]
        [--batch 4 --heads 16 --head-dim 128 --local-tokens 512 --dtype bfloat16 --impl auto]
        [--dense-heads 0 [--heads-on-fixed-queues]]

Same sweep as the reference's benchmark/benchmark_sparse_attn.py (its defaults at
lines 24-40 and 67: batch 4, 16 heads, head_dim 128, local window 512 tokens, block 64,
bf16, sequence lengths 2^10 .. 2^16, vert_stride in {1, 4, 16}, warm-up 25 / 100 timed
repetitions), next to PyTorch's dense causal scaled_dot_product_attention when that runs on
the box.  Prints one table per mode (milliseconds) and optionally writes a CSV.  The shape, the
dtype and the kernel family (`--impl generic` = the fp32-FMA kernels, `mfma` = matrix cores only)
can be changed, e.g. for fp32 on the matrix cores against the generic kernels.  `--dense-heads N`
makes the last N heads dense (num_dense_heads); `--heads-on-fixed-queues` then switches off the
rotation of heads over the hardware's workgroup queues that such uneven patterns get, for
comparison.
"""
import argparse
import csv
import math
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from dkernel_amd import LocalStrideSparseAttention, ops  # noqa: E402

B, H, D, BLOCK, LOCAL_TOKENS = 4, 16, 128, 64, 512
DTYPE = torch.bfloat16
DENSE_HEADS, FIXED_QUEUES = 0, False


def timeit(fn, warmup, reps):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(reps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / reps


def bench_one(L, vert, mode, warmup, reps):
    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(20)
    q, k, v, do = (torch.randn(B, L, H, D, generator=g, device=dev, dtype=DTYPE) for _ in range(4))
    sm = 1.0 / math.sqrt(D)
    mod = LocalStrideSparseAttention(H, L, BLOCK, LOCAL_TOKENS // BLOCK, vert, num_dense_heads=DENSE_HEADS).to(dev)
    if FIXED_QUEUES:
        mod.kwargs["uneven_heads"] = False
    nnz = int(mod.layout_csr_crow[:, -1].sum().item())
    flops = 4.0 * BLOCK * BLOCK * D * nnz * B * (1.0 if mode == "fwd" else 2.5)
    if mode == "fwd":
        with torch.no_grad():
            ms = timeit(lambda: mod(q, k, v, sm), warmup, reps)
    else:
        for t in (q, k, v):
            t.requires_grad_()
        o = mod(q, k, v, sm)
        ms = timeit(lambda: torch.autograd.grad(o, (q, k, v), do, retain_graph=True), warmup, reps)
    return ms, flops / (ms * 1e-3) / 1e12


def bench_dense(L, mode, warmup, reps):
    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(20)
    q, k, v, do = (torch.randn(B, H, L, D, generator=g, device=dev, dtype=DTYPE) for _ in range(4))
    f = torch.nn.functional.scaled_dot_product_attention
    if mode == "fwd":
        with torch.no_grad():
            return timeit(lambda: f(q, k, v, is_causal=True), warmup, reps)
    for t in (q, k, v):
        t.requires_grad_()
    o = f(q, k, v, is_causal=True)
    return timeit(lambda: torch.autograd.grad(o, (q, k, v), do, retain_graph=True), warmup, reps)


def main():
    global B, H, D, LOCAL_TOKENS, DTYPE, DENSE_HEADS, FIXED_QUEUES
    defaults = (B, H, D, LOCAL_TOKENS)
    ap = argparse.ArgumentParser()
    ap.add_argument("--mode", default="both", choices=["fwd", "bwd", "both"])
    ap.add_argument("--min-log2", type=int, default=10)
    ap.add_argument("--max-log2", type=int, default=16)
    ap.add_argument("--verts", default="1,4,16")
    ap.add_argument("--warmup", type=int, default=25)
    ap.add_argument("--reps", type=int, default=100)
    ap.add_argument("--no-dense", action="store_true")
    ap.add_argument("--csv", default=None)
    ap.add_argument("--batch", type=int, default=defaults[0])
    ap.add_argument("--heads", type=int, default=defaults[1])
    ap.add_argument("--head-dim", type=int, default=defaults[2])
    ap.add_argument("--local-tokens", type=int, default=defaults[3])
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float16", "float32"])
    ap.add_argument("--impl", default="auto", choices=["auto", "generic", "mfma"])
    ap.add_argument("--dense-heads", type=int, default=0)
    ap.add_argument("--heads-on-fixed-queues", action="store_true")
    args = ap.parse_args()
    DENSE_HEADS, FIXED_QUEUES = args.dense_heads, args.heads_on_fixed_queues
    B, H, D, LOCAL_TOKENS, DTYPE = args.batch, args.heads, args.head_dim, args.local_tokens, getattr(torch, args.dtype)
    ops.set_impl(args.impl)
    verts = [int(x) for x in args.verts.split(",")]
    rows = []
    for mode in (["fwd", "bwd"] if args.mode == "both" else [args.mode]):
        print(f"== {mode}: b={B} h={H} d={D} {args.dtype}, block {BLOCK}, local {LOCAL_TOKENS} tokens, kernels: {args.impl}"
              + (f", last {DENSE_HEADS} heads dense" + (", heads on fixed queues" if FIXED_QUEUES else "") if DENSE_HEADS else "")
              + "; ms (effective TFLOP/s)")
        print("seqlen".rjust(8) + "".join(f"vert={v}".rjust(22) for v in verts) + "dense sdpa".rjust(14))
        for lg in range(args.min_log2, args.max_log2 + 1):
            L = 1 << lg
            reps = max(5, args.reps // max(1, L // 8192))
            warm = max(2, args.warmup // max(1, L // 8192))
            line = str(L).rjust(8)
            for vert in verts:
                ms, tf = bench_one(L, vert, mode, warm, reps)
                rows.append({"mode": mode, "seqlen": L, "impl": f"sparse_vert{vert}", "ms": round(ms, 4), "tflops": round(tf, 1)})
                line += f"{ms:10.3f} ({tf:6.0f})".rjust(22)
            dense = None
            if not args.no_dense:
                try:
                    dense = bench_dense(L, mode, warm, reps)
                    rows.append({"mode": mode, "seqlen": L, "impl": "dense_sdpa", "ms": round(dense, 4), "tflops": ""})
                except Exception as exc:  # the dense comparator is optional
                    print(f"   dense sdpa failed at L={L}: {type(exc).__name__}", file=sys.stderr)
            line += (f"{dense:14.3f}" if dense is not None else "n/a".rjust(14))
            print(line, flush=True)
            torch.cuda.empty_cache()
    if args.csv:
        with open(args.csv, "w", newline="") as fh:
            w = csv.DictWriter(fh, fieldnames=["mode", "seqlen", "impl", "ms", "tflops"])
            w.writeheader()
            w.writerows(rows)


if __name__ == "__main__":
    main()
