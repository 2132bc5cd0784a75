"""Forward and backward of a user-defined pattern with global rows and columns (BigBird /
Longformer style: a window around the diagonal, the first blocks attended by and attending
everything, a few random blocks), causal or not.

    python benchmark/benchmark_global_rows.py [--heads 16 --batch 2 --head-dim 128]
        [--global-blocks 2 --window 3 --random 3] [--causal] [--last-row-first]

The long rows of such a pattern are its first ones.  `--last-row-first` switches off the
longest-first hand-out of rows that the module chooses for it (the forward and dQ kernels then
start from the last row, as they do for causal local-stride patterns), for comparison.
Prints ms and effective TFLOP/s (blocks of the pattern x 4 (forward) or 10 (backward) x 64 x 64 x
head_dim / time) for sequence lengths 4096 .. 32768.
"""
import argparse
import math
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from dkernel_amd import SparseAttention  # noqa: E402


def pattern(n, glob, window, rnd, causal):
    g = torch.Generator().manual_seed(1)
    i = torch.arange(n)
    pat = (i[:, None] - i[None, :]).abs() <= window
    pat[:glob, :] = True
    pat[:, :glob] = True
    pat |= torch.rand(n, n, generator=g) < rnd / n
    if causal:
        pat &= i[:, None] >= i[None, :]
    return pat


def timeit(fn, warmup=5, reps=20):
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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--heads", type=int, default=16)
    ap.add_argument("--batch", type=int, default=2)
    ap.add_argument("--head-dim", type=int, default=128)
    ap.add_argument("--global-blocks", type=int, default=2)
    ap.add_argument("--window", type=int, default=3)
    ap.add_argument("--random", type=float, default=3)
    ap.add_argument("--causal", action="store_true")
    ap.add_argument("--last-row-first", action="store_true")
    ap.add_argument("--min-log2", type=int, default=12)
    ap.add_argument("--max-log2", type=int, default=15)
    args = ap.parse_args()
    dev, D, H, B = "cuda:0", args.head_dim, args.heads, args.batch
    print(f"b={B} h={H} d={D} bf16, block 64, {args.global_blocks} global blocks, window {args.window}, "
          f"{args.random} random blocks per row, {'causal' if args.causal else 'not causal'}"
          + (", last row first" if args.last_row_first else "") + "; ms (effective TFLOP/s)")
    print("seqlen".rjust(8) + "longest row".rjust(14) + "mean row".rjust(10) + "fwd".rjust(20) + "bwd".rjust(20))
    for lg in range(args.min_log2, args.max_log2 + 1):
        L = 1 << lg
        pat = pattern(L // 64, args.global_blocks, args.window, args.random, args.causal)
        mod = SparseAttention(64, pat, causal=args.causal).to(dev)
        if args.last_row_first:
            mod.kwargs["unsorted_rows"] = False
        g = torch.Generator(device=dev).manual_seed(20)
        q, k, v, do = (torch.randn(B, L, H, D, generator=g, device=dev).to(torch.bfloat16) for _ in range(4))
        sm = 1 / math.sqrt(D)
        with torch.no_grad():
            fwd = timeit(lambda: mod(q, k, v, sm))
        for t in (q, k, v):
            t.requires_grad_()
        o = mod(q, k, v, sm)
        bwd = timeit(lambda: torch.autograd.grad(o, (q, k, v), do, retain_graph=True))
        blocks = int(pat.sum()) * H * B
        rows = pat.sum(1)
        tf = lambda ms, mult: mult * 64 * 64 * D * blocks / ms / 1e9  # noqa: E731
        print(f"{L:8d}{int(rows.max()):14d}{float(rows.float().mean()):10.1f}"
              + f"{fwd:10.3f} ({tf(fwd, 4):6.0f})".rjust(20) + f"{bwd:10.3f} ({tf(bwd, 10):6.0f})".rjust(20), flush=True)


if __name__ == "__main__":
    main()
