"""Decode-step sweep over batch size and context length: one new token per sequence over a
KV cache of `context` tokens per sequence (bf16, 32 q heads / 8 kv heads, head_dim 128, block 64,
local 16 blocks, vert_stride 8 -- the pattern of bench.py's decode workload).

    python benchmark/benchmark_decode.py [--paged PAGE_SIZE] [--head-major] [--csv out.csv]

Each step is replayed from a HIP graph (what a serving loop does), rotating over enough copies
of the cache that no step finds its keys in the 256 MB last-level cache.  Prints microseconds
per step, the K/V bytes the pattern makes the step read (every attended key and value once per
kv head) and that figure over the step time as a fraction of the 8 TB/s HBM peak.  The
reference has no decode benchmark (its benchmark/benchmark_sparse_attn.py times prefill only).
"""
import argparse
import csv
import math
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from dkernel_amd import LocalStrideSparseAttention  # noqa: E402

HQ, HKV, D, BLOCK, LOCAL, VERT = 32, 8, 128, 64, 16, 8
HBM_PEAK = 8.0e12


def attended_bytes(mod, batch, context):
    """K and V bytes of the keys the last token of a `context`-token sequence attends, all kv heads."""
    crow = mod.layout_csr_crow.cpu()
    col = mod.layout_csr_col.cpu()
    rb = (context - 1) // BLOCK
    tokens = 0
    for kvh in range(HKV):
        h = kvh * crow.size(0) // HKV
        cols = col[h, crow[h, rb]:crow[h, rb + 1]].tolist()
        tokens += sum(min(BLOCK, context - c * BLOCK) for c in cols)
    return batch * tokens * D * 2 * 2


def bench_one(batch, context, page, head_major=False):
    dev = "cuda:0"
    mod = LocalStrideSparseAttention(HQ, context, BLOCK, LOCAL, VERT, num_kv_heads=HKV,
                                     seq_dim=2 if head_major and not page else 1).to(dev)
    byts = attended_bytes(mod, batch, context)
    sm = 1.0 / math.sqrt(D)
    kv_bytes = batch * context * HKV * D * 2 * 2
    nset = max(1, min(16, -(-(1 << 30) // kv_bytes)))
    q = torch.randn(batch, 1, HQ, D, device=dev, dtype=torch.bfloat16)
    if page:
        pages_per_seq = -(-context // page)
        n_pages = batch * pages_per_seq
        shape = (n_pages, HKV, page, D) if head_major else (n_pages, page, HKV, D)
        pools = [(torch.randn(shape, device=dev, dtype=torch.bfloat16), torch.randn(shape, device=dev, dtype=torch.bfloat16))
                 for _ in range(nset)]
        if head_major:  # views (pages, page_size, kv heads, dim) of head-major pages
            pools = [(kp.transpose(1, 2), vp.transpose(1, 2)) for kp, vp in pools]
        table = torch.randperm(n_pages, device=dev).to(torch.int32).view(batch, pages_per_seq)
        lens = torch.full((batch,), context, dtype=torch.int32, device=dev)
        out = torch.empty(batch, HQ, D, device=dev, dtype=torch.bfloat16)
        steps = [lambda kp=kp, vp=vp: mod.paged_decode(q[:, 0], kp, vp, table, lens, sm, out=out) for kp, vp in pools]
    else:
        shape = (batch, HKV, context, D) if head_major else (batch, context, HKV, D)
        caches = [(torch.randn(shape, device=dev, dtype=torch.bfloat16), torch.randn(shape, device=dev, dtype=torch.bfloat16))
                  for _ in range(nset)]
        if head_major:
            q = q.transpose(1, 2)  # (batch, heads, 1, dim)
        lens = torch.full((batch,), context, dtype=torch.int32, device=dev)
        steps = [lambda k=k, v=v: mod(q, k, v, sm, seqlens=lens) for k, v in caches]

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for s in steps:
            s()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for s in steps:
            s()
    reps = max(3, min(100, int(3e5 / ((10.0 + byts / 4e6) * nset))))  # about 0.3 s per case
    for _ in range(3):
        graph.replay()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(reps):
        graph.replay()
    stop.record()
    torch.cuda.synchronize()
    us = start.elapsed_time(stop) * 1e3 / (reps * nset)
    return us, byts


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--paged", type=int, default=0, help="page size of a paged K/V cache (0: contiguous cache)")
    ap.add_argument("--head-major", action="store_true",
                    help="cache laid out (batch, kv heads, tokens, dim) / pages (kv heads, page_size, dim)")
    ap.add_argument("--batches", type=int, nargs="+", default=[1, 8, 32, 128])
    ap.add_argument("--contexts", type=int, nargs="+", default=[2048, 8192, 32768, 131072])
    ap.add_argument("--max-gib", type=float, default=40.0, help="skip cases whose K/V copies exceed this")
    ap.add_argument("--csv", default=None)
    a = ap.parse_args()
    if not torch.cuda.is_available():
        sys.exit("benchmark_decode.py needs a GPU")
    rows = []
    kind = f"paged cache, {a.paged}-token pages" if a.paged else "contiguous cache"
    kind += ", head-major" if a.head_major else ", token-major"
    print(f"== decode step: {HQ}/{HKV} heads, d={D}, bf16, block {BLOCK}, local {LOCAL} blocks, vert_stride {VERT}; "
          f"{kind}; us per step (attended K/V MB, % of 8 TB/s)", flush=True)
    print(f"{'batch':>6}" + "".join(f"{c:>26}" for c in a.contexts), flush=True)
    for b in a.batches:
        line = f"{b:>6}"
        for c in a.contexts:
            kv = b * c * HKV * D * 2 * 2
            if kv * max(1, min(16, -(-(1 << 30) // kv))) > a.max_gib * (1 << 30):
                line += f"{'-':>26}"
                continue
            us, byts = bench_one(b, c, a.paged, a.head_major)
            frac = byts / (us * 1e-6) / HBM_PEAK
            rows.append(dict(batch=b, context=c, us=round(us, 2), attended_mb=round(byts / 1e6, 2), hbm_frac=round(frac, 4)))
            line += f"{us:>10.1f} ({byts / 1e6:>7.1f}, {100 * frac:>4.1f}%)"
            torch.cuda.empty_cache()
        print(line, flush=True)
    if a.csv:
        with open(a.csv, "w", newline="") as f:
            w = csv.DictWriter(f, fieldnames=list(rows[0].keys()))
            w.writeheader()
            w.writerows(rows)


if __name__ == "__main__":
    main()
