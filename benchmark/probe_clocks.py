"""Shader clock and board power while a kernel runs back to back for a few seconds: the headline
sparse forward a plain bf16 GEMM of the vendor library (torch.matmul, 8192^3) and the forward + backward
benchmark workload, each on random and on all-zero operands.  Shows how far below the 2.4 GHz of the datasheet peak the part clocks
under matrix-core load with real data, and what rate the vendor's own GEMM sustains then.

    python benchmark/probe_clocks.py            (needs rocm-smi on PATH; reads, changes nothing)
"""
from __future__ import annotations

import math
import os
import re
import subprocess
import sys
import threading
import time

import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
from dkernel_amd import LocalStrideSparseAttention  # noqa: E402

DEV = "cuda:0"
SECONDS = 5.0


class Watch(threading.Thread):
    """Polls rocm-smi for the shader clock (MHz) and the package power (W)."""

    def __init__(self):
        super().__init__(daemon=True)
        self.samples: list[tuple[float, float]] = []
        self.stop = False

    def run(self):
        while not self.stop:
            try:
                out = subprocess.run(["rocm-smi", "--showclocks", "--showpower"], capture_output=True, text=True,
                                     timeout=20).stdout
            except (OSError, subprocess.SubprocessError):
                return
            clk = re.search(r"sclk clock level: \d+: \((\d+)Mhz\)", out)
            pw = re.search(r"Power \(W\): ([0-9.]+)", out)
            if clk:
                self.samples.append((float(clk.group(1)), float(pw.group(1)) if pw else float("nan")))
            time.sleep(0.3)


def measure(name, fn, flop):
    for _ in range(20):
        fn()
    torch.cuda.synchronize()
    w = Watch()
    w.start()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    calls, t0 = 0, time.time()
    start.record()
    while time.time() - t0 < SECONDS:
        for _ in range(200):
            fn()
        calls += 200
        torch.cuda.synchronize()
    stop.record()
    torch.cuda.synchronize()
    w.stop = True
    w.join()
    ms = start.elapsed_time(stop) / calls
    tail = w.samples[len(w.samples) // 2:]  # the settled half
    clk = sum(s[0] for s in tail) / max(len(tail), 1)
    pw = sum(s[1] for s in tail) / max(len(tail), 1)  # nan where the board does not report it
    print(f"{name:<46s} {ms:7.4f} ms  {flop / ms / 1e9:6.0f} TFLOP/s = {flop / ms / 1e9 / 25:4.1f} % of 2500   "
          f"sclk {clk:5.0f} MHz  power {pw:5.0f} W  ({len(w.samples)} samples)", flush=True)


def main():
    L, D = 8192, 128
    g = torch.Generator().manual_seed(20)
    mod = LocalStrideSparseAttention(32, L, 64, 16, 8, num_kv_heads=8).to(DEV)
    q = torch.randn(2, L, 32, D, generator=g).to(torch.bfloat16).to(DEV)
    k = torch.randn(2, L, 8, D, generator=g).to(torch.bfloat16).to(DEV)
    v = torch.randn(2, L, 8, D, generator=g).to(torch.bfloat16).to(DEV)
    sm = 1 / math.sqrt(D)
    fwd_flop = 4.0 * 64 * 64 * D * 87008 * 2  # listed blocks of the headline pattern, two batch entries
    a = torch.randn(8192, 8192, generator=g).to(torch.bfloat16).to(DEV)
    b = torch.randn(8192, 8192, generator=g).to(torch.bfloat16).to(DEV)
    gemm_flop = 2.0 * 8192 ** 3
    with torch.no_grad():
        measure("sparse forward (headline), random data", lambda: mod(q, k, v, sm, return_lse=True), fwd_flop)
        qz, kz, vz = torch.zeros_like(q), torch.zeros_like(k), torch.zeros_like(v)
        measure("sparse forward (headline), zeros", lambda: mod(qz, kz, vz, sm, return_lse=True), fwd_flop)
        measure("vendor GEMM 8192^3 bf16, random data", lambda: torch.matmul(a, b), gemm_flop)
        az, bz = torch.zeros_like(a), torch.zeros_like(b)
        measure("vendor GEMM 8192^3 bf16, zeros", lambda: torch.matmul(az, bz), gemm_flop)
        measure("sparse forward (headline), random data, again", lambda: mod(q, k, v, sm, return_lse=True), fwd_flop)
    # backward workload of bench.py: one batch entry, 32 heads (MHA); forward + backward per call, so the rate
    # quoted is that of the 3.5 x forward work (2 + 5 of the products counted)
    modb = LocalStrideSparseAttention(32, L, 64, 16, 8).to(DEV)
    for zeros in (False, True):
        qb, kb, vb, do = (torch.randn(1, L, 32, D, generator=g).to(torch.bfloat16).to(DEV) for _ in range(4))
        if zeros:
            qb, kb, vb, do = (torch.zeros_like(x) for x in (qb, kb, vb, do))
        qb, kb, vb = (x.requires_grad_() for x in (qb, kb, vb))

        def step():
            out = modb(qb, kb, vb, sm)
            out.backward(do)
            qb.grad = kb.grad = vb.grad = None

        measure(f"sparse forward + backward (MHA), {'zeros' if zeros else 'random data'}", step, 3.5 * 4.0 * 64 * 64 * D * 87008)


if __name__ == "__main__":
    main()
