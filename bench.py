"""Benchmark of the block-sparse attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-extra]

A step is one causal prefill forward (with LSE) over one synthetic batch of the
Phi-3-small-style configuration: B=2, L=8192, 32 q heads / 8 kv heads, head_dim
128, bf16, block 64, 16 local blocks, vertical stride 8.  Inputs are resident
in HBM before the timed region.  Prints ONE JSON line:

  value     effective (sparse-counted) TFLOP/s = 4*64*64*128 * active blocks / time
  roofline  the forward kernel against the dense bf16 MFMA peak: median of
            per-step HIP-event durations on the launch stream over the same
            timed steps (extra.bwd / extra.decode carry the same object)
  cpu_baseline  the reference's dense masked-attention checker (oracle port)
            timed on this box's host cores on a bounded sample
  extra     backward (B=1, 32 MHA heads) TFLOP/s and batched-decode us/step
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

MFMA_BF16_PEAK_TFLOPS = 2500.0   # MI355X dense bf16, vendor figure
HBM_PEAK_GBS = 8000.0            # MI355X HBM3E, vendor figure
# HBM bytes per launch come from rocprofv3 --pmc runs of this file (FETCH_SIZE scaled by the copy
# calibration + WRITE_SIZE), kept in profiles/hbm_traffic.json together with the library version
# and the kernels that were profiled.  Counters cannot be read from inside this process, so the
# figure is quoted, and only while the library still launches those kernels for the workload.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")
BS, LOCAL, VERT, D = 64, 16, 8, 128
WARM_GPU_SECONDS = 0.3           # untimed calls beyond --warmup until the clocks have settled


def block_flops(nnz_blocks, d=D, bs=BS):
    """QK^T and PV over one bs x bs block, diagonal blocks counted in full."""
    return 4.0 * bs * bs * d * nnz_blocks


def gen(shape, g, dtype):
    import torch
    return torch.randn(shape, generator=g, dtype=torch.float32).to(dtype)


def time_loop(fn, steps, warmup):
    """Wall-clock ms per step of `steps` back-to-back calls (no events between the steps: an
    event record between two 40 us launches costs several us of its own)."""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def time_steps(fn, steps, warmup):
    """Runs `warmup` untimed calls, keeps calling until the GPU has been busy for
    WARM_GPU_SECONDS, then times exactly `steps` calls.  Returns (wall ms per step over the
    whole timed region, median and mean HIP-event ms per step: one event pair per step on the
    launch stream)."""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    busy = 0.0
    while busy < WARM_GPU_SECONDS:
        a.record()
        for _ in range(20):
            fn()
        b.record()
        torch.cuda.synchronize()
        busy += a.elapsed_time(b) * 1e-3
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        marks[i].record()
        fn()
    marks[steps].record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    per_step = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(steps))
    median = per_step[steps // 2] if steps % 2 else 0.5 * (per_step[steps // 2 - 1] + per_step[steps // 2])
    return wall, median, marks[0].elapsed_time(marks[steps]) / steps


def quoted_traffic(leg, kernels, version):
    """(bytes per launch or None, note) for `leg` ("fwd", "bwd", "decode", "combine"): the profiled figure if it
    was taken from the kernels that just ran (names and library version agree), else None."""
    try:
        with open(TRAFFIC_FILE) as f:
            rec = json.load(f)
    except (OSError, ValueError) as e:
        return None, f"no traffic record ({e.__class__.__name__})"
    kernels = kernels.decode() if isinstance(kernels, bytes) else kernels
    ent = rec.get(leg)
    if ent is None:
        return None, f"no traffic record for {leg}"
    if rec.get("dk_version") != version:
        return None, f"traffic record is of library version {rec.get('dk_version')}, this is {version}: re-profile"
    if ent.get("kernels", "").strip() != kernels.strip():
        return None, f"traffic record is of kernels '{ent.get('kernels')}', this run launched '{kernels}': re-profile"
    return float(ent["fetch_bytes"]) + float(ent["write_bytes"]), rec.get("source", TRAFFIC_FILE)


def roofline(bound, work, ms, traffic, algorithmic_bytes):
    """work: FLOP (bound "mfma") or bytes (bound "hbm") per launch; ms: median launch duration."""
    if bound == "mfma":
        achieved, peak, unit = work / (ms * 1e-3) / 1e12, MFMA_BF16_PEAK_TFLOPS, "TFLOP/s"
    else:
        achieved, peak, unit = work / (ms * 1e-3) / 1e9, HBM_PEAK_GBS, "GB/s"
    return {"bound": bound, "achieved": round(achieved, 2), "peak": peak, "unit": unit,
            "frac": round(achieved / peak, 4), "traffic": traffic[0],
            "traffic_unit": "bytes per launch (rocprofv3 FETCH_SIZE / WRITE_SIZE, separate runs)",
            "traffic_source": traffic[1],
            "algorithmic_bytes": algorithmic_bytes, "kernel_ms": round(ms, 5)}


def cpu_baseline(seconds_budget=20.0):
    """The reference checker's dense masked attention (oracle port) on the host
    CPU, on a bounded sample of the same workload: whole heads of one batch
    element at L=8192, d=128, bf16 inputs, until the budget is spent."""
    import torch
    from oracle import attention as OA
    from oracle import layout as OL
    cores = os.cpu_count() or 1
    # the GPU box caps worker pools at 16 threads per GPU
    threads = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)), 16)
    torch.set_num_threads(threads)
    L, H, Hkv = 8192, 32, 8
    g = torch.Generator().manual_seed(20)
    bm = OL.block_mask(H, L, BS, LOCAL, VERT, num_kv_heads=Hkv)
    sm = 1.0 / math.sqrt(D)
    done_blocks, heads, t_total = 0, 0, 0.0
    tril = torch.tril(torch.ones(L, L, dtype=torch.bool))
    while t_total < seconds_budget and heads < 2 * H:  # both batch elements at most
        h = heads % H
        q, k, v = (gen((1, 1, L, D), g, torch.bfloat16) for _ in range(3))
        mask = torch.from_numpy(bm[h]).bool().repeat_interleave(BS, 0).repeat_interleave(BS, 1) & tril
        t0 = time.perf_counter()
        OA.reference_style_attention(q, k, v, mask[None, None], sm, seq_dim=2)
        t_total += time.perf_counter() - t0
        done_blocks += int(bm[h].sum())
        heads += 1
    return {
        "value": round(block_flops(done_blocks) / t_total / 1e12, 5),
        "unit": "TFLOP/s (effective, sparse-counted)",
        "cores": threads,
        "kind": "port",
        "sample": f"{heads} of 64 (batch, head) pairs at L=8192 d=128 bf16, dense masked torch attention, "
                  f"{t_total:.1f} s",
        "dense_tflops": round(4.0 * L * L * D * heads / t_total / 1e12, 5),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=25)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip backward / decode figures")
    ap.add_argument("--impl", default="auto", choices=["auto", "generic", "mfma"])
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run a plain 1 GiB device copy and exit (scale for the FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the path has no cross-GPU component in this build "
              "(heads and KV partitions shard without communication). Use --gpus 1.",
              file=sys.stderr)
        sys.exit(2)

    import torch
    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda:0").fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_bytes_read": 1 << 30, "copy_bytes_written": 1 << 30, "copies": 3}))
        return
    from dkernel_amd import LocalStrideSparseAttention, _lib, ops
    ops.set_impl(args.impl)
    lib = _lib.lib()
    version = lib.dk_version()
    dev = "cuda:0"
    torch.cuda.set_device(0)
    g = torch.Generator().manual_seed(20)
    sm = 1.0 / math.sqrt(D)

    # ---- C1: prefill forward -------------------------------------------------
    B, L, Hq, Hkv = 2, 8192, 32, 8
    mod = LocalStrideSparseAttention(Hq, L, BS, LOCAL, VERT, num_kv_heads=Hkv).to(dev)
    nnz = int(mod.layout_csr_crow[:, -1].sum().item())      # 87008 per batch element
    q = gen((B, L, Hq, D), g, torch.bfloat16).to(dev)
    k = gen((B, L, Hkv, D), g, torch.bfloat16).to(dev)
    v = gen((B, L, Hkv, D), g, torch.bfloat16).to(dev)
    with torch.no_grad():
        wall_ms, ev_ms, ev_mean = time_steps(lambda: mod(q, k, v, sm, return_lse=True), args.steps, args.warmup)
    fwd_kernels = lib.dk_last_kernels().decode()
    flops = block_flops(nnz) * B
    value = flops / (wall_ms * 1e-3) / 1e12
    # q + k + v read once, o + lse written once
    fwd_bytes = (2 * B * L * Hq * D + 2 * B * L * Hkv * D) * 2 + B * L * Hq * 4

    out = {
        "metric": "effective fwd TFLOP/s, causal block-sparse prefill, L=8192 d=128 bf16, 1 MI355X",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(wall_ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "prefill fwd + LSE: B=2 L=8192 Hq=32 Hkv=8 d=128 bf16, block 64, "
                               "local 16, vert 8, heterogeneous heads, causal",
                   "active_blocks_per_batch": nnz, "flop_per_step": flops, "impl": args.impl},
        "roofline": roofline("mfma", flops, ev_ms, quoted_traffic("fwd", fwd_kernels, version), fwd_bytes),
    }
    out["roofline"]["kernels"] = fwd_kernels
    out["roofline"]["kernel_ms_mean"] = round(ev_mean, 5)
    del q, k, v

    if not args.no_extra:
        extra = {}
        # ---- C2: backward, B=1, 32 MHA heads ---------------------------------
        mod2 = LocalStrideSparseAttention(32, L, BS, LOCAL, VERT).to(dev)
        nnz2 = int(mod2.layout_csr_crow[:, -1].sum().item())
        q2, k2, v2, do2 = (gen((1, L, 32, D), g, torch.bfloat16).to(dev) for _ in range(4))
        q2.requires_grad_(), k2.requires_grad_(), v2.requires_grad_()
        o2 = mod2(q2, k2, v2, sm)

        def bwd():
            torch.autograd.grad(o2, (q2, k2, v2), do2, retain_graph=True)
        steps2 = max(5, args.steps // 4)
        w2, e2, _ = time_steps(bwd, steps2, max(2, args.warmup // 4))
        with torch.no_grad():
            wf, ef, _ = time_steps(lambda: mod2(q2, k2, v2, sm), steps2, 2)
        bwd_flops = 2.5 * block_flops(nnz2)
        # q, k, v, o, dO read and dq, dk, dv written once (bf16), lse read (fp32)
        bwd_bytes = 8 * L * 32 * D * 2 + L * 32 * 4
        extra["bwd"] = {"workload": "dQ,dK,dV: B=1 L=8192 H=32 (MHA) d=128 bf16, same pattern "
                                    "(dQ pass + dK/dV pass, 5 of the 7 executed GEMMs counted)",
                        "tflops": round(bwd_flops / (e2 * 1e-3) / 1e12, 2),
                        "ms": round(e2, 4), "frac_of_mfma_peak":
                        round(bwd_flops / (e2 * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
                        "kernels": ops.last_bwd_kernels.decode(),
                        "roofline": roofline("mfma", bwd_flops, e2,
                                             quoted_traffic("bwd", ops.last_bwd_kernels, version), bwd_bytes),
                        "fwd_mha_tflops": round(block_flops(nnz2) / (ef * 1e-3) / 1e12, 2)}
        del q2, k2, v2, do2, o2
        # ---- C3: batched decode over left-padded KV --------------------------
        nseq, Lmax = 32, 8192
        lens = torch.randint(1024, 8193, (nseq,), generator=g)
        # Two K/V sets used in turn: one step touches ~180 MB, which would otherwise stay
        # resident in the 256 MB Infinity Cache and overstate the HBM rate.
        kv_sets = []
        for _ in range(2):
            kd = torch.zeros((nseq, Lmax, Hkv, D), dtype=torch.bfloat16)
            vd = torch.zeros_like(kd)
            for i, l in enumerate(lens.tolist()):
                kd[i, Lmax - l:] = gen((l, Hkv, D), g, torch.bfloat16)
                vd[i, Lmax - l:] = gen((l, Hkv, D), g, torch.bfloat16)
            kv_sets.append((kd.to(dev), vd.to(dev)))
        qd = gen((nseq, 1, Hq, D), g, torch.bfloat16).to(dev)
        left = (Lmax - lens).to(torch.int32).to(dev)
        # algorithmic bytes: K and V of every attended token, once per kv head
        byts = 0
        for l in lens.tolist():
            r = (l - 1) // BS
            for kvh in range(Hkv):
                nblk = min(r + 1, LOCAL) + sum(1 for j in range(0, max(r - LOCAL + 1, 0)) if (j + kvh) % VERT == 0)
                byts += (BS * (nblk - 1) + ((l - 1) % BS + 1)) * D * 2 * 2
        with torch.no_grad():
            step = [0]

            def decode_step():
                kd, vd = kv_sets[step[0] & 1]
                step[0] += 1
                return mod(qd, kd, vd, sm, left_paddings=left)
            _, ed_eager, _ = time_steps(decode_step, args.steps, args.warmup)
            dec_kernels = lib.dk_last_kernels().decode()
            wd = time_loop(decode_step, args.steps, 2)
            # An eager step is bounded by the Python launcher (the GPU idles between steps), so the
            # kernel's own duration is measured on a HIP graph of 8 steps (both K/V sets in turn,
            # what a serving loop would replay): median replay time / 8.
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for _ in range(4):
                    decode_step()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            step[0] = 0
            with torch.cuda.graph(graph):
                for _ in range(8):
                    decode_step()
            _, eg, _ = time_steps(graph.replay, max(10, args.steps), 3)
            ed = eg / 8
        dec_traffic = quoted_traffic("decode", dec_kernels, version)
        extra["decode"] = {"workload": "32 seqs x 1 token, Hq=32 Hkv=8 d=128 bf16, KV len U[1024,8192] left-padded, "
                                       "2 K/V sets alternated (working set > Infinity Cache)",
                           "us_per_step": round(wd * 1e3, 2), "graph_step_us": round(ed * 1e3, 2),
                           "eager_event_us": round(ed_eager * 1e3, 2),
                           "timing": "us_per_step: eager module calls back to back, wall clock; eager_event_us: the same "
                                     "with a HIP event between the steps (median); graph_step_us: HIP graph of 8 steps, "
                                     "median replay / 8 (every kernel of a step, no launch gaps: what rocprofv3 reports as "
                                     "the kernels' duration)",
                           "kernels": dec_kernels,
                           "algorithmic_MB": round(byts / 1e6, 2),
                           "achieved_GBs": round(byts / (ed * 1e-3) / 1e9, 1),
                           "frac_of_hbm_peak": round(byts / (ed * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                           "roofline": roofline("hbm", byts, ed, dec_traffic, byts),
                           "roofline_eager_events": roofline("hbm", byts, ed_eager, dec_traffic, byts)}
        extra["decode"]["kernel_us"] = extra["decode"]["graph_step_us"]   # former name of the same figure
        del kv_sets
        # ---- merge of two K/V partitions (combine_attn_partitions) at the packed configuration's size ----
        from dkernel_amd import combine_attn_partitions
        Tc, Hc = 16384, 16
        parts = [(gen((Tc, Hc, D), g, torch.bfloat16).to(dev), gen((Hc, Tc), g, torch.float32).to(dev)) for _ in range(2)]
        with torch.no_grad():
            _, ec, _ = time_steps(lambda: combine_attn_partitions(*parts), max(10, args.steps), 3)
        # two outputs read, one written (bf16), two log-sum-exps read (fp32)
        comb_bytes = 3 * Tc * Hc * D * 2 + 2 * Tc * Hc * 4
        comb_kernels = lib.dk_last_kernels().decode()
        extra["combine"] = {"workload": "2 partitions of packed (16384 tokens, 16 heads, d=128) bf16 outputs + fp32 LSE",
                            "us": round(ec * 1e3, 2), "kernels": comb_kernels,
                            "roofline": roofline("hbm", comb_bytes, ec, quoted_traffic("combine", comb_kernels, version),
                                                 comb_bytes)}
        out["extra"] = extra

    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
