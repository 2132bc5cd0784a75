"""Build-time check of the matrix-core kernels' register allocation (no GPU needed).

Every instantiation of the MFMA kernels must stay free of scratch memory: next to the
asynchronous HBM -> LDS tile copies a scratch reload waits for every copy in flight, and a
change that is neutral on the benchmark shapes has pushed other head dims into spills before
(forward 0.28 -> 0.78 ms at head_dim 192).  hipcc reports the usage of each kernel with
-Rpass-analysis=kernel-resource-usage; the files are compiled in parallel, each with the extra
flags the Makefile gives it (EXTRA_<file> lines).
"""
from __future__ import annotations

import concurrent.futures
import os
import re
import shutil
import subprocess

import pytest

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "dkernel_amd", "csrc")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-Rpass-analysis=kernel-resource-usage", "--cuda-device-only", "-c"]
# One head per workgroup at the 256-wide tile (one wave per SIMD, 512 registers): its spills sit
# outside the block loop and it measures as fast as before them.
ALLOWED = re.compile(r"mfma_fwd_kernelI\w+Li256ELi1E")


def _extra_flags(src):
    stem = os.path.splitext(src)[0]
    with open(os.path.join(CSRC, "Makefile")) as f:
        m = re.search(rf"^EXTRA_{stem}\s*:=\s*(.*)$", f.read(), re.M)
    return m.group(1).split() if m else []


def _usage(src, tmp):
    out = subprocess.run([HIPCC, *FLAGS, *_extra_flags(src), os.path.join(CSRC, src), "-o", os.path.join(tmp, src + ".o")],
                         capture_output=True, text=True, cwd=CSRC)
    assert out.returncode == 0, out.stderr[-2000:]
    usage, name = {}, None
    for line in out.stderr.splitlines():
        m = re.search(r"Function Name: (\S+)", line)
        if m:
            name = m.group(1)
        m = re.search(r"ScratchSize \[bytes/lane\]: (\d+)", line)
        if m and name:
            usage[name] = int(m.group(1))
    return usage


@pytest.mark.skipif(shutil.which(HIPCC) is None, reason="hipcc not installed")
def test_mfma_kernels_use_no_scratch(tmp_path):
    assert _extra_flags("mfma_fwd.hip"), "per-file flags of the Makefile not found"
    with concurrent.futures.ThreadPoolExecutor(4) as pool:
        results = list(pool.map(lambda s: _usage(s, str(tmp_path)),
                                ["mfma_fwd.hip", "mfma_bwd.hip", "decode.hip", "mfma_f32.hip"]))
    usage = {k: v for r in results for k, v in r.items()}
    assert len(usage) > 100, "kernel resource remarks not found"
    spilling = {k: v for k, v in usage.items() if v and not ALLOWED.search(k)}
    assert not spilling, f"kernels with scratch memory: {spilling}"
