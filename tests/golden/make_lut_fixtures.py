"""Writes tests/golden/lut_fixtures.npz: block masks and CSR/CSC look-up tables
produced by the reference's own host code (dkernel/utils.py, loaded by file
path) for a handful of small configurations, plus CRCs of the two headline
LUTs.  Run once in the build container, where /root/reference exists; the
fixtures (data only) are committed, the reference never travels.

    python tests/golden/make_lut_fixtures.py
"""
import importlib.util
import json
import os
import zlib

import numpy as np
import torch

REF = "/root/reference/dkernel/utils.py"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lut_fixtures.npz")

spec = importlib.util.spec_from_file_location("_ref_dkernel_utils", REF)
ref = importlib.util.module_from_spec(spec)
spec.loader.exec_module(ref)

MASK_CASES = {
    # name: kwargs of get_sparse_attn_mask
    "c0": dict(num_heads=8, seqlen=1024, block_size=64, local_blocks=4, vert_stride=4),
    "gqa": dict(num_heads=8, seqlen=1024, block_size=64, local_blocks=3, vert_stride=8, num_kv_heads=2),
    "dense_heads": dict(num_heads=6, seqlen=768, block_size=64, local_blocks=2, vert_stride=4,
                        num_kv_heads=3, num_dense_heads=1),
    "offset": dict(num_heads=4, seqlen=512, block_size=32, local_blocks=2, vert_stride=5,
                   head_sliding_offset=3),
    "homo": dict(num_heads=4, seqlen=512, block_size=32, local_blocks=2, vert_stride=3, homo_head=True),
    "ragged": dict(num_heads=2, seqlen=300, block_size=64, local_blocks=2, vert_stride=2),
    "past": dict(num_heads=2, seqlen=640, block_size=64, local_blocks=2, vert_stride=3, past_len=200),
    "noncausal": dict(num_heads=2, seqlen=512, block_size=32, local_blocks=2, vert_stride=4, causal=False),
    "noncausal_lr": dict(num_heads=1, seqlen=512, block_size=32, local_blocks=(3, 1), vert_stride=4,
                         causal=False),
    "partition": dict(num_heads=3, seqlen=256, block_size=32, local_blocks=4, vert_stride=4,
                      q_start_position=512, kv_start_position=256, kv_seqlen=256),
    "step": dict(num_heads=4, seqlen=512, block_size=32, local_blocks=1, vert_stride=8, head_sliding_step=3),
}

# (block_size, block_m, block_n, mask case) for merge_split_fwd_kernel_blocks
TILE_CASES = {
    "merge_16_128_16": (16, 128, 16, dict(num_heads=2, seqlen=512, block_size=16, local_blocks=2, vert_stride=4)),
    "merge_16_128_16_l1": (16, 128, 16, dict(num_heads=2, seqlen=512, block_size=16, local_blocks=1, vert_stride=4)),
    "mergesplit_64_128_32": (64, 128, 32, dict(num_heads=2, seqlen=1024, block_size=64, local_blocks=2, vert_stride=4)),
    "split_64_32_32": (64, 32, 32, dict(num_heads=2, seqlen=512, block_size=64, local_blocks=2, vert_stride=3)),
    "split_64_64_16": (64, 64, 16, dict(num_heads=1, seqlen=512, block_size=64, local_blocks=1, vert_stride=2)),
    "merge_32_64_32": (32, 64, 32, dict(num_heads=3, seqlen=512, block_size=32, local_blocks=2, vert_stride=4)),
}

out = {}
meta = {"mask": {}, "tile": {}}
for name, kw in MASK_CASES.items():
    (crow, col), bm, _ = ref.get_sparse_attn_mask(dtype=torch.uint8, **kw)
    out[f"mask/{name}/block_mask"] = bm.cpu().numpy()
    out[f"mask/{name}/crow"] = crow.cpu().numpy()
    out[f"mask/{name}/col"] = col.cpu().numpy()
    ccol, row = ref.dense_to_ccol_row(bm)
    out[f"mask/{name}/ccol"] = ccol.cpu().numpy()
    out[f"mask/{name}/row"] = row.cpu().numpy()
    out[f"mask/{name}/kv_eff"] = np.array(bool(ref.is_kv_cache_efficient(bm, kw["block_size"], kw["block_size"])))
    meta["mask"][name] = {k: (list(v) if isinstance(v, tuple) else v) for k, v in kw.items()}

for name, (bs, bm_, bn_, kw) in TILE_CASES.items():
    pattern = ref.get_sparse_attn_mask(dtype=torch.uint8, **kw)[1]
    crow, col = ref.merge_split_fwd_kernel_blocks(bs, pattern, bm_, bn_)
    out[f"tile/{name}/pattern"] = pattern.cpu().numpy()
    out[f"tile/{name}/crow"] = crow.cpu().numpy()
    out[f"tile/{name}/col"] = col.cpu().numpy()
    meta["tile"][name] = {"block_size": bs, "block_m": bm_, "block_n": bn_}

# headline LUT (32 q heads / 8 kv heads, L=8192, bs64 local16 vert8): crow + CRCs
kw = dict(num_heads=32, seqlen=8192, block_size=64, local_blocks=16, vert_stride=8, num_kv_heads=8)
(crow, col), bm, _ = ref.get_sparse_attn_mask(dtype=torch.uint8, **kw)
ccol, row = ref.dense_to_ccol_row(bm)
out["c1/crow"] = crow.cpu().numpy()
out["c1/ccol"] = ccol.cpu().numpy()
out["c1/crc"] = np.array([zlib.crc32(np.ascontiguousarray(x.cpu().numpy()).tobytes())
                          for x in (bm, col, row)], dtype=np.uint32)
out["c1/shapes"] = np.array([*col.shape, *row.shape], dtype=np.int64)
meta["c1"] = kw

out["meta_json"] = np.frombuffer(json.dumps(meta).encode(), dtype=np.uint8)
np.savez_compressed(OUT, **out)
print("wrote", OUT, os.path.getsize(OUT), "bytes,", len(out), "arrays")
