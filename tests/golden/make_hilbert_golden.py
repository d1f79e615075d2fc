"""Writes tests/golden/hilbert_golden.npz from the reference's own Hilbert encoder.

Run in the build container only (the reference checkout does not travel):
    python tests/golden/make_hilbert_golden.py

Why this function and no other: the bit/byte order of serialization/hilbert.py:143-152 and
:178-196 (uint8 views, flips, trailing-bit truncation) selects one particular Hilbert curve
among the many that satisfy bijectivity, adjacency and the octree hierarchy, so invariants
alone cannot pin it. z-order, the "-trans" swap and the batch packing have closed forms and
are pinned without the reference.

The fixture holds inputs and expected outputs only.
"""
import os
import sys

import numpy as np
import torch

sys.path.insert(0, "/root/reference")
from serialization.hilbert import encode as ref_hilbert_encode  # noqa: E402

out = {}
# every cell of the cube at depth 1..4
for d in (1, 2, 3, 4):
    r = np.arange(1 << d)
    cells = np.stack(np.meshgrid(r, r, r, indexing="ij"), -1).reshape(-1, 3).astype(np.int32)
    out[f"all_d{d}_in"] = cells
    out[f"all_d{d}_out"] = ref_hilbert_encode(torch.from_numpy(cells), 3, d).numpy()
# seeded random coordinates at the depths the workloads use, and the limits
rng = np.random.default_rng(20240607)
for d in (5, 8, 9, 12, 15, 16):
    pts = rng.integers(0, 1 << d, size=(512, 3), dtype=np.int64).astype(np.int32)
    pts[0] = 0
    pts[1] = (1 << d) - 1
    out[f"rand_d{d}_in"] = pts
    out[f"rand_d{d}_out"] = ref_hilbert_encode(torch.from_numpy(pts), 3, d).numpy()
# coordinates wider than the depth are truncated to their low bits
pts = rng.integers(0, 1 << 16, size=(256, 3), dtype=np.int64).astype(np.int32)
out["trunc_d9_in"] = pts
out["trunc_d9_out"] = ref_hilbert_encode(torch.from_numpy(pts), 3, 9).numpy()

path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hilbert_golden.npz")
np.savez_compressed(path, **out)
print("wrote", path, {k: v.shape for k, v in out.items() if k.endswith("_out")})
