"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch

DEV = "cuda:0"


def to_dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.to(DEV)


def rel_err(got, want):
    """max |got-want| / max |want| — the 'max-abs relative' measure of the parity bar."""
    got = got.detach().float().cpu()
    want = torch.as_tensor(want).detach().float()
    return float((got - want).abs().max() / want.abs().max().clamp_min(1e-12))


def unique_voxels(rng, n, extent, nb=1):
    """nb scenes of n distinct random cells each in [0,extent)^3: (grid (N,3) i32, batch, offset)."""
    grids, batch = [], []
    for b in range(nb):
        flat = rng.choice(extent ** 3, size=n, replace=False)
        g = np.stack([flat // (extent * extent), (flat // extent) % extent, flat % extent], 1)
        grids.append(g.astype(np.int32))
        batch.append(np.full(n, b, np.int64))
    return np.concatenate(grids), np.concatenate(batch), np.cumsum([n] * nb).astype(np.int64)
