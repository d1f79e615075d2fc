"""Device-side voxelisation and collation in front of PointTransformerV3.forward.

This is this package's own contract, not a mirror of anything in the reference: the reference tree holds the
model only, whose sole voxelisation is the fallback that derives grid_coord from coord with the batch-wide minimum
and truncation (model.py:88-96; Point does the same when grid_coord is missing). The transform a training
pipeline runs on the host before the model is not part of that tree, so which points survive here (voxel
boundaries, the point kept per voxel) is pinned only by this repository's brute-force check, not by parity
with such a pipeline. grid_sample computes floor((coord - minimum of the point's own scene) / grid_size), keeps
one point per voxel, and returns the dictionary the model's forward takes, for a whole batch at once."""
import torch

from . import ops


@torch.no_grad()   # not inference_mode: the returned features may enter a training step
def grid_sample(coord, offset, grid_size, feat=None, keys=(), mode="test", seed=None):
    """coord (N,3) float, offset (B,) cumulative scene ends, both on the GPU.

    Keeps one point of every grid_size voxel of every scene: the first in input order with mode "test", a
    member drawn uniformly with mode "train" (the draw follows `seed`, or torch's CPU generator when seed is
    None; it reproduces no other library's random stream). Returns a dict
    ready for PointTransformerV3.forward: coord, grid_coord, offset, grid_size, feat (if given,
    rows of the kept points), plus index (kept input rows) and inverse (voxel of every input point),
    and any extra per-point tensors passed in `keys` as (name, tensor) pairs, gathered alike."""
    if mode not in ("test", "train"):
        raise ValueError("mode must be 'test' or 'train'")
    pick = 0
    if mode == "train":
        pick = int(torch.randint(1, 2 ** 32, (1,)).item()) if seed is None else (int(seed) % (2 ** 32 - 1)) + 1
    vox = ops.voxelize(coord, offset, grid_size, seed=pick)
    index = vox["index"]
    out = dict(coord=coord[index], grid_coord=vox["grid_coord"], offset=vox["offset"], grid_size=grid_size,
               index=index, inverse=vox["inverse"])
    if feat is not None:
        out["feat"] = feat[index]
    for name, tensor in keys:
        out[name] = tensor[index]
    return out
