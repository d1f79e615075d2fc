"""Device-side voxelisation and collation in front of PointTransformerV3.forward.

Pointcept prepares a batch on the host (GridSample: grid coordinates relative to the scene minimum,
one point kept per voxel; then the scenes are concatenated with cumulative `offset`); the model
itself only has a fallback that derives grid_coord (model.py:88-96). grid_sample does that step
on the GPU for a whole batch at once and returns the dictionary the model's forward takes."""
import torch

from . import ops


@torch.no_grad()   # not inference_mode: the returned features may enter a training step
def grid_sample(coord, offset, grid_size, feat=None, keys=(), mode="test", seed=None):
    """coord (N,3) float, offset (B,) cumulative scene ends, both on the GPU.

    Keeps one point of every grid_size voxel of every scene: the first in input order with mode "test", a
    member drawn uniformly with mode "train" (GridSample's two modes; the draw follows `seed`, or torch's CPU
    generator when seed is None -- not numpy's stream, which the reference's pipeline uses). Returns a dict
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
