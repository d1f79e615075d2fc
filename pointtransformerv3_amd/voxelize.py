"""Device-side voxelisation and collation in front of PointTransformerV3.forward.

Pointcept prepares a batch on the host (GridSample: grid coordinates relative to the scene minimum,
one point kept per voxel; then the scenes are concatenated with cumulative `offset`); the model
itself only has a fallback that derives grid_coord (model.py:88-96). grid_sample does that step
on the GPU for a whole batch at once and returns the dictionary the model's forward takes."""
import torch

from . import ops


@torch.no_grad()   # not inference_mode: the returned features may enter a training step
def grid_sample(coord, offset, grid_size, feat=None, keys=()):
    """coord (N,3) float, offset (B,) cumulative scene ends, both on the GPU.

    Keeps the first point (in input order) of every grid_size voxel of every scene. Returns a dict
    ready for PointTransformerV3.forward: coord, grid_coord, offset, grid_size, feat (if given,
    rows of the kept points), plus index (kept input rows) and inverse (voxel of every input point),
    and any extra per-point tensors passed in `keys` as (name, tensor) pairs, gathered alike."""
    vox = ops.voxelize(coord, offset, grid_size)
    index = vox["index"]
    out = dict(coord=coord[index], grid_coord=vox["grid_coord"], offset=vox["offset"], grid_size=grid_size,
               index=index, inverse=vox["inverse"])
    if feat is not None:
        out["feat"] = feat[index]
    for name, tensor in keys:
        out[name] = tensor[index]
    return out
