"""The whole-model golden cases: their configurations, inputs and weights, all derived from seeds so
that the fixture file only has to hold the expected outputs.

Shared by make_forward_golden.py (which runs the reference's model.py on these cases in the build
container) and by the tests that compare the CPU oracle and the GPU product with what it wrote.
Nothing here comes from the reference: it is input data.
"""
import numpy as np
import torch

# name -> (model keyword arguments, scene sizes, what the fixture keeps: every stage's features or only those
# after the stem / poolings / unpoolings, and whether parameter gradients)
_SMALL = dict(in_channels=6, enc_channels=(32, 32, 64, 64, 64), enc_num_head=(2, 2, 4, 4, 4),
              dec_channels=(32, 32, 64, 64), dec_num_head=(2, 2, 4, 4))
CASES = {
    # fused-attention path, rows shuffled at every level, a scene longer than one patch (its last patch borrows
    # points), a scene shorter than one patch, two blocks per decoder stage (the first one convolves the skip
    # projection alone), five blocks in one stage (the order index wraps around)
    "flash_shuffle": (dict(_SMALL, enc_depths=(2, 1, 1, 5, 1), dec_depths=(2, 2, 1, 1), enc_patch_size=(48,) * 5,
                           dec_patch_size=(48,) * 4, shuffle_orders=True, enable_flash=True), (150, 40), dict(trace="full", grads=True)),
    # no fused attention: the patch shrinks to the smallest scene, float scores
    "no_flash": (dict(_SMALL, enc_depths=(1, 1, 1, 1, 1), dec_depths=(1, 1, 1, 1), enc_patch_size=(48,) * 5,
                      dec_patch_size=(48,) * 4, shuffle_orders=False, enable_flash=False, upcast_attention=True,
                      upcast_softmax=True), (110, 70), dict(trace="full", grads=False)),
    # the same with the relative position bias
    "no_flash_rpe": (dict(_SMALL, enc_depths=(1, 1, 1, 1, 1), dec_depths=(1, 1, 1, 1), enc_patch_size=(48,) * 5,
                          dec_patch_size=(48,) * 4, shuffle_orders=False, enable_flash=False, enable_rpe=True,
                          upcast_attention=True, upcast_softmax=True), (110, 70), dict(trace="coarse", grads=True)),
    # encoder only, the first pooling with stride 4 (two octree levels at once)
    "cls_stride4": (dict(_SMALL, enc_depths=(1, 1, 1, 1, 1), stride=(4, 2, 2, 2), enc_patch_size=(64,) * 5,
                         cls_mode=True, shuffle_orders=True, enable_flash=True), (200,), dict(trace="coarse", grads=False)),
    # decoder patches larger than the encoder's: the padding tables are cached on the Point by the stage's first
    # block (model.py:384-391), so the decoder blocks run on the encoder's patches
    "dec_patch_larger": (dict(_SMALL, enc_depths=(1, 1, 1, 1, 1), dec_depths=(1, 1, 1, 1), enc_patch_size=(32,) * 5,
                              dec_patch_size=(64,) * 4, shuffle_orders=False, enable_flash=True), (100, 30), dict(trace="coarse", grads=False)),
}
FLASH_FLAGS = dict(upcast_attention=False, upcast_softmax=False)


def model_kwargs(name):
    kw = dict(CASES[name][0])
    if kw.get("enable_flash", True):
        kw.update(FLASH_FLAGS)
    return kw


def case_seed(name):
    return 7000 + sorted(CASES).index(name)


def scene_inputs(name):
    """Surface-like voxel sets: every scene is a floor, a wall and a slanted sheet in a 32 x 32 x 16 cell box,
    distinct cells, scene sizes as the case says. Returns grid_coord (N,3) int32, coord (N,3) f32, feat (N,6) f32,
    offset (B,) int64."""
    rng = np.random.default_rng(case_seed(name))
    grids = []
    for n in CASES[name][1]:
        cells = set()
        while len(cells) < n:
            kind = rng.integers(0, 3)
            a, b = int(rng.integers(0, 32)), int(rng.integers(0, 32))
            if kind == 0:
                c = (a // 2, b // 2, int(rng.integers(0, 2)))
            elif kind == 1:
                c = (a // 2, int(rng.integers(12, 14)), b // 4)
            else:
                c = (a, b // 2, min(15, (a + b) // 4))
            cells.add(c)
        g = np.array(sorted(cells), dtype=np.int32)
        grids.append(g[rng.permutation(len(g))])
    grid = np.concatenate(grids)
    coord = ((grid.astype(np.float32) + rng.random(grid.shape, dtype=np.float32)) * 0.05).astype(np.float32)
    feat = rng.standard_normal((len(grid), 6)).astype(np.float32)
    offset = np.cumsum([len(g) for g in grids]).astype(np.int64)
    return grid, coord, feat, offset


def seeded_state_dict(names, shapes, seed):
    """Every tensor of a state_dict drawn from its name and shape alone, the same on every machine with this
    torch: weights ~ N(0, 1/fan_in), biases and running means ~ N(0, 0.1^2), norm scales 1 + N(0, 0.1^2),
    running variances U(0.5, 1.5), the relative position table N(0, 0.2^2)."""
    gen = torch.Generator().manual_seed(int(seed))
    sd = {}
    for name, shape in zip(names, shapes):
        shape = tuple(int(s) for s in shape)
        if name.endswith("num_batches_tracked"):
            sd[name] = torch.zeros(shape, dtype=torch.int64)
            continue
        r = torch.randn(shape, generator=gen) if len(shape) else torch.randn((), generator=gen)
        if name.endswith("running_var"):
            t = 0.5 + torch.rand(shape, generator=gen)
        elif name.endswith("running_mean") or name.endswith(".bias"):
            t = 0.1 * r
        elif name.endswith("rpe_table"):
            t = 0.2 * r
        elif len(shape) == 1:          # LayerNorm / BatchNorm scale
            t = 1.0 + 0.1 * r
        else:                          # Linear (out, in) and convolution (out, k, k, k, in) weights
            t = r / float(np.sqrt(r.numel() / shape[0]))
        sd[name] = t.float()
    return sd


def state_checksum(sd):
    return float(sum(v.double().abs().sum() for v in sd.values()))
