"""HIP encode / argsort / padding tables vs the CPU oracle: bit-exact."""
import os

import numpy as np
import pytest
import torch

from oracle import indexing as OI
from oracle import serialization as OS
from gpu_util import DEV, to_dev, unique_voxels

pytestmark = pytest.mark.gpu

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "hilbert_golden.npz"))


def ops():
    from pointtransformerv3_amd import ops as _ops
    return _ops


@pytest.mark.parametrize("name", sorted(k[:-3] for k in GOLD.files if k.endswith("_in")))
def test_hilbert_kernel_matches_reference_golden(name):
    depth = int(name.split("_d")[1])
    got = ops().encode_orders(to_dev(GOLD[name + "_in"]), None, depth, ["hilbert"])[0]
    assert np.array_equal(got.cpu().numpy(), GOLD[name + "_out"])


@pytest.mark.parametrize("depth", [1, 4, 8, 9, 12, 16])
@pytest.mark.parametrize("n", [1, 63, 100_003])
def test_encode_all_orders(depth, n):
    rng = np.random.default_rng(depth * 1000 + n)
    g = rng.integers(0, 1 << 16, size=(n, 3)).astype(np.int32)   # wider than depth: low bits are kept
    b = rng.integers(0, 4, size=n).astype(np.int64)
    got = ops().encode_orders(to_dev(g), to_dev(b), depth, list(OS.ORDERS)).cpu().numpy()
    for r, name in enumerate(OS.ORDERS):
        assert np.array_equal(got[r], OS.encode(g, b, depth, name)), name
    got1 = ops().encode_orders(to_dev(g), None, depth, ["hilbert-trans", "z"]).cpu().numpy()
    assert np.array_equal(got1[0], OS.encode(g, None, depth, "hilbert-trans"))
    assert np.array_equal(got1[1], OS.encode(g, None, depth, "z"))


def test_encode_mirror_of_reference_signature():
    from pointtransformerv3_amd.serialization import encode
    g = np.array([[1, 0, 0], [3, 0, 0], [256, 0, 0]], np.int32)
    assert encode(to_dev(g), None, 16, "z").tolist() == [4, 36, 1 << 26]
    b = to_dev(np.array([3, 3, 3], np.int64))
    assert encode(to_dev(g), b, 16, "z").tolist() == [(3 << 48) | 4, (3 << 48) | 36, (3 << 48) | (1 << 26)]


@pytest.mark.parametrize("name", sorted(k[:-3] for k in GOLD.files if k.endswith("_in")))
def test_hilbert_decode_kernel_inverts_reference_golden(name):
    """The codes the reference's hilbert.py encode wrote for these points decode back to the points."""
    from pointtransformerv3_amd.serialization import hilbert_decode
    depth = int(name.split("_d")[1])
    got = hilbert_decode(to_dev(GOLD[name + "_out"]), depth)
    # ("trunc" holds coordinates past the depth: encode keeps their low bits, decode returns those)
    assert got.dtype == torch.int64 and np.array_equal(got.cpu().numpy(), GOLD[name + "_in"] & ((1 << depth) - 1))


@pytest.mark.parametrize("depth", [1, 4, 8, 9, 12, 16])
@pytest.mark.parametrize("n", [1, 63, 100_003])
def test_decode_matches_oracle(depth, n):
    """Random codes (not only images of encode), with a batch index above the curve bits."""
    from pointtransformerv3_amd import serialization as PS
    rng = np.random.default_rng(100 * depth + n % 97)
    low = rng.integers(0, 1 << (3 * depth), size=n, dtype=np.int64)
    b = rng.integers(0, 1 << min(15, 63 - 3 * depth), size=n, dtype=np.int64)
    code = (b << np.int64(3 * depth)) | low
    for order, ref in (("z", OS.z_order_decode), ("hilbert", OS.hilbert_decode)):
        grid, batch = PS.decode(to_dev(code), depth, order)
        assert np.array_equal(grid.cpu().numpy(), ref(low, depth)), order
        assert np.array_equal(batch.cpu().numpy(), b), order
    assert np.array_equal(PS.z_order_decode(to_dev(low), depth).cpu().numpy(), OS.z_order_decode(low, depth))
    assert np.array_equal(PS.hilbert_decode(to_dev(low), depth).cpu().numpy(), OS.hilbert_decode(low, depth))
    # the transposed orders through the operator layer: decode of encode is the identity for all four
    g = rng.integers(0, 1 << depth, size=(n, 3)).astype(np.int32)
    codes = ops().encode_orders(to_dev(g), to_dev(b), depth, list(OS.ORDERS))
    for r, order in enumerate(OS.ORDERS):
        grid, batch = ops().decode_order(codes[r], depth, order)
        assert np.array_equal(grid.cpu().numpy(), g) and np.array_equal(batch.cpu().numpy(), b), order


def test_decode_round_trip_full_size():
    from pointtransformerv3_amd import serialization as PS
    rng = np.random.default_rng(5)
    g = to_dev(rng.integers(0, 1 << 16, size=(6_400_000, 3)).astype(np.int32))
    b = to_dev(np.sort(rng.integers(0, 4, size=6_400_000)).astype(np.int64))
    for order in ("z", "hilbert"):
        grid, batch = PS.decode(PS.encode(g, b, 16, order), 16, order)
        assert torch.equal(grid, g.long()) and torch.equal(batch, b)
    assert torch.equal(PS.z_order_decode(PS.z_order_encode(g, 16), 16), g.long())
    assert torch.equal(PS.hilbert_decode(PS.hilbert_encode(g, 16), 16), g.long())


def test_decode_mirror_of_reference_signature():
    from pointtransformerv3_amd.serialization import decode, z_order_decode
    from pointtransformerv3_amd._lib import Ptv3Error
    code = to_dev(np.array([4, 36, 1 << 26, (3 << 48) | 7], np.int64))
    grid, batch = decode(code, 16, "z")
    assert grid.tolist() == [[1, 0, 0], [3, 0, 0], [256, 0, 0], [1, 1, 1]] and batch.tolist() == [0, 0, 0, 3]
    assert z_order_decode(code[:0], 16).shape == (0, 3)
    with pytest.raises(AssertionError):
        decode(code, 16, "z-trans")             # default.py:29 takes "z" and "hilbert" only
    with pytest.raises(Ptv3Error):
        decode(code, 17, "z")


def test_encode_rejects_bad_depth_and_cpu_tensors():
    from pointtransformerv3_amd._lib import Ptv3Error
    g = to_dev(np.zeros((4, 3), np.int32))
    with pytest.raises(Ptv3Error):
        ops().encode_orders(g, None, 17, ["z"])
    with pytest.raises(Ptv3Error):
        ops().encode_orders(g.cpu(), None, 8, ["z"])


@pytest.mark.parametrize("n,extent,nb", [(1, 4, 1), (2047, 32, 1), (2049, 32, 2), (50_000, 64, 3)])
def test_argsort_unique_codes_bit_exact(n, extent, nb):
    rng = np.random.default_rng(n)
    g, batch, _ = unique_voxels(rng, n, extent, nb)
    depth, code, order, inverse = OS.serialize(g, batch)
    key_bits = 3 * depth + max(1, (nb - 1).bit_length())
    o, inv = ops().argsort_rows(to_dev(code), key_bits)
    assert np.array_equal(o.cpu().numpy(), order)
    assert np.array_equal(inv.cpu().numpy(), inverse)


def test_argsort_full_size_properties():
    # 4 x 100k-point scenes worth of codes at depth 16: sortedness + permutation validity
    rng = np.random.default_rng(5)
    n = 400_000
    g, batch, _ = unique_voxels(rng, n // 4, 200, 4)
    code = np.stack([OS.encode(g, batch, 16, o) for o in OS.ORDERS])
    o, inv = ops().argsort_rows(to_dev(code), 3 * 16 + 2)
    o, inv = o.cpu().numpy(), inv.cpu().numpy()
    for r in range(4):
        assert np.all(np.diff(code[r][o[r]]) > 0)
        assert np.array_equal(inv[r][o[r]], np.arange(n))
    assert np.array_equal(o, np.argsort(code, axis=1, kind="stable"))


def test_argsort_ties_are_stable():
    rng = np.random.default_rng(8)
    code = rng.integers(0, 50, size=(2, 10_000)).astype(np.int64)
    o, inv = ops().argsort_rows(to_dev(code), 6)
    assert np.array_equal(o.cpu().numpy(), np.argsort(code, axis=1, kind="stable"))


@pytest.mark.parametrize("counts,patch", [([2500], 1024), ([1500], 1024), ([1024], 1024), ([700], 1024),
                                          ([1300, 700, 2049], 512), ([5, 0, 40], 16), ([100_000], 1024)])
def test_pad_index(counts, patch):
    offset = np.cumsum(counts).astype(np.int64)
    pad, unpad, cu = OI.padding_tables(offset, patch)
    gp, gu, gc = ops().pad_index(to_dev(offset), offset.tolist(), patch)
    assert np.array_equal(gp.cpu().numpy(), pad)
    assert np.array_equal(gu.cpu().numpy(), unpad)
    assert gc.dtype == torch.int32 and np.array_equal(gc.cpu().numpy(), cu)


def test_attn_slots():
    rng = np.random.default_rng(1)
    n, patch = 2500, 1024
    order = rng.permutation(n).astype(np.int64)
    inverse = np.empty(n, np.int64)
    inverse[order] = np.arange(n)
    pad, unpad, _ = OI.padding_tables([n], patch)
    src, dst = ops().attn_slots(to_dev(order), to_dev(inverse), to_dev(pad), to_dev(unpad))
    want_src = order[pad]
    primary = unpad[inverse[want_src]] == np.arange(len(pad))
    assert np.array_equal(src.cpu().numpy(), want_src)
    assert np.array_equal(dst.cpu().numpy(), np.where(primary, want_src, -1))
    assert primary.sum() == n


def test_grid_max():
    rng = np.random.default_rng(3)
    for n in (1, 77, 300_001):
        g = rng.integers(-5, 70_000, size=(n, 3)).astype(np.int32)
        assert ops().grid_max(to_dev(g)).tolist() == g.max(0).tolist()
    # rows of a larger tensor: the first value is not on a 16-byte boundary
    g = rng.integers(-5, 70_000, size=(5003, 3)).astype(np.int32)
    dev = to_dev(g)
    for skip in (1, 2, 3, 5000, 5002):
        assert ops().grid_max(dev[skip:]).tolist() == g[skip:].max(0).tolist()


@pytest.mark.parametrize("sizes,grid", [([5000], 0.05), ([30_000, 1, 0, 12_345], 0.02), ([0, 700, 0], 0.1),
                                        ([200_000, 150_000], 0.02)])
def test_voxelize_matches_numpy(sizes, grid):
    from pointtransformerv3_amd import ops, voxelize
    rng = np.random.default_rng(sum(sizes))
    # points on a few planes plus noise, shifted per scene; duplicates of voxels are common
    coord = np.concatenate([np.concatenate([rng.random((n, 2)) * 6, rng.integers(0, 3, (n, 1)) + rng.normal(0, 0.004, (n, 1))], 1)
                            + rng.normal(0, 50, 3) for n in sizes]).astype(np.float32)
    offset = np.cumsum(sizes).astype(np.int64)
    wg, wi, winv, wends = OI.voxelize(coord, offset, grid)
    got = ops.voxelize(torch.from_numpy(coord).to(DEV), torch.from_numpy(offset).to(DEV), grid)
    assert np.array_equal(got["grid_coord"].cpu().numpy(), wg)
    assert np.array_equal(got["index"].cpu().numpy(), wi)
    assert np.array_equal(got["inverse"].cpu().numpy(), winv)
    assert np.array_equal(got["offset"].cpu().numpy(), wends)
    assert len(wi) < len(coord) or min(s for s in sizes if s) == 1   # the cases do merge points
    # the batch dictionary it makes runs through the model's own serialization
    feat = torch.from_numpy(rng.random((len(coord), 4)).astype(np.float32)).to(DEV)
    batch = voxelize.grid_sample(torch.from_numpy(coord).to(DEV), torch.from_numpy(offset).to(DEV), grid, feat=feat)
    assert batch["feat"].shape == (len(wi), 4) and torch.equal(batch["feat"], feat[batch["index"]])
    assert torch.equal(batch["coord"], torch.from_numpy(coord).to(DEV)[batch["index"]])


def test_voxelize_rejects_extents_beyond_16_bits():
    from pointtransformerv3_amd import ops
    coord = torch.tensor([[0.0, 0.0, 0.0], [700.0, 0.0, 0.0]], device=DEV)
    with pytest.raises(RuntimeError, match="16 bits"):
        ops.voxelize(coord, torch.tensor([2], device=DEV), 0.01)


def test_voxelize_train_mode_draws_a_uniform_member_of_every_voxel():
    """GridSample's train mode: one random member per voxel. Checked by what any correct draw satisfies: the same
    voxels as the first-point mode, every kept point inside its voxel, `inverse` consistent, another seed another
    draw, and over many two-point voxels each member kept about half of the time."""
    from pointtransformerv3_amd import ops, voxelize
    rng = np.random.default_rng(5)
    sizes = [60_000, 45_000]
    coord = np.concatenate([rng.random((n, 3)) * np.array([4.0, 4.0, 0.2]) + rng.normal(0, 20, 3) for n in sizes]).astype(np.float32)
    offset = np.cumsum(sizes).astype(np.int64)
    grid = 0.05
    wg, wi, winv, wends = OI.voxelize(coord, offset, grid)
    c, o = torch.from_numpy(coord).to(DEV), torch.from_numpy(offset).to(DEV)
    draws = [ops.voxelize(c, o, grid, seed=s) for s in (1, 2, 12345)]
    scene = np.searchsorted(offset, np.arange(len(coord)), side="right")
    first_voxel = winv                                            # voxel id (first-point numbering) of every input point
    for d in draws:
        idx = d["index"].cpu().numpy()
        assert len(idx) == len(wi) and np.all(np.diff(idx) > 0)   # kept points in input order, one per voxel
        assert np.array_equal(np.sort(first_voxel[idx]), np.arange(len(wi)))   # exactly one from every voxel
        assert np.array_equal(d["offset"].cpu().numpy(), wends)
        g = d["grid_coord"].cpu().numpy()
        assert np.array_equal(g, wg[first_voxel[idx]])            # its grid coordinate is its voxel's
        inv = d["inverse"].cpu().numpy()
        assert np.array_equal(first_voxel[idx[inv]], first_voxel) and np.array_equal(scene[idx[inv]], scene)
    a, b = draws[0]["index"].cpu().numpy(), draws[1]["index"].cpu().numpy()
    assert (a != b).mean() > 0.2
    # two-member voxels: the first member is kept in about half of them, for every seed
    counts = np.bincount(first_voxel, minlength=len(wi))
    pairs = np.nonzero(counts == 2)[0]
    assert len(pairs) > 3000
    for d in draws:
        idx = d["index"].cpu().numpy()
        kept_of = np.empty(len(wi), np.int64)
        kept_of[first_voxel[idx]] = idx
        frac = (kept_of[pairs] == wi[pairs]).mean()
        assert abs(frac - 0.5) < 4 * 0.5 / np.sqrt(len(pairs)), frac
    # seed 0 is the first-point mode; grid_sample's train mode keeps features and coordinates of the drawn points
    assert np.array_equal(ops.voxelize(c, o, grid, seed=0)["index"].cpu().numpy(), wi)
    feat = torch.from_numpy(rng.random((len(coord), 3)).astype(np.float32)).to(DEV)
    batch = voxelize.grid_sample(c, o, grid, feat=feat, mode="train", seed=7)
    assert torch.equal(batch["feat"], feat[batch["index"]]) and not np.array_equal(batch["index"].cpu().numpy(), wi)
