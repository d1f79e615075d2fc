"""HIP patch attention vs the CPU fp32 oracle.
Tolerances (max-abs error relative to max-abs reference): 1e-4 in fp32, 2e-2 in fp16/bf16."""
import numpy as np
import pytest
import torch

from oracle import functional as OF
from oracle import indexing as OI
from gpu_util import DEV, rel_err, to_dev

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-4, torch.float16: 2e-2, torch.bfloat16: 2e-2}


def ops():
    from pointtransformerv3_amd import ops as _ops
    return _ops


def _case(counts, patch, heads, dtype, seed, scale_in=1.0, head_dim=16):
    rng = np.random.default_rng(seed)
    g = torch.Generator().manual_seed(seed)
    n = int(sum(counts))
    C = heads * head_dim
    offset = np.cumsum(counts).astype(np.int64)
    # a per-scene random permutation plays the role of the serialized order
    order = np.concatenate([s + rng.permutation(c) for s, c in zip(np.concatenate([[0], offset[:-1]]), counts)]).astype(np.int64)
    inverse = np.empty(n, np.int64)
    inverse[order] = np.arange(n)
    qkv = (torch.randn(n, 3 * C, generator=g) * scale_in).to(dtype)
    pad, unpad, cu = OI.padding_tables(offset, patch)
    want = OF.serialized_attention_core(qkv.float(), order, inverse, pad, unpad, cu, heads)
    o = ops()
    gp, gu, gc = o.pad_index(to_dev(offset), offset.tolist(), patch)
    src, dst = o.attn_slots(to_dev(order), to_dev(inverse), gp, gu)
    got = o.patch_attention(qkv.to(DEV), heads, src, dst, gc, patch, head_dim ** -0.5)
    return got, want


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("head_dim", [8, 32, 64])
def test_attention_other_head_dims(dtype, head_dim):
    """Head dims other than 16 (model.py:441-443 allows any channels // num_heads) take the thread-per-query
    kernel: same bar, ragged last patch and two scenes."""
    got, want = _case([700, 333], 256, 3, dtype, seed=head_dim, head_dim=head_dim)
    assert got.dtype == dtype and got.shape == want.shape
    assert rel_err(got, want) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_attention_sequences_beyond_the_mfma_kernels_lds(dtype):
    """Patch 3072: sequences of 3072 keys are more than the MFMA kernel keeps in LDS (2368); the half-precision
    call then runs on the thread-per-query kernel instead of failing."""
    got, want = _case([7000, 500], 3072, 2, dtype, seed=21)
    assert rel_err(got, want) < TOL[dtype]
    from pointtransformerv3_amd import _lib
    with pytest.raises(_lib.Ptv3Error):          # a head dim outside 8, 16, 32, 64 is still refused
        _case([100], 32, 2, dtype, seed=1, head_dim=24)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("counts,patch", [([64], 32), ([100], 32), ([37], 64), ([300, 17, 129], 128),
                                          ([2500], 1024), ([1024, 1500], 1024)])
def test_attention_parity(dtype, counts, patch):
    got, want = _case(counts, patch, 4, dtype, seed=len(counts) * 100 + patch)
    assert got.dtype == dtype and got.shape == want.shape
    assert rel_err(got, want) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("counts,heads", [([700], 2), ([513, 1024, 600], 3), ([1000, 33, 1023], 1), ([40_000], 8),
                                          ([5000, 3000, 777], 32), ([1024], 1)])
def test_attention_patch_1024_launch_shapes(dtype, counts, heads):
    """Patch 1024 in half precision, the shape of every released model: sequences shorter than the patch (ragged
    last step, a 33-point scene), more items than resident work-groups (a last partial round cut into query
    ranges), fewer items than work-groups, one item."""
    got, want = _case(counts, 1024, heads, dtype, seed=sum(counts) + heads)
    assert got.dtype == dtype and got.shape == want.shape
    assert torch.isfinite(got.float()).all()
    assert rel_err(got, want) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_attention_is_deterministic(dtype):
    """Two launches over the same input give the same bits."""
    o = ops()
    rng = np.random.default_rng(5)
    counts, heads, patch = [3000, 1500], 4, 1024
    n, C = sum(counts), heads * 16
    offset = np.cumsum(counts).astype(np.int64)
    order = np.concatenate([s + rng.permutation(c) for s, c in zip([0, counts[0]], counts)]).astype(np.int64)
    inverse = np.empty(n, np.int64)
    inverse[order] = np.arange(n)
    qkv = torch.randn(n, 3 * C, generator=torch.Generator().manual_seed(5)).to(dtype).to(DEV)
    gp, gu, gc = o.pad_index(to_dev(offset), offset.tolist(), patch)
    src, dst = o.attn_slots(to_dev(order), to_dev(inverse), gp, gu)
    a = o.patch_attention(qkv, heads, src, dst, gc, patch, 0.25)
    b = o.patch_attention(qkv, heads, src, dst, gc, patch, 0.25)
    assert torch.equal(a, b) and torch.isfinite(a.float()).all()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_attention_large_logits(dtype):
    # |q.k| * scale reaches the tens: the running-max path must keep softmax finite and exact
    got, want = _case([1500], 1024, 2, dtype, seed=9, scale_in=3.0)
    assert torch.isfinite(got.float()).all()
    assert rel_err(got, want) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("scale_in", [1.6, 1.9, 2.4])
def test_attention_mixed_shift_paths(dtype, scale_in):
    # |q||k| bounds straddle the limit below which the kernel skips the running-maximum shift, so
    # query tiles of one launch take different paths; ragged last step, filler slots, two scenes
    got, want = _case([1111, 2300], 1024, 3, dtype, seed=int(scale_in * 10), scale_in=scale_in)
    assert torch.isfinite(got.float()).all()
    assert rel_err(got, want) < TOL[dtype]


def test_attention_config1_shape_fp32():
    # 16 patches of 1024, C=64, 4 heads, fp32
    got, want = _case([16384], 1024, 4, torch.float32, seed=1)
    assert rel_err(got, want) < 1e-4


def test_baseline_config1_serialization_then_one_attention_block_fp32():
    """Baseline configuration 1 as written: 16,384 points uniform in a 5 m cube at grid 0.02 m; z-order and
    Hilbert codes and orders at the adaptive depth (8) and at depth 16, bit-exact; then one SerializedAttention
    (patch 1024, C = 64, 4 heads, seeded weights) on the CPU reference path -- no fused attention, fp32."""
    from oracle import serialization as OS
    from pointtransformerv3_amd import Point, synthetic
    from pointtransformerv3_amd.modules import SerializedAttention
    sc = synthetic.cube_scene(16_384, 1000, 0.02)
    grid = sc["grid_coord"]
    n = len(grid)
    assert n == 16_384 and int(grid.max()).bit_length() == 8
    offset = np.array([n], np.int64)
    batch = np.zeros(n, np.int64)
    orders = ["z", "hilbert"]
    points = {}
    for depth in (None, 16):
        p = Point(grid_coord=torch.from_numpy(grid).to(DEV), offset=torch.from_numpy(offset).to(DEV),
                  feat=torch.zeros(n, 1, device=DEV))
        p.serialization(order=orders, depth=depth)
        want_depth, code, order, inverse = OS.serialize(grid, batch, orders, depth=depth)
        assert p.serialized_depth == want_depth == (8 if depth is None else 16)
        assert np.array_equal(p.serialized_code.cpu().numpy(), code)
        assert np.array_equal(p.serialized_order.cpu().numpy(), order)
        assert np.array_equal(p.serialized_inverse.cpu().numpy(), inverse)
        points[depth] = (p, order, inverse)
    # the block: Linear -> patch attention along the Hilbert order -> Linear
    C, heads, patch = 64, 4, 1024
    torch.manual_seed(1001)
    attn = SerializedAttention(C, heads, patch_size=patch, order_index=1, enable_flash=False).eval()
    sd = {k: v.clone() for k, v in attn.state_dict().items()}
    feat = torch.randn(n, C, generator=torch.Generator().manual_seed(1002))
    p, order, inverse = points[16]
    p.feat = feat.to(DEV)
    with torch.inference_mode():
        got = attn.to(DEV)(p).feat
    assert attn.patch_size == patch and got.dtype == torch.float32
    pad, unpad, cu = OI.padding_tables(offset, patch)
    assert len(cu) == 17
    qkv = torch.nn.functional.linear(feat, sd["qkv.weight"], sd["qkv.bias"])
    core = OF.serialized_attention_core(qkv, order[1], inverse[1], pad, unpad, cu, heads)
    want = torch.nn.functional.linear(core, sd["proj.weight"], sd["proj.bias"])
    assert rel_err(got, want) < 1e-4


def test_baseline_config2_attention_bf16_every_patch():
    """Baseline configuration 2 as written: one room scene of ~100k voxelised points at 2 cm, its Hilbert order
    (adaptive depth), patch 1024, C = 512, 32 heads, q/k/v ~ N(0,1)/4 in bf16. Every patch and head is checked,
    the borrowed tail patch included."""
    from pointtransformerv3_amd import synthetic
    sc = synthetic.room_scene(106_000, 2000, 0.02)
    grid = sc["grid_coord"]
    n, patch, heads, C = len(grid), 1024, 32, 512
    assert 95_000 < n < 106_000 and n % patch != 0
    o = ops()
    depth = int(grid.max()).bit_length()
    code = o.encode_orders(to_dev(grid), torch.zeros(n, dtype=torch.int64, device=DEV), depth, ["hilbert"])
    order_d, inverse_d = o.argsort_rows(code, 3 * depth + 1)
    order, inverse = order_d[0].cpu().numpy(), inverse_d[0].cpu().numpy()
    from oracle import serialization as OS
    assert np.array_equal(order, OS.serialize(grid, np.zeros(n, np.int64), ["hilbert"])[2][0])
    qkv = (torch.randn(n, 3 * C, generator=torch.Generator().manual_seed(2)) / 4).to(torch.bfloat16)
    pad, unpad, cu = OI.padding_tables([n], patch)
    assert len(cu) - 1 == -(-n // patch) and len(pad) == (len(cu) - 1) * patch
    gp, gu, gc = o.pad_index(to_dev(np.array([n])), [n], patch)
    src, dst = o.attn_slots(order_d[0], inverse_d[0], gp, gu)
    got = o.patch_attention(qkv.to(DEV), heads, src, dst, gc, patch, 0.25)
    assert torch.isfinite(got.float()).all()
    want = OF.serialized_attention_core(qkv.float(), order, inverse, pad, unpad, cu, heads)
    assert rel_err(got, want) < 2e-2
    # the tail: the last r points sit in a patch completed with the K - r points in front of them
    last = order[n - (n % patch):]
    assert rel_err(got[torch.as_tensor(last, device=DEV)], want[torch.as_tensor(last)]) < 2e-2


@pytest.mark.parametrize("counts,patch", [([64], 64), ([700, 300], 256), ([2500], 1024)])
def test_attention_rpe_parity_fp32(counts, patch):
    """Relative position bias path (fp32): kernel vs the CPU oracle, table drawn like the reference's."""
    heads, seed = 4, 31
    rng = np.random.default_rng(seed)
    g = torch.Generator().manual_seed(seed)
    n = int(sum(counts))
    C = heads * 16
    offset = np.cumsum(counts).astype(np.int64)
    starts = np.concatenate([[0], offset[:-1]])
    order = np.concatenate([s + rng.permutation(c) for s, c in zip(starts, counts)]).astype(np.int64)
    inverse = np.empty(n, np.int64)
    inverse[order] = np.arange(n)
    qkv = torch.randn(n, 3 * C, generator=g)
    grid = rng.integers(0, 60, size=(n, 3)).astype(np.int32)
    pos_bnd = int((4 * patch) ** (1 / 3) * 2)
    table = torch.randn(3 * (2 * pos_bnd + 1), heads, generator=g) * 0.5
    pad, unpad, cu = OI.padding_tables(offset, patch)
    want = OF.serialized_attention_core(qkv, order, inverse, pad, unpad, cu, heads, rpe=(grid, table, pos_bnd))
    o = ops()
    gp, gu, gc = o.pad_index(to_dev(offset), offset.tolist(), patch)
    src, dst = o.attn_slots(to_dev(order), to_dev(inverse), gp, gu)
    got = o.patch_attention_rpe(qkv.to(DEV), heads, src, dst, gc, patch, 16 ** -0.5, to_dev(grid), table.to(DEV), pos_bnd)
    assert rel_err(got, want) < 1e-4
    zero = o.patch_attention_rpe(qkv.to(DEV), heads, src, dst, gc, patch, 16 ** -0.5, to_dev(grid),
                                 torch.zeros_like(table).to(DEV), pos_bnd)
    plain = o.patch_attention(qkv.to(DEV), heads, src, dst, gc, patch, 16 ** -0.5)
    assert rel_err(zero, plain.cpu()) < 1e-5


def test_attention_module_with_rpe():
    """SerializedAttention(enable_rpe=True, enable_flash=False) as the reference builds it (model.py:319-490):
    the patch shrinks to the smallest scene, the bias table is the module's parameter `rpe.rpe_table`."""
    from pointtransformerv3_amd import Point
    from pointtransformerv3_amd.modules import SerializedAttention
    rng = np.random.default_rng(8)
    torch.manual_seed(8)
    C, heads = 64, 4
    attn = SerializedAttention(C, heads, patch_size=128, order_index=0, enable_rpe=True, enable_flash=False).eval()
    assert attn.rpe.rpe_table.shape == (3 * (2 * int((4 * 128) ** (1 / 3) * 2) + 1), heads)
    assert "rpe.rpe_table" in attn.state_dict()
    counts = [150, 260]
    n = sum(counts)
    grid = rng.integers(0, 40, size=(n, 3)).astype(np.int32)
    offset = np.cumsum(counts).astype(np.int64)
    feat = torch.randn(n, C)
    p = Point(feat=feat.to(DEV), grid_coord=torch.from_numpy(grid).to(DEV), offset=torch.from_numpy(offset).to(DEV))
    p.serialization(order=["z"])
    with torch.inference_mode():
        got = attn.to(DEV)(p).feat.cpu()
    patch = 128                                              # min(150, 260, 128)
    order, inverse = p.serialized_order[0].cpu().numpy(), p.serialized_inverse[0].cpu().numpy()
    pad, unpad, cu = OI.padding_tables(offset, patch)
    sd = {k: v.cpu() for k, v in attn.state_dict().items()}
    qkv = torch.nn.functional.linear(feat, sd["qkv.weight"], sd["qkv.bias"])
    core = OF.serialized_attention_core(qkv, order, inverse, pad, unpad, cu, heads,
                                        rpe=(grid, sd["rpe.rpe_table"], attn.rpe.pos_bnd))
    want = torch.nn.functional.linear(core, sd["proj.weight"], sd["proj.bias"])
    assert rel_err(got, want) < 1e-4
