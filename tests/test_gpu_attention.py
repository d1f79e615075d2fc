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


def _case(counts, patch, heads, dtype, seed, scale_in=1.0):
    rng = np.random.default_rng(seed)
    g = torch.Generator().manual_seed(seed)
    n = int(sum(counts))
    C = heads * 16
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
    got = o.patch_attention(qkv.to(DEV), heads, src, dst, gc, patch, 16 ** -0.5)
    return got, want


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("counts,patch", [([64], 32), ([100], 32), ([37], 64), ([300, 17, 129], 128),
                                          ([2500], 1024), ([1024, 1500], 1024)])
def test_attention_parity(dtype, counts, patch):
    got, want = _case(counts, patch, 4, dtype, seed=len(counts) * 100 + patch)
    assert got.dtype == dtype and got.shape == want.shape
    assert rel_err(got, want) < TOL[dtype]


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


def test_attention_config2_shape_bf16_sampled():
    # one 100k-point scene, C=512, 32 heads, bf16, q/k/v ~ N(0,1)/4; the oracle checks a
    # sample of patches (first, middle, last-with-fillers), every head
    n, patch, heads, C = 100_000, 1024, 32, 512
    rng = np.random.default_rng(2)
    g = torch.Generator().manual_seed(2)
    order = rng.permutation(n).astype(np.int64)
    inverse = np.empty(n, np.int64)
    inverse[order] = np.arange(n)
    qkv = (torch.randn(n, 3 * C, generator=g) / 4).to(torch.bfloat16)
    pad, unpad, cu = OI.padding_tables([n], patch)
    o = ops()
    gp, gu, gc = o.pad_index(to_dev(np.array([n])), [n], patch)
    src, dst = o.attn_slots(to_dev(order), to_dev(inverse), gp, gu)
    got = o.patch_attention(qkv.to(DEV), heads, src, dst, gc, patch, 0.25).float().cpu()
    assert torch.isfinite(got).all()
    rows = order[pad]
    for p in (0, 48, 96, 97):
        s, e = int(cu[p]), int(cu[p + 1])
        want = OF.patch_attention(qkv[rows[s:e]].float(), [0, e - s], heads)
        primary = unpad[inverse[rows[s:e]]] == np.arange(s, e)
        sel = torch.as_tensor(rows[s:e][primary])
        err = (got[sel] - want[torch.as_tensor(primary)]).abs().max() / want.abs().max()
        assert err < 2e-2, (p, float(err))
