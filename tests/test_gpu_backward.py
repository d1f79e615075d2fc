"""HIP backward kernels (attention, submanifold convolution, segment reduction, unpooling) and the
whole model's parameter gradients vs autograd over the CPU oracle.
Tolerances (max-abs error relative to max-abs reference): 1e-4 in fp32, 2e-2 in fp16 / bf16."""
import numpy as np
import pytest
import torch

from oracle import functional as OF
from oracle import grad as OG
from oracle import indexing as OI
from oracle.forward import ptv3_forward
from gpu_util import DEV, rel_err, to_dev, unique_voxels

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-4, torch.float16: 2e-2, torch.bfloat16: 2e-2}


def ops():
    from pointtransformerv3_amd import ops as _ops
    return _ops


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("counts,patch", [([64], 32), ([100], 32), ([37], 64), ([3], 64), ([300, 17, 129], 128),
                                          ([2500], 1024), ([1024, 1500], 1024)])
def test_attention_backward_parity(dtype, counts, patch):
    from pointtransformerv3_amd.autograd import PatchAttention
    heads, seed = 4, len(counts) * 100 + patch
    rng = np.random.default_rng(seed)
    g = torch.Generator().manual_seed(seed)
    n, C = int(sum(counts)), heads * 16
    offset = np.cumsum(counts).astype(np.int64)
    starts = np.concatenate([[0], offset[:-1]])
    order = np.concatenate([s + rng.permutation(c) for s, c in zip(starts, counts)]).astype(np.int64)
    inverse = np.empty(n, np.int64)
    inverse[order] = np.arange(n)
    qkv = torch.randn(n, 3 * C, generator=g).to(dtype)
    dout = torch.randn(n, C, generator=g).to(dtype)
    pad, unpad, cu = OI.padding_tables(offset, patch)
    want = OG.serialized_attention_grad(qkv.float(), dout.float(), order, inverse, pad, unpad, cu, heads)
    o = ops()
    gp, gu, gc = o.pad_index(to_dev(offset), offset.tolist(), patch)
    src, dst = o.attn_slots(to_dev(order), to_dev(inverse), gp, gu)
    x = qkv.to(DEV).requires_grad_(True)
    out = PatchAttention.apply(x, heads, src, dst, gc, patch, 16 ** -0.5)
    out.backward(dout.to(DEV))
    assert x.grad.dtype == dtype and x.grad.shape == want.shape
    assert torch.isfinite(x.grad.float()).all()
    assert rel_err(x.grad, want) < TOL[dtype]
    # each third on its own scale: dq and dk are much smaller than dv
    for part in range(3):
        sl = slice(part * C, (part + 1) * C)
        assert rel_err(x.grad[:, sl], want[:, sl]) < TOL[dtype], part


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("counts,patch,p", [([100], 32, 0.25), ([300, 17, 129], 128, 0.1), ([2500], 1024, 0.5)])
def test_attention_dropout_forward_and_backward_parity(dtype, counts, patch, p):
    """Attention dropout: the kernels' mask is a hash of (seed, head, query slot, key slot) that the oracle
    restates, so result and gradient are compared exactly like without dropout; the kept fraction is 1 - p."""
    from pointtransformerv3_amd.autograd import PatchAttention
    heads, seed = 4, 1000 + patch
    rng = np.random.default_rng(seed)
    g = torch.Generator().manual_seed(seed)
    n, C = int(sum(counts)), heads * 16
    offset = np.cumsum(counts).astype(np.int64)
    starts = np.concatenate([[0], offset[:-1]])
    order = np.concatenate([s + rng.permutation(c) for s, c in zip(starts, counts)]).astype(np.int64)
    inverse = np.empty(n, np.int64)
    inverse[order] = np.arange(n)
    qkv = torch.randn(n, 3 * C, generator=g).to(dtype)
    dout = torch.randn(n, C, generator=g).to(dtype)
    pad, unpad, cu = OI.padding_tables(offset, patch)
    xr = qkv.float().clone().requires_grad_(True)
    want = OF.serialized_attention_core(xr, order, inverse, pad, unpad, cu, heads, dropout=(p, seed))
    want.backward(dout.float())
    plain = OF.serialized_attention_core(qkv.float(), order, inverse, pad, unpad, cu, heads)
    assert rel_err(want, plain) > 0.05                                   # the mask does something
    keep = OF.dropout_keep_mask(seed, 1, np.arange(len(pad)), np.arange(min(len(pad), 512)), p)
    assert abs(keep.mean() - (1 - p)) < 0.01
    o = ops()
    gp, gu, gc = o.pad_index(to_dev(offset), offset.tolist(), patch)
    src, dst = o.attn_slots(to_dev(order), to_dev(inverse), gp, gu)
    x = qkv.to(DEV).requires_grad_(True)
    out = PatchAttention.apply(x, heads, src, dst, gc, patch, 16 ** -0.5, p, seed)
    out.backward(dout.to(DEV))
    assert rel_err(out, want) < TOL[dtype]
    assert rel_err(x.grad, xr.grad) < TOL[dtype]
    # another seed, another mask; the same seed, the same result
    again = PatchAttention.apply(x.detach(), heads, src, dst, gc, patch, 16 ** -0.5, p, seed)
    other = PatchAttention.apply(x.detach(), heads, src, dst, gc, patch, 16 ** -0.5, p, seed + 1)
    assert torch.equal(again, out.detach()) and rel_err(other, want) > 0.05


@pytest.mark.parametrize("drop_p", [0.0, 0.2])
@pytest.mark.parametrize("counts,patch", [([64], 64), ([700, 300], 256), ([1500], 512)])
def test_attention_rpe_backward_parity_fp32(counts, patch, drop_p):
    """Relative position bias path (with and without attention dropout): result, gradients of qkv and of the bias
    table vs autograd over the CPU oracle."""
    from pointtransformerv3_amd.autograd import PatchAttentionRpe
    heads, seed = 4, 33
    rng = np.random.default_rng(seed)
    g = torch.Generator().manual_seed(seed)
    n, C = int(sum(counts)), heads * 16
    offset = np.cumsum(counts).astype(np.int64)
    starts = np.concatenate([[0], offset[:-1]])
    order = np.concatenate([s + rng.permutation(c) for s, c in zip(starts, counts)]).astype(np.int64)
    inverse = np.empty(n, np.int64)
    inverse[order] = np.arange(n)
    grid = rng.integers(0, 40, size=(n, 3)).astype(np.int32)
    pos_bnd = int((4 * patch) ** (1 / 3) * 2)
    table = (torch.randn(3 * (2 * pos_bnd + 1), heads, generator=g) * 0.3)
    qkv = torch.randn(n, 3 * C, generator=g)
    dout = torch.randn(n, C, generator=g)
    pad, unpad, cu = OI.padding_tables(offset, patch)
    xq = qkv.clone().requires_grad_(True)
    tb = table.clone().requires_grad_(True)
    dropout = (drop_p, 77) if drop_p else None
    want = OF.serialized_attention_core(xq, order, inverse, pad, unpad, cu, heads, rpe=(grid, tb, pos_bnd), dropout=dropout)
    want.backward(dout)
    o = ops()
    gp, gu, gc = o.pad_index(to_dev(offset), offset.tolist(), patch)
    src, dst = o.attn_slots(to_dev(order), to_dev(inverse), gp, gu)
    x = qkv.to(DEV).requires_grad_(True)
    t = table.to(DEV).requires_grad_(True)
    out = PatchAttentionRpe.apply(x, t, heads, src, dst, gc, patch, 0.25, to_dev(grid), pos_bnd, drop_p, 77)
    out.backward(dout.to(DEV))
    assert rel_err(out, want) < 1e-4
    assert rel_err(x.grad, xq.grad) < 1e-4
    assert rel_err(t.grad, tb.grad) < 1e-4


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_attention_backward_recomputes_lse_when_not_kept(dtype):
    """The backward entry point without the forward's log-sum-exp rows: same result as with them."""
    heads, patch, counts = 2, 128, [300, 77]
    rng = np.random.default_rng(7)
    g = torch.Generator().manual_seed(7)
    n, C = sum(counts), heads * 16
    offset = np.cumsum(counts).astype(np.int64)
    order = np.concatenate([s + rng.permutation(c) for s, c in zip([0, counts[0]], counts)]).astype(np.int64)
    inverse = np.empty(n, np.int64)
    inverse[order] = np.arange(n)
    o = ops()
    gp, gu, gc = o.pad_index(to_dev(offset), offset.tolist(), patch)
    src, dst = o.attn_slots(to_dev(order), to_dev(inverse), gp, gu)
    qkv = torch.randn(n, 3 * C, generator=g).to(dtype).to(DEV)
    dout = torch.randn(n, C, generator=g).to(dtype).to(DEV)
    args = (heads, src, dst, gc, patch, 0.25)
    out, lse = o.patch_attention_lse(qkv, *args)
    assert torch.equal(out, o.patch_attention(qkv, *args))
    kept = o.patch_attention_bwd(qkv, out, dout, *args, lse=lse)
    redone = o.patch_attention_bwd(qkv, out, dout, *args)
    assert rel_err(redone, kept.float().cpu()) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("cin,cout,ks,n", [(6, 32, 5, 1500), (32, 32, 3, 2000), (64, 64, 3, 3000), (128, 128, 3, 1200),
                                           (48, 80, 3, 700)])
def test_subm_conv_backward_parity(dtype, cin, cout, ks, n):
    from pointtransformerv3_amd.sparse import SparseConvTensor, SubMConv3d
    rng = np.random.default_rng(cin + cout + ks)
    grid, batch, _ = unique_voxels(rng, n, 20, nb=2)
    idx = np.concatenate([batch[:, None], grid], 1).astype(np.int32)
    torch.manual_seed(cin * 7 + ks)
    conv = SubMConv3d(cin, cout, ks, bias=True, indice_key="k")
    feat = torch.randn(len(idx), cin).to(dtype)
    dout = torch.randn(len(idx), cout).to(dtype)
    w = conv.weight.detach().to(dtype).float()
    b = conv.bias.detach().to(dtype).float()
    nbr = OI.subm_kmap(idx, ks)
    dfeat, dw, db = OG.subm_conv_grad(feat.float(), nbr, w, b, dout.float())
    conv = conv.to(DEV, dtype)
    x = feat.to(DEV).requires_grad_(True)
    sp = SparseConvTensor(x, to_dev(idx), [32, 32, 32], 2)
    out = conv(sp).features
    assert rel_err(out, OF.subm_conv(feat.float(), nbr, w, b)) < TOL[dtype]
    out.backward(dout.to(DEV))
    assert rel_err(x.grad, dfeat) < TOL[dtype]
    assert rel_err(conv.weight.grad, dw) < TOL[dtype]
    assert rel_err(conv.bias.grad, db) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("n,k,nout", [(5000, 32, 96), (70001, 128, 512), (333, 512, 64), (1, 8, 8), (20000, 72, 40)])
def test_linear_backward_parity(dtype, n, k, nout):
    """The Linear autograd function (row kernel forward, row-reduction kernel for the weight gradient)
    against torch CPU autograd in fp32 on the same rounded inputs."""
    from pointtransformerv3_amd.autograd import Linear
    g = torch.Generator().manual_seed(n + k)
    x = torch.randn(n, k, generator=g).to(dtype)
    w = (torch.randn(nout, k, generator=g) / k ** 0.5).to(dtype)
    b = torch.randn(nout, generator=g).to(dtype)
    dout = torch.randn(n, nout, generator=g).to(dtype)
    xr, wr, br = (t.float().clone().requires_grad_(True) for t in (x, w, b))
    torch.nn.functional.linear(xr, wr, br).backward(dout.float())
    xg, wg, bg = (t.detach().to(DEV).requires_grad_(True) for t in (x, w, b))
    out = Linear.apply(xg, wg, bg)
    out.backward(dout.to(DEV))
    assert rel_err(out, torch.nn.functional.linear(x.float(), w.float(), b.float())) < TOL[dtype]
    assert rel_err(xg.grad, xr.grad) < TOL[dtype]
    assert rel_err(wg.grad, wr.grad) < TOL[dtype]
    assert rel_err(bg.grad, br.grad) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("n,c", [(1, 32), (4097, 32), (3000, 64), (2500, 128), (1111, 256), (700, 512)])
def test_layer_norm_backward_parity(dtype, n, c):
    from pointtransformerv3_amd.autograd import LayerNorm
    g = torch.Generator().manual_seed(n + c)
    x = (torch.randn(n, c, generator=g) * 2 + 0.5).to(dtype)
    w = (torch.rand(c, generator=g) + 0.5).to(dtype)
    b = torch.randn(c, generator=g).to(dtype)
    dout = torch.randn(n, c, generator=g).to(dtype)
    xr, wr, br = (t.float().clone().requires_grad_(True) for t in (x, w, b))
    want = torch.nn.functional.layer_norm(xr, (c,), wr, br, 1e-5)
    want.backward(dout.float())
    xg, wg, bg = (t.detach().to(DEV).requires_grad_(True) for t in (x, w, b))
    out = LayerNorm.apply(xg, wg, bg, 1e-5)
    out.backward(dout.to(DEV))
    assert rel_err(out, want) < TOL[dtype]
    assert rel_err(xg.grad, xr.grad) < TOL[dtype]
    assert rel_err(wg.grad, wr.grad) < TOL[dtype]
    assert rel_err(bg.grad, br.grad) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("n,c,gelu,training", [(5000, 32, True, True), (777, 64, False, True), (2, 128, True, True),
                                               (3001, 256, True, False), (900, 512, True, True)])
def test_batch_norm_act_parity(dtype, n, c, gelu, training):
    """BatchNorm1d (+ GELU) as one autograd node: result, running averages and all gradients against torch CPU in
    fp32 on the same rounded inputs; a mean far from zero checks that the variance does not cancel."""
    from pointtransformerv3_amd.autograd import BatchNormAct
    g = torch.Generator().manual_seed(n + c)
    x = (torch.randn(n, c, generator=g) * 1.5 + 6.0).to(dtype)
    dout = torch.randn(n, c, generator=g).to(dtype)
    ref = torch.nn.BatchNorm1d(c, eps=1e-3, momentum=0.01)
    with torch.no_grad():
        ref.weight.copy_(torch.rand(c, generator=g) + 0.5)
        ref.bias.copy_(torch.randn(c, generator=g))
        ref.running_mean.copy_(torch.randn(c, generator=g) + 6.0)
        ref.running_var.copy_(torch.rand(c, generator=g) + 1.5)
    import copy
    mod = copy.deepcopy(ref).to(DEV)
    ref.train(training)
    mod.train(training)
    xr = x.float().clone().requires_grad_(True)
    want = ref(xr)
    want = torch.nn.functional.gelu(want) if gelu else want
    want.backward(dout.float())
    xg = x.detach().to(DEV).requires_grad_(True)
    out = BatchNormAct.apply(xg, mod.weight, mod.bias, mod, gelu)
    out.backward(dout.to(DEV))
    tol = TOL[dtype] if dtype != torch.float32 else 2e-4   # sums over thousands of rows in another order
    assert out.dtype == dtype and rel_err(out, want) < tol
    assert rel_err(xg.grad, xr.grad) < tol
    assert rel_err(mod.weight.grad, ref.weight.grad) < tol
    assert rel_err(mod.bias.grad, ref.bias.grad) < tol
    assert rel_err(mod.running_mean, ref.running_mean) < 1e-4 and rel_err(mod.running_var, ref.running_var) < 1e-3
    assert int(mod.num_batches_tracked) == int(ref.num_batches_tracked)


@pytest.mark.parametrize("with_mask", [False, True])
@pytest.mark.parametrize("skip_dtype,branch_dtype", [(torch.float32, torch.float32), (torch.float32, torch.bfloat16),
                                                     (torch.float16, torch.float16)])
def test_add_layer_norm_backward_parity(skip_dtype, branch_dtype, with_mask):
    """Residual add (+ per-row stochastic-depth factor) and the following LayerNorm as one autograd node: both
    results and all four gradients against torch CPU autograd, with a gradient arriving at the sum as well."""
    from pointtransformerv3_amd.autograd import AddLayerNorm
    n, c = 3001, 64
    g = torch.Generator().manual_seed(4)
    skip = torch.randn(n, c, generator=g).to(skip_dtype)
    branch = torch.randn(n, c, generator=g).to(branch_dtype)
    mask = ((torch.rand(n, 1, generator=g) < 0.7).float() / 0.7).to(branch_dtype) if with_mask else None
    w = (torch.rand(c, generator=g) + 0.5)
    b = torch.randn(c, generator=g)
    ds = torch.randn(n, c, generator=g)
    dy = torch.randn(n, c, generator=g)
    sr, br, wr, bb = (t.float().clone().requires_grad_(True) for t in (skip, branch, w, b))
    s_want = sr + br * (mask.float() if with_mask else 1.0)
    y_want = torch.nn.functional.layer_norm(s_want, (c,), wr, bb, 1e-5)
    torch.autograd.backward([s_want, y_want], [ds, dy])
    sg, bg, wg, bg2 = (t.detach().to(DEV).requires_grad_(True) for t in (skip, branch, w, b))
    s_got, y_got = AddLayerNorm.apply(sg, bg, None if mask is None else mask.to(DEV), wg, bg2, 1e-5)
    torch.autograd.backward([s_got, y_got], [ds.to(DEV).to(s_got.dtype), dy.to(DEV).to(y_got.dtype)])
    tol = TOL[torch.promote_types(skip_dtype, branch_dtype)]
    assert rel_err(s_got, s_want) < tol and rel_err(y_got, y_want) < tol
    assert rel_err(sg.grad, sr.grad) < tol
    assert rel_err(bg.grad, br.grad) < TOL[branch_dtype]
    assert rel_err(wg.grad, wr.grad) < tol
    assert rel_err(bg2.grad, bb.grad) < tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("reduce", ["max", "min", "sum", "mean"])
def test_segment_reduce_backward_parity(dtype, reduce):
    from pointtransformerv3_amd.autograd import SegmentReduce
    rng = np.random.default_rng(11)
    n, c, m = 5000, 64, 1300
    indices = rng.permutation(n)
    cuts = np.sort(rng.choice(np.arange(1, n), m - 1, replace=False))
    idx_ptr = np.concatenate([[0], cuts, [n]]).astype(np.int64)
    g = torch.Generator().manual_seed(3)
    src = torch.randn(n, c, generator=g).to(dtype)
    dout = torch.randn(m, c, generator=g).to(dtype)
    want = OG.segment_csr_grad(src.float(), indices, idx_ptr, reduce, dout.float())
    x = src.to(DEV).requires_grad_(True)
    SegmentReduce.apply(x, to_dev(indices), to_dev(idx_ptr), reduce).backward(dout.to(DEV))
    # half-precision sources can tie inside a cluster: compare where the oracle's pick is unambiguous
    if dtype == torch.float32 or reduce in ("sum", "mean"):
        assert rel_err(x.grad, want) < TOL[dtype]
    else:
        got = x.grad.float().cpu()
        per_cluster = torch.zeros(m, c).index_add_(0, torch.repeat_interleave(torch.arange(m), torch.as_tensor(np.diff(idx_ptr))),
                                                   got[torch.as_tensor(indices)])
        assert torch.allclose(per_cluster, dout.float(), atol=1e-3)   # every cluster hands its gradient to one member
        assert ((got != 0) == (want != 0)).float().mean() > 0.999


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_unpool_add_backward_parity(dtype):
    from pointtransformerv3_amd.autograd import UnpoolAdd
    rng = np.random.default_rng(12)
    n, c, m = 4000, 32, 900
    cluster = np.sort(np.concatenate([np.arange(m), rng.integers(0, m, size=n - m)]))
    perm = rng.permutation(n)
    cluster = cluster[perm]                      # cluster id per parent row
    indices = np.argsort(cluster, kind="stable")  # member lists
    idx_ptr = np.concatenate([[0], np.cumsum(np.bincount(cluster, minlength=m))]).astype(np.int64)
    g = torch.Generator().manual_seed(5)
    parent = torch.randn(n, c, generator=g).to(dtype).to(DEV).requires_grad_(True)
    child = torch.randn(m, c, generator=g).to(dtype).to(DEV).requires_grad_(True)
    dout = torch.randn(n, c, generator=g).to(dtype)
    out = UnpoolAdd.apply(parent, child, to_dev(cluster), to_dev(indices), to_dev(idx_ptr))
    out.backward(dout.to(DEV))
    dparent, dchild = OG.unpool_add_grad(dout.float(), cluster, m)
    assert rel_err(parent.grad, dparent) < TOL[dtype]
    assert rel_err(child.grad, dchild) < TOL[dtype]


def _small_model(**kw):
    from pointtransformerv3_amd import PointTransformerV3
    cfg = dict(enc_depths=(1, 1, 1, 1, 1), dec_depths=(1, 1, 1, 1), enc_patch_size=(256,) * 5, dec_patch_size=(256,) * 4,
               shuffle_orders=False, drop_path=0.0)
    cfg.update(kw)
    return PointTransformerV3(**cfg), cfg


def _scene(n=1500, scenes=2, seed=21):
    from pointtransformerv3_amd import synthetic
    sc = [synthetic.room_scene(n, seed + i, 0.05) for i in range(scenes)]
    d = synthetic.collate(sc)
    return d, synthetic.room_features(d["coord"], seed)


def test_model_parameter_gradients_fp32_against_oracle_autograd():
    """Every parameter's gradient of a random linear functional of the output, BatchNorm on running statistics
    (what the oracle forward restates), attention in float (enable_flash=False) so that 1e-4 applies."""
    torch.manual_seed(0)
    model, cfg = _small_model(enable_flash=False)
    model.eval()
    d, feat = _scene()
    torch.manual_seed(5)
    perms = [None] + [torch.randperm(4).numpy() for _ in range(4)]
    sd = {k: v.detach().clone().requires_grad_(v.is_floating_point() and "running" not in k)
          for k, v in model.state_dict().items()}
    okw = {k: v for k, v in cfg.items() if k not in ("shuffle_orders", "drop_path")}
    want_out = ptv3_forward(sd, d["grid_coord"], feat, d["offset"], perms=perms, **okw)
    g = torch.Generator().manual_seed(9)
    probe = torch.randn(want_out.shape, generator=g)
    (want_out * probe).sum().backward()

    model = model.to(DEV)
    data = dict(feat=torch.from_numpy(feat).to(DEV), grid_coord=torch.from_numpy(d["grid_coord"]).to(DEV),
                offset=torch.from_numpy(d["offset"]).to(DEV))
    torch.manual_seed(5)
    out = model(data).feat
    assert rel_err(out, want_out) < 1e-4
    (out * probe.to(DEV)).sum().backward()
    worst = 0.0
    for name, p in model.named_parameters():
        assert p.grad is not None, name
        err = rel_err(p.grad, sd[name].grad)
        worst = max(worst, err)
        assert err < 2e-3, (name, err)   # sums over thousands of points in another order than the oracle's
    assert worst > 0.0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_training_step_under_autocast(dtype):
    """Training mode end to end: batch statistics, stochastic depth, autocast; gradients finite and a few
    optimizer steps lower the loss."""
    torch.manual_seed(1)
    model, _ = _small_model(drop_path=0.1, shuffle_orders=True)
    model = model.to(DEV).train()
    d, feat = _scene(n=2500)
    data = lambda: dict(feat=torch.from_numpy(feat).to(DEV), grid_coord=torch.from_numpy(d["grid_coord"]).to(DEV),
                        offset=torch.from_numpy(d["offset"]).to(DEV))
    target = torch.from_numpy(feat[:, :3]).to(DEV)
    head = torch.nn.Linear(64, 3).to(DEV)
    opt = torch.optim.AdamW(list(model.parameters()) + list(head.parameters()), lr=2e-3)
    before = model.embedding.stem.norm.running_mean.clone()
    losses = []
    for _ in range(8):
        opt.zero_grad()
        with torch.autocast("cuda", dtype=dtype):
            out = model(data()).feat
            loss = torch.nn.functional.mse_loss(head(out).float(), target)
        # autocast runs layer_norm in float, so the residual stream behind the first xCPE norm is float
        assert out.dtype == torch.float32
        loss.backward()
        assert all(torch.isfinite(p.grad).all() for p in model.parameters() if p.grad is not None)
        assert all(p.grad is not None for p in model.parameters())
        opt.step()
        losses.append(float(loss.detach()))
    assert not torch.equal(before, model.embedding.stem.norm.running_mean)
    assert losses[-1] < losses[0]


@pytest.mark.parametrize("variant", ["pdnorm", "post_norm", "cls_mode", "no_flash_fp32", "input_gradient", "rpe", "attn_drop"])
def test_training_step_of_model_variants(variant):
    """One forward + backward of the model built other ways: every parameter that takes part gets a finite
    gradient (PDNorm only trains the norms of the condition it is given)."""
    kw, autocast, extra = {}, torch.bfloat16, {}
    if variant == "pdnorm":
        kw = dict(pdnorm_bn=True, pdnorm_ln=True)
        extra = dict(condition="S3DIS")
    elif variant == "post_norm":
        kw = dict(pre_norm=False)
    elif variant == "cls_mode":
        kw = dict(cls_mode=True)
    elif variant == "no_flash_fp32":
        kw, autocast = dict(enable_flash=False), None
    elif variant == "attn_drop":
        kw = dict(attn_drop=0.1, proj_drop=0.1)
    elif variant == "rpe":
        kw, autocast = dict(enable_flash=False, enable_rpe=True, upcast_attention=True, upcast_softmax=True), None
    torch.manual_seed(3)
    model, _ = _small_model(drop_path=0.2, shuffle_orders=True, **kw)
    model = model.to(DEV).train()
    d, feat = _scene(n=1200)
    x = torch.from_numpy(feat).to(DEV).requires_grad_(variant == "input_gradient")
    data = dict(feat=x, grid_coord=torch.from_numpy(d["grid_coord"]).to(DEV), offset=torch.from_numpy(d["offset"]).to(DEV),
                **extra)
    if autocast is None:
        out = model(data).feat
    else:
        with torch.autocast("cuda", dtype=autocast):
            out = model(data).feat
    out.float().square().mean().backward()
    missing = [n for n, p in model.named_parameters() if p.grad is None]
    if variant == "pdnorm":
        assert missing and all(".norm." in n and ".norm.1." not in n for n in missing), missing[:5]
    else:
        assert not missing, missing[:5]
    assert all(torch.isfinite(p.grad).all() for p in model.parameters() if p.grad is not None)
    if variant == "input_gradient":
        assert x.grad is not None and torch.isfinite(x.grad).all() and x.grad.abs().max() > 0


def test_training_on_the_output_of_grid_sample():
    """Raw points -> device voxelisation -> a training step: the batch must be usable under autograd."""
    from pointtransformerv3_amd import synthetic, voxelize
    raw = [synthetic.room_points(6000, 70 + i).astype(np.float32) for i in range(2)]
    coord = torch.from_numpy(np.concatenate(raw)).to(DEV)
    offset = torch.from_numpy(np.cumsum([len(r) for r in raw])).to(DEV)
    feat = torch.rand(len(coord), 6, generator=torch.Generator().manual_seed(1)).to(DEV)
    batch = voxelize.grid_sample(coord, offset, 0.05, feat=feat)
    torch.manual_seed(2)
    model, _ = _small_model()
    model = model.to(DEV).train()
    with torch.autocast("cuda", dtype=torch.float16):
        out = model({k: batch[k] for k in ("feat", "grid_coord", "coord", "offset")}).feat
    out.float().square().mean().backward()
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in model.parameters())


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_parameter_casts_in_one_launch(dtype):
    """ptv3_cast_params behind ops.cast_cached: plain, transposed and mirrored copies of fp32 masters equal
    torch's own conversion bit for bit, follow in-place updates (all stale copies in one sweep, written in
    place) and a replaced storage, for shapes that are not multiples of the tile or the vector width."""
    o = ops()
    g = torch.Generator().manual_seed(11)
    shapes = [(96, 32), (13, 64), (64, 27, 64), (32, 5, 5, 5, 6), (70, 3, 130), (1, 7), (4099,)]
    params = [torch.nn.Parameter(torch.randn(*s, generator=g).to(DEV)) for s in shapes]

    def want(p, layout):
        src = p.detach()
        if layout == "transpose":
            src = src.t()
        elif layout == "mirror":
            src = src.reshape(p.shape[0], -1, p.shape[-1]).flip(1).permute(2, 1, 0)
        return src.to(dtype).contiguous()

    def layouts(p):
        return ["plain"] + (["transpose"] if p.dim() == 2 else []) + (["mirror"] if p.dim() >= 2 else [])

    held = {}
    for i, p in enumerate(params):
        for layout in layouts(p):
            got = o.cast_cached(p, dtype, layout)
            if dtype == torch.float32 and layout == "plain":
                assert got is p
                continue
            assert got.dtype == dtype and got.is_contiguous() and torch.equal(got, want(p, layout)), (i, layout)
            assert o.cast_cached(p, dtype, layout) is got
            held[(i, layout)] = got
    with torch.no_grad():
        for p in params:
            p.mul_(1.5).add_(0.25)
    first = next(iter(held))
    o.cast_cached(params[first[0]], dtype, first[1])            # one call refreshes every stale copy ...
    for (i, layout), got in held.items():
        assert torch.equal(got, want(params[i], layout)), (i, layout)   # ... in place
        assert o.cast_cached(params[i], dtype, layout) is got
    params[2].data = torch.randn(64, 27, 64, generator=g).to(DEV)
    assert torch.equal(o.cast_cached(params[2], dtype, "mirror"), want(params[2], "mirror"))
    odd = torch.nn.Parameter(torch.randn(1001, generator=g).to(DEV)[1:])   # storage offset: 4-byte alignment only
    if dtype != torch.float32:
        assert torch.equal(o.cast_cached(odd, dtype), odd.detach().to(dtype))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("n,c", [(1000, 32), (777, 64), (2048, 128), (300, 256), (129, 512), (1, 64)])
def test_mlp_function_parity(dtype, n, c):
    """The MLP under autograd with the GELU taken into fc1's kernel (forward) and into fc2's input gradient
    (backward), model.py:493-516: output, input gradient and the four parameter gradients vs torch autograd over
    the same fp32 masters in float64."""
    from pointtransformerv3_amd.modules import MLP
    torch.manual_seed(n + c)
    mlp = MLP(c, 4 * c, c).to(DEV)
    x = torch.randn(n, c, device=DEV, dtype=dtype, requires_grad=True)
    dy = torch.randn(n, c, device=DEV, dtype=dtype)
    with torch.autocast("cuda", dtype=dtype):
        y = mlp(x)
    assert y.dtype == dtype and "Mlp" in type(y.grad_fn).__name__
    y.backward(dy)

    ref = MLP(c, 4 * c, c).double()
    ref.load_state_dict({k: v.double().cpu() for k, v in mlp.state_dict().items()})
    xr = x.detach().double().cpu().requires_grad_(True)
    h = torch.nn.functional.linear(xr, ref.fc1.weight, ref.fc1.bias)
    yr = torch.nn.functional.linear(torch.nn.functional.gelu(h), ref.fc2.weight, ref.fc2.bias)
    yr.backward(dy.double().cpu())
    assert rel_err(y, yr) < TOL[dtype]
    assert rel_err(x.grad, xr.grad) < TOL[dtype]
    for name, p in mlp.named_parameters():
        assert rel_err(p.grad, dict(ref.named_parameters())[name].grad) < TOL[dtype], name


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_linear_gelu_kernels_against_their_parts(dtype):
    """ptv3_linear_gelu_fwd writes the same rows as the plain kernel followed by torch's GELU of them, and
    ptv3_linear_gelu_bwd the product of the plain kernel's rows with gelu'(pre), to one rounding."""
    o = ops()
    torch.manual_seed(5)
    for n, k, nout in [(5000, 64, 256), (333, 256, 1024), (64, 512, 2048), (31, 32, 128)]:
        x = torch.randn(n, k, device=DEV, dtype=dtype)
        w = (torch.randn(nout, k, device=DEV) / k ** 0.5).to(dtype)
        b = torch.randn(nout, device=DEV).to(dtype)
        pre, act = o.linear_gelu(x, w, b)
        plain = o.linear_rows(x, w, b)
        assert torch.equal(pre, plain)
        assert rel_err(act, torch.nn.functional.gelu(plain.float()).cpu()) < 4e-3
        d = o.linear_gelu_bwd(x, w, pre)
        z = pre.double().requires_grad_(True)
        torch.nn.functional.gelu(z).backward(o.linear_rows(x, w).double())
        assert rel_err(d, z.grad.cpu()) < 4e-3


@pytest.mark.parametrize("skip_dtype,branch_dtype", [(torch.float32, torch.bfloat16), (torch.float32, torch.float16),
                                                     (torch.float32, torch.float32), (torch.float16, torch.float16)])
@pytest.mark.parametrize("n,c", [(1000, 32), (77, 512), (1, 8), (4099, 64)])
def test_residual_add_function(skip_dtype, branch_dtype, n, c):
    """ptv3_scaled_add behind ResidualAdd: skip + branch * mask (model.py:602-604 with model.py:583's factor)
    and its two gradients vs torch in float64."""
    from pointtransformerv3_amd.autograd import ResidualAdd
    g = torch.Generator().manual_seed(n * c)
    skip = torch.randn(n, c, generator=g).to(skip_dtype).to(DEV).requires_grad_(True)
    branch = torch.randn(n, c, generator=g).to(branch_dtype).to(DEV).requires_grad_(True)
    mask = (torch.bernoulli(torch.full((n, 1), 0.7), generator=g) / 0.7).to(branch_dtype).to(DEV)
    dout = torch.randn(n, c, generator=g).to(skip_dtype).to(DEV)
    out = ResidualAdd.apply(skip, branch, mask)
    out.backward(dout)
    assert out.dtype == skip_dtype and skip.grad.dtype == skip_dtype and branch.grad.dtype == branch_dtype
    want = skip.detach().double() + branch.detach().double() * mask.double()
    tol = 1e-6 if skip_dtype == torch.float32 else 1e-3
    assert rel_err(out, want.cpu()) < tol
    assert torch.equal(skip.grad, dout)
    tol = 1e-6 if branch_dtype == torch.float32 else (1e-3 if branch_dtype == torch.float16 else 4e-3)
    assert rel_err(branch.grad, (dout.double() * mask.double()).cpu()) < tol


@pytest.mark.parametrize("fused", [False, True])
def test_parameter_casts_follow_the_optimizer(fused):
    """torch's fused optimizers write the parameters without touching their version counters: the remembered
    half-precision copies are declared stale by a hook on every optimizer step (ops.invalidate_casts)."""
    o = ops()
    p = torch.nn.Parameter(torch.randn(64, 32, device=DEV))
    opt = torch.optim.AdamW([p], lr=1e-1, fused=fused)
    held = o.cast_cached(p, torch.bfloat16)
    before = held.clone()
    p.grad = torch.ones_like(p)
    opt.step()
    got = o.cast_cached(p, torch.bfloat16)
    assert got is held and torch.equal(got, p.detach().to(torch.bfloat16)) and not torch.equal(got, before)
    assert torch.equal(o.cast_cached(p, torch.bfloat16, "transpose"), p.detach().t().to(torch.bfloat16).contiguous())
    with torch.no_grad():
        p.data.mul_(2.0)          # behind autograd's back: only an explicit call can tell
    o.invalidate_casts()
    assert torch.equal(o.cast_cached(p, torch.bfloat16), p.detach().to(torch.bfloat16))


def test_packed_convolution_weight_follows_a_fused_optimizer():
    """The tile convolution's repacked weight (inference between training epochs) is redone after an optimizer
    step that leaves the parameter's version counter alone."""
    from pointtransformerv3_amd.sparse import SubMConv3d
    o = ops()
    conv = SubMConv3d(64, 64, kernel_size=3, bias=True, indice_key="k").to(DEV)
    opt = torch.optim.AdamW(conv.parameters(), lr=1e-1, fused=True)
    held = conv._packed_weight(torch.float16)
    assert conv._packed_weight(torch.float16) is held
    first = held.clone()                      # the copy is redone in place, like the half-precision casts
    conv.weight.grad = torch.ones_like(conv.weight)
    opt.step()
    second = conv._packed_weight(torch.float16)
    want = o.conv_pack_weight(conv.weight.detach().reshape(64, -1, 64), 27, torch.float16)
    assert torch.equal(second, want) and not torch.equal(second, first)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("cin,cout,ks", [(64, 64, 3), (128, 128, 3), (8, 32, 5), (256, 128, 3)])
def test_conv_weight_gradient_from_pair_lists(dtype, cin, cout, ks):
    """ptv3_subm_conv_wgrad_pairs (ranges of each tap's own pair list) against ptv3_subm_conv_wgrad (compaction
    of the neighbour map) on the same inputs: the same sums in another order, and the same bias gradient."""
    o = ops()
    rng = np.random.default_rng(cin + cout + ks)
    grid, batch, _ = unique_voxels(rng, 6000, 24, nb=2)
    indices = torch.cat([to_dev(batch).int()[:, None], to_dev(grid)], 1).contiguous()   # (N, 4) batch, x, y, z
    nbr = o.kmap_build(indices, ks, tap_major=True)
    plan = o.conv_plan(nbr, tap_major=True)
    n = grid.shape[0]
    x = torch.randn(n, cin, device=DEV).to(dtype)
    dy = torch.randn(n, cout, device=DEV).to(dtype)
    dw_a, db_a = o.subm_conv_wgrad(x, dy, nbr, with_bias=True)
    dw_b, db_b = o.subm_conv_wgrad_pairs(x, dy, plan, with_bias=True)
    assert rel_err(dw_b, dw_a.cpu()) < 1e-5 and rel_err(db_b, db_a.cpu()) < 1e-5


@pytest.mark.parametrize("with_mask", [False, True])
@pytest.mark.parametrize("c", [32, 64, 128, 256, 512])
@pytest.mark.parametrize("skip_dtype,branch_dtype", [(torch.float32, torch.bfloat16), (torch.float32, torch.float32),
                                                     (torch.float16, torch.float16)])
def test_add_layer_norm_with_the_branch_norm_in_front(skip_dtype, branch_dtype, with_mask, c):
    """s = skip + LayerNorm_pre(branch) * mask, y = LayerNorm(s) as one node (the xCPE's norm, the first residual
    connection of a Block and norm1, model.py:546-554, :589-592): both results and all six gradients against
    torch CPU autograd in float32, with a gradient arriving at the sum as well."""
    from pointtransformerv3_amd.autograd import AddLayerNorm
    n = 1501 if c >= 256 else 3001
    g = torch.Generator().manual_seed(c)
    skip = torch.randn(n, c, generator=g).to(skip_dtype)
    branch = (torch.randn(n, c, generator=g) * 2 + 0.5).to(branch_dtype)
    mask = ((torch.rand(n, 1, generator=g) < 0.7).float() / 0.7).to(branch_dtype) if with_mask else None
    w, pw = torch.rand(c, generator=g) + 0.5, torch.rand(c, generator=g) + 0.5
    b, pb = torch.randn(c, generator=g), torch.randn(c, generator=g)
    ds, dy = torch.randn(n, c, generator=g), torch.randn(n, c, generator=g)
    ref = [t.float().clone().requires_grad_(True) for t in (skip, branch, w, b, pw, pb)]
    pre = torch.nn.functional.layer_norm(ref[1], (c,), ref[4], ref[5], 1e-6)
    s_want = ref[0] + pre * (mask.float() if with_mask else 1.0)
    y_want = torch.nn.functional.layer_norm(s_want, (c,), ref[2], ref[3], 1e-5)
    torch.autograd.backward([s_want, y_want], [ds, dy])
    got = [t.detach().to(DEV).requires_grad_(True) for t in (skip, branch, w, b, pw, pb)]
    s_got, y_got = AddLayerNorm.apply(got[0], got[1], None if mask is None else mask.to(DEV), got[2], got[3], 1e-5, None,
                                      got[4], got[5], 1e-6)
    torch.autograd.backward([s_got, y_got], [ds.to(DEV).to(s_got.dtype), dy.to(DEV).to(y_got.dtype)])
    tol = TOL[torch.promote_types(skip_dtype, branch_dtype)]
    assert rel_err(s_got, s_want) < tol and rel_err(y_got, y_want) < tol
    for i, name in enumerate(["skip", "branch", "weight", "bias", "pre_weight", "pre_bias"]):
        assert rel_err(got[i].grad, ref[i].grad) < (TOL[branch_dtype] if i == 1 else tol), name
