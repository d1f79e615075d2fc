"""HIP kmap / submanifold conv / pooling kernels vs the CPU oracle.
Integer outputs bit-exact; conv within 1e-4 (fp32) / 2e-2 (fp16, bf16) max-abs relative."""
import numpy as np
import pytest
import torch

from oracle import functional as OF
from oracle import indexing as OI
from oracle import serialization as OS
from gpu_util import DEV, rel_err, to_dev, unique_voxels

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-4, torch.float16: 2e-2, torch.bfloat16: 2e-2}


def ops():
    from pointtransformerv3_amd import ops as _ops
    return _ops


def _indices(rng, n, extent, nb):
    g, batch, offset = unique_voxels(rng, n, extent, nb)
    return np.concatenate([batch[:, None].astype(np.int32), g], 1), g, batch, offset


@pytest.mark.parametrize("ks", [3, 5])
@pytest.mark.parametrize("n,extent,nb", [(1, 4, 1), (500, 10, 2), (30_000, 48, 2)])
def test_kmap_bit_exact(ks, n, extent, nb):
    rng = np.random.default_rng(n + ks)
    idx, *_ = _indices(rng, n, extent, nb)
    got = ops().kmap_build(to_dev(idx), ks).cpu().numpy()
    assert np.array_equal(got, OI.subm_kmap(idx, ks))


def test_kmap_room_200k_properties():
    from pointtransformerv3_amd import synthetic
    g = synthetic.room_voxels(200_000, 3000)["grid_coord"]
    idx = np.concatenate([np.zeros((len(g), 1), np.int32), g], 1)
    got = ops().kmap_build(to_dev(idx), 3).cpu().numpy()
    assert np.array_equal(got[:, 13], np.arange(len(g)))
    i, k = np.nonzero(got >= 0)
    assert np.array_equal(got[got[i, k], 26 - k], i)
    assert np.array_equal(got, OI.subm_kmap(idx, 3))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("ks,cin,cout,n", [(3, 32, 32, 3000), (3, 64, 64, 5000), (3, 128, 128, 700),
                                           (5, 16, 32, 2000), (3, 64, 64, 70_000)])
def test_subm_conv_parity(dtype, ks, cin, cout, n):
    rng = np.random.default_rng(cin + n)
    g = torch.Generator().manual_seed(cin + n)
    idx, *_ = _indices(rng, n // 2, 40 if n > 10_000 else 14, 2)
    nbr = OI.subm_kmap(idx, ks)
    feat = torch.randn(len(idx), cin, generator=g).to(dtype)
    bound = 1.0 / np.sqrt(ks ** 3 * cin)
    w = ((torch.rand(cout, ks, ks, ks, cin, generator=g) * 2 - 1) * bound).to(dtype)
    b = ((torch.rand(cout, generator=g) * 2 - 1) * bound).to(dtype) if ks == 3 else None
    want = OF.subm_conv(feat.float(), nbr, w.float(), None if b is None else b.float())
    got = ops().subm_conv(feat.to(DEV), to_dev(nbr), w.to(DEV), None if b is None else b.to(DEV))
    assert got.dtype == dtype
    assert rel_err(got, want) < TOL[dtype]


def test_pool_clusters_and_gather_bit_exact():
    rng = np.random.default_rng(4)
    idx, g, batch, offset = _indices(rng, 20_000, 40, 3)
    depth, code, order, inverse = OS.serialize(g, batch)
    want = OI.pool_clusters(code, g, batch, 1)
    o = ops()
    cluster, idx_ptr, head, m = o.pool_clusters(to_dev(code[0]), to_dev(order[0]), 3)
    assert m == len(want["counts"])
    assert np.array_equal(cluster.cpu().numpy(), want["cluster"])
    assert np.array_equal(idx_ptr.cpu().numpy(), want["idx_ptr"])
    # the reference takes whichever member an unstable sort puts first (model.py:660-664);
    # only values shared by all members are read through it, so membership is the contract
    assert np.array_equal(want["cluster"][head.cpu().numpy()], np.arange(m))
    pc, pg, pb, p4 = o.pool_gather(to_dev(code), 3, to_dev(g), 1, to_dev(batch), head)
    assert np.array_equal(pc.cpu().numpy(), want["code"])
    assert np.array_equal(pg.cpu().numpy(), want["grid_coord"])
    assert np.array_equal(pb.cpu().numpy(), want["batch"])
    # the sparse tensor's indices are [batch, x, y, z] of the pooled points (model.py:165-167)
    assert np.array_equal(p4.cpu().numpy(), np.concatenate([want["batch"][:, None], want["grid_coord"]], 1))
    # pooled scene ends, read back with the cluster count, equal bincount(batch).cumsum (model.py:43-45, :66-67)
    res = o.pool_clusters(to_dev(code[0]), to_dev(order[0]), 3, to_dev(offset))
    assert res[3] == m and torch.equal(res[0], cluster)
    want_off = np.cumsum(np.bincount(want["batch"], minlength=len(offset)))
    assert np.array_equal(res[4].cpu().numpy(), want_off) and res[5] == want_off.tolist()
    # rows written in shuffled order (model.py:675-679) are the rows of the unshuffled tables
    rows = [2, 0, 3, 1]
    po, pi = o.pool_orders(to_dev(order), cluster, m)
    qc, _, _, _ = o.pool_gather(to_dev(code), 3, to_dev(g), 1, to_dev(batch), head, rows)
    qo, qi = o.pool_orders(to_dev(order), cluster, m, rows)
    assert torch.equal(qc, pc[rows]) and torch.equal(qo, po[rows]) and torch.equal(qi, pi[rows])


def test_offset2batch_matches_repeat_interleave():
    from pointtransformerv3_amd import point as P
    for sizes in ([5], [3, 0, 4], [1000, 1, 70_000, 12], [0, 0, 9]):
        offset = torch.tensor(sizes).cumsum(0)
        n = int(offset[-1])
        want = torch.arange(len(sizes)).repeat_interleave(torch.tensor(sizes))
        got = P.offset2batch(offset.to(DEV), n)
        assert got.dtype == torch.int64 and torch.equal(got.cpu(), want)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_segment_reduce_and_unpool(dtype):
    rng = np.random.default_rng(6)
    g0 = torch.Generator().manual_seed(6)
    idx, g, batch, offset = _indices(rng, 6000, 24, 2)
    depth, code, order, inverse = OS.serialize(g, batch)
    pc = OI.pool_clusters(code, g, batch, 1)
    feat = torch.randn(len(g), 48, generator=g0).to(dtype)
    o = ops()
    got = o.segment_reduce(feat.to(DEV), to_dev(pc["indices"]), to_dev(pc["idx_ptr"]), "max")
    want = OF.segment_csr(feat.float(), pc["indices"], pc["idx_ptr"], "max")
    assert torch.equal(got.float().cpu(), want)   # max picks an input value: exact
    coord = torch.rand(len(g), 3, generator=g0)
    gotm = o.segment_reduce(coord.to(DEV), to_dev(pc["indices"]), to_dev(pc["idx_ptr"]), "mean")
    assert rel_err(gotm, OF.segment_csr(coord, pc["indices"], pc["idx_ptr"], "mean")) < 1e-6
    child = torch.randn(len(pc["counts"]), 48, generator=g0).to(dtype)
    gotu = o.unpool_add(feat.to(DEV), child.to(DEV), to_dev(pc["cluster"]))
    wantu = OF.unpool_add(feat.float(), child.float(), pc["cluster"])
    assert rel_err(gotu, wantu) < (1e-6 if dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("c", [32, 64, 128, 256, 512, 48])
def test_layer_norm_modes(dtype, c):
    import torch.nn.functional as F
    g = torch.Generator().manual_seed(c)
    n = 3001
    x = (torch.randn(n, c, generator=g) * 2 + 0.5).to(dtype)
    r = torch.randn(n, c, generator=g).to(dtype)
    w, b = (torch.rand(c, generator=g) + 0.5).to(dtype), torch.randn(c, generator=g).to(dtype)
    w2, b2 = (torch.rand(c, generator=g) + 0.5).to(dtype), torch.randn(c, generator=g).to(dtype)
    tol = 1e-5 if dtype == torch.float32 else 1e-2

    def ln(v, ww, bb):
        return F.layer_norm(v.float(), (c,), ww.float(), bb.float(), 1e-5)

    o = ops()
    dv = lambda t: t.to(DEV)
    assert rel_err(o.layer_norm(dv(x), dv(w), dv(b)), ln(x, w, b)) < tol
    assert rel_err(o.layer_norm(dv(x), dv(w), dv(b), residual=dv(r), mode=1), r.float() + ln(x, w, b).to(dtype).float()) < tol
    s, z = o.layer_norm(dv(x), dv(w), dv(b), residual=dv(r), mode=2)
    want_s = (x.float() + r.float()).to(dtype)
    assert rel_err(s, want_s.float()) < tol and rel_err(z, ln(want_s, w, b)) < tol
    s2, z2 = o.layer_norm(dv(x), dv(w), dv(b), residual=dv(r), mode=2, shift=dv(b2))
    assert rel_err(s2, want_s.float() + b2.float()) < tol and torch.equal(z2, z)
    y, z = o.layer_norm(dv(x), dv(w), dv(b), residual=dv(r), mode=3, weight2=dv(w2), bias2=dv(b2))
    want_y = (r.float() + ln(x, w, b).to(dtype).float()).to(dtype)
    assert rel_err(y, want_y.float()) < tol and rel_err(z, ln(want_y, w2, b2)) < tol


@pytest.mark.parametrize("ks,n,extent", [(3, 1, 4), (3, 777, 12), (5, 3000, 20), (3, 40_000, 48)])
def test_conv_plan_bit_exact(ks, n, extent):
    rng = np.random.default_rng(n)
    idx, *_ = _indices(rng, n, extent, 2)
    nbr = OI.subm_kmap(idx, ks)
    plan = ops().conv_plan(to_dev(nbr))
    act = nbr >= 0
    assert plan.n_pairs == int(act.sum())
    # output-major slots: exclusive row-major rank of every active (voxel, tap)
    want_row_ptr = np.concatenate([[0], np.cumsum(act.sum(1))])
    assert np.array_equal(plan.row_ptr.cpu().numpy(), want_row_ptr)
    assert np.array_equal(plan.tap_ptr.cpu().numpy(), np.concatenate([[0], np.cumsum(act.sum(0))]))
    slot_of = np.cumsum(act.reshape(-1)).reshape(act.shape) - 1
    vi, ti = np.nonzero(act.T)[1], np.nonzero(act.T)[0]    # tap-major enumeration, voxels ascending
    assert np.array_equal(plan.pair_in.cpu().numpy()[:plan.n_pairs], nbr[vi, ti])
    assert np.array_equal(plan.pair_slot.cpu().numpy()[:plan.n_pairs], slot_of[vi, ti])


@pytest.mark.parametrize("ks,n,extent,nb", [(3, 1, 4, 1), (3, 777, 12, 2), (5, 3000, 20, 2), (3, 40_000, 48, 3),
                                            (5, 30_000, 40, 2), (3, 5000, 300, 1)])
def test_conv_plan_direct_equals_plan_of_map(ks, n, extent, nb):
    # the pair lists built straight from the coordinates are those of the stored map, bit for bit
    rng = np.random.default_rng(ks * 1000 + n)
    idx, *_ = _indices(rng, n, extent, nb)
    o = ops()
    dev_idx = to_dev(idx)
    ref = o.conv_plan(o.kmap_build(dev_idx, ks, tap_major=True), tap_major=True)
    got = o.conv_plan_direct(dev_idx, ks)
    assert got.n_pairs == ref.n_pairs and got.taps == ref.taps and got.n == ref.n
    assert torch.equal(got.tap_ptr, ref.tap_ptr) and torch.equal(got.row_ptr, ref.row_ptr)
    assert torch.equal(got.pair_in[:got.n_pairs], ref.pair_in[:ref.n_pairs])
    assert torch.equal(got.pair_slot[:got.n_pairs], ref.pair_slot[:ref.n_pairs])
    # and the oracle's map, tap-major, lists the same pairs
    nbr = OI.subm_kmap(idx, ks)
    t_idx, v_idx = np.nonzero(nbr.T >= 0)
    assert got.n_pairs == len(t_idx)
    assert np.array_equal(got.pair_in[:got.n_pairs].cpu().numpy(), nbr.T[t_idx, v_idx])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("ks,cin,cout,n,extent", [(3, 32, 32, 3000, 20), (3, 64, 64, 50_000, 60), (3, 128, 128, 9000, 24),
                                                  (3, 256, 256, 2000, 12), (3, 512, 512, 600, 8), (5, 16, 32, 20_000, 40),
                                                  (3, 192, 192, 1500, 12), (3, 256, 160, 1500, 12), (3, 128, 256, 4000, 16),
                                                  (3, 384, 72, 900, 10), (3, 128, 128, 2, 4), (3, 256, 256, 20_000, 30), (3, 512, 512, 7000, 16),
                                                  (3, 256, 512, 3000, 14), (3, 256, 256, 2, 2)])
def test_subm_conv_pairs_parity(dtype, ks, cin, cout, n, extent):
    rng = np.random.default_rng(cin + n)
    g = torch.Generator().manual_seed(cin + n)
    idx, *_ = _indices(rng, n // 2, extent, 2)
    nbr = OI.subm_kmap(idx, ks)
    feat = torch.randn(len(idx), cin, generator=g).to(dtype)
    bound = 1.0 / np.sqrt(ks ** 3 * cin)
    w = ((torch.rand(cout, ks, ks, ks, cin, generator=g) * 2 - 1) * bound).to(dtype)
    b = ((torch.rand(cout, generator=g) * 2 - 1) * bound).to(dtype) if ks == 3 else None
    want = OF.subm_conv(feat.float(), nbr, w.float(), None if b is None else b.float())
    o = ops()
    plan = o.conv_plan(to_dev(nbr))
    got = o.subm_conv_pairs(feat.to(DEV), plan, w.to(DEV), None if b is None else b.to(DEV))
    assert got.dtype == dtype
    assert rel_err(got, want) < TOL[dtype]


def test_tap_major_layout_is_the_transpose():
    rng = np.random.default_rng(12)
    g = torch.Generator().manual_seed(12)
    idx, *_ = _indices(rng, 5000, 24, 2)
    o = ops()
    for ks in (3, 5):
        a = o.kmap_build(to_dev(idx), ks)
        b = o.kmap_build(to_dev(idx), ks, tap_major=True)
        assert b.shape == (ks ** 3, len(idx)) and torch.equal(a.t().contiguous(), b)
        pa, pb = o.conv_plan(a), o.conv_plan(b, tap_major=True)
        assert pa.n_pairs == pb.n_pairs
        for f in ("tap_ptr", "row_ptr", "pair_in", "pair_slot"):
            assert torch.equal(getattr(pa, f), getattr(pb, f)), f
    nbr, nbr_t = o.kmap_build(to_dev(idx), 3), o.kmap_build(to_dev(idx), 3, tap_major=True)
    for dtype in (torch.float32, torch.float16):
        feat = torch.randn(len(idx), 64, generator=g).to(dtype).to(DEV)
        w = (torch.randn(64, 27, 64, generator=g) * 0.05).to(dtype).to(DEV)
        assert torch.equal(o.subm_conv(feat, nbr, w), o.subm_conv(feat, nbr_t, w, tap_major=True))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("c,n", [(32, 1), (32, 5000), (64, 33), (64, 70_001), (128, 1), (128, 300), (128, 40_001),
                                 (256, 63), (256, 64), (256, 20_001), (512, 65), (512, 9000),
                                 # more row groups than resident work-groups: rounds of 2 + 2, 3 + 2, 3 + 3 + 2 and
                                 # 2 + 1 groups per wave, the last round partly past the end
                                 (256, 32_768), (256, 32_773), (128, 114_691), (512, 24_577), (512, 16_385)])
def test_mlp_fused_parity(dtype, c, n):
    import torch.nn.functional as F
    g = torch.Generator().manual_seed(c + n)
    x = torch.randn(n, c, generator=g).to(dtype)
    r = torch.randn(n, c, generator=g).to(dtype)
    w1 = (torch.randn(4 * c, c, generator=g) / c ** 0.5).to(dtype)
    b1 = (torch.randn(4 * c, generator=g) * 0.5).to(dtype)
    w2 = (torch.randn(c, 4 * c, generator=g) / (4 * c) ** 0.5).to(dtype)
    b2 = (torch.randn(c, generator=g) * 0.5).to(dtype)
    h = F.gelu(F.linear(x.float(), w1.float(), b1.float()))
    want = r.float() + F.linear(h, w2.float(), b2.float())
    got = ops().mlp_fused(*(t.to(DEV) for t in (x, r, w1, b1, w2, b2)))
    assert got.dtype == dtype and rel_err(got, want) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("c,n", [(128, 1), (128, 40_001), (256, 64), (256, 20_001), (512, 9000), (256, 32_773), (512, 16_385)])
def test_mlp_fused_packed_weights_give_the_same_bits(dtype, c, n):
    """The packed weight stream only changes where the kernel finds its operands: against the torch fp32 layers
    within the half-precision bar, and bit for bit what the kernel gives on the layers' own layout."""
    import torch.nn.functional as F
    o = ops()
    g = torch.Generator().manual_seed(3 * c + n)
    x = torch.randn(n, c, generator=g).to(dtype)
    r = torch.randn(n, c, generator=g).to(dtype)
    w1 = (torch.randn(4 * c, c, generator=g) / c ** 0.5).to(dtype)
    b1 = (torch.randn(4 * c, generator=g) * 0.5).to(dtype)
    w2 = (torch.randn(c, 4 * c, generator=g) / (4 * c) ** 0.5).to(dtype)
    b2 = (torch.randn(c, generator=g) * 0.5).to(dtype)
    want = r.float() + F.linear(F.gelu(F.linear(x.float(), w1.float(), b1.float())), w2.float(), b2.float())
    dx, dr, dw1, db1, dw2, db2 = (t.to(DEV) for t in (x, r, w1, b1, w2, b2))
    packed = o.mlp_pack_weights(dw1, dw2, dtype)
    # the packed copy is a permutation of the two matrices' elements
    assert torch.equal(packed.view(torch.int16).sort().values,
                       torch.cat([dw1.flatten(), dw2.flatten()]).view(torch.int16).sort().values)
    got = o.mlp_fused_packed(dx, dr, packed, db1, db2)
    assert got.dtype == dtype and rel_err(got, want) < TOL[dtype]
    assert torch.equal(got, o.mlp_fused(dx, dr, dw1, db1, dw2, db2))


def test_mlp_fused_module_repacks_after_a_parameter_write():
    from pointtransformerv3_amd.modules import MLP
    o = ops()
    torch.manual_seed(5)
    mlp = MLP(128, 512).half().to(DEV)
    x = torch.randn(500, 128, device=DEV).half()
    r = torch.randn(500, 128, device=DEV).half()
    plain = lambda: o.mlp_fused(x, r, mlp.fc1.weight, mlp.fc1.bias, mlp.fc2.weight, mlp.fc2.bias)
    other = MLP(256, 1024).half().to(DEV)     # a second stale module rides on the same launch
    o._MLP_PACK_USERS.add(other)
    first = o.mlp_fused_module(x, r, mlp)
    assert torch.equal(first, plain())
    held = mlp._packed_stream[torch.float16][1]
    for m in (mlp, other):                    # the batch packs what the single call packs
        assert torch.equal(m._packed_stream[torch.float16][1],
                           o.mlp_pack_weights(m.fc1.weight, m.fc2.weight, torch.float16))
    with torch.no_grad():
        mlp.fc2.weight.mul_(0.5)              # bumps the version counter
    second = o.mlp_fused_module(x, r, mlp)
    assert torch.equal(second, plain()) and not torch.equal(second, first)
    assert mlp._packed_stream[torch.float16][1] is held     # redone in place
    mlp.fc1.weight.data.mul_(2.0)             # no version bump: callers announce it
    o.invalidate_casts()
    assert torch.equal(o.mlp_fused_module(x, r, mlp), plain())
    assert "_packed_stream" not in mlp.state_dict()


def _tail_modules(c, dtype, seed):
    """proj, norm2 and the MLP of a block at width c with weights that are no identity anywhere."""
    from pointtransformerv3_amd.modules import MLP, LayerNorm
    torch.manual_seed(seed)
    proj, ln, mlp = torch.nn.Linear(c, c), LayerNorm(c), MLP(c, 4 * c)
    with torch.no_grad():
        ln.weight.uniform_(0.5, 1.5)
        ln.bias.uniform_(-0.5, 0.5)
        for lin in (proj, mlp.fc1, mlp.fc2):
            lin.bias.uniform_(-0.5, 0.5)
    return [m.to(dtype).to(DEV) for m in (proj, ln, mlp)]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("c,n", [(128, 1), (128, 191), (128, 40_001), (128, 114_691), (256, 64), (256, 97), (256, 20_001),
                                 (256, 32_773)])
def test_block_tail_wide_parity(dtype, c, n):
    """The second half of a block in one kernel (projection, residual, LayerNorm, MLP, residual) against the same
    layers in torch fp32 on the same half-precision inputs and weights, and against the two kernels it replaces."""
    import torch.nn.functional as F
    o = ops()
    proj, ln, mlp = _tail_modules(c, dtype, c + n)
    g = torch.Generator().manual_seed(7 * c + n)
    attn = torch.randn(n, c, generator=g).to(dtype).to(DEV)
    short = (torch.randn(n, c, generator=g) * 2 + 0.75).to(dtype).to(DEV)    # rows with a mean well off zero
    f = lambda t: t.float()
    total = f(short) + F.linear(f(attn), f(proj.weight), f(proj.bias))
    normed = F.layer_norm(total, (c,), f(ln.weight), f(ln.bias), ln.eps)
    want = total + F.linear(F.gelu(F.linear(normed, f(mlp.fc1.weight), f(mlp.fc1.bias))), f(mlp.fc2.weight), f(mlp.fc2.bias))
    got = o.block_tail_wide(attn, short, proj, ln, mlp)
    assert got.dtype == dtype and got.shape == (n, c) and rel_err(got, want.cpu()) < TOL[dtype]
    feat, nrm = o.linear_ln(attn, proj, short, ln, 2)
    two = o.mlp_fused_module(nrm, feat, mlp)
    assert rel_err(got, two.cpu()) < TOL[dtype] / 4      # same layers, roundings at slightly different places


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("c,n", [(128, 1), (128, 191), (128, 40_001), (128, 114_691), (256, 64), (256, 97), (256, 20_001),
                                 (256, 32_773)])
def test_block_head_wide_parity(dtype, c, n):
    """The first half of a block behind its convolution in one kernel (Linear, LayerNorm, residual, LayerNorm, qkv)
    against the same layers in torch fp32 on the same half-precision inputs and weights, and against the two kernels
    it replaces."""
    import torch.nn.functional as F
    from pointtransformerv3_amd.modules import LayerNorm
    o = ops()
    torch.manual_seed(c + n)
    lin, lnc, ln1, qkv = torch.nn.Linear(c, c), LayerNorm(c), LayerNorm(c, eps=1e-4), torch.nn.Linear(c, 3 * c)
    with torch.no_grad():
        for ln in (lnc, ln1):
            ln.weight.uniform_(0.5, 1.5)
            ln.bias.uniform_(-0.5, 0.5)
        for m in (lin, qkv):
            m.bias.uniform_(-0.5, 0.5)
    lin, lnc, ln1, qkv = [m.to(dtype).to(DEV) for m in (lin, lnc, ln1, qkv)]
    g = torch.Generator().manual_seed(5 * c + n)
    conv = (torch.randn(n, c, generator=g) + 0.5).to(dtype).to(DEV)
    short = (torch.randn(n, c, generator=g) * 2 + 0.75).to(dtype).to(DEV)
    f = lambda t: t.float()
    want_feat = f(short) + F.layer_norm(F.linear(f(conv), f(lin.weight), f(lin.bias)), (c,), f(lnc.weight), f(lnc.bias), lnc.eps)
    want_qkv = F.linear(F.layer_norm(want_feat, (c,), f(ln1.weight), f(ln1.bias), ln1.eps), f(qkv.weight), f(qkv.bias))
    feat, got = o.block_head_wide(conv, short, lin, lnc, ln1, qkv)
    assert feat.dtype == dtype and feat.shape == (n, c) and got.dtype == dtype and got.shape == (n, 3 * c)
    assert rel_err(feat, want_feat.cpu()) < TOL[dtype] and rel_err(got, want_qkv.cpu()) < TOL[dtype]
    ln1.eps = lnc.eps                      # the two-kernel route takes one epsilon for both norms
    feat1, got1 = o.block_head_wide(conv, short, lin, lnc, ln1, qkv)
    feat2, normed = o.linear_ln(conv, lin, short, lnc, 3, ln2=ln1)
    assert rel_err(feat1, feat2.cpu()) < TOL[dtype] / 4 and rel_err(got1, o.linear(normed, qkv).cpu()) < TOL[dtype] / 4


def test_block_head_wide_repacks_after_a_parameter_write():
    from pointtransformerv3_amd.modules import LayerNorm
    o = ops()
    torch.manual_seed(13)
    lin, lnc, ln1, qkv = [m.half().to(DEV) for m in (torch.nn.Linear(256, 256), LayerNorm(256), LayerNorm(256),
                                                      torch.nn.Linear(256, 768))]
    conv = torch.randn(300, 256, device=DEV).half()
    short = torch.randn(300, 256, device=DEV).half()
    f0, q0 = o.block_head_wide(conv, short, lin, lnc, ln1, qkv)
    pack = qkv._head_weights
    held = pack._packed_stream[torch.float16][1]
    assert held.numel() == 4 * 256 * 256
    both = torch.cat([lin.weight.detach().flatten(), qkv.weight.detach().flatten()])
    assert torch.equal(held.view(torch.int16).sort().values, both.view(torch.int16).sort().values)
    kept = qkv.weight.detach().clone()
    with torch.no_grad():
        qkv.weight.mul_(0.5)
    f1, q1 = o.block_head_wide(conv, short, lin, lnc, ln1, qkv)
    assert torch.equal(f0, f1) and not torch.equal(q0, q1) and pack._packed_stream[torch.float16][1] is held
    with torch.no_grad():
        qkv.weight.copy_(kept)
        lin.weight.mul_(0.5)
    f2, q2 = o.block_head_wide(conv, short, lin, lnc, ln1, qkv)
    assert not torch.equal(f0, f2) and qkv._head_weights is pack
    assert "_head_weights" not in qkv.state_dict() and "_packed_stream" not in qkv.state_dict()


def test_block_tail_wide_repacks_after_a_parameter_write():
    o = ops()
    proj, ln, mlp = _tail_modules(128, torch.float16, 11)
    attn = torch.randn(700, 128, device=DEV).half()
    short = torch.randn(700, 128, device=DEV).half()
    first = o.block_tail_wide(attn, short, proj, ln, mlp)
    held = proj._packed_stream[torch.float16][1]
    assert held.numel() == 128 * 128
    assert torch.equal(held.view(torch.int16).sort().values, proj.weight.detach().flatten().view(torch.int16).sort().values)
    kept = proj.weight.detach().clone()
    with torch.no_grad():
        proj.weight.mul_(0.5)
    second = o.block_tail_wide(attn, short, proj, ln, mlp)
    assert not torch.equal(first, second) and proj._packed_stream[torch.float16][1] is held
    with torch.no_grad():
        proj.weight.copy_(kept)
    assert torch.equal(o.block_tail_wide(attn, short, proj, ln, mlp), first)
    assert "_packed_stream" not in proj.state_dict()


def test_gelu_of_the_fused_kernels_over_every_fp16_input():
    """The GELU the Linear / MLP / block kernels evaluate (one v_exp_f32 and a degree-7 polynomial in its exponent)
    against the correctly rounded erf GELU of nn.GELU, for every finite fp16 input: an identity Linear with the GELU
    epilogue passes each value through the device code. At most one ulp off, and for well under 0.1 % of the inputs."""
    o = ops()
    bits = torch.arange(0, 0x7c00, dtype=torch.int32)
    bits = torch.cat([bits, bits[1:] + 0x8000]).to(torch.int16)       # every finite fp16 value once (one zero)
    x = bits.view(torch.float16)
    pad = (-len(x)) % 32
    x = torch.cat([x, torch.zeros(pad, dtype=torch.float16)]).reshape(-1, 32)
    got = o.linear_rows(x.to(DEV), torch.eye(32, dtype=torch.float16, device=DEV), None, gelu=True).cpu()
    xd = x.double()
    want = (0.5 * xd * (1.0 + torch.special.erf(xd / 2.0 ** 0.5))).to(torch.float16)
    both_zero = (got == 0) & (want == 0)                              # -0 against +0 in the far negative tail
    differ = (got != want) & ~both_zero
    ulps = (got.view(torch.int16).int() - want.view(torch.int16).int()).abs()[differ]
    assert torch.isfinite(got.float()).all()
    assert differ.sum().item() <= 64 and (ulps.numel() == 0 or ulps.max().item() == 1), (differ.sum().item(), ulps.max())


def test_gelu_of_the_fused_kernels_at_infinities_and_nan():
    """Non-finite inputs (a first-layer sum beyond the half-precision range): NaN stays NaN and +-inf give NaN too
    (the polynomial meets inf * 0; torch's CPU kernels return NaN or the limits inf / -0 depending on the machine's
    vector path) -- a blow-up is never turned into a finite number. Finite neighbours against torch. Each row
    carries its value in column 0 and the weight copies that column to every output, so no product mixes inf with 0."""
    o = ops()
    vals = torch.tensor([float("inf"), float("-inf"), float("nan"), 3.0, -2.0, 65504.0, -65504.0, 0.0])
    x = torch.zeros(32, 32, dtype=torch.float16)
    x[:8, 0] = vals.half()
    w = torch.zeros(32, 32, dtype=torch.float16)
    w[:, 0] = 1.0
    got = o.linear_rows(x.to(DEV), w.to(DEV), None, gelu=True).cpu()[:8].float()
    assert bool(torch.isnan(got[:3]).all()) and bool(torch.isfinite(got[3:]).all())
    want = torch.nn.functional.gelu(vals[3:].double()).float()[:, None].expand(5, 32)
    assert rel_err(got[3:], want) < 1e-3


def _lin(cin, cout, g, dtype, bias=True):
    m = torch.nn.Linear(cin, cout, bias=bias)
    with torch.no_grad():
        m.weight.copy_(torch.randn(cout, cin, generator=g) / cin ** 0.5)
        if bias:
            m.bias.copy_(torch.randn(cout, generator=g) * 0.5)
    return m.to(dtype)


def _ln(c, g, dtype):
    m = torch.nn.LayerNorm(c)
    with torch.no_grad():
        m.weight.copy_(torch.rand(c, generator=g) + 0.5)
        m.bias.copy_(torch.randn(c, generator=g) * 0.3)
    return m.to(dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("c", [32, 64])
@pytest.mark.parametrize("n", [1, 33, 5000, 70_001])
def test_block_head_fused_parity(dtype, c, n):
    """shortcut + LN(Linear(conv)) and Linear(LN(that)) against the separate fp32 layers."""
    g = torch.Generator().manual_seed(11 * c + n)
    conv = torch.randn(n, c, generator=g).to(dtype)
    short = torch.randn(n, c, generator=g).to(dtype)
    cpe1, lnc, ln1 = _lin(c, c, g, dtype), _ln(c, g, dtype), _ln(c, g, dtype)
    qkv = _lin(c, 3 * c, g, dtype, bias=(n % 2 == 1))
    with torch.no_grad():
        f32 = lambda m: m.float()
        want_feat = short.float() + f32(_clone(lnc))(f32(_clone(cpe1))(conv.float()))
        want_qkv = f32(_clone(qkv))(f32(_clone(ln1))(want_feat))
        mods = [m.to(DEV) for m in (cpe1, lnc, ln1, qkv)]
        feat, out = ops().block_head_fused(conv.to(DEV), short.to(DEV), *mods)
    assert feat.dtype == dtype and out.shape == (n, 3 * c)
    assert rel_err(feat, want_feat) < TOL[dtype]
    assert rel_err(out, want_qkv) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("c", [32, 64])
@pytest.mark.parametrize("n", [1, 33, 5000, 70_001])
def test_block_tail_fused_parity(dtype, c, n):
    """feat = shortcut + proj(attn); feat + fc2(GELU(fc1(LN(feat)))) against the separate fp32 layers."""
    import torch.nn.functional as F
    g = torch.Generator().manual_seed(13 * c + n)
    attn = torch.randn(n, c, generator=g).to(dtype)
    short = torch.randn(n, c, generator=g).to(dtype)
    proj, ln2 = _lin(c, c, g, dtype), _ln(c, g, dtype)
    fc1, fc2 = _lin(c, 4 * c, g, dtype), _lin(4 * c, c, g, dtype)
    with torch.no_grad():
        f32 = lambda m: _clone(m).float()
        feat = short.float() + f32(proj)(attn.float())
        want = feat + f32(fc2)(F.gelu(f32(fc1)(f32(ln2)(feat))))
        mods = [m.to(DEV) for m in (proj, ln2, fc1, fc2)]
        got = ops().block_tail_fused(attn.to(DEV), short.to(DEV), *mods)
    assert got.dtype == dtype and rel_err(got, want) < TOL[dtype]


def _clone(module):
    import copy
    return copy.deepcopy(module)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("half_stats", [False, True])
def test_bn_act_parity(dtype, half_stats):
    import torch.nn.functional as F
    g = torch.Generator().manual_seed(3)
    n, c = 4097, 64
    x = (torch.randn(n, c, generator=g) * 2).to(dtype)
    mean, var = torch.randn(c, generator=g), torch.rand(c, generator=g) + 0.5
    w, b = (torch.rand(c, generator=g) + 0.5).to(dtype), torch.randn(c, generator=g).to(dtype)
    sd = dtype if half_stats else torch.float32
    mean, var = mean.to(sd), var.to(sd)
    y = F.batch_norm(x.float(), mean.float(), var.float(), w.float(), b.float(), False, 0.0, 1e-3)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    o = ops()
    dv = lambda t: t.to(DEV)
    assert rel_err(o.bn_act(dv(x), dv(mean), dv(var), dv(w), dv(b), 1e-3, False), y) < tol
    assert rel_err(o.bn_act(dv(x), dv(mean), dv(var), dv(w), dv(b), 1e-3, True), F.gelu(y.to(dtype).float())) < tol


@pytest.mark.parametrize("n,extent,nb", [(1, 4, 1), (3000, 16, 2), (60_000, 64, 3)])
def test_pool_orders_equal_argsort_of_pooled_codes(n, extent, nb):
    rng = np.random.default_rng(n)
    idx, g, batch, offset = _indices(rng, n, extent, nb)
    depth, code, order, inverse = OS.serialize(g, batch)
    want = OI.pool_clusters(code, g, batch, 1)
    o = ops()
    # also with the rows in another order than (z, z-trans, hilbert, hilbert-trans)
    for perm in ([0, 1, 2, 3], [2, 0, 3, 1]):
        c, od = code[perm], order[perm]
        w = OI.pool_clusters(c, g, batch, 1)
        cluster, idx_ptr, head, m = o.pool_clusters(to_dev(c[0]), to_dev(od[0]), 3)
        po, pi = o.pool_orders(to_dev(od), cluster, m)
        assert np.array_equal(po.cpu().numpy(), w["order"]) and np.array_equal(pi.cpu().numpy(), w["inverse"])
        pc, _, _, _ = o.pool_gather(to_dev(c), 3, to_dev(g), 1, to_dev(batch), head)
        so, si = o.argsort_rows(pc, 3 * (depth - 1) + 2)
        assert torch.equal(so, po) and torch.equal(si, pi)
    assert m == len(want["counts"])


def test_subm_conv_config3_full_size_fp16():
    """Baseline config 3 at full size: 200,000 room voxels, 64 -> 64 channels, fp16, Kaiming-uniform
    weights. The pair form from the direct plan is checked (a) against the dense output-stationary form,
    (b) row by row against a float64 evaluation of the definition on 3,000 sampled voxels using the
    neighbour map, whose symmetry and centre column are checked in passing, (c) for linearity; (d) the form the
    module's dispatch picks here (sparse tiles) against the same float64 rows."""
    from pointtransformerv3_amd import synthetic
    vox = synthetic.room_voxels(200_000, 3000)["grid_coord"]
    idx = np.concatenate([np.zeros((len(vox), 1), np.int32), vox], 1)
    g = torch.Generator().manual_seed(3)
    n, c = len(idx), 64
    feat = torch.randn(n, c, generator=g).half()
    bound = 1.0 / np.sqrt(27 * c)
    w = ((torch.rand(c, 3, 3, 3, c, generator=g) * 2 - 1) * bound).half()
    b = ((torch.rand(c, generator=g) * 2 - 1) * bound).half()
    o = ops()
    dev_idx = to_dev(idx)
    plan = o.conv_plan_direct(dev_idx, 3)
    got = o.subm_conv_pairs(feat.to(DEV), plan, w.to(DEV), b.to(DEV))
    nbr = o.kmap_build(dev_idx, 3)
    dense = o.subm_conv(feat.to(DEV), nbr, w.to(DEV), b.to(DEV))
    assert rel_err(got, dense.float().cpu()) < 2e-2                       # (a)
    nb = nbr.cpu().numpy()
    assert plan.n_pairs == int((nb >= 0).sum())
    assert np.array_equal(nb[:, 13], np.arange(n))
    rows, taps = np.nonzero(nb >= 0)
    assert np.array_equal(nb[nb[rows, taps], 26 - taps], rows)            # pair symmetry
    rng = np.random.default_rng(0)
    sample = rng.choice(n, 3000, replace=False)
    wf = w.double().reshape(c, 27, c).numpy()
    ff = feat.double().numpy()
    want = np.tile(b.double().numpy(), (len(sample), 1))
    for t in range(27):
        src = nb[sample, t]
        ok = src >= 0
        want[ok] += ff[src[ok]] @ wf[:, t, :].T
    err = np.abs(got.float().cpu().numpy()[sample] - want).max() / np.abs(want).max()
    assert err < 2e-2, err                                                # (b)
    # (d) the form the module's dispatch picks at this width and sparsity (the one the benchmark times): the module
    # call itself, with a spy on the wrapper that confirms which kernel ran, against the same float64 rows
    from pointtransformerv3_amd import ops as ops_mod, sparse
    conv = sparse.SubMConv3d(c, c, kernel_size=3, bias=True, indice_key="cfg3").to(DEV).half()
    with torch.no_grad():
        conv.weight.copy_(w.reshape(conv.weight.shape))
        conv.bias.copy_(b)
    x = sparse.SparseConvTensor(feat.to(DEV), dev_idx, [int(v) + 1 for v in vox.max(0)], 1)
    calls = []
    real = ops_mod.subm_conv_sparse
    ops_mod.subm_conv_sparse = lambda *a, **k: (calls.append(1), real(*a, **k))[1]
    try:
        with torch.inference_mode():
            picked = conv(x).features
    finally:
        ops_mod.subm_conv_sparse = real
    assert calls == [1]                                                   # the sparse tile form
    err = np.abs(picked.float().cpu().numpy()[sample] - want).max() / np.abs(want).max()
    assert err < 2e-2, err
    assert rel_err(picked, dense.float().cpu()) < 2e-2
    twice = o.subm_conv_pairs((feat * 2).to(DEV), plan, w.to(DEV), None)
    once = o.subm_conv_pairs(feat.to(DEV), plan, w.to(DEV), None)
    assert rel_err(twice, 2 * once.float().cpu()) < 2e-3                  # (c)


@pytest.mark.parametrize("ks", [3, 5])
def test_voxel_hash_edge_coordinates(ks):
    """Voxels at the corners of the coordinate range (0 and 65535), many scene ids, neighbours across
    4x4x4 block borders in every direction, a lone voxel: map and direct pair lists against the oracle."""
    rng = np.random.default_rng(ks)
    parts = []
    for b, base in ((0, 0), (1, 65535 - 7), (37, 4), (1023, 32760)):
        g = rng.integers(0, 8, size=(150, 3)) + base
        parts.append(np.concatenate([np.full((150, 1), b), g], 1))
    parts.append(np.array([[5, 0, 0, 0], [5, 65535, 65535, 65535], [5, 3, 4, 3], [5, 4, 4, 4], [6, 100, 200, 300]]))
    idx = np.unique(np.concatenate(parts).astype(np.int32), axis=0)
    idx = idx[rng.permutation(len(idx))]
    want = OI.subm_kmap(idx, ks)
    o = ops()
    assert np.array_equal(o.kmap_build(to_dev(idx), ks).cpu().numpy(), want)
    plan = o.conv_plan_direct(to_dev(idx), ks)
    t_idx, v_idx = np.nonzero(want.T >= 0)
    assert plan.n_pairs == len(t_idx)
    assert np.array_equal(plan.pair_in[:plan.n_pairs].cpu().numpy(), want.T[t_idx, v_idx])
    assert np.array_equal(plan.row_ptr.cpu().numpy(), np.concatenate([[0], np.cumsum((want >= 0).sum(1))]))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("k,nout,n,gelu,bias", [(32, 64, 50_001, False, True), (64, 64, 31, False, True), (64, 128, 4000, True, False),
                                                (128, 128, 1, False, True), (128, 384, 40_001, False, True), (128, 512, 777, True, True),
                                                (256, 768, 9000, False, True), (256, 1024, 5000, True, True), (256, 96, 33, False, False),
                                                (512, 512, 2500, False, True), (512, 2048, 1000, True, True), (512, 1536, 64, False, True),
                                                (256, 256, 37_681, False, True), (256, 1024, 37_681, True, True), (256, 256, 4097, False, False),
                                                (256, 768, 16_384, False, True)])
def test_linear_rows_parity(dtype, k, nout, n, gelu, bias):
    import torch.nn.functional as F
    g = torch.Generator().manual_seed(k + nout + n)
    x = torch.randn(n, k, generator=g).to(dtype)
    w = (torch.randn(nout, k, generator=g) / k ** 0.5).to(dtype)
    b = (torch.randn(nout, generator=g) * 0.5).to(dtype) if bias else None
    want = F.linear(x.float(), w.float(), None if b is None else b.float())
    if gelu:
        want = F.gelu(want)
    got = ops().linear_rows(x.to(DEV), w.to(DEV), None if b is None else b.to(DEV), gelu)
    assert got.dtype == dtype and got.shape == (n, nout)
    assert rel_err(got, want) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("k,nout,n,resid,bias", [(1024, 256, 37_681, True, False), (2048, 512, 8617, True, False),
                                                 (512, 1536, 8617, False, True), (128, 128, 1, False, True),
                                                 (384, 128, 129, True, True), (1024, 256, 127, True, True)])
def test_linear_gemm_parity(dtype, k, nout, n, resid, bias):
    """The tiled GEMM of the long contractions: resid + x W^T + b, added in fp32, rounded once, written over resid."""
    import torch.nn.functional as F
    g = torch.Generator().manual_seed(k + nout + n)
    x = torch.randn(n, k, generator=g).to(dtype)
    w = (torch.randn(nout, k, generator=g) / k ** 0.5).to(dtype)
    b = (torch.randn(nout, generator=g) * 0.5).to(dtype) if bias else None
    r = torch.randn(n, nout, generator=g).to(dtype) if resid else None
    want = F.linear(x.float(), w.float(), None if b is None else b.float())
    if resid:
        want = want + r.float()
    r_dev = None if r is None else r.to(DEV)
    got = ops().linear_gemm(x.to(DEV), w.to(DEV), None if b is None else b.to(DEV), r_dev)
    assert got.dtype == dtype and got.shape == (n, nout)
    if resid:
        assert got.data_ptr() == r_dev.data_ptr()
    assert rel_err(got, want) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("k,nout,n,gelu,stats_f32,affine", [(512, 256, 3001, True, True, True), (256, 256, 777, True, False, True),
                                                            (64, 64, 40_001, True, True, True), (128, 64, 5, False, True, False),
                                                            (32, 128, 1000, True, True, True), (256, 128, 2048, False, False, True)])
def test_linear_bn_act_parity(dtype, k, nout, n, gelu, stats_f32, affine):
    """Linear -> BatchNorm1d (inference) -> GELU in one kernel (model.py:726-735) against torch in fp32."""
    import torch.nn.functional as F
    torch.manual_seed(k * 7 + nout + n)
    lin = torch.nn.Linear(k, nout)
    bn = torch.nn.BatchNorm1d(nout, affine=affine).eval()
    bn.running_mean.normal_(0, 0.3)
    bn.running_var.uniform_(0.5, 2.0)
    if affine:
        bn.weight.data.uniform_(0.5, 1.5)
        bn.bias.data.normal_(0, 0.3)
    x = torch.randn(n, k).to(dtype)
    lin_h = lin.to(dtype)
    with torch.no_grad():
        want = bn(F.linear(x.float(), lin_h.weight.float(), lin_h.bias.float()))
        if gelu:
            want = F.gelu(want)
    lin_d, bn_d = lin_h.to(DEV), bn.to(DEV)
    if not stats_f32:
        bn_d = bn_d.to(dtype)
    got = ops().linear_bn_act(x.to(DEV), lin_d, bn_d, gelu)
    assert got.dtype == dtype and got.shape == (n, nout)
    assert rel_err(got, want) < TOL[dtype]
    # the same as the two-kernel path it replaces, up to one rounding of the intermediate
    two = ops().bn_act(ops().linear_rows(x.to(DEV), lin_d.weight, lin_d.bias), bn_d.running_mean, bn_d.running_var,
                       bn_d.weight, bn_d.bias, bn_d.eps, gelu)
    assert rel_err(got, two.float().cpu()) < (2e-3 if dtype == torch.float16 else 1.6e-2)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("c,n,extent", [(64, 3000, 20), (64, 50_000, 60), (128, 9000, 24), (128, 2000, 12), (64, 2, 4),
                                        (128, 900, 8), (64, 40_001, 90), (128, 6000, 40), (64, 400, 6)])
def test_subm_conv_tiles_parity(dtype, c, n, extent):
    """Tile form of the xCPE convolution (sums kept on chip) against the oracle, from sparse scans to
    nearly full grids (every tap of most voxels present), and the same bits on every run."""
    rng = np.random.default_rng(c + n)
    g = torch.Generator().manual_seed(c + n)
    idx, *_ = _indices(rng, n // 2, extent, 2)
    nbr = OI.subm_kmap(idx, 3)
    feat = torch.randn(len(idx), c, generator=g).to(dtype)
    bound = 1.0 / np.sqrt(27 * c)
    w = ((torch.rand(c, 3, 3, 3, c, generator=g) * 2 - 1) * bound * 3).to(dtype)
    b = ((torch.rand(c, generator=g) * 2 - 1) * 0.2).to(dtype)
    want = OF.subm_conv(feat.float(), nbr, w.float(), b.float())
    o = ops()
    plan = o.conv_plan_direct(to_dev(idx), 3)
    # the output-major words list every voxel's neighbours in tap order
    sp = plan.slot_pair().cpu().numpy()[:plan.n_pairs]
    v_idx, t_idx = np.nonzero(nbr >= 0)
    assert np.array_equal(sp >> 24, t_idx) and np.array_equal(sp & 0xFFFFFF, nbr[v_idx, t_idx])
    packed = o.conv_pack_weight(w.to(DEV), 27, dtype)
    got = o.subm_conv_tiles(feat.to(DEV), plan, packed, b.to(DEV))
    assert got.dtype == dtype and got.shape == (len(idx), c)
    assert rel_err(got, want) < TOL[dtype]
    again = o.subm_conv_tiles(feat.to(DEV), plan, packed, b.to(DEV))
    assert torch.equal(got, again)
    nob = o.subm_conv_tiles(feat.to(DEV), plan, packed, None)
    assert rel_err(nob, OF.subm_conv(feat.float(), nbr, w.float(), None)) < TOL[dtype]
    if c == 128:
        # tiles of 96 outputs instead of 128: a voxel's sum is taken in tap order either way, so the same bits
        for tv in (96, 128):
            assert torch.equal(o.subm_conv_tiles(feat.to(DEV), plan, packed, b.to(DEV), tile_voxels=tv), got)
        t96, t128 = plan.tiles(96), plan.tiles(128)
        assert t96[0].shape[0] == -(-len(idx) // 96) and t128[0].shape[0] == -(-len(idx) // 128)
        assert int(t96[0][:, 27].sum()) == plan.n_pairs == int(t128[0][:, 27].sum())   # every pair in one tile
        assert torch.equal(t96[2], t128[2])                                              # per-voxel tap sets
    else:
        with pytest.raises(Exception):
            o.subm_conv_tiles(feat.to(DEV), plan, packed, b.to(DEV), tile_voxels=96)     # 96 is for 128 channels


def test_tile_size_choice_follows_the_rounds():
    o = ops()
    assert o.tile_voxels_for(146_195, 128) == 96      # 2.2 rounds of 128-voxel tiles, 2.97 of 96-voxel ones
    assert o.tile_voxels_for(60_000, 128) == 128      # one round either way
    assert o.tile_voxels_for(10_000_000, 128) == 128  # many rounds: the larger tile amortises its weights better
    assert o.tile_voxels_for(146_195, 64) == 128


def test_repack_conv_weights_batch_equals_single_packs():
    """One launch repacks every stale convolution weight; each result equals the single-weight packing, float
    masters included (their half copy is made first), and only stale copies are touched."""
    from pointtransformerv3_amd.sparse import SubMConv3d
    o = ops()
    torch.manual_seed(4)
    mods = [SubMConv3d(c, c, 3).to(DEV) for c in (32, 64, 128, 64)] + [SubMConv3d(6, 32, 5).to(DEV)]
    mods[1].half()
    for dtype in (torch.float16, torch.bfloat16):
        o.repack_conv_weights(mods, dtype, torch.device(DEV))
        assert not hasattr(mods[4], "_packed") or dtype not in mods[4]._packed     # 5x5x5, cin != cout: not packable
        for m in mods[:4]:
            c = m.in_channels
            if m.weight.dtype == torch.float16 and dtype == torch.bfloat16:
                want = o.conv_pack_weight(m.weight.detach().to(dtype).reshape(c, 27, c), 27, dtype)
            else:
                want = o.conv_pack_weight(m.weight.detach().reshape(c, 27, c), 27, dtype)
            assert torch.equal(m._packed[dtype][1], want), (c, dtype)
    # nothing stale: no launch, same tensors; one weight written through .data after invalidate: only that one changes
    before = [m._packed[torch.float16][1].clone() for m in mods[:4]]
    o.repack_conv_weights(mods, torch.float16, torch.device(DEV))
    assert all(torch.equal(a, m._packed[torch.float16][1]) for a, m in zip(before, mods[:4]))
    mods[2].weight.data.mul_(3.0)
    o.invalidate_casts()
    o.repack_conv_weights(mods, torch.float16, torch.device(DEV))
    assert not torch.equal(before[2], mods[2]._packed[torch.float16][1])
    assert torch.equal(before[0], mods[0]._packed[torch.float16][1])
    assert torch.equal(mods[2]._packed[torch.float16][1],
                       o.conv_pack_weight(mods[2].weight.detach().reshape(128, 27, 128), 27, torch.float16))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("c,n,extent", [(64, 3000, 20), (64, 50_000, 60), (32, 9000, 24), (32, 2000, 12), (64, 2, 4),
                                        (32, 900, 8), (64, 40_001, 90), (32, 60_000, 120), (64, 400, 6), (32, 2, 3),
                                        (64, 2400, 11), (32, 1900, 10)])
def test_subm_conv_sparse_parity(dtype, c, n, extent):
    """Sparse tile form of the xCPE convolution (an MFMA row is a pair, sums in LDS) against the oracle, from
    scans with a neighbour or two per voxel to full grids (all 27 taps, several blocks per tap), the same bits
    on every run, and the same result as the other two forms up to the rounding of their sums."""
    rng = np.random.default_rng(c + n)
    g = torch.Generator().manual_seed(c + n)
    idx, *_ = _indices(rng, n // 2, extent, 2)
    nbr = OI.subm_kmap(idx, 3)
    feat = torch.randn(len(idx), c, generator=g).to(dtype)
    bound = 1.0 / np.sqrt(27 * c)
    w = ((torch.rand(c, 3, 3, 3, c, generator=g) * 2 - 1) * bound * 3).to(dtype)
    b = ((torch.rand(c, generator=g) * 2 - 1) * 0.2).to(dtype)
    want = OF.subm_conv(feat.float(), nbr, w.float(), b.float())
    o = ops()
    plan = o.conv_plan_direct(to_dev(idx), 3)
    packed = o.conv_pack_weight(w.to(DEV), 27, dtype)
    got = o.subm_conv_sparse(feat.to(DEV), plan, packed, b.to(DEV))
    assert got.dtype == dtype and got.shape == (len(idx), c)
    assert rel_err(got, want) < TOL[dtype]
    again = o.subm_conv_sparse(feat.to(DEV), plan, packed, b.to(DEV))
    assert torch.equal(got, again)
    nob = o.subm_conv_sparse(feat.to(DEV), plan, packed, None)
    assert rel_err(nob, OF.subm_conv(feat.float(), nbr, w.float(), None)) < TOL[dtype]
    pairs = o.subm_conv_pairs(feat.to(DEV), plan, w.reshape(c, 27, c).to(DEV), b.to(DEV))
    assert rel_err(got, pairs.float().cpu()) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("c,n,mode", [(128, 5001, 3), (128, 77, 2), (256, 3000, 3), (256, 40_001, 2), (256, 1, 3), (128, 33, 3),
                                      (256, 37_681, 3), (256, 60_001, 2), (256, 50_000, 3), (256, 49_152, 2), (256, 49_153, 3),
                                      (256, 12_289, 2), (256, 191, 3)])
def test_linear_ln_parity(dtype, c, n, mode):
    """Square Linear + LayerNorm(s) + residual in one kernel (model.py:541-545,587-597) against torch in
    fp32 and against the two kernels it replaces (same rounding points, other summation order)."""
    import torch.nn.functional as F
    torch.manual_seed(c + n + mode)
    lin = torch.nn.Linear(c, c).to(dtype)
    ln1, ln2 = torch.nn.LayerNorm(c), torch.nn.LayerNorm(c)
    for ln in (ln1, ln2):
        ln.weight.data.uniform_(0.5, 1.5)
        ln.bias.data.normal_(0, 0.3)
    ln1, ln2 = ln1.to(dtype), ln2.to(dtype)
    x = torch.randn(n, c).to(dtype)
    res = torch.randn(n, c).to(dtype)
    shift = (torch.randn(c) * 0.2).to(dtype)
    o = ops()
    with torch.no_grad():
        y = F.linear(x.float(), lin.weight.float(), lin.bias.float())
        if mode == 3:
            s = res.float() + F.layer_norm(y, (c,), ln1.weight.float(), ln1.bias.float(), ln1.eps)
            want0, want1 = s, F.layer_norm(s, (c,), ln2.weight.float(), ln2.bias.float(), ln2.eps)
        else:
            s = res.float() + y
            want0, want1 = s + shift.float(), F.layer_norm(s, (c,), ln1.weight.float(), ln1.bias.float(), ln1.eps)
        lin_d, l1, l2 = lin.to(DEV), ln1.to(DEV), ln2.to(DEV)   # (moves the modules)
        if mode == 3:
            got0, got1 = o.linear_ln(x.to(DEV), lin_d, res.to(DEV), l1, 3, ln2=l2)
            two0, two1 = o.layer_norm(o.linear_rows(x.to(DEV), lin_d.weight, lin_d.bias), l1.weight, l1.bias, l1.eps,
                                      residual=res.to(DEV), mode=3, weight2=l2.weight, bias2=l2.bias)
        else:
            got0, got1 = o.linear_ln(x.to(DEV), lin_d, res.to(DEV), l1, 2, shift=shift.to(DEV))
            two0, two1 = o.layer_norm(o.linear_rows(x.to(DEV), lin_d.weight, lin_d.bias), l1.weight, l1.bias, l1.eps,
                                      residual=res.to(DEV), mode=2, shift=shift.to(DEV))
    assert got0.dtype == dtype and got0.shape == (n, c) and got1.shape == (n, c)
    assert rel_err(got0, want0) < TOL[dtype] and rel_err(got1, want1) < TOL[dtype]
    ulp = 2e-3 if dtype == torch.float16 else 1.6e-2
    assert rel_err(got0, two0.float().cpu()) < ulp and rel_err(got1, two1.float().cpu()) < ulp


@pytest.mark.parametrize("n,extent,nb", [(1, 4, 1), (2500, 14, 2), (50_000, 60, 3), (20_000, 300, 1)])
def test_conv_plan_inner_equals_direct_3x3x3(n, extent, nb):
    """The 3x3x3 pair lists derived from the 5x5x5 ones (their inner 27 taps) are the lists built directly."""
    rng = np.random.default_rng(n + extent)
    idx, *_ = _indices(rng, n, extent, nb)
    o = ops()
    dev_idx = to_dev(idx)
    pend5 = o.conv_plan_direct_start(dev_idx, 5)
    plan5 = o.conv_plan_direct_finish(pend5)
    got = o.conv_plan_inner(plan5, pend5)
    ref = o.conv_plan_direct(dev_idx, 3)
    assert got.n_pairs == ref.n_pairs and got.taps == 27 and got.n == ref.n
    assert torch.equal(got.tap_ptr, ref.tap_ptr) and torch.equal(got.row_ptr, ref.row_ptr)
    assert torch.equal(got.pair_in[:got.n_pairs], ref.pair_in[:ref.n_pairs])
    assert torch.equal(got.pair_slot[:got.n_pairs], ref.pair_slot[:ref.n_pairs])
