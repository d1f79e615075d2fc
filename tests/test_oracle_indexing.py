"""Pins the index-bookkeeping and floating-point oracles against closed forms, hand-worked
cases, brute force on tiny inputs and stock library routines."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import cnative
from oracle import functional as OF
from oracle import indexing as OI
from oracle import serialization as S


# ---------------------------------------------------------------- padding tables
def test_padding_hand_case_2500():
    pad, unpad, cu = OI.padding_tables([2500], 1024)
    assert len(pad) == 3072 and len(unpad) == 2500
    assert np.array_equal(pad[:2500], np.arange(2500))
    assert np.array_equal(pad[2500:], np.arange(1476, 2048))  # filler slots look one patch back
    assert np.array_equal(unpad, np.arange(2500))
    assert cu.dtype == np.int32 and cu.tolist() == [0, 1024, 2048, 3072]


@pytest.mark.parametrize("n,want_pad,want_cu", [
    (1500, 2048, [0, 1024, 2048]), (1024, 1024, [0, 1024]), (700, 700, [0, 700]), (2048, 2048, [0, 1024, 2048])])
def test_padding_single_scene(n, want_pad, want_cu):
    pad, unpad, cu = OI.padding_tables([n], 1024)
    assert len(pad) == want_pad and cu.tolist() == want_cu
    assert np.array_equal(pad[unpad], np.arange(n))


def test_padding_two_scenes_slice_semantics():
    # re-derive with the slice-copy formulation on python lists
    offset, K = [1300, 1300 + 700, 1300 + 700 + 2049], 512
    pad, unpad, cu = OI.padding_tables(offset, K)
    cnt = np.diff(offset, prepend=0)
    want_pad, want_unpad, want_cu, o, op = [], [], [], 0, 0
    for n in cnt.tolist():
        npad = n if n <= K else ((n + K - 1) // K) * K
        local = list(range(npad))
        if npad != n:
            r = n % K
            local[npad - K + r:npad] = local[npad - 2 * K + r:npad - K]
        want_pad += [o + v for v in local]
        want_unpad += [op + j for j in range(n)]
        want_cu += list(range(op, op + npad, K))
        o += n
        op += npad
    want_cu.append(op)
    assert pad.tolist() == want_pad and unpad.tolist() == want_unpad and cu.tolist() == want_cu
    # every patch of a padded scene is full and stays inside its scene
    batch = OI.offset2batch(offset)
    for s, e in zip(cu[:-1], cu[1:]):
        assert len(set(batch[pad[s:e]].tolist())) == 1


def test_offset_batch_helpers():
    off = np.array([3, 3, 7])
    assert OI.offset2bincount(off).tolist() == [3, 0, 4]
    assert OI.offset2batch(off).tolist() == [0, 0, 0, 2, 2, 2, 2]
    assert OI.batch2offset([0, 0, 1, 1, 1]).tolist() == [2, 5]


# ---------------------------------------------------------------- kernel map
def _random_voxels(rng, n, extent, nb=2):
    cells = np.stack(np.meshgrid(*[np.arange(extent)] * 3, indexing="ij"), -1).reshape(-1, 3)
    rows = []
    for b in range(nb):
        pick = rng.permutation(len(cells))[:n]
        rows.append(np.concatenate([np.full((n, 1), b), cells[pick]], 1))
    return np.concatenate(rows).astype(np.int32)


@pytest.mark.parametrize("ks", [3, 5])
def test_kmap_three_ways(ks):
    rng = np.random.default_rng(ks)
    idx = _random_voxels(rng, 300, 9)
    a = OI.subm_kmap(idx, ks)
    assert np.array_equal(a, OI.subm_kmap_bruteforce(idx, ks))
    assert np.array_equal(a, cnative.kmap(idx, ks))
    V = ks ** 3
    assert np.array_equal(a[:, V // 2], np.arange(len(idx)))  # centre tap is the voxel itself
    i, k = np.nonzero(a >= 0)
    assert np.array_equal(a[a[i, k], V - 1 - k], i)  # nbr[i,k]=j <=> nbr[j,V-1-k]=i
    # scenes never see each other
    assert np.array_equal(idx[a[i, k], 0], idx[i, 0])


# ---------------------------------------------------------------- conv
@pytest.mark.parametrize("ks,cin,cout", [(3, 5, 7), (5, 4, 6)])
def test_subm_conv_equals_dense_conv3d_at_active_sites(ks, cin, cout):
    rng = np.random.default_rng(11)
    idx = _random_voxels(rng, 200, 8)
    g = torch.Generator().manual_seed(5)
    feat = torch.randn(len(idx), cin, generator=g)
    w = torch.randn(cout, ks, ks, ks, cin, generator=g)
    b = torch.randn(cout, generator=g)
    got = OF.subm_conv(feat, OI.subm_kmap(idx, ks), w, b)
    want = OF.subm_conv_dense(feat, idx, w, b)
    assert torch.allclose(got, want, rtol=1e-5, atol=1e-5)


# ---------------------------------------------------------------- attention
def test_attention_vs_sdpa_and_bruteforce():
    g = torch.Generator().manual_seed(1)
    H, D = 2, 16
    cu = [0, 8, 16, 21]
    qkv = torch.randn(21, 3 * H * D, generator=g)
    got = OF.patch_attention(qkv, cu, H)
    assert np.allclose(got.numpy(), OF.patch_attention_bruteforce(qkv.numpy(), cu, H), atol=1e-5)
    for s, e in zip(cu[:-1], cu[1:]):
        q, k, v = qkv[s:e].reshape(e - s, 3, H, D).permute(1, 2, 0, 3)
        want = F.scaled_dot_product_attention(q, k, v).transpose(0, 1).reshape(e - s, H * D)
        assert torch.allclose(got[s:e], want, atol=1e-5)
    # keys may be shuffled inside a patch without changing any query's output
    perm = torch.cat([torch.randperm(8, generator=g), 8 + torch.arange(13)])
    got_p = OF.patch_attention(qkv[perm], cu, H)
    assert torch.allclose(got_p, got[perm], atol=1e-5)


def test_serialized_attention_core_keeps_primary_slot():
    g = torch.Generator().manual_seed(2)
    N, K, H, D = 37, 16, 2, 4
    qkv = torch.randn(N, 3 * H * D, generator=g)
    order = torch.randperm(N, generator=g).numpy()
    inverse = np.empty(N, np.int64)
    inverse[order] = np.arange(N)
    pad, unpad, cu = OI.padding_tables([N], K)
    got = OF.serialized_attention_core(qkv, order, inverse, pad, unpad, cu, H)
    # per point: it sits at rank inverse[n]; its patch is rank // K, except that the last
    # (short) patch is completed with the points just before it
    sorted_qkv = qkv[order]
    for n in range(N):
        r = int(inverse[n])
        p = r // K
        lo, hi = p * K, min((p + 1) * K, N)
        if hi - lo < K:
            lo = hi - K
        blk = sorted_qkv[lo:hi]
        ref = OF.patch_attention_bruteforce(blk.numpy(), [0, hi - lo], H)[r - lo]
        assert np.allclose(got[n].numpy(), ref, atol=1e-5)


# ---------------------------------------------------------------- pooling
def test_pool_clusters_bruteforce():
    rng = np.random.default_rng(9)
    idx = _random_voxels(rng, 400, 10, nb=2)
    g, batch = idx[:, 1:], idx[:, 0].astype(np.int64)
    depth, code, order, inverse = S.serialize(g, batch)
    pc = OI.pool_clusters(code, g, batch, 1)
    # group by (batch, coarse cell) with a dictionary; rank groups by shifted row-0 code
    groups = {}
    for n in range(len(g)):
        groups.setdefault((int(batch[n]), *(g[n] >> 1).tolist()), []).append(n)
    keys = sorted(groups, key=lambda kk: int(code[0][groups[kk][0]]) >> 3)
    M = len(keys)
    assert len(pc["counts"]) == M
    for m, kk in enumerate(keys):
        mem = groups[kk]
        assert set(np.nonzero(pc["cluster"] == m)[0].tolist()) == set(mem)
        assert pc["counts"][m] == len(mem)
        assert sorted(pc["indices"][pc["idx_ptr"][m]:pc["idx_ptr"][m + 1]].tolist()) == sorted(mem)
        assert pc["grid_coord"][m].tolist() == list(kk[1:]) and pc["batch"][m] == kk[0]
    # pooled codes equal the codes of the pooled cells one level up, for every order
    for r, name in enumerate(S.ORDERS):
        assert np.array_equal(pc["code"][r], S.encode(pc["grid_coord"], pc["batch"], depth - 1, name))
        assert np.all(np.diff(pc["code"][r][pc["order"][r]]) > 0)
    assert np.array_equal(pc["order"][0], np.arange(M))


def test_segment_csr_and_unpool():
    src = torch.tensor([[1., 5.], [3., -2.], [0., 7.], [4., 4.]])
    indices, ptr = np.array([2, 0, 3, 1]), np.array([0, 1, 4])
    assert OF.segment_csr(src, indices, ptr, "max").tolist() == [[0., 7.], [4., 5.]]
    assert OF.segment_csr(src, indices, ptr, "mean").tolist() == [[0., 7.], [8 / 3, 7 / 3]] or \
        np.allclose(OF.segment_csr(src, indices, ptr, "mean").numpy(), [[0., 7.], [8 / 3, 7 / 3]])
    out = OF.unpool_add(torch.ones(3, 2), torch.tensor([[1., 2.], [10., 20.]]), [1, 0, 1])
    assert out.tolist() == [[11., 21.], [2., 3.], [11., 21.]]


def test_rpe_bias_and_attention_with_bias():
    """Relative position bias (model.py:297-316, :468-469). Pins: a per-pair loop straight from the
    definition; a hand case (offset (+1, 0, -40) with pos_bnd 3 reads table rows 4, 7+3, 14+0); the
    clamp; a zero table changes nothing; softmax with the bias equals torch's
    scaled_dot_product_attention with the bias passed as an additive mask."""
    rng = np.random.default_rng(5)
    g = torch.Generator().manual_seed(5)
    L, H, bnd = 37, 3, 3
    rnum = 2 * bnd + 1
    coord = rng.integers(0, 12, size=(L, 3))
    table = torch.randn(3 * rnum, H, generator=g)
    bias = OF.rpe_bias(coord, table, bnd)
    assert bias.shape == (H, L, L)
    for i, j in ((0, 0), (3, 17), (36, 5), (11, 30)):
        want = torch.zeros(H)
        for a in range(3):
            d = int(np.clip(coord[i, a] - coord[j, a], -bnd, bnd))
            want += table[a * rnum + d + bnd]
        assert torch.allclose(bias[:, i, j], want, atol=1e-6)
    two = OF.rpe_bias(np.array([[5, 2, 0], [4, 2, 40]]), table, bnd)     # query 0 - key 1 = (+1, 0, -40)
    assert torch.allclose(two[:, 0, 1], table[4] + table[rnum + 3] + table[2 * rnum + 0], atol=1e-6)
    assert torch.allclose(two[:, 1, 0], table[2] + table[rnum + 3] + table[2 * rnum + 6], atol=1e-6)
    qkv = torch.randn(L, 3 * H * 16, generator=g)
    plain = OF.patch_attention(qkv, [0, L], H)
    assert torch.allclose(OF.patch_attention(qkv, [0, L], H, rpe=(coord, torch.zeros_like(table), bnd)), plain, atol=1e-6)
    got = OF.patch_attention(qkv, [0, L], H, rpe=(coord, table, bnd))
    assert not torch.allclose(got, plain, atol=1e-3)
    q, k, v = qkv.reshape(L, 3, H, 16).permute(1, 2, 0, 3)
    want = F.scaled_dot_product_attention(q[None], k[None], v[None], attn_mask=bias[None])[0]
    assert torch.allclose(got, want.transpose(0, 1).reshape(L, H * 16), atol=1e-5)


def test_voxelize_against_dictionary_and_scene_generator():
    from pointtransformerv3_amd import synthetic
    rng = np.random.default_rng(31)
    sizes = [400, 0, 1, 900]
    coord = np.concatenate([rng.random((n, 3)) * 2 + rng.normal(0, 20, 3) for n in sizes]).astype(np.float32)
    offset = np.cumsum(sizes)
    grid = 0.25
    g, index, inverse, ends = OI.voxelize(coord, offset, grid)
    # brute force: walk the points, remember the first of every (scene, cell)
    seen, want_g, want_i, want_inv, want_ends, start = {}, [], [], [], [], 0
    for s, end in enumerate(offset):
        lo = coord[start:end].min(0) if end > start else None
        for i in range(start, end):
            cell = tuple(np.floor((coord[i] - lo) / np.float32(grid)).astype(np.int64))
            if (s, cell) not in seen:
                seen[(s, cell)] = len(want_i)
                want_g.append(cell); want_i.append(i)
            want_inv.append(seen[(s, cell)])
        want_ends.append(len(want_i))
        start = end
    assert np.array_equal(g, np.array(want_g)) and np.array_equal(index, want_i)
    assert np.array_equal(inverse, want_inv) and np.array_equal(ends, want_ends)
    assert len(index) < len(coord)
    # one scene: the generator of the benchmark scenes does the same (in the precision of its points)
    pts = synthetic.room_points(5000, 3).astype(np.float32)
    g1, keep = synthetic.voxelize_unique(pts, np.float32(0.05))
    g2, i2, _, _ = OI.voxelize(pts, [len(pts)], 0.05)
    assert np.array_equal(g1, g2) and np.array_equal(keep, i2)
