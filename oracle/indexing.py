"""CPU oracle for the index bookkeeping of the PTv3 forward path (TEST INFRASTRUCTURE).

Only tests, the smoke check and the CPU-baseline leg of the benchmark may import this.

* offset/batch helpers            -> model.py:28-45
* patch padding tables            -> model.py:382-438
* grid-pooling clusters           -> model.py:640-695
* submanifold neighbour map       -> the semantics spconv's SubMConv3d implements for the
  call sites model.py:546-552 and :767-774 (spconv itself is not part of the reference
  checkout; the map is pinned against a dense convolution in the tests)
"""
import numpy as np


def offset2bincount(offset):
    offset = np.asarray(offset, dtype=np.int64)
    return np.diff(offset, prepend=np.int64(0))


def offset2batch(offset):
    cnt = offset2bincount(offset)
    return np.repeat(np.arange(len(cnt), dtype=np.int64), cnt)


def batch2offset(batch):
    return np.cumsum(np.bincount(np.asarray(batch, dtype=np.int64))).astype(np.int64)


def padding_tables(offset, patch):
    """model.py:392-437, written per scene and per slot instead of with slice copies.

    Returns (pad (Npad,), unpad (N,), cu_seqlens (P+1,) int32). A scene longer than one
    patch is rounded up to whole patches and the tail of its last patch is filled with
    the `patch - r` points that precede the last `r` real ones (model.py:412-423)."""
    offset = np.asarray(offset, dtype=np.int64)
    cnt = offset2bincount(offset)
    pad, unpad, cu = [], [], []
    base = 0
    start = 0
    for n in cnt.tolist():
        n_pad = -(-n // patch) * patch if n > patch else n  # model.py:394-404
        slot = np.arange(n_pad, dtype=np.int64)
        src = np.where(slot < n, slot, slot - patch)  # filler slots look one patch back
        pad.append(start + src)
        unpad.append(base + np.arange(n, dtype=np.int64))
        cu.append(np.arange(base, base + n_pad, patch, dtype=np.int64))
        base += n_pad
        start += n
    cu.append(np.array([base], dtype=np.int64))
    return (
        np.concatenate(pad) if pad else np.zeros(0, np.int64),
        np.concatenate(unpad) if unpad else np.zeros(0, np.int64),
        np.concatenate(cu).astype(np.int32),
    )


def pool_clusters(code, grid_coord, batch, pooling_depth=1):
    """model.py:652-695 (no shuffle): clusters are numbered by ascending row-0 code
    shifted right by 3*pooling_depth bits.

    Returns a dict with cluster (N,), counts (M,), idx_ptr (M+1,), indices (N,)
    [points grouped by cluster, stable], head (M,), and the pooled code (k,M),
    order (k,M), inverse (k,M), grid_coord (M,3), batch (M,)."""
    code = np.asarray(code, dtype=np.int64) >> np.int64(3 * pooling_depth)
    uniq, cluster, counts = np.unique(code[0], return_inverse=True, return_counts=True)
    cluster = cluster.astype(np.int64)
    indices = np.argsort(cluster, kind="stable").astype(np.int64)
    idx_ptr = np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)
    head = indices[idx_ptr[:-1]]
    pcode = code[:, head]
    order = np.argsort(pcode, axis=1, kind="stable").astype(np.int64)
    inverse = np.empty_like(order)
    for r in range(order.shape[0]):
        inverse[r, order[r]] = np.arange(order.shape[1], dtype=np.int64)
    return dict(
        cluster=cluster,
        counts=counts.astype(np.int64),
        idx_ptr=idx_ptr,
        indices=indices,
        head=head,
        code=pcode,
        order=order,
        inverse=inverse,
        grid_coord=np.asarray(grid_coord)[head] >> pooling_depth,
        batch=np.asarray(batch)[head],
    )


def kernel_offsets(ks):
    """Row-major (kx,ky,kz) enumeration, offset = k - ks//2."""
    r = ks // 2
    return np.array(
        [(a - r, b - r, c - r) for a in range(ks) for b in range(ks) for c in range(ks)],
        dtype=np.int64,
    )


def subm_kmap(indices, ks=3):
    """nbr (N, ks^3) int32: index of the active voxel at coord_i + offset_k, else -1.

    indices is (N,4) [batch,x,y,z] with non-negative coordinates (model.py:167-169).
    Vectorised: pack -> sort -> searchsorted per offset."""
    idx = np.asarray(indices, dtype=np.int64)
    n = idx.shape[0]
    off = kernel_offsets(ks)
    nbr = np.full((n, off.shape[0]), -1, dtype=np.int32)
    if n == 0:
        return nbr

    def pack(b, x, y, z):
        return (b << 51) | ((x + 4) << 34) | ((y + 4) << 17) | (z + 4)

    keys = pack(idx[:, 0], idx[:, 1], idx[:, 2], idx[:, 3])
    perm = np.argsort(keys, kind="stable")
    skeys = keys[perm]
    for k, (dx, dy, dz) in enumerate(off.tolist()):
        q = pack(idx[:, 0], idx[:, 1] + dx, idx[:, 2] + dy, idx[:, 3] + dz)
        pos = np.searchsorted(skeys, q)
        pos_c = np.minimum(pos, n - 1)
        hit = skeys[pos_c] == q
        nbr[hit, k] = perm[pos_c[hit]].astype(np.int32)
    return nbr


def subm_kmap_bruteforce(indices, ks=3):
    """Dictionary lookup, for tiny inputs only; independent of subm_kmap's packing."""
    idx = [tuple(int(v) for v in row) for row in np.asarray(indices)]
    table = {v: i for i, v in enumerate(idx)}
    off = kernel_offsets(ks).tolist()
    nbr = np.full((len(idx), len(off)), -1, dtype=np.int32)
    for i, (b, x, y, z) in enumerate(idx):
        for k, (dx, dy, dz) in enumerate(off):
            nbr[i, k] = table.get((b, x + dx, y + dy, z + dz), -1)
    return nbr


def voxelize(coord, offset, grid_size):
    """Voxelisation in front of the model: per scene grid_coord = floor((p - scene min) / grid_size)
    in float32, the first point (input order) of every voxel kept.

    The reference checkout has no file for this step (it is Pointcept's GridSample + collate, outside
    the checkout; model.py:88-96 is only the fallback that derives grid_coord): parity with it is
    unpinned. What is pinned is this function against a dictionary brute force and against the
    generator of the benchmark scenes (tests/test_oracle_indexing.py).
    Returns grid_coord (M,3) int32, index (M,) kept input rows ascending, inverse (N,) voxel of every
    point, ends (B,) cumulative kept counts."""
    coord = np.asarray(coord, np.float32)
    grids, index, inverse, ends = [], [], np.empty(len(coord), np.int64), []
    start, kept = 0, 0
    for end in offset:
        p = coord[start:end]
        if len(p):
            g = np.floor((p - p.min(0)) / np.float32(grid_size)).astype(np.int64)
            key = (g[:, 0] << 42) | (g[:, 1] << 21) | g[:, 2]
            _, first, inv = np.unique(key, return_index=True, return_inverse=True)
            rank = np.argsort(np.argsort(first))          # voxels numbered by their first point
            order = np.sort(first)
            grids.append(g[order].astype(np.int32))
            index.append(order + start)
            inverse[start:end] = rank[inv] + kept
            kept += len(order)
        ends.append(kept)
        start = end
    g_all = np.concatenate(grids) if grids else np.zeros((0, 3), np.int32)
    i_all = np.concatenate(index) if index else np.zeros(0, np.int64)
    return g_all, i_all, inverse, np.array(ends, np.int64)
