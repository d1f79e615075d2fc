"""ptv3_pool_clusters_static (the entry point that allocates nothing) against ptv3_pool_clusters, through the
C ABI, bit for bit: two calls in a row on the same GPU, the second on a smaller input, so that whatever the
first call left in the library's fixed buffer is still there when the second one runs."""
import numpy as np
import pytest
import torch

from gpu_util import DEV

pytestmark = pytest.mark.gpu


def _both(lib, _lib, n, n_scenes, seed, shift=3):
    rng = np.random.default_rng(seed)
    # sorted-run structure like a serialized level: scene id above bit 48, clusters of 1..8 points
    sizes = np.diff(np.sort(np.concatenate([[0, n], rng.choice(np.arange(1, n), n_scenes - 1, replace=False)])))
    code = np.concatenate([(np.int64(b) << 48) | np.sort(rng.integers(0, 1 << 30, size=s, dtype=np.int64))
                           for b, s in enumerate(sizes)])
    perm = rng.permutation(n)
    code0 = torch.from_numpy(code[np.argsort(perm)]).to(DEV)          # point order
    order0 = torch.argsort(code0, stable=True)
    offset = torch.from_numpy(np.cumsum(sizes).astype(np.int64)).to(DEV)
    stream = torch.cuda.current_stream().cuda_stream
    outs = []
    for static in (False, True):
        cluster = torch.full((n,), -7, dtype=torch.int64, device=DEV)
        idx_ptr = torch.full((n + 1,), -7, dtype=torch.int64, device=DEV)
        head = torch.full((n,), -7, dtype=torch.int64, device=DEV)
        count = torch.full((1 + n_scenes,), -7, dtype=torch.int64, device=DEV)
        args = [code0.data_ptr(), order0.data_ptr(), n, shift, offset.data_ptr(), n_scenes, cluster.data_ptr(),
                idx_ptr.data_ptr(), head.data_ptr(), count.data_ptr()]
        if static:
            # the warm-up call (n = 0: looks the buffer's address up, launches nothing), then the real one, which
            # must leave the amount of free device memory as it found it
            _lib.check(lib.ptv3_pool_clusters_static(None, None, 0, shift, None, 0, None, None, None, None, stream),
                       "ptv3_pool_clusters_static warm-up")
            torch.cuda.synchronize()
            free_before = torch.cuda.mem_get_info()[0]
            _lib.check(lib.ptv3_pool_clusters_static(*args, stream), "ptv3_pool_clusters_static")
            torch.cuda.synchronize()
            assert torch.cuda.mem_get_info()[0] == free_before
        else:
            nbytes = lib.ptv3_pool_clusters_workspace_bytes(n)
            ws = torch.empty(nbytes, dtype=torch.uint8, device=DEV)
            _lib.check(lib.ptv3_pool_clusters(*args, ws.data_ptr(), nbytes, stream), "ptv3_pool_clusters")
        torch.cuda.synchronize()
        outs.append((cluster.cpu(), idx_ptr.cpu(), head.cpu(), count.cpu()))
    return outs


def test_static_entry_point_matches_the_workspace_one_twice_in_a_row():
    from pointtransformerv3_amd import _lib
    lib = _lib.load()
    for n, nb, seed in ((300_001, 4, 1), (70_003, 3, 2)):     # the second call is the smaller one
        (c0, p0, h0, k0), (c1, p1, h1, k1) = _both(lib, _lib, n, nb, seed)
        m = int(k0[0])
        assert 0 < m < n and int(k1[0]) == m
        assert torch.equal(c0, c1) and torch.equal(k0, k1)
        assert torch.equal(p0[: m + 1], p1[: m + 1]) and torch.equal(h0[:m], h1[:m])
        # and they are the clusters: run starts of code >> shift in sorted order
        assert int(c1.max()) == m - 1 and int(p1[m]) == n
