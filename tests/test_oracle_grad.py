"""Pins the gradient oracle: autograd over the CPU restatements against central finite differences
(float64) and against the closed forms the HIP backward kernels implement."""
import numpy as np
import torch

from oracle import functional as OF
from oracle import grad as OG
from oracle import indexing as OI


def _fd(fn, x, dout, eps=1e-5):
    """d(sum(fn(x) * dout)) / dx by central differences, float64."""
    x = np.asarray(x, np.float64)
    g = np.zeros_like(x)
    it = np.nditer(x, flags=["multi_index"])
    for _ in it:
        i = it.multi_index
        xp, xm = x.copy(), x.copy()
        xp[i] += eps
        xm[i] -= eps
        g[i] = ((fn(xp) - fn(xm)) * dout).sum() / (2 * eps)
    return g


def test_attention_gradient_against_finite_differences_and_closed_form():
    rng = np.random.default_rng(0)
    heads, C = 2, 32
    cu = [0, 5, 12]
    qkv = rng.standard_normal((12, 3 * C))
    dout = rng.standard_normal((12, C))
    closed = OG.patch_attention_grad_closed_form(qkv, dout, cu, heads)
    fd = _fd(lambda x: OF.patch_attention_bruteforce(x, cu, heads), qkv, dout)
    assert np.abs(closed - fd).max() < 1e-6 * np.abs(fd).max()
    x = torch.tensor(qkv, dtype=torch.float32, requires_grad=True)
    OF.patch_attention(x, cu, heads).backward(torch.tensor(dout, dtype=torch.float32))
    assert np.abs(x.grad.numpy() - closed).max() < 1e-5 * np.abs(closed).max()


def test_serialized_attention_gradient_adds_the_filler_slots_share():
    # two scenes, the second padded with filler slots that repeat earlier rows: their key / value
    # gradient must arrive at the repeated rows
    rng = np.random.default_rng(1)
    counts, patch, heads = [8, 11], 4, 1
    n, C = sum(counts), 16
    offset = np.cumsum(counts)
    starts = np.concatenate([[0], offset[:-1]])
    order = np.concatenate([s + rng.permutation(c) for s, c in zip(starts, counts)]).astype(np.int64)
    inverse = np.empty(n, np.int64)
    inverse[order] = np.arange(n)
    pad, unpad, cu = OI.padding_tables(offset, patch)
    assert len(pad) > n
    qkv = rng.standard_normal((n, 3 * C)).astype(np.float32)
    dout = rng.standard_normal((n, C)).astype(np.float32)
    got = OG.serialized_attention_grad(qkv, dout, order, inverse, pad, unpad, cu, heads).numpy()
    # closed form on the padded rows, then the scatter-add of the gather qkv[order[pad]]
    rows = order[pad]
    dpad = np.zeros((len(pad), C))
    primary = unpad[inverse[rows]] == np.arange(len(pad))
    dpad[primary] = dout[rows[primary]]
    gp = OG.patch_attention_grad_closed_form(qkv[rows], dpad, cu, heads)
    want = np.zeros((n, 3 * C))
    np.add.at(want, rows, gp)
    assert np.abs(got - want).max() < 1e-5 * np.abs(want).max()


def test_subm_conv_gradient_against_finite_differences_and_closed_form():
    rng = np.random.default_rng(2)
    pts = np.unique(rng.integers(0, 4, size=(40, 3)), axis=0)
    idx = np.concatenate([np.zeros((len(pts), 1), np.int64), pts], 1)
    nbr = OI.subm_kmap(idx, 3)
    cin, cout = 3, 2
    feat = rng.standard_normal((len(pts), cin))
    w = rng.standard_normal((cout, 3, 3, 3, cin))
    dout = rng.standard_normal((len(pts), cout))
    dfeat, dw = OG.subm_conv_grad_closed_form(feat, nbr, w, dout)
    fwd = lambda f, ww: OF.subm_conv(torch.tensor(f, dtype=torch.float64).float(), nbr, torch.tensor(ww).float()).double().numpy()
    # float32 forward: a coarse step keeps the differences above rounding
    fd_feat = _fd(lambda f: fwd(f, w), feat, dout, eps=1e-2)
    fd_w = _fd(lambda ww: fwd(feat, ww), w, dout, eps=1e-2).reshape(cout, 27, cin)
    assert np.abs(dfeat - fd_feat).max() < 2e-3 * np.abs(fd_feat).max()
    assert np.abs(dw - fd_w).max() < 2e-3 * np.abs(fd_w).max()
    a_feat, a_w, _ = OG.subm_conv_grad(feat, nbr, w, None, dout)
    assert np.abs(a_feat.numpy() - dfeat).max() < 1e-5 * np.abs(dfeat).max()
    assert np.abs(a_w.numpy().reshape(cout, 27, cin) - dw).max() < 1e-5 * np.abs(dw).max()


def test_submanifold_neighbour_maps_are_mirror_symmetric():
    # nbr[i][t] = j  <=>  nbr[j][V-1-t] = i: what lets the input gradient reuse the forward kernels
    rng = np.random.default_rng(3)
    pts = np.unique(rng.integers(0, 6, size=(120, 3)), axis=0)
    idx = np.concatenate([rng.integers(0, 2, size=(len(pts), 1)), pts], 1)
    for ks in (3, 5):
        nbr = OI.subm_kmap(idx, ks)
        v = ks ** 3
        i, t = np.nonzero(nbr >= 0)
        assert (nbr[nbr[i, t], v - 1 - t] == i).all()


def test_segment_max_gradient_and_the_differentiable_branch():
    rng = np.random.default_rng(4)
    n, c, m = 23, 5, 7
    indices = rng.permutation(n)
    cuts = np.sort(rng.choice(np.arange(1, n), m - 1, replace=False))
    idx_ptr = np.concatenate([[0], cuts, [n]])
    src = rng.standard_normal((n, c)).astype(np.float32)
    dout = rng.standard_normal((m, c)).astype(np.float32)
    for reduce in ("max", "min", "sum", "mean"):
        plain = OF.segment_csr(src, indices, idx_ptr, reduce)
        x = torch.tensor(src, requires_grad=True)
        assert torch.allclose(OF.segment_csr(x, indices, idx_ptr, reduce), plain, atol=1e-6)
        got = OG.segment_csr_grad(src, indices, idx_ptr, reduce, dout).numpy()
        want = np.zeros((n, c))
        for s in range(m):
            rows = indices[idx_ptr[s]:idx_ptr[s + 1]]
            for ch in range(c):
                if reduce in ("max", "min"):
                    pick = rows[np.argmax(src[rows, ch]) if reduce == "max" else np.argmin(src[rows, ch])]
                    want[pick, ch] = dout[s, ch]
                else:
                    want[rows, ch] = dout[s, ch] / (len(rows) if reduce == "mean" else 1)
        assert np.abs(got - want).max() < 1e-6


def test_unpool_add_gradient():
    rng = np.random.default_rng(5)
    cluster = rng.integers(0, 4, size=15)
    dout = rng.standard_normal((15, 3)).astype(np.float32)
    dparent, dchild = OG.unpool_add_grad(dout, cluster, 4)
    p = torch.zeros(15, 3, requires_grad=True)
    ch = torch.zeros(4, 3, requires_grad=True)
    OF.unpool_add(p, ch, cluster).backward(torch.tensor(dout))
    assert torch.allclose(dparent, p.grad) and torch.allclose(dchild, ch.grad, atol=1e-6)


def test_dropout_mask_statistics():
    """The attention-dropout mask both the kernels and the oracle use: kept fraction 1 - p, rows and columns
    balanced, and no visible dependence between heads, seeds or neighbouring slots."""
    q = np.arange(3000, 5048)
    k = np.arange(100, 2148)
    for p in (0.1, 0.3, 0.5):
        m = OF.dropout_keep_mask(7, 0, q, k, p)
        assert abs(m.mean() - (1 - p)) < 3e-3
        assert np.abs(m.mean(0) - (1 - p)).max() < 0.06 and np.abs(m.mean(1) - (1 - p)).max() < 0.06
    a = OF.dropout_keep_mask(7, 0, q, k, 0.5).astype(np.float64) - 0.5
    for other in (OF.dropout_keep_mask(7, 1, q, k, 0.5), OF.dropout_keep_mask(8, 0, q, k, 0.5),
                  OF.dropout_keep_mask(7, 0, q + 1, k, 0.5), OF.dropout_keep_mask(7, 0, q, k + 1, 0.5)):
        b = other.astype(np.float64) - 0.5
        assert abs((a * b).mean() / 0.25) < 5e-3          # correlation of two masks of four million bits
    assert np.array_equal(OF.dropout_keep_mask(7, 0, q, k, 0.5), OF.dropout_keep_mask(7, 0, q, k, 0.5))
    assert OF.dropout_keep_mask(1, 0, q, k, 0.0).all()
