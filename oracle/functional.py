"""CPU fp32 oracle for the floating-point kernels of the PTv3 forward path
(TEST INFRASTRUCTURE — only tests, the smoke check and the CPU-baseline leg of the
benchmark may import this).

Stock torch CPU operators stand in for the third-party CUDA packages the reference calls:

* patch attention   -> the non-flash arithmetic of model.py:458-474 (== what
  flash_attn_varlen_qkvpacked_func computes at model.py:476-482 with dropout 0),
  looped per sequence so the (P,H,K,K) score tensor is never materialised
* submanifold conv  -> gather + GEMM over the neighbour map (spconv.SubMConv3d call
  sites model.py:546-552, :767-774)
* segment reductions-> torch_scatter.segment_csr call sites model.py:684-689
* unpooling add     -> model.py:746
"""
import numpy as np
import torch
import torch.nn.functional as F


def rpe_bias(coord, table, pos_bnd):
    """Relative position bias of one patch (model.py:297-316, :375-379): coord (L, 3) integer grid
    coordinates in patch order, table (3 * R, H) with R = 2 * pos_bnd + 1. Returns (H, L, L) with
    entry [h, i, j] = sum over axes a of table[a * R + clamp(coord[i, a] - coord[j, a]) + pos_bnd, h]."""
    coord = torch.as_tensor(np.asarray(coord), dtype=torch.int64)
    table = torch.as_tensor(table, dtype=torch.float32)
    rnum = 2 * pos_bnd + 1
    rel = coord[:, None, :] - coord[None, :, :]                                   # (L, L, 3): query - key
    idx = rel.clamp(-pos_bnd, pos_bnd) + pos_bnd + torch.arange(3) * rnum
    return table[idx.reshape(-1)].reshape(idx.shape + (-1,)).sum(2).permute(2, 0, 1)


def dropout_keep_mask(seed, head, q_slots, k_slots, p):
    """The attention-dropout mask of this build's kernels (flash_attn's own random stream, model.py:480, cannot
    be reproduced): element (query slot, key slot) of a head is kept when a 32-bit hash of (seed, head, q, k)
    is at least p * 2^32. q_slots (Lq,), k_slots (Lk,) are padded slot numbers. Returns (Lq, Lk) bool."""
    m32 = np.uint64(0xFFFFFFFF)
    q = np.asarray(q_slots, dtype=np.uint64)[:, None]
    k = np.asarray(k_slots, dtype=np.uint64)[None, :]
    x = ((q * np.uint64(0x9E3779B1)) & m32) ^ (((k + np.uint64(0x7F4A7C15)) * np.uint64(0x85EBCA77)) & m32)
    x = x ^ ((np.uint64(head + 1) * np.uint64(0xC2B2AE3D)) & m32) ^ np.uint64(seed & 0xFFFFFFFF)
    x ^= x >> np.uint64(16)
    x = (x * np.uint64(0x7FEB352D)) & m32
    x ^= x >> np.uint64(15)
    x = (x * np.uint64(0x846CA68B)) & m32
    x ^= x >> np.uint64(16)
    return x >= np.uint64(min(int(p * 4294967296.0), 0xFFFFFFFF))


def patch_attention(qkv, cu_seqlens, num_heads, scale=None, rpe=None, dropout=None):
    """qkv: (Npad, 3*C) fp32 rows already in padded serialized order, channel layout
    [3][H][D] (model.py:461,477). rpe = (coord (Npad, 3) in the same order, table, pos_bnd) adds the
    relative position bias to the scores (model.py:468-469). dropout = (p, seed): softmax probabilities are
    zeroed where dropout_keep_mask says so and the rest divided by 1 - p (model.py:470, :480). Returns (Npad, C)."""
    qkv = torch.as_tensor(qkv, dtype=torch.float32)
    npad, c3 = qkv.shape
    C = c3 // 3
    D = C // num_heads
    scale = D ** -0.5 if scale is None else scale
    cu = [int(v) for v in cu_seqlens]
    out = torch.empty(npad, C, dtype=torch.float32)
    for s, e in zip(cu[:-1], cu[1:]):
        blk = qkv[s:e].reshape(e - s, 3, num_heads, D).permute(1, 2, 0, 3)  # (3,H,L,D)
        q, k, v = blk[0], blk[1], blk[2]
        score = (q * scale) @ k.transpose(-2, -1)
        if rpe is not None:
            score = score + rpe_bias(np.asarray(rpe[0])[s:e], rpe[1], rpe[2])
        attn = torch.softmax(score, dim=-1)
        if dropout is not None and dropout[0] > 0:
            slots = np.arange(s, e)
            keep = np.stack([dropout_keep_mask(dropout[1], h, slots, slots, dropout[0]) for h in range(num_heads)])
            attn = attn * torch.from_numpy(keep).to(attn.dtype) / (1.0 - dropout[0])
        out[s:e] = (attn @ v).transpose(0, 1).reshape(e - s, C)
    return out


def patch_attention_bruteforce(qkv, cu_seqlens, num_heads, scale=None):
    """Triple loop in float64 numpy; toy sizes only."""
    qkv = np.asarray(qkv, dtype=np.float64)
    npad, c3 = qkv.shape
    C = c3 // 3
    D = C // num_heads
    scale = D ** -0.5 if scale is None else scale
    out = np.zeros((npad, C))
    cu = [int(v) for v in cu_seqlens]
    for s, e in zip(cu[:-1], cu[1:]):
        for h in range(num_heads):
            q = qkv[s:e, h * D:(h + 1) * D]
            k = qkv[s:e, C + h * D:C + (h + 1) * D]
            v = qkv[s:e, 2 * C + h * D:2 * C + (h + 1) * D]
            for i in range(e - s):
                sc = (k @ q[i]) * scale
                w = np.exp(sc - sc.max())
                out[s + i, h * D:(h + 1) * D] = (w / w.sum()) @ v
    return out


def serialized_attention_core(feat_qkv, order, inverse, pad, unpad, cu_seqlens, num_heads,
                              scale=None, rpe=None, dropout=None):
    """model.py:452-484: gather rows into padded serialized order, attend inside each
    patch, keep each point's primary slot. feat_qkv: (N, 3C); rpe = (grid_coord (N, 3) in point
    order, table, pos_bnd). Returns (N, C)."""
    feat_qkv = torch.as_tensor(feat_qkv, dtype=torch.float32)
    gidx = torch.as_tensor(np.asarray(order)[np.asarray(pad)])
    back = torch.as_tensor(np.asarray(unpad)[np.asarray(inverse)])
    if rpe is not None:
        rpe = (np.asarray(rpe[0])[gidx.numpy()], rpe[1], rpe[2])
    out = patch_attention(feat_qkv[gidx], cu_seqlens, num_heads, scale, rpe, dropout)
    return out[back]


def subm_conv(feat, nbr, weight, bias=None):
    """out[i] = sum_k W[:,k,:] @ feat[nbr[i,k]] (+ bias); rows with nbr == -1 contribute 0.

    feat (N,Cin); nbr (N,V) int; weight (Cout, ks,ks,ks, Cin) — the layout spconv 2.x
    gives SubMConv3d.weight (an assumption: spconv is not in the reference checkout);
    cross-correlation, offset index k = (kx*ks+ky)*ks+kz."""
    feat = torch.as_tensor(feat, dtype=torch.float32)
    weight = torch.as_tensor(weight, dtype=torch.float32)
    nbr = torch.as_tensor(np.asarray(nbr), dtype=torch.int64)
    cout, cin = weight.shape[0], weight.shape[-1]
    V = nbr.shape[1]
    w = weight.reshape(cout, V, cin)
    out = torch.zeros(feat.shape[0], cout, dtype=torch.float32)
    for k in range(V):
        col = nbr[:, k]
        hit = (col >= 0).nonzero(as_tuple=True)[0]
        if hit.numel() == 0:
            continue
        out.index_add_(0, hit, feat[col[hit]] @ w[:, k, :].t())
    if bias is not None:
        out += torch.as_tensor(bias, dtype=torch.float32)
    return out


def subm_conv_dense(feat, indices, weight, bias=None):
    """The same convolution through torch's dense conv3d on a densified grid; tiny grids
    only. Pins offset enumeration, weight layout and cross-correlation of subm_conv."""
    feat = torch.as_tensor(feat, dtype=torch.float32)
    weight = torch.as_tensor(weight, dtype=torch.float32)
    idx = torch.as_tensor(np.asarray(indices), dtype=torch.int64)
    cout, ks, cin = weight.shape[0], weight.shape[1], weight.shape[-1]
    B = int(idx[:, 0].max()) + 1
    X, Y, Z = (int(idx[:, a].max()) + 1 for a in (1, 2, 3))
    dense = torch.zeros(B, cin, X, Y, Z)
    dense[idx[:, 0], :, idx[:, 1], idx[:, 2], idx[:, 3]] = feat
    w = weight.permute(0, 4, 1, 2, 3).contiguous()  # (Cout,Cin,kx,ky,kz)
    y = F.conv3d(dense, w, None if bias is None else torch.as_tensor(bias, dtype=torch.float32),
                 padding=ks // 2)
    return y[idx[:, 0], :, idx[:, 1], idx[:, 2], idx[:, 3]]


def segment_csr(src, indices, idx_ptr, reduce="max"):
    """reduce(src[indices[idx_ptr[m]:idx_ptr[m+1]]]) per segment m (model.py:684-689).
    Segments are never empty on this path. A src that takes a gradient goes through torch operators
    (same values) so that autograd can differentiate it: the gradient of max / min lands on the
    attaining member, split evenly should several tie (torch_scatter picks one of them)."""
    if isinstance(src, torch.Tensor) and src.requires_grad:
        return _segment_csr_autograd(src, indices, idx_ptr, reduce)
    src = np.asarray(torch.as_tensor(src, dtype=torch.float32))[np.asarray(indices)]
    starts = np.asarray(idx_ptr[:-1], dtype=np.int64)
    if reduce == "max":
        out = np.maximum.reduceat(src, starts, axis=0)
    elif reduce == "min":
        out = np.minimum.reduceat(src, starts, axis=0)
    else:
        out = np.add.reduceat(src.astype(np.float64), starts, axis=0)
        if reduce == "mean":
            out = out / np.diff(np.asarray(idx_ptr, dtype=np.int64))[:, None]
        out = out.astype(np.float32)
    return torch.from_numpy(np.ascontiguousarray(out))


def _segment_csr_autograd(src, indices, idx_ptr, reduce):
    ptr = torch.as_tensor(np.asarray(idx_ptr), dtype=torch.int64)
    rows = src[torch.as_tensor(np.asarray(indices), dtype=torch.int64)]
    m = ptr.numel() - 1
    seg = torch.repeat_interleave(torch.arange(m), ptr[1:] - ptr[:-1])[:, None].expand_as(rows)
    op = {"max": "amax", "min": "amin", "sum": "sum", "mean": "mean"}[reduce]
    return torch.zeros(m, src.shape[1], dtype=src.dtype).scatter_reduce(0, seg, rows, op, include_self=False)


def unpool_add(parent_feat, child_feat, cluster):
    """model.py:746."""
    parent_feat = torch.as_tensor(parent_feat, dtype=torch.float32)
    child_feat = torch.as_tensor(child_feat, dtype=torch.float32)
    return parent_feat + child_feat[torch.as_tensor(np.asarray(cluster), dtype=torch.int64)]
