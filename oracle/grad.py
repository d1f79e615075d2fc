"""Gradient oracle for the backward kernels (TEST INFRASTRUCTURE — only tests may import this).

The gradients are torch autograd's over the CPU restatements of oracle/functional.py, so they inherit
what pins those. Two things are checked on top, in tests/test_oracle_grad.py: central finite differences
of the restatements in float64 (which would catch a restatement that autograd cannot see through), and
the closed forms below against autograd.

Closed forms (what the HIP kernels implement):
  attention, per sequence and head, P = softmax(scale Q K^T), D_i = <dO_i, O_i>:
      dV = P^T dO,  dS = P o (dO V^T - D),  dQ = scale dS K,  dK = scale dS^T Q
      (the backward of flash_attn_varlen_qkvpacked_func at model.py:476-482; the gathers qkv[order] and
      feat[inverse] around it, model.py:455-484, become a scatter-add and a gather)
  submanifold convolution out[i] = sum_t W[:,t,:] x[nbr[i,t]] (model.py:546-552):
      dx[j] = sum_{i,t: nbr[i,t]=j} W[:,t,:]^T dout[i],   dW[:,t,:] = sum_i dout[i] x[nbr[i,t]]^T
  segment max (model.py:684-689): the gradient of a cluster goes to the member attaining the maximum
  unpooling add (model.py:746): dparent = dout, dchild[c] = sum_{i: cluster[i]=c} dout[i]
"""
import numpy as np
import torch

from . import functional as OF


def _leaf(a, dtype):
    return torch.as_tensor(np.asarray(a), dtype=dtype).clone().requires_grad_(True)


def serialized_attention_grad(feat_qkv, dout, order, inverse, pad, unpad, cu_seqlens, num_heads, scale=None):
    """d(sum(out * dout)) / d(feat_qkv) for oracle.functional.serialized_attention_core: (N, 3C)."""
    x = _leaf(feat_qkv, torch.float32)
    out = OF.serialized_attention_core(x, order, inverse, pad, unpad, cu_seqlens, num_heads, scale)
    out.backward(torch.as_tensor(np.asarray(dout), dtype=torch.float32))
    return x.grad


def patch_attention_grad_closed_form(qkv, dout, cu_seqlens, num_heads, scale=None):
    """The closed form above in float64 numpy for rows already in padded order: (Npad, 3C)."""
    qkv = np.asarray(qkv, dtype=np.float64)
    dout = np.asarray(dout, dtype=np.float64)
    npad, c3 = qkv.shape
    C = c3 // 3
    D = C // num_heads
    scale = D ** -0.5 if scale is None else scale
    grad = np.zeros_like(qkv)
    cu = [int(v) for v in cu_seqlens]
    for s, e in zip(cu[:-1], cu[1:]):
        for h in range(num_heads):
            sl = slice(h * D, (h + 1) * D)
            q, k, v = qkv[s:e, sl], qkv[s:e, C + h * D:C + (h + 1) * D], qkv[s:e, 2 * C + h * D:2 * C + (h + 1) * D]
            g = dout[s:e, sl]
            sc = scale * q @ k.T
            p = np.exp(sc - sc.max(1, keepdims=True))
            p /= p.sum(1, keepdims=True)
            o = p @ v
            ds = p * (g @ v.T - (g * o).sum(1, keepdims=True))
            grad[s:e, sl] = scale * ds @ k
            grad[s:e, C + h * D:C + (h + 1) * D] = scale * ds.T @ q
            grad[s:e, 2 * C + h * D:2 * C + (h + 1) * D] = p.T @ g
    return grad


def subm_conv_grad(feat, nbr, weight, bias, dout):
    """(dfeat, dweight, dbias) of oracle.functional.subm_conv; nbr (N, V) voxel-major."""
    x, w = _leaf(feat, torch.float32), _leaf(weight, torch.float32)
    b = None if bias is None else _leaf(bias, torch.float32)
    OF.subm_conv(x, nbr, w, b).backward(torch.as_tensor(np.asarray(dout), dtype=torch.float32))
    return x.grad, w.grad, None if b is None else b.grad


def subm_conv_grad_closed_form(feat, nbr, weight, dout):
    """The closed form above in float64 numpy: (dfeat, dweight (Cout, V, Cin))."""
    feat, dout = np.asarray(feat, np.float64), np.asarray(dout, np.float64)
    nbr = np.asarray(nbr)
    cout, cin = weight.shape[0], weight.shape[-1]
    w = np.asarray(weight, np.float64).reshape(cout, -1, cin)
    dfeat, dw = np.zeros_like(feat), np.zeros_like(w)
    for t in range(nbr.shape[1]):
        hit = np.nonzero(nbr[:, t] >= 0)[0]
        src = nbr[hit, t]
        np.add.at(dfeat, src, dout[hit] @ w[:, t, :])
        dw[:, t, :] = dout[hit].T @ feat[src]
    return dfeat, dw


def segment_csr_grad(src, indices, idx_ptr, reduce, dout):
    """dsrc of oracle.functional.segment_csr."""
    x = _leaf(src, torch.float32)
    OF.segment_csr(x, indices, idx_ptr, reduce).backward(torch.as_tensor(np.asarray(dout), dtype=torch.float32))
    return x.grad


def unpool_add_grad(dout, cluster, m):
    """(dparent, dchild) of oracle.functional.unpool_add for child of m rows."""
    dout = torch.as_tensor(np.asarray(dout), dtype=torch.float32)
    child = torch.zeros(m, dout.shape[1]).index_add_(0, torch.as_tensor(np.asarray(cluster), dtype=torch.int64), dout)
    return dout, child
