"""torch.autograd.Function wrappers of the sparse operators that have HIP backward kernels: patch
attention (the reference relies on flash_attn's backward, model.py:476-482), submanifold convolution
(spconv's, model.py:546-552, :767-774), segment reduction (torch_scatter's, model.py:684-689) and the
unpooling add (index_select's, model.py:746). Dense layers keep torch's own autograd."""
import torch

from . import ops


class PatchAttention(torch.autograd.Function):
    @staticmethod
    def forward(ctx, qkv, num_heads, slot_src, slot_dst, cu_seqlens, max_seqlen, scale, dropout_p=0.0, seed=0):
        args = (num_heads, slot_src, slot_dst, cu_seqlens, max_seqlen, scale)
        out, ctx.lse = ops.patch_attention_lse(qkv, *args, dropout_p=dropout_p, seed=seed)
        ctx.save_for_backward(qkv, out)
        ctx.args, ctx.dropout = args, (dropout_p, seed)
        return out

    @staticmethod
    def backward(ctx, dout):
        qkv, out = ctx.saved_tensors
        p, seed = ctx.dropout
        return (ops.patch_attention_bwd(qkv, out, dout, *ctx.args, lse=ctx.lse, dropout_p=p, seed=seed),) + (None,) * 8


class PatchAttentionRpe(torch.autograd.Function):
    """Patch attention with the relative position bias (fp32, model.py:297-316, :463-471); the table takes a
    gradient too."""

    @staticmethod
    def forward(ctx, qkv, rpe_table, num_heads, slot_src, slot_dst, cu_seqlens, max_seqlen, scale, grid_coord, pos_bnd,
                dropout_p=0.0, seed=0):
        args = (num_heads, slot_src, slot_dst, cu_seqlens, max_seqlen, scale, grid_coord)
        out = ops.patch_attention_rpe(qkv, *args, rpe_table.detach(), pos_bnd, dropout_p, seed)
        ctx.save_for_backward(qkv, out, rpe_table)
        ctx.args, ctx.pos_bnd, ctx.dropout = args, pos_bnd, (dropout_p, seed)
        return out

    @staticmethod
    def backward(ctx, dout):
        qkv, out, table = ctx.saved_tensors
        dqkv, dtable = ops.patch_attention_rpe_bwd(qkv, out, dout, *ctx.args, table, ctx.pos_bnd, *ctx.dropout)
        return (dqkv, dtable.to(table.dtype)) + (None,) * 10


class SubMConv(torch.autograd.Function):
    """module is the SubMConv3d whose forward dispatch (pair, tile or dense form) is reused for the
    input gradient; sparse is the SparseConvTensor that owns the neighbour maps."""

    @staticmethod
    def forward(ctx, feat, weight, bias, sparse, module):
        cout, cin = weight.shape[0], weight.shape[-1]
        w = ops.cast_cached(weight, feat.dtype).detach().reshape(cout, -1, cin)
        b = None if bias is None else ops.cast_cached(bias, feat.dtype).detach()
        out = module.convolve(sparse, feat.detach(), w, b)
        ctx.save_for_backward(feat, weight)
        ctx.sparse, ctx.module, ctx.has_bias = sparse, module, bias is not None
        ctx.bias_dtype = None if bias is None else bias.dtype
        return out

    @staticmethod
    def backward(ctx, dout):
        feat, weight = ctx.saved_tensors
        sparse, module = ctx.sparse, ctx.module
        cout, cin = weight.shape[0], weight.shape[-1]
        dout = dout.contiguous()
        dfeat = dweight = dbias = None
        if ctx.needs_input_grad[0]:
            # the same convolution with mirrored taps and the weight transposed
            wt = ops.cast_cached(weight, dout.dtype, "mirror")
            if dout.dtype != torch.float32 and cin % 16:   # the half-precision forms write outputs in 16s
                wt = torch.nn.functional.pad(wt, (0, 0, 0, 0, 0, -cin % 16))
            dfeat = module.convolve(sparse, dout, wt, None)[:, :cin].to(feat.dtype)
        if ctx.needs_input_grad[1]:
            x = feat.detach()
            if x.dtype != torch.float32 and cin % 8:
                x = torch.nn.functional.pad(x, (0, -cin % 8))   # the matrix-core kernel reads channels 8 at a time
            want_bias = ctx.has_bias and ctx.needs_input_grad[2]
            if x.dtype != torch.float32 and cout % 8 == 0 and min(x.shape[1], cout) < ops.OUTER_WIDE_CHANNELS:
                # the forward's pair lists: no neighbour map to build, no compaction, ranges of equal length
                # (half the time on the 64 x 64 block kernel; the 128 x 128 one measured 10 % slower that way:
                # it wants more and shorter work-groups than full ranges give it)
                dw, db = ops.subm_conv_wgrad_pairs(x, dout, sparse.conv_plan(module.kernel_size, module.indice_key),
                                                   with_bias=True)
            else:
                nbr = sparse.neighbour_map(module.kernel_size, module.indice_key)
                dw, db = ops.subm_conv_wgrad(x, dout, nbr, with_bias=True)
            dweight = dw[:, :, :cin].reshape(weight.shape).to(weight.dtype)
            if want_bias and db is not None:
                dbias = db.to(ctx.bias_dtype)
        if dbias is None and ctx.has_bias and ctx.needs_input_grad[2]:
            dbias = dout.sum(0, dtype=torch.float32).to(ctx.bias_dtype)
        return dfeat, dweight, dbias, None, None


class Linear(torch.autograd.Function):
    """x W^T + b for half-precision rows; weight and bias may be fp32 masters (autocast)."""

    @staticmethod
    def forward(ctx, x, weight, bias):
        w = ops.cast_cached(weight, x.dtype)
        b = None if bias is None else ops.cast_cached(bias, x.dtype)
        if ops.linear_rows_pays(x, w):
            out = ops.linear_rows(x, w, b)
        else:
            out = torch.nn.functional.linear(x, w, b)
        ctx.save_for_backward(x, weight)
        ctx.bias_dtype = None if bias is None else bias.dtype
        return out

    @staticmethod
    def backward(ctx, dout):
        x, weight = ctx.saved_tensors
        dout = dout.contiguous()
        dx = None
        if ctx.needs_input_grad[0]:
            wt = ops.cast_cached(weight, dout.dtype, "transpose")   # (K, Nout): dx = dout wt^T
            if ops.linear_rows_pays(dout, wt):
                dx = ops.linear_rows(dout, wt)   # many rows, few channels: the row kernel again
            else:
                dx = dout @ ops.cast_cached(weight, dout.dtype)
        want_bias = ctx.bias_dtype is not None and ctx.needs_input_grad[2]
        dw = db = None
        if ctx.needs_input_grad[1]:
            dw, db = ops.linear_wgrad(x, dout, with_bias=True)
            dw = dw.to(weight.dtype)
        if want_bias:
            db = db.to(ctx.bias_dtype) if db is not None else dout.sum(0, dtype=torch.float32).to(ctx.bias_dtype)
        return dx, dw, db if want_bias else None


class Mlp(torch.autograd.Function):
    """fc2(gelu(fc1 x)) (model.py:493-516 without dropout) for half-precision rows; weights and biases may be
    fp32 masters. The GELU's input and output are both kept, as autograd would keep them."""

    @staticmethod
    def forward(ctx, x, w1, b1, w2, b2):
        dt = x.dtype
        pre, act = ops.linear_gelu(x, ops.cast_cached(w1, dt), None if b1 is None else ops.cast_cached(b1, dt))
        cw2, cb2 = ops.cast_cached(w2, dt), None if b2 is None else ops.cast_cached(b2, dt)
        if ops.linear_rows_pays(act, cw2):
            out = ops.linear_rows(act, cw2, cb2)
        else:
            out = torch.nn.functional.linear(act, cw2, cb2)
        ctx.save_for_backward(x, pre, act, w1, w2)
        ctx.bias_dtypes = tuple(None if b is None else b.dtype for b in (b1, b2))
        return out

    @staticmethod
    def backward(ctx, dout):
        x, pre, act, w1, w2 = ctx.saved_tensors
        dout = dout.contiguous()
        dt = dout.dtype
        dpre = ops.linear_gelu_bwd(dout, ops.cast_cached(w2, dt, "transpose"), pre)
        dx = None
        if ctx.needs_input_grad[0]:
            w1t = ops.cast_cached(w1, dt, "transpose")   # (in, hidden): dx = dpre w1t^T
            dx = ops.linear_rows(dpre, w1t) if ops.linear_rows_pays(dpre, w1t) else dpre @ ops.cast_cached(w1, dt)
        grads = []
        for inp, dy, w, bias_dtype, wi in ((x, dpre, w1, ctx.bias_dtypes[0], 1), (act, dout, w2, ctx.bias_dtypes[1], 3)):
            dw = db = None
            if ctx.needs_input_grad[wi]:
                dw, db = ops.linear_wgrad(inp, dy, with_bias=True)
                dw = dw.to(w.dtype)
            if bias_dtype is not None and ctx.needs_input_grad[wi + 1]:
                db = db.to(bias_dtype) if db is not None else dy.sum(0, dtype=torch.float32).to(bias_dtype)
            else:
                db = None
            grads += [dw, db]
        return (dx, *grads)


class LayerNorm(torch.autograd.Function):
    """Row-wise LayerNorm, statistics in fp32, result in out_dtype (x's when None: autocast asks for float
    where the result joins the residual stream, half precision where only a Linear reads it). Mean and rstd
    are not kept: the backward kernel recomputes them from x."""

    @staticmethod
    def forward(ctx, x, weight, bias, eps, out_dtype=None):
        ctx.save_for_backward(x, weight)
        ctx.eps, ctx.bias_dtype = eps, bias.dtype
        return ops.add_layer_norm(None, x, None, weight.detach(), bias.detach(), eps, out_dtype=out_dtype)[1]

    @staticmethod
    def backward(ctx, dout):
        x, weight = ctx.saved_tensors
        _, dx, dw, db = ops.add_layer_norm_bwd(x, dout, None, None, weight.detach(), ctx.eps, branch_dtype=x.dtype)
        return dx, dw.to(weight.dtype), db.to(ctx.bias_dtype), None, None


class AddLayerNorm(torch.autograd.Function):
    """s = skip + branch * mask, y = LayerNorm(s): a residual connection followed by the next pre-norm
    (model.py:589-604; mask is the stochastic-depth factor per row, or None), one kernel each way. Returns
    (s, y), y in out_dtype; the backward kernel adds the gradient arriving at s to the LayerNorm's own, so
    autograd has nothing to accumulate, and writes each input's gradient in that input's dtype.
    With pre_weight, pre_bias, pre_eps the branch first goes through a LayerNorm of its own in the same pass
    (s = skip + LayerNorm_pre(branch) * mask: the xCPE's norm, model.py:546-554); sum_dtype then says what that
    norm's result would have been added in (float under autocast, which runs layer_norm in float)."""

    @staticmethod
    def forward(ctx, skip, branch, mask, weight, bias, eps, out_dtype=None, pre_weight=None, pre_bias=None, pre_eps=0.0,
                sum_dtype=None):
        pre = None if pre_weight is None else (pre_weight.detach(), pre_bias.detach(), pre_eps)
        s, y = ops.add_layer_norm(skip, branch, mask, weight.detach(), bias.detach(), eps, sum_dtype=sum_dtype,
                                  out_dtype=out_dtype, pre=pre)
        ctx.save_for_backward(s, weight, mask, *(() if pre is None else (branch, pre_weight)))
        ctx.eps, ctx.pre_eps, ctx.dtypes = eps, pre_eps, (skip.dtype, branch.dtype, bias.dtype)
        ctx.pre_bias_dtype = None if pre is None else pre_bias.dtype
        return s, y

    @staticmethod
    def backward(ctx, ds, dy):
        s, weight, mask, *rest = ctx.saved_tensors
        skip_dtype, branch_dtype, bias_dtype = ctx.dtypes
        pre = (rest[0], rest[1].detach(), ctx.pre_eps) if rest else None
        out = ops.add_layer_norm_bwd(s, dy, ds, mask, weight.detach(), ctx.eps,
                                     skip_dtype=skip_dtype if ctx.needs_input_grad[0] else None,
                                     branch_dtype=branch_dtype if ctx.needs_input_grad[1] else None, pre=pre)
        dskip, dbranch, dw, db = out[:4]
        dpw = dpb = None
        if pre is not None:
            dpw, dpb = out[4].to(rest[1].dtype), out[5].to(ctx.pre_bias_dtype)
        return dskip, dbranch, None, dw.to(weight.dtype), db.to(bias_dtype), None, None, dpw, dpb, None, None


class SplitCast(torch.autograd.Function):
    """(x, x in half precision) for a float x with two readers, one of which reads halves (the residual stream at
    the head of a Block: the skip connection and the xCPE convolution under autocast, model.py:589-592). Going
    back, the float and the half-precision gradient are added by one kernel instead of a conversion followed
    by autograd's accumulation."""

    @staticmethod
    def forward(ctx, x, dtype):
        return x.view_as(x), x.to(dtype)

    @staticmethod
    def backward(ctx, dx, dhalf):
        if dx is None or dhalf is None:
            return (dx if dhalf is None else dhalf.to(torch.float32)), None
        return ops.scaled_add(dx, dhalf, None, dx.dtype), None


class ResidualAdd(torch.autograd.Function):
    """skip + branch * mask (model.py:602-604 with the stochastic-depth factor per row) in skip's dtype, the
    branch read in its own; going back skip's gradient is the incoming one as it is and the branch's one
    kernel, instead of autocast's conversions around an addcmul."""

    @staticmethod
    def forward(ctx, skip, branch, mask):
        ctx.save_for_backward(mask)
        ctx.branch_dtype = branch.dtype
        return ops.scaled_add(skip, branch, mask, skip.dtype)

    @staticmethod
    def backward(ctx, dout):
        (mask,) = ctx.saved_tensors
        dbranch = ops.scaled_add(None, dout, mask, ctx.branch_dtype) if ctx.needs_input_grad[1] else None
        return (dout if ctx.needs_input_grad[0] else None), dbranch, None


class BatchNormAct(torch.autograd.Function):
    """nn.BatchNorm1d (batch statistics and running-average update in training mode, the running statistics
    otherwise), optionally followed by exact GELU (model.py:776-779, :707-710, :729-735), as one node: the
    pre-activation is not kept, the backward kernels recompute it from x."""

    @staticmethod
    def forward(ctx, x, weight, bias, bn, gelu):
        batch = bn.training or bn.running_mean is None
        if batch:
            track = bn.track_running_stats and bn.running_mean is not None and bn.running_mean.dtype == torch.float32
            momentum = bn.momentum
            if track and bn.num_batches_tracked is not None:
                bn.num_batches_tracked += 1
                if momentum is None:
                    momentum = 1.0 / float(bn.num_batches_tracked)
            stats = ops.batch_norm_stats(x, bn.eps, momentum or 0.0, bn.running_mean if track else None,
                                         bn.running_var if track else None)
            mean, var = stats[0], stats[2]
        else:
            mean, var = bn.running_mean.float(), bn.running_var.float()
            stats = torch.stack([mean, torch.rsqrt(var + bn.eps)])
        out = ops.bn_act(x, mean, var, None if weight is None else weight.detach(),
                         None if bias is None else bias.detach(), bn.eps, gelu)
        ctx.save_for_backward(x, weight, bias, stats)
        ctx.gelu, ctx.batch = gelu, batch
        return out

    @staticmethod
    def backward(ctx, dout):
        x, weight, bias, stats = ctx.saved_tensors
        dx, dw, db = ops.batch_norm_bwd(x, dout, stats, None if weight is None else weight.detach(),
                                        None if bias is None else bias.detach(), ctx.gelu, ctx.batch)
        return (dx, None if weight is None else dw.to(weight.dtype), None if bias is None else db.to(bias.dtype),
                None, None)


class SegmentReduce(torch.autograd.Function):
    @staticmethod
    def forward(ctx, src, indices, idx_ptr, reduce):
        out = ops.segment_reduce(src, indices, idx_ptr, reduce)
        ctx.save_for_backward(src, out)
        ctx.args = (indices, idx_ptr, reduce)
        return out

    @staticmethod
    def backward(ctx, dout):
        src, out = ctx.saved_tensors
        return ops.segment_reduce_bwd(src, out, dout, *ctx.args), None, None, None


class UnpoolAdd(torch.autograd.Function):
    """parent + child[cluster]; indices / idx_ptr are the pooling's member lists of the clusters, over which
    the gradient of child is a segment sum (no atomics)."""

    @staticmethod
    def forward(ctx, parent, child, cluster, indices, idx_ptr):
        ctx.args = (indices, idx_ptr)
        ctx.child_dtype = child.dtype
        return ops.unpool_add(parent, child, cluster)

    @staticmethod
    def backward(ctx, dout):
        dout = dout.contiguous()
        dchild = ops.segment_reduce(dout, *ctx.args, "sum").to(ctx.child_dtype) if ctx.needs_input_grad[1] else None
        return dout, dchild, None, None, None
