"""The building blocks of PTv3 as thin host glue over the HIP kernels.

Module and parameter names follow model.py:177-783 of the reference, so its state_dicts load
unchanged. Dense layers (Linear / LayerNorm / BatchNorm / GELU) are torch's; serialization,
attention, sparse convolution and pooling run in libptv3_hip.so.
"""
import math
from collections import OrderedDict

import torch
import torch.nn as nn

from . import ops
from ._lib import Ptv3Error
from .autograd import (AddLayerNorm, BatchNormAct, LayerNorm as LayerNormFn, ResidualAdd, SegmentReduce, SplitCast,
                       UnpoolAdd)
from .point import AttrDict, Point, offset2bincount
from .sparse import SparseConvTensor, SubMConv3d, is_spconv_module


class DropPath(nn.Module):
    """Stochastic depth per sample row (stands in for timm's DropPath, model.py:17,583)."""

    def __init__(self, drop_prob=0.0, scale_by_keep=True):
        super().__init__()
        self.drop_prob, self.scale_by_keep = drop_prob, scale_by_keep

    def mask(self, x):
        """The per-row factor (0 or 1 / keep) forward multiplies x by, or None when it is the identity."""
        if self.drop_prob == 0.0 or not self.training:
            return None
        keep = 1.0 - self.drop_prob
        mask = x.new_empty((x.shape[0],) + (1,) * (x.ndim - 1)).bernoulli_(keep)
        if keep > 0.0 and self.scale_by_keep:
            mask.div_(keep)
        return mask

    def forward(self, x):
        mask = self.mask(x)
        return x if mask is None else x * mask


class LayerNorm(nn.LayerNorm):
    """nn.LayerNorm (same parameters and state_dict) evaluated by the row-wise HIP kernel."""

    def forward(self, x):
        if x.dim() != 2 or len(self.normalized_shape) != 1 or self.weight is None or self.bias is None:
            return super().forward(x)
        if ops.wants_grad(x, self.weight, self.bias):
            if x.is_cuda and x.shape[1] in ops.LAYER_NORM_BWD_CHANNELS:
                # autocast runs layer_norm in float and hands out a float result
                out_dtype = torch.float32 if torch.is_autocast_enabled() else None
                return LayerNormFn.apply(x, self.weight, self.bias, self.eps, out_dtype)
            return super().forward(x)
        return ops.layer_norm(x, self.weight, self.bias, self.eps)


def _fusable_bn(module, feat):
    """Inference-mode BatchNorm1d over (N, C) GPU features that the one-pass kernel covers."""
    return (type(module) is nn.BatchNorm1d and not module.training and module.track_running_stats
            and module.running_mean is not None and feat.is_cuda and feat.dim() == 2 and feat.shape[1] % 8 == 0
            and not ops.wants_grad(feat, module.weight, module.bias))


def _trainable_bn(module, feat):
    """BatchNorm1d over (N, C) GPU features under autograd that the training kernels cover."""
    return (type(module) is nn.BatchNorm1d and feat.is_cuda and feat.dim() == 2
            and feat.shape[1] in ops.BATCH_NORM_TRAIN_CHANNELS and feat.shape[0] > 1
            and (module.running_mean is None or module.running_mean.dtype == torch.float32)
            and (module.weight is None) == (module.bias is None)
            and ops.wants_grad(feat, module.weight, module.bias))


def _exact_gelu(module):
    return type(module) is nn.GELU and module.approximate == "none"


class PointModule(nn.Module):
    """Marker base class: PointSequential hands the whole Point to subclasses (model.py:177-183)."""


class PointSequential(PointModule):
    """Sequential container that knows three kinds of children (model.py:186-252):
    PointModules get the Point, sparse convolutions get point.sparse_conv_feat, anything
    else gets point.feat."""

    def __init__(self, *args, **kwargs):
        super().__init__()
        if len(args) == 1 and isinstance(args[0], OrderedDict):
            for name, module in args[0].items():
                self.add_module(name, module)
        else:
            for i, module in enumerate(args):
                self.add_module(str(i), module)
        for name, module in kwargs.items():
            if name in self._modules:
                raise ValueError("name exists.")
            self.add_module(name, module)

    def __getitem__(self, idx):
        if not (-len(self) <= idx < len(self)):
            raise IndexError("index {} is out of range".format(idx))
        return list(self._modules.values())[idx]

    def __len__(self):
        return len(self._modules)

    def add(self, module, name=None):
        if name is None:
            name = str(len(self._modules))
            if name in self._modules:
                raise KeyError("name exists")
        self.add_module(name, module)

    def forward(self, input):
        modules = list(self._modules.values())
        skip = 0
        for i, module in enumerate(modules):
            if skip:   # already applied together with the module(s) before it
                skip -= 1
                continue
            nxt = modules[i + 1] if i + 1 < len(modules) else None
            if (isinstance(input, Point) and type(module) is nn.Linear and ops.linear_rows_pays(input.feat, module.weight)
                    and _fusable_bn(nxt, input.feat)):
                # Linear -> BatchNorm1d (-> GELU), the projections of the unpooling stages, in one kernel
                with_act = _exact_gelu(modules[i + 2] if i + 2 < len(modules) else None)
                input.feat = ops.linear_bn_act(input.feat, module, nxt, with_act)
                if "sparse_conv_feat" in input:
                    input.sparse_conv_feat = input.sparse_conv_feat.replace_feature(input.feat)
                skip = 2 if with_act else 1
                continue
            if isinstance(input, Point) and _trainable_bn(module, input.feat):
                # training: batch statistics, the GELU behind it and their backward as one autograd node
                with_act = _exact_gelu(nxt)
                input.feat = BatchNormAct.apply(input.feat, module.weight, module.bias, module, with_act)
                if "sparse_conv_feat" in input:
                    input.sparse_conv_feat = input.sparse_conv_feat.replace_feature(input.feat)
                skip = int(with_act)
                continue
            if isinstance(input, Point) and _fusable_bn(module, input.feat):
                with_act = _exact_gelu(nxt)
                input.feat = ops.bn_act(input.feat, module.running_mean, module.running_var, module.weight,
                                        module.bias, module.eps, with_act)
                if "sparse_conv_feat" in input:
                    input.sparse_conv_feat = input.sparse_conv_feat.replace_feature(input.feat)
                skip = int(with_act)
                continue
            if isinstance(module, PointModule):
                input = module(input)
            elif is_spconv_module(module):
                if isinstance(input, Point):
                    input.sparse_conv_feat = module(input.sparse_conv_feat)
                    input.feat = input.sparse_conv_feat.features
                else:
                    input = module(input)
            elif isinstance(input, Point):
                input.feat = ops.linear(input.feat, module) if type(module) is nn.Linear else module(input.feat)
                if "sparse_conv_feat" in input:
                    input.sparse_conv_feat = input.sparse_conv_feat.replace_feature(input.feat)
            elif isinstance(input, SparseConvTensor):
                if input.indices.shape[0] != 0:
                    input = input.replace_feature(module(input.features))
            else:
                input = module(input)
        return input


class PDNorm(PointModule):
    """Per-dataset (de)coupled normalisation of PPT training (model.py:255-294); plain torch."""

    def __init__(self, num_features, norm_layer, context_channels=256,
                 conditions=("ScanNet", "S3DIS", "Structured3D"), decouple=True, adaptive=False):
        super().__init__()
        self.conditions, self.decouple, self.adaptive = conditions, decouple, adaptive
        if decouple:
            self.norm = nn.ModuleList([norm_layer(num_features) for _ in conditions])
        else:
            self.norm = norm_layer
        if adaptive:
            self.modulation = nn.Sequential(nn.SiLU(), nn.Linear(context_channels, 2 * num_features, bias=True))

    def forward(self, point):
        assert {"feat", "condition"}.issubset(point.keys())
        condition = point.condition if isinstance(point.condition, str) else point.condition[0]
        if self.decouple:
            assert condition in self.conditions
            norm = self.norm[self.conditions.index(condition)]
        else:
            norm = self.norm
        point.feat = norm(point.feat)
        if self.adaptive:
            assert "context" in point.keys()
            shift, scale = self.modulation(point.context).chunk(2, dim=1)
            point.feat = point.feat * (1.0 + scale) + shift
        return point


class RPE(nn.Module):
    """Relative position bias table (model.py:297-316): one learned value per axis, clamped grid
    offset and head. The attention kernel reads the table directly; forward() is the reference's
    dense (N, H, K, K) bias for callers that want it."""

    def __init__(self, patch_size, num_heads):
        super().__init__()
        self.patch_size, self.num_heads = patch_size, num_heads
        self.pos_bnd = int((4 * patch_size) ** (1 / 3) * 2)
        self.rpe_num = 2 * self.pos_bnd + 1
        self.rpe_table = nn.Parameter(torch.zeros(3 * self.rpe_num, num_heads))
        nn.init.trunc_normal_(self.rpe_table, std=0.02)

    def forward(self, coord):
        idx = (coord.clamp(-self.pos_bnd, self.pos_bnd) + self.pos_bnd
               + torch.arange(3, device=coord.device) * self.rpe_num)
        out = self.rpe_table.index_select(0, idx.reshape(-1))
        return out.view(idx.shape + (-1,)).sum(3).permute(0, 3, 1, 2)


class SerializedAttention(PointModule):
    """Attention inside patches of the serialized point sequence (model.py:319-490).

    The qkv projection and the output projection are torch Linears; everything between them —
    gathering rows into padded serialized order, softmax(q k^T) v per patch and head,
    scattering rows back — is one HIP kernel launch reading through int32 slot tables that
    are built once per (Point, order) and cached on the Point."""

    def __init__(self, channels, num_heads, patch_size, qkv_bias=True, qk_scale=None, attn_drop=0.0,
                 proj_drop=0.0, order_index=0, enable_rpe=False, enable_flash=True,
                 upcast_attention=True, upcast_softmax=True):
        super().__init__()
        assert channels % num_heads == 0
        self.channels, self.num_heads = channels, num_heads
        self.scale = qk_scale or (channels // num_heads) ** -0.5
        self.order_index = order_index
        self.upcast_attention, self.upcast_softmax = upcast_attention, upcast_softmax
        self.enable_rpe, self.enable_flash = enable_rpe, enable_flash
        if enable_flash:
            assert enable_rpe is False, "Set enable_rpe to False when enable Flash Attention"
            assert upcast_attention is False, "Set upcast_attention to False when enable Flash Attention"
            assert upcast_softmax is False, "Set upcast_softmax to False when enable Flash Attention"
            self.patch_size = patch_size
        else:
            # without the fused path the reference shrinks the patch to the smallest scene so
            # that no padding is ever needed (model.py:359-363, :441-444)
            self.patch_size_max = patch_size
            self.patch_size = 0
        assert 0.0 <= attn_drop < 1.0
        self.attn_drop = attn_drop   # applied inside the attention kernels in training mode (model.py:470, :480)
        self.qkv = nn.Linear(channels, channels * 3, bias=qkv_bias)
        self.proj = nn.Linear(channels, channels)
        self.proj_drop = nn.Dropout(proj_drop)
        self.rpe = RPE(patch_size, num_heads) if enable_rpe else None

    @torch.no_grad()
    def get_padding_and_inverse(self, point):
        """pad / unpad / cu_seqlens, cached on the Point under the reference's keys
        (model.py:382-438)."""
        if not {"pad", "unpad", "cu_seqlens_key"}.issubset(point.keys()):
            pad, unpad, cu = ops.pad_index(point.offset, point.offset_host(), self.patch_size)
            point["pad"], point["unpad"], point["cu_seqlens_key"] = pad, unpad, cu
            point["_pad_patch"] = self.patch_size
        return point["pad"], point["unpad"], point["cu_seqlens_key"]

    def _cached_patch(self, point):
        """Longest sequence of the padding tables cached on the Point. The first attention layer that
        reaches a Point makes them and every later one reuses them under the same keys (model.py:384-391),
        so the decoder blocks of a stage attend over the patches its encoder blocks defined. The kernels size
        their staging from this value, never from the layer's own patch size."""
        built_for = point.get("_pad_patch")
        if built_for is None:   # tables put on the Point by the caller: measure them
            cu = point["cu_seqlens_key"]
            built_for = int((cu[1:] - cu[:-1]).max()) if cu.numel() > 1 else 0
            point["_pad_patch"] = built_for
        if self.enable_flash and built_for > self.patch_size:
            # the reference would hand flash_attn sequences longer than its max_seqlen (model.py:479)
            raise Ptv3Error(f"the padding tables cached on this Point hold patches of {built_for} points, more than "
                            f"this layer's patch_size {self.patch_size}: undefined in the reference; use patch "
                            f"sizes that do not shrink from the encoder to the decoder of a stage")
        if not self.enable_flash and built_for != self.patch_size:
            # model.py:461 would reshape rows padded for one patch size into patches of another
            raise Ptv3Error(f"the padding tables cached on this Point were made for patches of {built_for} points, "
                            f"this layer wants {self.patch_size}: not supported without the fused path")
        return built_for

    @torch.no_grad()
    def _slots(self, point):
        key = f"_attn_slots_{self.order_index}"
        if key not in point:
            pad, unpad, _ = self.get_padding_and_inverse(point)
            point[key] = ops.attn_slots(point.serialized_order[self.order_index],
                                        point.serialized_inverse[self.order_index], pad, unpad)
        return point[key]

    def attend(self, point, qkv):
        """softmax(q k^T * scale) v inside the patches of this layer's order, for packed
        qkv (N, 3C) in point order; returns (N, C) in point order (model.py:452-484)."""
        if not self.enable_flash:
            sizes = offset2bincount(torch.as_tensor(point.offset_host()))
            self.patch_size = min(int(sizes.min()), self.patch_size_max)
        _, _, cu_seqlens = self.get_padding_and_inverse(point)
        max_seqlen = self._cached_patch(point)
        slot_src, slot_dst = self._slots(point)
        grad = ops.wants_grad(qkv, self.rpe.rpe_table if self.enable_rpe else None)
        drop_p = self.attn_drop if self.training else 0.0
        if drop_p > 0.0:
            from .autograd import PatchAttention, PatchAttentionRpe
            seed = int(torch.randint(0, 2 ** 31 - 1, (1,)).item())   # torch's CPU generator: follows torch.manual_seed
            if self.enable_rpe:
                out = PatchAttentionRpe.apply(qkv.float(), self.rpe.rpe_table, self.num_heads, slot_src, slot_dst,
                                              cu_seqlens, max_seqlen, self.scale, point.grid_coord,
                                              self.rpe.pos_bnd, drop_p, seed)
                return out.to(qkv.dtype)
            half = qkv.half() if (self.enable_flash and qkv.dtype == torch.float32) else qkv
            return PatchAttention.apply(half, self.num_heads, slot_src, slot_dst, cu_seqlens, max_seqlen,
                                        self.scale, drop_p, seed).to(qkv.dtype)
        if grad and self.enable_rpe:
            from .autograd import PatchAttentionRpe
            out = PatchAttentionRpe.apply(qkv.float(), self.rpe.rpe_table, self.num_heads, slot_src, slot_dst, cu_seqlens,
                                          max_seqlen, self.scale, point.grid_coord, self.rpe.pos_bnd)
            return out.to(qkv.dtype)
        if grad:
            from .autograd import PatchAttention
            half = qkv.half() if (self.enable_flash and qkv.dtype == torch.float32) else qkv
            return PatchAttention.apply(half, self.num_heads, slot_src, slot_dst, cu_seqlens, max_seqlen,
                                        self.scale).to(qkv.dtype)
        if self.enable_rpe:
            # bias from the grid offsets of (query, key) inside the patch, added before the softmax; the
            # reference takes this path in float (upcast_attention / upcast_softmax, model.py:463-471)
            out = ops.patch_attention_rpe(qkv.float(), self.num_heads, slot_src, slot_dst, cu_seqlens, max_seqlen,
                                          self.scale, point.grid_coord, self.rpe.rpe_table, self.rpe.pos_bnd)
            return out.to(qkv.dtype)
        if self.enable_flash and qkv.dtype == torch.float32:
            # the fused path of the reference always computes in half precision (model.py:477,483)
            return ops.patch_attention(qkv.half(), self.num_heads, slot_src, slot_dst, cu_seqlens,
                                       max_seqlen, self.scale).to(qkv.dtype)
        return ops.patch_attention(qkv, self.num_heads, slot_src, slot_dst, cu_seqlens,
                                   max_seqlen, self.scale)

    def forward(self, point):
        feat = self.attend(point, ops.linear(point.feat, self.qkv))
        feat = ops.linear(feat, self.proj)
        feat = self.proj_drop(feat)
        point.feat = feat
        return point


class MLP(nn.Module):
    """fc1 -> act -> drop -> fc2 -> drop (model.py:493-516)."""

    def __init__(self, in_channels, hidden_channels=None, out_channels=None, act_layer=nn.GELU, drop=0.0):
        super().__init__()
        out_channels = out_channels or in_channels
        hidden_channels = hidden_channels or in_channels
        self.fc1 = nn.Linear(in_channels, hidden_channels)
        self.act = act_layer()
        self.fc2 = nn.Linear(hidden_channels, out_channels)
        self.drop = nn.Dropout(drop)

    def forward(self, x):
        if (ops.wants_grad(x, *self.parameters()) and type(self.act) is nn.GELU and self.act.approximate == "none"
                and not (self.training and self.drop.p > 0)):
            y = ops.mlp(x, self.fc1, self.fc2)
            if y is not None:
                return y
        return self.drop(ops.linear(self.drop(self.act(ops.linear(x, self.fc1))), self.fc2))


class Block(PointModule):
    """xCPE conv + attention + MLP, each with a residual (model.py:519-606)."""

    def __init__(self, channels, num_heads, patch_size=48, mlp_ratio=4.0, qkv_bias=True, qk_scale=None,
                 attn_drop=0.0, proj_drop=0.0, drop_path=0.0, norm_layer=LayerNorm, act_layer=nn.GELU,
                 pre_norm=True, order_index=0, cpe_indice_key=None, enable_rpe=False, enable_flash=True,
                 upcast_attention=True, upcast_softmax=True):
        super().__init__()
        self.channels, self.pre_norm = channels, pre_norm
        self.cpe = PointSequential(
            SubMConv3d(channels, channels, kernel_size=3, bias=True, indice_key=cpe_indice_key),
            nn.Linear(channels, channels),
            norm_layer(channels),
        )
        self.norm1 = PointSequential(norm_layer(channels))
        self.attn = SerializedAttention(
            channels=channels, patch_size=patch_size, num_heads=num_heads, qkv_bias=qkv_bias,
            qk_scale=qk_scale, attn_drop=attn_drop, proj_drop=proj_drop, order_index=order_index,
            enable_rpe=enable_rpe, enable_flash=enable_flash, upcast_attention=upcast_attention,
            upcast_softmax=upcast_softmax)
        self.norm2 = PointSequential(norm_layer(channels))
        self.mlp = PointSequential(MLP(in_channels=channels, hidden_channels=int(channels * mlp_ratio),
                                       out_channels=channels, act_layer=act_layer, drop=proj_drop))
        self.drop_path = PointSequential(DropPath(drop_path) if drop_path > 0.0 else nn.Identity())

    def _plain_layernorms(self):
        """True when the three norms are affine LayerNorms this file can fuse with the residual
        adds around them (the default model); PDNorm or post-norm blocks take the modular path."""
        mods = (self.cpe[2], self.norm1[0], self.norm2[0])
        return (self.pre_norm and all(type(m) is LayerNorm and m.weight is not None for m in mods)
                and not (self.training and not isinstance(self.drop_path[0], nn.Identity)))

    def forward(self, point):
        if not self._plain_layernorms() or (torch.is_grad_enabled() and ops.wants_grad(point.feat, *self.parameters())):
            return self._forward_modular(point)   # module by module: every one of them has a backward
        ln_cpe, ln1, ln2 = self.cpe[2], self.norm1[0], self.norm2[0]
        mlp = self.mlp[0]
        plain_mlp = (type(mlp) is MLP and mlp.fc1.bias is not None and mlp.fc2.bias is not None
                     and not (self.training and mlp.drop.p > 0))
        exact_gelu = type(mlp.act) is nn.GELU and mlp.act.approximate == "none" if plain_mlp else False
        fusable = (plain_mlp and exact_gelu and mlp.fc1.out_features == 4 * self.channels
                   and point.feat.dtype != torch.float32)
        fused = fusable and self.channels in ops.MLP_FUSED_CHANNELS            # whole block head and tail
        fused_mlp = fusable and self.channels in ops.MLP_ONLY_FUSED_PAYS          # the MLP alone
        # xCPE: conv reads the sparse view, which lags behind feat in the first decoder block
        conv = self.cpe[0](point.sparse_conv_feat).features
        if fused and type(self.cpe[1]) is nn.Linear and not (self.training and self.attn.proj_drop.p > 0):
            # thin channels, many points: every dense layer is bound by its N x C tensors going to
            # HBM and back, so the block runs as conv, head kernel, attention, tail kernel
            feat, qkv = ops.block_head_fused(conv, point.feat, self.cpe[1], ln_cpe, ln1, self.attn.qkv)
            attn = self.attn.attend(point, qkv)
            feat = ops.block_tail_fused(attn, feat, self.attn.proj, ln2, mlp.fc1, mlp.fc2)
            point.feat = feat
            point.sparse_conv_feat = point.sparse_conv_feat.replace_feature(feat)
            return point
        same_eps = ln_cpe.eps == ln1.eps
        qkv = None
        if (fused_mlp and self.channels in ops.BLOCK_HEAD_WIDE_PAYS and type(self.cpe[1]) is nn.Linear
                and self.cpe[1].bias is not None and type(self.attn.qkv) is nn.Linear and self.attn.qkv.bias is not None
                and self.attn.enable_flash):
            # cpe Linear, its LayerNorm, the residual, the attention's pre-norm and qkv in one kernel
            feat, qkv = ops.block_head_wide(conv, point.feat, self.cpe[1], ln_cpe, ln1, self.attn.qkv)
        elif ops.linear_ln_ok(conv, self.cpe[1]) and same_eps:
            # cpe Linear, its LayerNorm, the residual and the attention's pre-norm in one kernel
            feat, normed = ops.linear_ln(conv, self.cpe[1], point.feat, ln_cpe, 3, ln2=ln1)
        else:
            branch = ops.linear(conv, self.cpe[1]) if type(self.cpe[1]) is nn.Linear else self.cpe[1](conv)
            # feat = shortcut + LN(branch) and its pre-norm for attention, in one pass
            feat, normed = ops.layer_norm(branch, ln_cpe.weight, ln_cpe.bias, ln_cpe.eps, residual=point.feat,
                                          mode=3, weight2=ln1.weight, bias2=ln1.bias)
        # feat += attention branch, plus the pre-norm for the MLP.
        # When fc2 runs as a separate GEMM it accumulates onto the stored sum (beta = 1), so its
        # bias is added to that sum here: feat + fc2(h) + b2 without a separate add pass
        shift = mlp.fc2.bias if (plain_mlp and not fused_mlp) else None
        if qkv is None:
            point.feat = normed
            qkv = ops.linear(normed, self.attn.qkv)
        attn_out = self.attn.attend(point, qkv)
        if (fused_mlp and self.channels in ops.BLOCK_TAIL_WIDE_CHANNELS and type(self.attn.proj) is nn.Linear
                and self.attn.proj.bias is not None and not (self.training and self.attn.proj_drop.p > 0)):
            # proj, the residual, the MLP's pre-norm and the MLP with its residual in one kernel
            feat = ops.block_tail_wide(attn_out, feat, self.attn.proj, ln2, mlp)
            point.feat = feat
            point.sparse_conv_feat = point.sparse_conv_feat.replace_feature(feat)
            return point
        if ops.linear_ln_ok(attn_out, self.attn.proj) and not (self.training and self.attn.proj_drop.p > 0):
            # proj, the residual and the MLP's pre-norm in one kernel
            feat, normed = ops.linear_ln(attn_out, self.attn.proj, feat, ln2, 2, shift=shift)
        else:
            branch = self.attn.proj_drop(ops.linear(attn_out, self.attn.proj))
            feat, normed = ops.layer_norm(branch, ln2.weight, ln2.bias, ln2.eps, residual=feat, mode=2, shift=shift)
        if fused_mlp:
            # fc1 + GELU + fc2 + residual in one kernel, the 4C-wide hidden tensor never leaves the CU
            feat = ops.mlp_fused_module(normed, feat, mlp)
        elif plain_mlp:
            hidden = ops.linear(normed, mlp.fc1, gelu=True) if exact_gelu else mlp.act(mlp.fc1(normed))
            feat = feat.contiguous()
            if ops.linear_gemm_ok(hidden, mlp.fc2.weight) and feat.dtype == hidden.dtype:
                feat = ops.linear_gemm(hidden, mlp.fc2.weight, None, resid=feat)   # onto the stored sum, in place
            else:
                feat = ops.linear_any(hidden, mlp.fc2.weight, None, resid=feat.to(hidden.dtype))
        else:
            feat = feat + mlp(normed)
        point.feat = feat
        point.sparse_conv_feat = point.sparse_conv_feat.replace_feature(feat)
        return point

    def _forward_training(self, point):
        """Pre-norm block with plain LayerNorms under autograd: as _forward_modular, with each residual add
        (and its stochastic-depth factor) taken together with the LayerNorm that follows it."""
        ln1, ln2 = self.norm1[0], self.norm2[0]
        drop = self.drop_path[0]
        path_mask = drop.mask if isinstance(drop, DropPath) else (lambda x: None)
        # under autocast the normalised rows are only ever read by a Linear, which would cast them to half
        # precision first: the kernel writes them in that dtype (the same single rounding), the sums stay float
        normed_dtype = torch.get_autocast_dtype("cuda") if torch.is_autocast_enabled() else None
        skip = point.feat
        conv, lin, ln_cpe = self.cpe[0], self.cpe[1], self.cpe[2]
        if (type(lin) is nn.Linear and type(ln_cpe) is LayerNorm and ln_cpe.weight is not None
                and ln_cpe.bias is not None and "sparse_conv_feat" in point):
            # the xCPE's own norm rides on the kernel of the residual add and norm1 behind it
            sparse = point.sparse_conv_feat
            if (normed_dtype is not None and skip.dtype == torch.float32 and skip.requires_grad
                    and self.channels % 8 == 0 and sparse.features is skip):
                skip, half = SplitCast.apply(skip, normed_dtype)   # one kernel adds the two gradients going back
                sparse = sparse.replace_feature(half)
            branch = ops.linear(conv(sparse).features, lin)
            # autocast's layer_norm hands out float, so the sum (the residual stream from here on) is float
            feat, point.feat = AddLayerNorm.apply(skip, branch, None, ln1.weight, ln1.bias, ln1.eps, normed_dtype,
                                                  ln_cpe.weight, ln_cpe.bias, ln_cpe.eps,
                                                  torch.float32 if normed_dtype is not None else None)
        else:
            point = self.cpe(point)
            feat, point.feat = AddLayerNorm.apply(skip, point.feat, None, ln1.weight, ln1.bias, ln1.eps, normed_dtype)
        point = self.attn(point)
        feat, point.feat = AddLayerNorm.apply(feat, point.feat, path_mask(point.feat), ln2.weight, ln2.bias, ln2.eps,
                                              normed_dtype)
        point = self.mlp(point)
        mask = path_mask(point.feat)
        if mask is None:
            point.feat = feat + point.feat
        elif self.channels % 8 == 0 and all(t.dtype in ops.DTYPE_CODES for t in (feat, point.feat, mask)):
            point.feat = ResidualAdd.apply(feat, point.feat, mask)
        else:
            point.feat = torch.addcmul(feat, point.feat, mask)
        point.sparse_conv_feat = point.sparse_conv_feat.replace_feature(point.feat)
        return point

    def _forward_modular(self, point):
        if (self.pre_norm and point.feat.is_cuda and self.channels in ops.LAYER_NORM_BWD_CHANNELS
                and all(type(m[0]) is LayerNorm and m[0].weight is not None and m[0].bias is not None
                        for m in (self.norm1, self.norm2))
                and isinstance(self.drop_path[0], (DropPath, nn.Identity))
                and ops.wants_grad(point.feat, *self.parameters())):
            return self._forward_training(point)
        skip = point.feat
        point = self.cpe(point)
        point.feat = skip + point.feat

        skip = point.feat
        if self.pre_norm:
            point = self.norm1(point)
        point = self.drop_path(self.attn(point))
        point.feat = skip + point.feat
        if not self.pre_norm:
            point = self.norm1(point)

        skip = point.feat
        if self.pre_norm:
            point = self.norm2(point)
        point = self.drop_path(self.mlp(point))
        point.feat = skip + point.feat
        if not self.pre_norm:
            point = self.norm2(point)
        # the sparse view is refreshed only here (model.py:605); the conv of the NEXT block
        # therefore sees exactly this tensor
        point.sparse_conv_feat = point.sparse_conv_feat.replace_feature(point.feat)
        return point


class SerializedPooling(PointModule):
    """Grid pooling along the serialized order (model.py:609-712).

    Points whose row-0 code agrees after dropping 3*log2(stride) bits form a cluster. Because
    serialized_order[0] already sorts those codes, clusters are runs: one flag+scan kernel
    numbers them (no unique, no sort), a gather kernel produces the pooled codes, coordinates
    and scene ids, and a segment kernel reduces the projected features."""

    # kernel sizes of the convolutions that follow on the pooled points (the xCPE of every Block is
    # 3x3x3, model.py:546-552): their pair lists are started as soon as the pooled coordinates exist
    plan_kernel_sizes = (3,)
    # stride of the pooling module that follows on this one's output, if any: its clusters are started
    # as soon as the pooled codes exist
    next_stride = None

    def __init__(self, in_channels, out_channels, stride=2, norm_layer=None, act_layer=None,
                 reduce="max", shuffle_orders=True, traceable=True):
        super().__init__()
        self.in_channels, self.out_channels = in_channels, out_channels
        assert stride == 2 ** (math.ceil(stride) - 1).bit_length()   # 2, 4, 8
        self.stride = stride
        assert reduce in ["sum", "mean", "min", "max"]
        self.reduce, self.shuffle_orders, self.traceable = reduce, shuffle_orders, traceable
        self.proj = nn.Linear(in_channels, out_channels)
        self.norm = PointSequential(norm_layer(out_channels)) if norm_layer is not None else None
        self.act = PointSequential(act_layer()) if act_layer is not None else None

    def pooled_index(self, point, pending=None):
        """Everything of the pooled level that follows from the parent's coordinates alone (model.py:652-679, :690,
        :695, :700-703): clusters, the pooled codes / coordinates / scene ids, the pooled orders and inverses, the
        first halves of the pooled level's pair lists. `pending`: the cluster kernels when the caller has queued
        them already. One host wait (the cluster count). Returns the pooled Point, without features."""
        pooling_depth = (math.ceil(self.stride) - 1).bit_length()
        if pooling_depth > point.serialized_depth:
            pooling_depth = 0
        assert {"serialized_code", "serialized_order", "serialized_inverse", "serialized_depth"}.issubset(
            point.keys()), "Run point.serialization() point cloud before SerializedPooling"
        shift = 3 * pooling_depth
        depth = point.serialized_depth - pooling_depth

        # clusters in ascending order of the (shifted) row-0 code
        indices = point.serialized_order[0]
        if pending is None:
            pending = self._clusters_started(point)
        cluster, idx_ptr, head, m, offset, offset_host = ops.pool_clusters_finish(pending)
        # the shuffle of the orders (model.py:675-679) is applied while the pooled tables are written
        perm = torch.randperm(point.serialized_code.shape[0]).tolist() if self.shuffle_orders else None   # CPU generator
        code, grid_coord, batch, indices4 = ops.pool_gather(point.serialized_code, shift, point.grid_coord,
                                                            pooling_depth, point.batch, head, perm)
        # pair lists of the convolutions on the pooled points: first half queued now, finished at first use
        plans = {ks: ops.conv_plan_direct_start(indices4, ks) for ks in self.plan_kernel_sizes}
        # pooled orders: the distinct clusters met when walking the parent along each curve (same
        # result as argsort of the pooled codes, model.py:667-674, without sorting)
        order, inverse = ops.pool_orders(point.serialized_order, cluster, m, perm)
        # the clusters' mean coordinates (model.py:687-689) follow from the input coordinates, not from the features
        extra = {"coord": ops.segment_reduce(point.coord.float(), indices, idx_ptr, "mean")} if "coord" in point else {}
        return Point(AttrDict(
            **extra,
            grid_coord=grid_coord,
            serialized_code=code,
            serialized_order=order,
            serialized_inverse=inverse,
            serialized_depth=depth,
            batch=batch,
            offset=offset,   # what batch2offset(batch) would compute (model.py:66-67), without its host syncs
            _offset_host=offset_host,
            _sparse_indices=indices4,   # [batch, x, y, z] int32, what sparsify() would concatenate
            _pending_plans=plans,
            _pool_members=(indices, idx_ptr),   # the clusters' member lists: the unpooling's backward sums over them
            _pooling_inverse=cluster,
            # max(x >> d) == max(x) >> d: the pooled grid extent needs no reduction and no sync
            _grid_max_host=[v >> pooling_depth for v in point.grid_max_host()],
        ))

    def _clusters_started(self, point):
        """The cluster kernels of this pooling on `point`: those Point.pool_ahead queued, or queued now."""
        pooling_depth = (math.ceil(self.stride) - 1).bit_length()
        if pooling_depth > point.serialized_depth:
            pooling_depth = 0
        ahead = point.pop("_pending_pool", None)   # started when the codes came into being (Point.pool_ahead)
        if ahead is not None and ahead[0] == 3 * pooling_depth:
            return ahead[1]
        return ops.pool_clusters_start(point.serialized_code[0], point.serialized_order[0], 3 * pooling_depth, point.offset)

    def forward(self, point):
        pooled = point.pop("_pooled_ahead", None)   # the pooled level's index, when the model built it beforehand
        built_ahead = pooled is not None
        if not built_ahead:
            pending = self._clusters_started(point)
            projected = ops.linear(point.feat, self.proj)   # needs no cluster count: runs while the count travels
            pooled = self.pooled_index(point, pending)
        else:
            projected = ops.linear(point.feat, self.proj)
        indices, idx_ptr = pooled["_pool_members"]
        cluster = pooled.pop("_pooling_inverse")
        pooled["feat"] = (SegmentReduce.apply(projected, indices, idx_ptr, self.reduce) if ops.wants_grad(projected)
                          else ops.segment_reduce(projected, indices, idx_ptr, self.reduce))
        for key in ("condition", "context"):
            if key in point:
                pooled[key] = point[key]
        if self.traceable:
            pooled["pooling_inverse"] = cluster
            pooled["pooling_parent"] = point
        norm = self.norm[0] if self.norm is not None and len(self.norm) == 1 else None
        act = self.act[0] if self.act is not None and len(self.act) == 1 else None
        if norm is not None and _trainable_bn(norm, pooled.feat) and _exact_gelu(act):
            pooled.feat = BatchNormAct.apply(pooled.feat, norm.weight, norm.bias, norm, True)
        elif norm is not None and _fusable_bn(norm, pooled.feat) and _exact_gelu(act):
            pooled.feat = ops.bn_act(pooled.feat, norm.running_mean, norm.running_var, norm.weight, norm.bias,
                                     norm.eps, True)
        else:
            if self.norm is not None:
                pooled = self.norm(pooled)
            if self.act is not None:
                pooled = self.act(pooled)
        pooled.sparsify()
        if not built_ahead and self.next_stride is not None:
            pooled.pool_ahead(self.next_stride)
        return pooled


class SerializedUnpooling(PointModule):
    """Project child and parent, then parent += child[cluster] (model.py:715-750)."""

    def __init__(self, in_channels, skip_channels, out_channels, norm_layer=None, act_layer=None,
                 traceable=False):
        super().__init__()
        self.proj = PointSequential(nn.Linear(in_channels, out_channels))
        self.proj_skip = PointSequential(nn.Linear(skip_channels, out_channels))
        if norm_layer is not None:
            self.proj.add(norm_layer(out_channels))
            self.proj_skip.add(norm_layer(out_channels))
        if act_layer is not None:
            self.proj.add(act_layer())
            self.proj_skip.add(act_layer())
        self.traceable = traceable

    def forward(self, point):
        assert "pooling_parent" in point.keys()
        assert "pooling_inverse" in point.keys()
        parent = point.pop("pooling_parent")
        inverse = point.pop("pooling_inverse")
        point = self.proj(point)
        parent = self.proj_skip(parent)
        # only .feat is updated; parent.sparse_conv_feat keeps the skip projection, which is
        # what the first decoder block's conv reads in the reference as well (model.py:746)
        if ops.wants_grad(parent.feat, point.feat):
            parent.feat = UnpoolAdd.apply(parent.feat, point.feat, inverse, *point["_pool_members"])
        else:
            parent.feat = ops.unpool_add(parent.feat, point.feat, inverse)
        if self.traceable:
            parent["unpooling_parent"] = point
        return parent


class Embedding(PointModule):
    """Stem: 5x5x5 submanifold conv -> norm -> act (model.py:753-783)."""

    def __init__(self, in_channels, embed_channels, norm_layer=None, act_layer=None):
        super().__init__()
        self.in_channels, self.embed_channels = in_channels, embed_channels
        self.stem = PointSequential(conv=SubMConv3d(in_channels, embed_channels, kernel_size=5, padding=1,
                                                    bias=False, indice_key="stem"))
        if norm_layer is not None:
            self.stem.add(norm_layer(embed_channels), name="norm")
        if act_layer is not None:
            self.stem.add(act_layer(), name="act")

    def forward(self, point):
        return self.stem(point)
