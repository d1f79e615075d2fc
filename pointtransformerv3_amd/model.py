"""PointTransformerV3 with the constructor and forward contract of model.py:786-982 of the
reference, running on the gfx950 HIP kernels of this package."""
from functools import partial

import torch
import torch.nn as nn

from .modules import (MLP, Block, DropPath, Embedding, LayerNorm, PDNorm, PointModule, PointSequential,  # noqa: F401
                      SerializedAttention, SerializedPooling, SerializedUnpooling)
from . import ops
from .point import Point, batch2offset, offset2batch, offset2bincount  # noqa: F401
from .sparse import SparseConvTensor, SubMConv3d  # noqa: F401


class PointTransformerV3(PointModule):
    def __init__(
        self,
        in_channels=6,
        order=("z", "z-trans", "hilbert", "hilbert-trans"),
        stride=(2, 2, 2, 2),
        enc_depths=(2, 2, 2, 6, 2),
        enc_channels=(32, 64, 128, 256, 512),
        enc_num_head=(2, 4, 8, 16, 32),
        enc_patch_size=(1024, 1024, 1024, 1024, 1024),
        dec_depths=(2, 2, 2, 2),
        dec_channels=(64, 64, 128, 256),
        dec_num_head=(4, 4, 8, 16),
        dec_patch_size=(1024, 1024, 1024, 1024),
        mlp_ratio=4,
        qkv_bias=True,
        qk_scale=None,
        attn_drop=0.0,
        proj_drop=0.0,
        drop_path=0.3,
        pre_norm=True,
        shuffle_orders=True,
        enable_rpe=False,
        enable_flash=True,
        upcast_attention=False,
        upcast_softmax=False,
        cls_mode=False,
        pdnorm_bn=False,
        pdnorm_ln=False,
        pdnorm_decouple=True,
        pdnorm_adaptive=False,
        pdnorm_affine=True,
        pdnorm_conditions=("ScanNet", "S3DIS", "Structured3D"),
    ):
        super().__init__()
        self.num_stages = len(enc_depths)
        self.order = [order] if isinstance(order, str) else order
        self.cls_mode = cls_mode
        # Opt-in: the index work of every level (curve codes and orders, clusters, pooled tables, pair and tile lists,
        # attention tables: no feature is touched) runs first, on a stream of its own that does not wait for what
        # the current stream holds, so in a loop of forwards it runs beside the feature kernels of the forward before
        # and the feature pass that follows never waits for the host. Only for callers whose inputs are complete when
        # forward() is called (nothing that produces them is still queued on the current stream); evaluation mode only.
        self.overlap_index_prologue = False
        self._prologue_state = None
        self.shuffle_orders = shuffle_orders
        n = self.num_stages
        assert n == len(stride) + 1 == len(enc_channels) == len(enc_num_head) == len(enc_patch_size)
        assert cls_mode or n == len(dec_depths) + 1 == len(dec_channels) + 1
        assert cls_mode or n == len(dec_num_head) + 1 == len(dec_patch_size) + 1

        pd = dict(conditions=pdnorm_conditions, decouple=pdnorm_decouple, adaptive=pdnorm_adaptive)
        bn = partial(nn.BatchNorm1d, eps=1e-3, momentum=0.01)
        if pdnorm_bn:
            bn = partial(PDNorm, norm_layer=partial(nn.BatchNorm1d, eps=1e-3, momentum=0.01,
                                                    affine=pdnorm_affine), **pd)
        ln = LayerNorm
        if pdnorm_ln:
            ln = partial(PDNorm, norm_layer=partial(LayerNorm, elementwise_affine=pdnorm_affine), **pd)
        act = nn.GELU

        def make_block(channels, heads, patch, rate, i, stage):
            return Block(channels=channels, num_heads=heads, patch_size=patch, mlp_ratio=mlp_ratio,
                         qkv_bias=qkv_bias, qk_scale=qk_scale, attn_drop=attn_drop, proj_drop=proj_drop,
                         drop_path=rate, norm_layer=ln, act_layer=act, pre_norm=pre_norm,
                         order_index=i % len(self.order), cpe_indice_key=f"stage{stage}",
                         enable_rpe=enable_rpe, enable_flash=enable_flash,
                         upcast_attention=upcast_attention, upcast_softmax=upcast_softmax)

        self.embedding = Embedding(in_channels=in_channels, embed_channels=enc_channels[0],
                                   norm_layer=bn, act_layer=act)
        self.stride = tuple(stride)

        # encoder: stochastic-depth rate grows linearly over all encoder blocks
        rates = [r.item() for r in torch.linspace(0, drop_path, sum(enc_depths))]
        self.enc = PointSequential()
        for s in range(n):
            stage = PointSequential()
            if s > 0:
                down = SerializedPooling(in_channels=enc_channels[s - 1], out_channels=enc_channels[s],
                                         stride=stride[s - 1], norm_layer=bn, act_layer=act)
                down.next_stride = stride[s] if s < n - 1 else None   # the pooling that follows on its output
                stage.add(down, name="down")
            first = sum(enc_depths[:s])
            for i in range(enc_depths[s]):
                stage.add(make_block(enc_channels[s], enc_num_head[s], enc_patch_size[s], rates[first + i], i, s),
                          name=f"block{i}")
            if len(stage) != 0:
                self.enc.add(module=stage, name=f"enc{s}")

        # decoder: walks the stages back up; rates are laid out per stage and reversed inside
        if not cls_mode:
            rates = [r.item() for r in torch.linspace(0, drop_path, sum(dec_depths))]
            widths = list(dec_channels) + [enc_channels[-1]]
            self.dec = PointSequential()
            for s in reversed(range(n - 1)):
                first = sum(dec_depths[:s])
                stage_rates = rates[first:first + dec_depths[s]][::-1]
                stage = PointSequential()
                stage.add(SerializedUnpooling(in_channels=widths[s + 1], skip_channels=enc_channels[s],
                                              out_channels=widths[s], norm_layer=bn, act_layer=act), name="up")
                for i in range(dec_depths[s]):
                    stage.add(make_block(widths[s], dec_num_head[s], dec_patch_size[s], stage_rates[i], i, s),
                              name=f"block{i}")
                self.dec.add(module=stage, name=f"dec{s}")

    def _level0_kernel_sizes(self):
        return self._levels()[0]["kernel_sizes"]

    def _levels(self):
        """Per level of the encoder, what the index work needs to know of the modules: the pooling module in front
        of the level, the convolutions that share its pair lists (encoder and decoder stage) and the attention
        layers whose tables can be made ahead. Walked once: the module structure is taken as fixed from the first
        forward on."""
        held = self.__dict__.get("_levels_held")
        if held is None:
            held = []
            for s, stage in enumerate(self.enc._modules.values()):
                dec = self.dec._modules.get(f"dec{s}") if not self.cls_mode else None
                enc_side = [self.embedding] * (s == 0) + [stage]
                both = enc_side + [dec] * (dec is not None)
                convs = [m for st in both for m in st.modules() if isinstance(m, SubMConv3d)]
                blocks = [b for st in (stage, dec) if st is not None for b in st._modules.values() if isinstance(b, Block)]
                same = blocks and all(b.attn.enable_flash and b.attn.patch_size == blocks[0].attn.patch_size for b in blocks)
                sizes = {m.kernel_size for st in enc_side for m in st.modules() if isinstance(m, SubMConv3d)}
                held.append(dict(down=stage._modules.get("down"), convs=convs, attention=blocks if same else [],
                                 kernel_sizes=tuple(sorted(sizes, reverse=True))))
            object.__setattr__(self, "_levels_held", held)   # not a submodule, not a parameter: stays out of state_dict
        return held

    def forward(self, data_dict):
        """data_dict: feat, grid_coord (or coord + grid_size), offset or batch. Returns the Point
        whose feat is (N, dec_channels[0]) in the original point order."""
        # whoever writes the parameters behind autograd's back (fused optimizer kernels, .data, weight surgery
        # under no_grad) leaves no trace on them: the derived copies (half-precision casts of float masters,
        # the tile convolutions' packed weights) are redone once per forward, in evaluation as well
        ops.invalidate_casts()
        point = self._index_prologue(data_dict)
        point = self.embedding(point)
        point = self.enc(point)
        if not self.cls_mode:
            point = self.dec(point)
        if self._prologue_state is not None:
            self._prologue_state.forward_queued(point)
        return point

    def _level0_index(self, data_dict, everything=False):
        """Everything of level 0 that follows from the coordinates alone (model.py:966-970): the Point, its curve
        codes and orders, the stem's pair lists, the clusters of the first pooling. `everything`: also what the
        modules would otherwise make at their first use, on every level (the caller has put this on a stream of its
        own): pair and tile lists of the convolutions, padding and slot tables of the attention, and the whole index
        of the pooled levels (_pooled_index_ahead)."""
        point = Point(data_dict)
        # the pair lists of the stem and of the first stage's xCPE depend on the coordinates only:
        # their first halves are queued behind the first host read-back and run while the host waits
        point.plan_ahead(self._level0_kernel_sizes())
        point.serialization(order=self.order, shuffle_orders=self.shuffle_orders)
        if self.stride:
            point.pool_ahead(self.stride[0])   # the first pooling's clusters need the codes only
        point.sparsify()
        if everything:
            level0 = self._levels()[0]
            for m in level0["convs"]:
                m.lists_ahead(point.sparse_conv_feat)
            for b in level0["attention"]:
                b.attn._slots(point)
            self._pooled_index_ahead(point)
        return point

    def _pooled_index_ahead(self, point):
        """The index of every pooled level (clusters, pooled codes / coordinates / orders, pair and tile lists,
        attention tables: model.py:652-679, :165-172, :382-438 read coordinates only), level by level, each left on
        its parent Point under "_pooled_ahead" for the pooling module to pick up. The pooling stages draw their row
        shuffles from torch's CPU generator in module order here as they would in the forward: evaluation mode only
        (stochastic depth and dropout draw from the same generator in between)."""
        parent, made = point, []
        for level in self._levels()[1:]:
            down = level["down"]
            if not isinstance(down, SerializedPooling):
                break
            pooled = down.pooled_index(parent)   # waits for this level's cluster count; its pair counts are queued
            if down.next_stride is not None:
                pooled.pool_ahead(down.next_stride)
            parent["_pooled_ahead"] = pooled
            made.append((level, pooled))
            parent = pooled
        # the pair counts of all levels are on their way by now: one wait in effect, instead of one per level between
        # the levels' cluster kernels
        for level, pooled in made:
            ready = {}
            for ks, pend in pooled.pop("_pending_plans").items():
                ready[ks] = ops.conv_plan_direct_finish(pend)
                for m in level["convs"]:
                    if m.kernel_size == ks:
                        m.tiles_ahead(ready[ks])
            pooled["_ready_plans"] = ready
            for b in level["attention"]:
                b.attn._slots(pooled)

    def _index_prologue(self, data_dict):
        feat = data_dict.get("feat")
        if (not self.overlap_index_prologue or self.training or torch.is_grad_enabled() or feat is None
                or not feat.is_cuda or ops.Readback.blocking):
            self._prologue_state = None
            return self._level0_index(data_dict)
        if self._prologue_state is None or self._prologue_state.device != feat.device:
            self._prologue_state = ops.PrologueOverlap(feat.device)
        with self._prologue_state.scope():
            point = self._level0_index(data_dict, everything=feat.dtype != torch.float32)
        return point
