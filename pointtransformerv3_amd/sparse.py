"""Sparse-convolution tensor and submanifold convolution on the HIP kmap / implicit-GEMM
kernels. Stands in for the two spconv types the reference touches (model.py:165-172,
:233-236, :546-552, :767-774): same constructor arguments and attribute names."""
import math
import weakref

import torch
import torch.nn as nn

from . import ops


class SparseConvTensor:
    """features (N,C), indices (N,4) int32 [batch,x,y,z], spatial_shape, batch_size.
    Neighbour maps are cached per indice_key in `indice_dict` and shared by every tensor
    derived through replace_feature, like spconv's."""

    def __init__(self, features, indices, spatial_shape, batch_size, indice_dict=None):
        self.features = features
        self.indices = indices
        self.spatial_shape = list(spatial_shape)
        self.batch_size = batch_size
        self.indice_dict = {} if indice_dict is None else indice_dict

    def replace_feature(self, features):
        return SparseConvTensor(features, self.indices, self.spatial_shape, self.batch_size,
                                self.indice_dict)

    def neighbour_map(self, kernel_size, indice_key=None):
        """Tap-major (taps, N) int32 neighbour map, built once per indice_key."""
        key = (indice_key, kernel_size) if indice_key is not None else None
        if key is not None and key in self.indice_dict:
            return self.indice_dict[key]
        nbr = ops.kmap_build(self.indices, kernel_size, tap_major=True)   # (taps, N)
        if key is not None:
            self.indice_dict[key] = nbr
        return nbr

    def _finish_pending(self, kernel_size):
        """Second half of a pair-list construction started ahead; the 3x3x3 lists that were asked to be
        derived from these 5x5x5 lists are made right behind them and parked under ("ready", 3)."""
        pend = self.indice_dict.pop(("pending", kernel_size))
        plan = ops.conv_plan_direct_finish(pend)
        for k in [k for k in self.indice_dict if isinstance(k, tuple) and k[0] == "derive" and self.indice_dict[k] == kernel_size]:
            self.indice_dict[("ready", k[1])] = ops.conv_plan_inner(plan, pend)
            del self.indice_dict[k]
        return plan

    def conv_plan(self, kernel_size, indice_key=None):
        """Pair lists of the neighbour map (see ops.conv_plan), cached like the map itself; built
        straight from the coordinates unless the map has been built already."""
        key = ("plan", indice_key, kernel_size) if indice_key is not None else None
        if key is not None and key in self.indice_dict:
            return self.indice_dict[key]
        if indice_key is not None and (indice_key, kernel_size) in self.indice_dict:
            plan = ops.conv_plan(self.indice_dict[(indice_key, kernel_size)], tap_major=True)
        elif ("ready", kernel_size) in self.indice_dict:
            plan = self.indice_dict.pop(("ready", kernel_size))
        elif ("pending", kernel_size) in self.indice_dict:
            plan = self._finish_pending(kernel_size)
        elif ("derive", kernel_size) in self.indice_dict and ("pending", self.indice_dict[("derive", kernel_size)]) in self.indice_dict:
            # asked for before the lists it derives from were finished: finish those (kept for their own conv)
            src = self.indice_dict[("derive", kernel_size)]
            self.indice_dict[("ready", src)] = self._finish_pending(src)
            plan = self.indice_dict.pop(("ready", kernel_size))
        else:
            plan = ops.conv_plan_direct(self.indices, kernel_size)
        if key is not None:
            self.indice_dict[key] = plan
        return plan


class SubMConv3d(nn.Module):
    """Submanifold 3-D convolution: output sites = input sites. weight has spconv 2.x's
    (out, k, k, k, in) layout so checkpoints keep loading; `padding` is accepted and unused,
    as submanifold convolutions are centred by construction."""

    # above this fraction of active (voxel, tap) pairs the dense output-stationary kernel is used
    # (no pair-matrix round trip, but MFMA work for every tap); a 2 cm surface scan goes from 0.05
    # at full resolution to 0.5 at the coarsest level, where the two forms measure about equal
    PAIR_MODE_MAX_DENSITY = 0.6
    # from this many pairs per voxel on, the tile form (sums kept on chip, no pair matrix through memory)
    # measured faster than the pair form at 64 and 128 channels; sparser levels stay on the pair form
    TILE_MODE_MIN_PAIRS_PER_VOXEL = 4.0
    # 32 and 64 channels: the sparse tile form (work in proportion to the pairs) up to this many pairs per voxel;
    # measured faster than both other forms from 2.5 to 10 pairs per voxel, a full grid (27) is the tile form's case
    SPARSE_MODE_MAX_PAIRS_PER_VOXEL = 14.0

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1,
                 groups=1, bias=True, indice_key=None):
        super().__init__()
        assert stride == 1 and dilation == 1 and groups == 1
        assert kernel_size in (3, 5), "the kmap kernel covers 3x3x3 and 5x5x5"
        self.in_channels, self.out_channels = in_channels, out_channels
        self.kernel_size, self.indice_key = kernel_size, indice_key
        k = kernel_size
        self.weight = nn.Parameter(torch.empty(out_channels, k, k, k, in_channels))
        self.bias = nn.Parameter(torch.empty(out_channels)) if bias else None
        self.reset_parameters()

    def reset_parameters(self):
        fan_in = self.kernel_size ** 3 * self.in_channels
        bound = 1.0 / math.sqrt(fan_in)   # kaiming_uniform(a=sqrt(5)) on fan_in
        nn.init.uniform_(self.weight, -bound, bound)
        if self.bias is not None:
            nn.init.uniform_(self.bias, -bound, bound)

    def _packed_weight(self, dtype):
        """The weight in the tile kernels' fragment order, repacked when the parameter may have changed -- together
        with every other convolution's that is stale, in one launch (ops.repack_conv_weights)."""
        w = self.weight
        held = self._packed.get(dtype) if isinstance(getattr(self, "_packed", None), dict) else None
        if held is None or held[0] != (ops.parameter_stamp(w), w.device):
            _PACKED_USERS.add(self)
            ops.repack_conv_weights(_PACKED_USERS, dtype, w.device)
            held = self._packed[dtype]
        return held[1]

    def _tile_form(self, plan, cin, cout):
        """Which of the two forms that walk the plan's tile lists takes this convolution in half precision:
        "sparse", "tile" or None (pair or dense form)."""
        if self.kernel_size != 3 or cin != cout or plan.n >= (1 << 24):
            return None
        if cin in ops.CONV_SPARSE_CHANNELS and plan.n_pairs <= self.SPARSE_MODE_MAX_PAIRS_PER_VOXEL * plan.n:
            return "sparse"
        if cin in ops.CONV_TILE_CHANNELS and plan.n_pairs >= self.TILE_MODE_MIN_PAIRS_PER_VOXEL * plan.n:
            return "tile"
        return None

    def lists_ahead(self, x):
        """Makes (and caches on x, under this module's indice_key) the index lists the half-precision forward of this
        module will ask for: the pair lists, and the tile lists where a tile form takes the layer. They follow from
        the coordinates alone."""
        self.tiles_ahead(x.conv_plan(self.kernel_size, self.indice_key))

    def tiles_ahead(self, plan):
        """The tile lists of `plan` that this module's half-precision forward will ask for, if it takes a tile form."""
        form = self._tile_form(plan, self.in_channels, self.out_channels)
        if form == "sparse":
            plan.tiles(128)
        elif form == "tile":
            plan.tiles(ops.tile_voxels_for(plan.n, self.in_channels))

    def convolve(self, x, feat, weight, bias, packed=None):
        """The convolution of feat (N, Cin) over x's neighbourhoods with weight (Cout, V, Cin), on whichever
        form fits: dense output-stationary (fp32, or many active taps), pair lists, tiles, or sparse tiles.
        packed() hands out the weight in the tile kernels' order when the caller has it cached."""
        cout, _, cin = weight.shape
        if feat.dtype == torch.float32:
            nbr = x.neighbour_map(self.kernel_size, self.indice_key)
            return ops.subm_conv(feat, nbr, weight, bias, tap_major=True)
        if cin % 16 != 0:
            # the MFMA kernels consume input channels 16 at a time: zero-pad the thin stem input
            pad = 16 - cin % 16
            feat = nn.functional.pad(feat, (0, pad))
            weight = nn.functional.pad(weight, (0, pad))
        plan = x.conv_plan(self.kernel_size, self.indice_key)
        form = self._tile_form(plan, cin, cout)
        if form is not None:
            tiles = packed() if packed is not None else ops.conv_pack_weight(weight, 27, feat.dtype)
            return (ops.subm_conv_sparse if form == "sparse" else ops.subm_conv_tiles)(feat, plan, tiles, bias)
        weight = weight.to(feat.dtype)
        if plan.density() <= self.PAIR_MODE_MAX_DENSITY and cout % 8 == 0:
            return ops.subm_conv_pairs(feat, plan, weight, bias)
        return ops.subm_conv(feat, x.neighbour_map(self.kernel_size, self.indice_key), weight, bias, tap_major=True)

    def forward(self, x):
        feat = x.features
        if torch.is_autocast_enabled():
            feat = feat.to(torch.get_autocast_dtype("cuda"))
        if ops.wants_grad(feat, self.weight, self.bias):
            from .autograd import SubMConv
            return x.replace_feature(SubMConv.apply(feat, self.weight, self.bias, x, self))
        weight = self.weight.reshape(self.out_channels, -1, self.in_channels)
        return x.replace_feature(self.convolve(x, feat, weight, self.bias, lambda: self._packed_weight(feat.dtype)))


# the convolutions that have been asked for packed weights: one stale weight has all stale ones repacked together
_PACKED_USERS = weakref.WeakSet()


ops._IDLE_WORK.append(lambda: [ops.repack_conv_weights(_PACKED_USERS, dtype, device) for device, dtype in list(ops._PACK_TABLES)])


def is_spconv_module(module):
    return isinstance(module, SubMConv3d)
