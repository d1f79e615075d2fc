"""The Point dictionary of PTv3 and its two preparation steps, serialization and
sparsification, on top of the HIP kernels.

Interface (keys, method names, arguments) follows model.py:28-174 of the reference so user
code that builds a data_dict keeps working. What differs is where the work happens: all k
curve codes come from one fused kernel, the k argsorts and inverse permutations from one
batched radix sort, and the host learns the three things it needs (grid extent, hence depth
and sparse shape, and scene sizes) from a single device->host copy that is cached on the
Point.
"""
import math

import torch

from . import ops


@torch.inference_mode()
def offset2bincount(offset):
    """Scene sizes from cumulative scene ends (model.py:28-32)."""
    return torch.diff(offset, prepend=offset.new_zeros(1))


@torch.inference_mode()
def offset2batch(offset, n=None):
    """Scene id per point from cumulative scene ends (model.py:35-40). With the number of points
    given, the result is sized without reading the offsets back to the host."""
    if n is not None and offset.is_cuda:
        return ops.offset2batch(offset, n)
    sizes = offset2bincount(offset)
    ids = torch.arange(sizes.numel(), device=offset.device, dtype=torch.long)
    return ids.repeat_interleave(sizes, output_size=n)


@torch.inference_mode()
def batch2offset(batch):
    """Cumulative scene ends from sorted scene ids (model.py:43-45)."""
    return batch.bincount().cumsum(0).long()


class AttrDict(dict):
    """dict whose items are also attributes (stands in for addict.Dict, model.py:11,48)."""

    def __getattr__(self, name):
        try:
            return self[name]
        except KeyError:
            raise AttributeError(name) from None

    def __setattr__(self, name, value):
        self[name] = value

    def __delattr__(self, name):
        try:
            del self[name]
        except KeyError:
            raise AttributeError(name) from None


class Point(AttrDict):
    """Batched point cloud as a dictionary (model.py:48-79).

    Recognised keys: coord, grid_coord, grid_size, feat, offset, batch, and — written by the
    methods below — serialized_depth/code/order/inverse, sparse_shape, sparse_conv_feat.
    Keys starting with an underscore are host-side caches of this implementation."""

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        if "batch" not in self and "offset" in self:
            n = next((self[k].shape[0] for k in ("feat", "coord", "grid_coord") if k in self), None)
            self["batch"] = offset2batch(self["offset"], n)
        elif "offset" not in self and "batch" in self:
            self["offset"] = batch2offset(self["batch"])

    # ---- host-side facts: scene ends and grid extent, read in one device->host copy, cached
    def _fetch_host(self):
        want_offset = "_offset_host" not in self
        want_grid = "_grid_max_host" not in self and ("grid_coord" in self or {"grid_size", "coord"} <= self.keys())
        parts = []
        if want_offset:
            parts.append(self["offset"].long())
        if want_grid:
            self._ensure_grid_coord()
            parts.append(ops.grid_max(self["grid_coord"]).long())
        both = torch.cat(parts) if len(parts) > 1 else parts[0]
        if both.is_cuda:
            read = ops.Readback(both)
            for ks in self.pop("_plan_ahead", ()):   # queued behind the read-back, runs while the host waits
                self.start_plan(ks)
            host = [int(v) for v in read.get()]
        else:
            host = [int(v) for v in both.tolist()]
        if want_offset:
            nb = self["offset"].shape[0]
            self["_offset_host"], host = host[:nb], host[nb:]
        if want_grid:
            self["_grid_max_host"] = host

    def offset_host(self):
        """Cumulative scene ends as a Python list."""
        if "_offset_host" not in self:
            self._fetch_host()
        return self["_offset_host"]

    def grid_max_host(self):
        """Per-axis maximum of grid_coord as a Python list of 3 ints."""
        if "_grid_max_host" not in self:
            self._fetch_host()
        return self["_grid_max_host"]

    def _ensure_grid_coord(self):
        if "grid_coord" not in self:
            # fallback voxelisation of the reference (model.py:88-96)
            assert {"grid_size", "coord"}.issubset(self.keys())
            shifted = self["coord"] - self["coord"].min(0)[0]
            self["grid_coord"] = torch.div(shifted, self["grid_size"], rounding_mode="trunc").int()

    # ---- serialization ---------------------------------------------------------------
    def serialization(self, order="z", depth=None, shuffle_orders=False):
        """Curve codes, sort order and inverse for every requested order (model.py:81-136).

        Writes serialized_depth (int) and serialized_code / serialized_order /
        serialized_inverse, each (k, N) int64."""
        assert "batch" in self
        self._ensure_grid_coord()
        orders = [order] if isinstance(order, str) else list(order)
        if depth is None:
            depth = max(self.grid_max_host()).bit_length()   # model.py:98-101
        self["serialized_depth"] = depth
        n_scenes = len(self.offset_host())
        assert depth * 3 + n_scenes.bit_length() <= 63       # model.py:103
        assert depth <= 16                                    # model.py:108

        if shuffle_orders:
            # model.py:127-132 permutes the rows of code / order / inverse afterwards; a row depends
            # on nothing but its order, so encoding the orders in permuted sequence gives the same tables
            perm = torch.randperm(len(orders)).tolist()       # CPU generator, as model.py:129
            orders = [orders[i] for i in perm]
        code = ops.encode_orders(self["grid_coord"], self["batch"], depth, orders)
        key_bits = 3 * depth + max(1, (n_scenes - 1).bit_length())
        sort_order, inverse = ops.argsort_rows(code, key_bits)

        self["serialized_code"] = code
        self["serialized_order"] = sort_order
        self["serialized_inverse"] = inverse

    # ---- pair lists of the convolutions, started ahead of their first use ------------------
    def _sparse_indices_tensor(self):
        indices = self.get("_sparse_indices")
        if indices is None:
            indices = torch.cat([self["batch"].unsqueeze(-1).int(), self["grid_coord"].int()], dim=1).contiguous()
            self["_sparse_indices"] = indices
        return indices

    def plan_ahead(self, kernel_sizes):
        """Ask for the pair lists of these kernel sizes to be started at the next host read-back (or now
        if the host facts are cached already): they depend on the coordinates only."""
        if "_offset_host" in self and "_grid_max_host" in self:
            for ks in kernel_sizes:
                self.start_plan(ks)
        else:
            self["_plan_ahead"] = tuple(kernel_sizes)

    def start_plan(self, ks):
        if not self["feat"].is_cuda:
            return
        self._ensure_grid_coord()
        pending = self.setdefault("_pending_plans", {})
        if ks == 3 and 5 in pending:
            # the 3x3x3 lists are the inner taps of the 5x5x5 ones: derived when those are finished
            self.setdefault("_derived_plans", {})[3] = 5
        elif ks not in pending:
            pending[ks] = ops.conv_plan_direct_start(self._sparse_indices_tensor(), ks)

    def pool_ahead(self, stride):
        """Queue the cluster kernels of the grid pooling with this stride now (model.py:652-664 reads
        nothing but the serialized codes): when the pooling module runs, the cluster count is on the host."""
        if "serialized_code" not in self or not self["serialized_code"].is_cuda:
            return
        depth = (math.ceil(stride) - 1).bit_length()
        if depth > self["serialized_depth"]:
            depth = 0
        self["_pending_pool"] = (3 * depth, ops.pool_clusters_start(self["serialized_code"][0], self["serialized_order"][0],
                                                                     3 * depth, self["offset"]))

    # ---- sparsify --------------------------------------------------------------------
    def sparsify(self, pad=96):
        """Attach the sparse-conv view of the features (model.py:138-174)."""
        from .sparse import SparseConvTensor

        assert {"feat", "batch"}.issubset(self.keys())
        self._ensure_grid_coord()
        if "sparse_shape" in self:
            sparse_shape = self["sparse_shape"]
        else:
            sparse_shape = [v + pad for v in self.grid_max_host()]
        indices = self._sparse_indices_tensor()
        self["sparse_shape"] = sparse_shape
        sct = SparseConvTensor(features=self["feat"], indices=indices, spatial_shape=sparse_shape,
                               batch_size=len(self.offset_host()))
        for ks, pend in self.pop("_pending_plans", {}).items():
            sct.indice_dict[("pending", ks)] = pend
        for ks, plan in self.pop("_ready_plans", {}).items():   # finished before the features existed
            sct.indice_dict[("ready", ks)] = plan
        for ks, src in self.pop("_derived_plans", {}).items():
            sct.indice_dict[("derive", ks)] = src
        self["sparse_conv_feat"] = sct
