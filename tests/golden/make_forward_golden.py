"""Writes tests/golden/forward_golden.npz by running the reference's own model.py on the cases of
forward_cases.py.

Run in the build container only (the reference checkout does not travel):
    python tests/golden/make_forward_golden.py

Why: the reference has no tests, and whole-model behaviour rests on how model.py composes its pieces --
which tensor the first decoder block convolves (model.py:233-246, :746), which order a block attends along
(:905, :955), that clusters are numbered by the row that is first after the shuffle (:128-132, :653), that the
padding tables are cached per Point (:384-391), the BatchNorm epsilon (:848), the order of operations in Block
(:586-606), pooling (:639-712) and unpooling (:739-750). A restatement written from a reading of that file
cannot check its own reading; this script lets the reference's classes run as written.

What it pins and what it does not: model.py imports five third-party packages that are neither in the reference
checkout nor installed here (addict, timm, spconv, torch_scatter, flash_attn). Local stand-ins are registered
for them below, each a few lines of stock torch that is independent of this repository's oracle:
  addict.Dict                               an attribute dictionary
  timm.models.layers.DropPath               identity in eval mode
  spconv.pytorch.SubMConv3d                 torch.nn.functional.conv3d on the densified grid, read back at the
                                            active sites, weight (Cout, k, k, k, Cin)
  torch_scatter.segment_csr                 a loop over the segments
  flash_attn.flash_attn_varlen_qkvpacked_func   scaled_dot_product_attention per sequence on the fp16 input
So the fixture pins the COMPOSITION -- everything in model.py itself -- and nothing about the arithmetic inside
those packages (tap order, weight layout, accumulation order: still unpinned, still defined by the oracle's
dense-convolution / softmax / reduceat equivalences).

The fixture holds expected outputs only; inputs and weights are regenerated from seeds (forward_cases.py).
"""
import importlib
import os
import sys
import types

import numpy as np
import torch
import torch.nn as nn
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
sys.dont_write_bytecode = True
import forward_cases as FC  # noqa: E402


# ---------------------------------------------------------------- stand-ins for the absent packages
class AttrDict(dict):
    def __getattr__(self, key):
        try:
            return self[key]
        except KeyError:
            raise AttributeError(key)

    def __setattr__(self, key, value):
        self[key] = value


class DropPath(nn.Module):
    def __init__(self, drop_prob=0.0):
        super().__init__()
        self.drop_prob = drop_prob

    def forward(self, x):
        assert not self.training, "the fixtures are made in eval mode"
        return x


class SparseConvTensor:
    def __init__(self, features, indices, spatial_shape, batch_size):
        self.features, self.indices, self.spatial_shape, self.batch_size = features, indices, spatial_shape, batch_size

    def replace_feature(self, feature):
        return SparseConvTensor(feature, self.indices, self.spatial_shape, self.batch_size)


class SparseModule(nn.Module):
    pass


class SubMConv3d(SparseModule):
    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1, groups=1,
                 bias=True, indice_key=None):
        super().__init__()
        assert stride == 1 and dilation == 1 and groups == 1
        self.kernel_size = kernel_size
        self.weight = nn.Parameter(torch.zeros(out_channels, kernel_size, kernel_size, kernel_size, in_channels))
        self.bias = nn.Parameter(torch.zeros(out_channels)) if bias else None

    def forward(self, x):
        idx = x.indices.long()
        b, i, j, k = idx[:, 0], idx[:, 1], idx[:, 2], idx[:, 3]
        dense = torch.zeros(int(b.max()) + 1, int(i.max()) + 1, int(j.max()) + 1, int(k.max()) + 1,
                            x.features.shape[1], dtype=x.features.dtype)
        dense = dense.index_put((b, i, j, k), x.features).permute(0, 4, 1, 2, 3)
        # a submanifold convolution keeps the active sites and pads as far as the kernel reaches, whatever
        # `padding` says
        y = F.conv3d(dense, self.weight.permute(0, 4, 1, 2, 3), self.bias, padding=self.kernel_size // 2)
        return x.replace_feature(y[b, :, i, j, k])


def segment_csr(src, indptr, reduce="sum"):
    rows = []
    for a, e in zip(indptr[:-1].tolist(), indptr[1:].tolist()):
        seg = src[a:e]
        rows.append({"max": lambda s: s.max(0).values, "min": lambda s: s.min(0).values, "sum": lambda s: s.sum(0),
                     "mean": lambda s: s.mean(0)}[reduce](seg))
    return torch.stack(rows)


def flash_attn_varlen_qkvpacked_func(qkv, cu_seqlens, max_seqlen, dropout_p=0.0, softmax_scale=None):
    assert qkv.dtype == torch.float16 and dropout_p == 0
    out = torch.empty(qkv.shape[0], qkv.shape[2], qkv.shape[3], dtype=torch.float16)
    cu = cu_seqlens.tolist()
    for a, e in zip(cu[:-1], cu[1:]):
        assert e - a <= max_seqlen
        q, k, v = qkv[a:e].float().permute(1, 2, 0, 3)        # each (H, L, D)
        out[a:e] = F.scaled_dot_product_attention(q, k, v, scale=softmax_scale).permute(1, 0, 2).half()
    return out


def _module(name, **attrs):
    m = types.ModuleType(name)
    m.__dict__.update(attrs)
    sys.modules[name] = m
    return m


_module("addict", Dict=AttrDict)
_module("timm")
_module("timm.models")
_module("timm.models.layers", DropPath=DropPath)
_spmod = _module("spconv.pytorch.modules", is_spconv_module=lambda m: isinstance(m, SparseModule),
                 SparseModule=SparseModule)
_sp = _module("spconv.pytorch", SubMConv3d=SubMConv3d, SparseConvTensor=SparseConvTensor, modules=_spmod)
_module("spconv", pytorch=_sp)
_module("torch_scatter", segment_csr=segment_csr)
_module("flash_attn", flash_attn_varlen_qkvpacked_func=flash_attn_varlen_qkvpacked_func)

# model.py imports its serialization package relatively, so it is loaded as part of the namespace package
# /root/reference
sys.path.insert(0, "/root")
ref = importlib.import_module("reference.model")


# ---------------------------------------------------------------- the cases
def run_case(name, out):
    kw = FC.model_kwargs(name)
    keep = FC.CASES[name][2]
    grid, coord, feat, offset = FC.scene_inputs(name)
    torch.manual_seed(0)
    model = ref.PointTransformerV3(**kw).eval()
    names = list(model.state_dict().keys())
    shapes = [tuple(v.shape) for v in model.state_dict().values()]
    sd = FC.seeded_state_dict(names, shapes, FC.case_seed(name))
    model.load_state_dict(sd)

    draws = []
    randperm = torch.randperm

    def recording_randperm(n, *a, **k):
        p = randperm(n, *a, **k)
        draws.append(p.clone())
        return p

    trace, levels, clusters, hooks = {}, [], [], []
    stage_names = [n for n, m in model.named_modules()
                   if n == "embedding" or n.endswith(".down") or n.endswith(".up") or ".block" in n and n.count(".") == 2]

    def note(prefix):
        def hook(module, args, result):
            trace[prefix] = result.feat.detach().clone()
            if prefix == "embedding" or prefix.endswith(".down"):
                levels.append(result)
                # the decoder pops this key again (model.py:743)
                clusters.append(result.pooling_inverse.clone() if "pooling_inverse" in result.keys() else None)
        return hook

    for n, m in model.named_modules():
        if n in stage_names:
            hooks.append(m.register_forward_hook(note(n)))
    # what the convolution of the first block of every decoder stage reads (the skip projection alone)
    conv_in = {}
    for n, m in model.named_modules():
        if n.startswith("dec.") and n.endswith("block0.cpe.0"):
            hooks.append(m.register_forward_hook(
                lambda module, args, result, n=n: conv_in.__setitem__(n, args[0].features.detach().clone())))

    data = dict(feat=torch.from_numpy(feat).requires_grad_(False), coord=torch.from_numpy(coord),
                grid_coord=torch.from_numpy(grid), offset=torch.from_numpy(offset))
    torch.manual_seed(FC.case_seed(name))
    torch.randperm = recording_randperm
    try:
        point = model(data)
    finally:
        torch.randperm = randperm
    res = point.feat

    # gradients of a seeded linear functional of the output with respect to every parameter
    probe = torch.randn(res.shape, generator=torch.Generator().manual_seed(FC.case_seed(name) + 1))
    (res * probe).sum().backward()

    pre = name + "/"
    out[pre + "names"] = np.frombuffer("\n".join(names).encode(), dtype=np.uint8)
    out[pre + "shapes"] = np.frombuffer("\n".join(",".join(map(str, s)) for s in shapes).encode(), dtype=np.uint8)
    out[pre + "state_checksum"] = np.float64(FC.state_checksum(sd))
    out[pre + "n_draws"] = np.int64(len(draws))
    for i, p in enumerate(draws):
        out[pre + f"perm{i}"] = p.numpy()
    out[pre + "out"] = res.detach().numpy()
    for k, v in trace.items():
        if keep["trace"] == "full" or ".block" not in k:
            out[pre + "trace/" + k] = v.numpy()
    for k, v in (conv_in.items() if keep["trace"] == "full" else ()):
        out[pre + "conv_in/" + k] = v.numpy()
    for li, lv in enumerate(levels):
        lp = pre + f"level{li}/"
        out[lp + "code"] = lv.serialized_code.numpy()
        out[lp + "order"] = lv.serialized_order.numpy()
        out[lp + "inverse"] = lv.serialized_inverse.numpy()
        out[lp + "grid_coord"] = lv.grid_coord.numpy()
        out[lp + "batch"] = lv.batch.numpy()
        out[lp + "depth"] = np.int64(lv.serialized_depth)
        if clusters[li] is not None:
            out[lp + "cluster"] = clusters[li].numpy()
        if "pad" in lv.keys():
            out[lp + "pad"] = lv.pad.numpy()
            out[lp + "unpad"] = lv.unpad.numpy()
            out[lp + "cu_seqlens"] = lv.cu_seqlens_key.numpy()
    if keep["grads"]:
        # one row per parameter in named_parameters() order: its first 64 elements as they are (zero padded),
        # and the sum and absolute sum of all of them
        heads, sums = [], []
        for n, p in model.named_parameters():
            g = p.grad.detach().reshape(-1)
            heads.append(F.pad(g[:64], (0, max(0, 64 - g.numel()))).numpy())
            sums.append([float(g.double().sum()), float(g.double().abs().sum())])
        out[pre + "grad_names"] = np.frombuffer("\n".join(n for n, _ in model.named_parameters()).encode(), dtype=np.uint8)
        out[pre + "grad_head"] = np.stack(heads)
        out[pre + "grad_sums"] = np.array(sums)
    for h in hooks:
        h.remove()
    print(f"{name}: N={len(grid)} out={tuple(res.shape)} stages={len(trace)} draws={len(draws)} "
          f"levels={[int(l.feat.shape[0]) for l in levels]}")


if __name__ == "__main__":
    out = {}
    for case in FC.CASES:
        run_case(case, out)
    path = os.path.join(HERE, "forward_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, f"{os.path.getsize(path) / 1024:.0f} KiB, {len(out)} arrays")
