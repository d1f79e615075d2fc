"""CPU fp32 oracle of the whole PTv3 forward, written as straight-line functional code over a
state_dict (TEST INFRASTRUCTURE — only tests, the smoke check and the CPU-baseline leg of
the benchmark may import this; it shares no code with the shipped modules).

Follows model.py:966-982 of the reference and, inside it, :781-783 (stem), :586-606 (block),
:440-490 (attention), :639-712 (pooling), :739-750 (unpooling), including the behaviours that
results depend on:
  * the last patch of a scene is completed with real neighbours, not masked (:412-423)
  * clusters are numbered by whichever order is row 0 after shuffling (:128-132, :653)
  * the first decoder block convolves the skip projection alone while its shortcut carries
    skip + upsampled child (:746 updates .feat only)
  * decoder blocks reuse the encoder stage's neighbour map (same indice_key, :906,:956)
Row shuffles are passed in explicitly (`perms`) so no RNG is involved.
"""
import numpy as np
import torch
import torch.nn.functional as F

from . import functional as OF
from . import indexing as OI
from . import serialization as OS

DEFAULTS = dict(
    order=("z", "z-trans", "hilbert", "hilbert-trans"), stride=(2, 2, 2, 2),
    enc_depths=(2, 2, 2, 6, 2), enc_channels=(32, 64, 128, 256, 512), enc_num_head=(2, 4, 8, 16, 32),
    enc_patch_size=(1024,) * 5, dec_depths=(2, 2, 2, 2), dec_channels=(64, 64, 128, 256),
    dec_num_head=(4, 4, 8, 16), dec_patch_size=(1024,) * 4, cls_mode=False, enable_flash=True,
    # model.py:477 hands flash_attn qkv.half() and gets fp16 back whatever the model's dtype: True restates that
    # rounding (what the reference computes in a float model); False keeps float throughout (what a float
    # model computes here, and what half-precision runs are compared with)
    flash_half=False)


def _linear(sd, name, x):
    return F.linear(x, sd[name + ".weight"], sd.get(name + ".bias"))


def _ln(sd, name, x):
    w = sd[name + ".weight"]
    return F.layer_norm(x, (w.numel(),), w, sd[name + ".bias"], 1e-5)


def _bn(sd, name, x):
    # eval mode, eps 1e-3 (model.py:848)
    return F.batch_norm(x, sd[name + ".running_mean"], sd[name + ".running_var"], sd[name + ".weight"],
                        sd[name + ".bias"], False, 0.0, 1e-3)


def _kmap(level, ks):
    if ks not in level["kmaps"]:
        idx = np.concatenate([level["batch"][:, None], level["grid_coord"]], 1)
        level["kmaps"][ks] = OI.subm_kmap(idx, ks)
    return level["kmaps"][ks]


def _attention(sd, name, level, x, heads, patch, order_index):
    rpe = None
    if name + ".rpe.rpe_table" in sd:
        # the table is sized by the configured patch size, whatever the patch shrinks to (model.py:298-303, :371)
        rpe = (level["grid_coord"], sd[name + ".rpe.rpe_table"], int((4 * patch) ** (1 / 3) * 2))
    if not level["flash"]:
        # without the fused path the patch shrinks to the smallest scene (model.py:441-444)
        patch = min(int(OI.offset2bincount(level["offset"]).min()), patch)
    # the tables are made by the first block that reaches this Point and kept under fixed keys (model.py:384-391):
    # decoder blocks of a stage run on the tables its encoder blocks made, whatever their own patch size
    if "pad" not in level:
        level["pad"] = (patch, OI.padding_tables(level["offset"], patch))
    built_for, (pad, unpad, cu) = level["pad"]
    if level["flash"]:
        # flash_attn takes the patch as max_seqlen (model.py:479): sequences longer than that are outside its contract
        assert built_for <= patch, f"cached patches of {built_for} points exceed this block's patch size {patch}"
    else:
        # model.py:461 reshapes the cached padded rows into patches of the current size
        assert built_for == patch, "patch sizes that differ within a stage are not restated for the non-fused path"
    qkv = _linear(sd, name + ".qkv", x)
    if level["flash"] and level["flash_half"]:
        qkv = qkv.half().float()                                                  # model.py:477
    out = OF.serialized_attention_core(qkv, level["order"][order_index], level["inverse"][order_index],
                                       pad, unpad, cu, heads, rpe=rpe)
    if level["flash"] and level["flash_half"]:
        out = out.half().float()                    # flash_attn returns fp16, model.py:483 casts it back
    return _linear(sd, name + ".proj", out)


def _block(sd, name, level, heads, patch, order_index):
    feat = level["feat"]
    # xCPE on the sparse view, which may lag behind feat (first decoder block)
    y = OF.subm_conv(level["sparse_feat"], _kmap(level, 3), sd[name + ".cpe.0.weight"], sd[name + ".cpe.0.bias"])
    y = _ln(sd, name + ".cpe.2", _linear(sd, name + ".cpe.1", y))
    feat = feat + y
    feat = feat + _attention(sd, name + ".attn", level, _ln(sd, name + ".norm1.0", feat), heads, patch, order_index)
    h = _ln(sd, name + ".norm2.0", feat)
    h = _linear(sd, name + ".mlp.0.fc2", F.gelu(_linear(sd, name + ".mlp.0.fc1", h)))
    feat = feat + h
    level["feat"] = feat
    level["sparse_feat"] = feat


def _pool(sd, name, parent, perm, stride=2, argmax=None):
    # model.py:640-651: pooling depth = bit length of (stride - 1), 0 when deeper than the codes
    pooling_depth = (int(np.ceil(stride)) - 1).bit_length()
    if pooling_depth > parent["depth"]:
        pooling_depth = 0
    pc = OI.pool_clusters(parent["code"], parent["grid_coord"], parent["batch"], pooling_depth)
    code, order, inverse = pc["code"], pc["order"], pc["inverse"]
    if perm is not None:
        code, order, inverse = code[perm], order[perm], inverse[perm]
    rows = _linear(sd, name + ".proj", parent["feat"])
    if argmax is None:
        feat = OF.segment_csr(rows, pc["indices"], pc["idx_ptr"], "max")
    else:
        # the member that attains each cluster's maximum is given (row numbers of the parent, one per cluster and
        # channel): where several members come within rounding of each other a half-precision run may pick another
        # one than float arithmetic does, and a gradient check against that run has to follow its choice
        feat = rows.gather(0, torch.as_tensor(argmax, dtype=torch.int64))
    feat = F.gelu(_bn(sd, name + ".norm.0", feat))
    return dict(feat=feat, sparse_feat=feat, grid_coord=pc["grid_coord"], batch=pc["batch"],
                offset=OI.batch2offset(pc["batch"]), code=code, order=order, inverse=inverse,
                depth=parent["depth"] - pooling_depth, kmaps={}, cluster=pc["cluster"], parent=parent,
                flash=parent["flash"], flash_half=parent["flash_half"])


def _unpool(sd, name, child):
    parent = child["parent"]
    up = F.gelu(_bn(sd, name + ".proj.1", _linear(sd, name + ".proj.0", child["feat"])))
    skip = F.gelu(_bn(sd, name + ".proj_skip.1", _linear(sd, name + ".proj_skip.0", parent["feat"])))
    parent["sparse_feat"] = skip
    parent["feat"] = OF.unpool_add(skip, up, child["cluster"])
    return parent


def ptv3_forward(state_dict, grid_coord, feat, offset, perms=None, trace=None, pool_argmax=None, **config):
    """Returns the (N, dec_channels[0]) output features in original point order (fp32 torch).

    perms: None (no shuffling) or a list of row permutations, one for the initial
    serialization followed by one per pooling stage.
    trace: optional dict; receives the feature tensor after the stem and after every
    pooling / unpooling / block, keyed by the module's state_dict prefix.
    pool_argmax: optional list, one (clusters, channels) array of parent row numbers per pooling stage: the
    members whose projected value is taken as each cluster's maximum (see _pool); None = the true maxima."""
    cfg = dict(DEFAULTS)
    cfg.update(config)
    sd = {k: torch.as_tensor(v).float() for k, v in state_dict.items()}
    orders = [cfg["order"]] if isinstance(cfg["order"], str) else list(cfg["order"])
    k = len(orders)
    grid_coord = np.asarray(grid_coord)
    offset = np.asarray(offset, dtype=np.int64)
    batch = OI.offset2batch(offset)
    perms = [None] * (len(cfg["stride"]) + 1) if perms is None else list(perms)

    depth, code, order, inverse = OS.serialize(grid_coord, batch, orders)
    if perms[0] is not None:
        code, order, inverse = code[perms[0]], order[perms[0]], inverse[perms[0]]
    x = torch.as_tensor(feat).float()
    level = dict(feat=x, sparse_feat=x, grid_coord=grid_coord, batch=batch, offset=offset, code=code,
                 order=order, inverse=inverse, depth=depth, kmaps={}, flash=bool(cfg["enable_flash"]),
                 flash_half=bool(cfg["flash_half"]))

    # stem (model.py:766-779): 5x5x5 conv without bias, BN, GELU
    y = OF.subm_conv(x, _kmap(level, 5), sd["embedding.stem.conv.weight"], None)
    y = F.gelu(_bn(sd, "embedding.stem.norm", y))
    level["feat"] = level["sparse_feat"] = y
    def note(name, lv):
        if trace is not None:
            trace[name] = lv["feat"]
            trace[name + "#level"] = lv   # integer structures of the level, for debugging

    note("embedding", level)

    assert all(st == 2 ** ((int(st) - 1).bit_length()) for st in cfg["stride"])   # model.py:646
    n_stage = len(cfg["enc_depths"])
    for s in range(n_stage):
        if s > 0:
            level = _pool(sd, f"enc.enc{s}.down", level, perms[s], cfg["stride"][s - 1],
                          None if pool_argmax is None else pool_argmax[s - 1])
            note(f"enc.enc{s}.down", level)
        for i in range(cfg["enc_depths"][s]):
            _block(sd, f"enc.enc{s}.block{i}", level, cfg["enc_num_head"][s], cfg["enc_patch_size"][s], i % k)
            note(f"enc.enc{s}.block{i}", level)
    if not cfg["cls_mode"]:
        for s in reversed(range(n_stage - 1)):
            level = _unpool(sd, f"dec.dec{s}.up", level)
            note(f"dec.dec{s}.up", level)
            for i in range(cfg["dec_depths"][s]):
                _block(sd, f"dec.dec{s}.block{i}", level, cfg["dec_num_head"][s], cfg["dec_patch_size"][s], i % k)
                note(f"dec.dec{s}.block{i}", level)
    return level["feat"]
