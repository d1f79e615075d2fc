"""The CPU oracle's whole-model forward against tests/golden/forward_golden.npz, which was written by the
reference's own model.py classes running as written (tests/golden/make_forward_golden.py says with which
stand-ins for the packages model.py imports). This pins how oracle/forward.py composes its pieces: the order
of operations in a block, the stale convolution input of the first decoder block, the order index of every
block, clusters numbered by the first row after the shuffle, the per-Point cache of the padding tables, the
BatchNorm epsilon, stride-4 pooling, cls_mode, the non-fused attention path and the relative position bias.

Bars: integer structures bit-exact; features within 1e-5 of the largest value of the stage on the non-fused
path (both sides are fp32 on the CPU; the conv stand-in sums its taps in another order than the oracle;
measured 1e-6). On the fused path model.py:477 rounds qkv to fp16 and flash_attn returns fp16: a difference in
the last float bit in front of that rounding can move an element by half an fp16 step (5e-4 relative), and those
steps add up over the stages -- measured 2e-4 at the output, bar 5e-4. A compositional mistake (wrong tensor,
wrong order index, wrong cluster numbering) shows as an error of order one on either path."""
import os
import sys

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
import forward_cases as FC  # noqa: E402

from oracle.forward import ptv3_forward  # noqa: E402

GOLD = np.load(os.path.join(HERE, "golden", "forward_golden.npz"))
ORACLE_KEYS = ("order", "stride", "enc_depths", "enc_channels", "enc_num_head", "enc_patch_size", "dec_depths",
               "dec_channels", "dec_num_head", "dec_patch_size", "cls_mode", "enable_flash")


def load_case(name):
    """(model kwargs, inputs, state_dict, perms as ptv3_forward takes them) of one golden case."""
    pre = name + "/"
    names = bytes(GOLD[pre + "names"]).decode().split("\n")
    shapes = [tuple(int(v) for v in s.split(",") if v) for s in bytes(GOLD[pre + "shapes"]).decode().split("\n")]
    sd = FC.seeded_state_dict(names, shapes, FC.case_seed(name))
    assert abs(FC.state_checksum(sd) - float(GOLD[pre + "state_checksum"])) < 1e-6 * float(GOLD[pre + "state_checksum"]), \
        "the seeded weights did not come out as on the machine that wrote the fixture"
    kw = FC.model_kwargs(name)
    draws = [GOLD[pre + f"perm{i}"] for i in range(int(GOLD[pre + "n_draws"]))]
    n_pool = len(kw.get("stride", (2, 2, 2, 2)))
    # model.py:128-132 draws once when the model shuffles, model.py:676-680 once per pooling stage
    perms = ([draws.pop(0)] if kw["shuffle_orders"] else [None]) + draws
    assert len(perms) == n_pool + 1
    return kw, FC.scene_inputs(name), sd, perms


def oracle_kwargs(kw):
    return {k: v for k, v in kw.items() if k in ORACLE_KEYS}


def close(got, want, tol=1e-5):
    got, want = torch.as_tensor(got).float(), torch.as_tensor(want).float()
    assert got.shape == want.shape, (got.shape, want.shape)
    return float((got - want).abs().max()) <= tol * float(want.abs().max())


@pytest.mark.parametrize("name", list(FC.CASES))
def test_oracle_forward_matches_reference_run(name):
    kw, (grid, coord, feat, offset), sd, perms = load_case(name)
    trace = {}
    out = ptv3_forward(sd, grid, feat, offset, perms=perms, trace=trace, flash_half=True, **oracle_kwargs(kw))
    pre = name + "/"
    # integer structures of every level
    levels = [trace["embedding#level"]] + [trace[f"enc.enc{s}.down#level"] for s in range(1, 5)]
    for li, lv in enumerate(levels):
        lp = pre + f"level{li}/"
        assert int(GOLD[lp + "depth"]) == lv["depth"]
        for key in ("code", "order", "inverse", "grid_coord", "batch"):
            assert np.array_equal(GOLD[lp + key], np.asarray(lv[key])), (li, key)
        if lp + "cluster" in GOLD.files:
            assert np.array_equal(GOLD[lp + "cluster"], np.asarray(lv["cluster"])), li
        if lp + "pad" in GOLD.files:
            built_for, (pad, unpad, cu) = lv["pad"]
            assert np.array_equal(GOLD[lp + "pad"], pad) and np.array_equal(GOLD[lp + "unpad"], unpad)
            assert np.array_equal(GOLD[lp + "cu_seqlens"], cu) and GOLD[lp + "cu_seqlens"].dtype == np.int32
    # features after every stage the fixture kept
    stages = [k[len(pre + "trace/"):] for k in GOLD.files if k.startswith(pre + "trace/")]
    assert len(stages) >= 5
    tol = 5e-4 if kw["enable_flash"] else 1e-5
    for st in stages:
        # no fp16 rounding has happened before the first attention
        assert close(trace[st], GOLD[pre + "trace/" + st], 1e-5 if st == "embedding" else tol), st
    assert close(out, GOLD[pre + "out"], tol)


def test_first_decoder_block_convolves_the_skip_projection_alone():
    """model.py:746 adds the upsampled child to parent.feat only; the sparse tensor the next convolution reads
    (model.py:233-236) still holds the skip projection. The fixture recorded what that convolution was given."""
    name = "flash_shuffle"
    kw, (grid, coord, feat, offset), sd, perms = load_case(name)
    trace = {}
    ptv3_forward(sd, grid, feat, offset, perms=perms, trace=trace, flash_half=True, **oracle_kwargs(kw))
    seen = 0
    for key in GOLD.files:
        if not key.startswith(name + "/conv_in/"):
            continue
        stage = key[len(name + "/conv_in/"):].split(".block0")[0]          # dec.dec{s}
        conv_in = torch.from_numpy(GOLD[key])
        after_up = trace[stage + ".up"]
        assert conv_in.shape == after_up.shape
        # not the sum the shortcut carries ...
        assert not close(conv_in, after_up, 1e-3)
        # ... but GELU(BN(Linear(parent))) of the skip branch, which the oracle keeps as the sparse view
        lv = trace[stage + ".up#level"]
        skip = torch.nn.functional.gelu(torch.nn.functional.batch_norm(
            torch.nn.functional.linear(trace_parent_feat(trace, stage), sd[stage + ".up.proj_skip.0.weight"],
                                       sd[stage + ".up.proj_skip.0.bias"]),
            sd[stage + ".up.proj_skip.1.running_mean"], sd[stage + ".up.proj_skip.1.running_var"],
            sd[stage + ".up.proj_skip.1.weight"], sd[stage + ".up.proj_skip.1.bias"], False, 0.0, 1e-3))
        assert close(conv_in, skip, 5e-4), stage
        assert len(lv["feat"]) == len(conv_in)
        seen += 1
    assert seen == 4


def trace_parent_feat(trace, stage):
    """Features of the encoder stage that dec.dec{s} unpools onto: the output of its last block."""
    s = int(stage[-1])
    blocks = sorted(k for k in trace if k.startswith(f"enc.enc{s}.block") and "#" not in k)
    return trace[blocks[-1]]


@pytest.mark.parametrize("name", [n for n in FC.CASES if FC.CASES[n][2]["grads"]])
def test_oracle_autograd_matches_reference_run(name):
    """Parameter gradients of a seeded linear functional of the output: autograd through the oracle against
    autograd through the reference's classes."""
    kw, (grid, coord, feat, offset), sd, perms = load_case(name)
    leaves = {k: v.clone().requires_grad_(v.is_floating_point() and "running" not in k) for k, v in sd.items()}
    out = ptv3_forward(leaves, grid, feat, offset, perms=perms, flash_half=True, **oracle_kwargs(kw))
    probe = torch.randn(out.shape, generator=torch.Generator().manual_seed(FC.case_seed(name) + 1))
    (out * probe).sum().backward()
    pre = name + "/"
    names = bytes(GOLD[pre + "grad_names"]).decode().split("\n")
    heads, sums = GOLD[pre + "grad_head"], GOLD[pre + "grad_sums"]
    assert len(names) == len(heads) > 100
    scale = max(float(np.abs(heads).max()), 1e-12)
    tol = 1e-2 if kw["enable_flash"] else 1e-4
    for i, n in enumerate(names):
        g = leaves[n].grad.reshape(-1)
        k = min(64, g.numel())
        # float path: both sides are fp32 autograd (measured 1e-5). Fused path: the gradients pass the fp16
        # roundings of model.py:477 / :483 on the way back as well and the forward values differ by rounding
        # flips (measured 2e-3); a compositional mistake is an error of order one
        ref_scale = max(float(np.abs(heads[i]).max()), 1e-3 * scale)
        assert float(np.abs(g[:k].numpy() - heads[i][:k]).max()) <= tol * ref_scale, n
        assert abs(float(g.double().abs().sum()) - sums[i][1]) <= tol * max(sums[i][1], 1e-3 * scale), n
