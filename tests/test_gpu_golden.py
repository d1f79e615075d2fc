"""The GPU model against tests/golden/forward_golden.npz directly: outputs written by the reference's own
model.py classes (tests/golden/make_forward_golden.py), no oracle of this repository in between.

The product draws its row shuffles from torch's CPU generator in the reference's call sequence
(model.py:129, :677), so seeding it like the fixture run reproduces the same permutations.

Bars: integer structures bit-exact. Features: non-fused path in fp32 < 1e-4 of the largest value; fused path
(the reference rounds qkv and the attention result to fp16 there, model.py:477-483, and so does the product
in a float model) < 2e-3 in a float model, < 2e-2 in an fp16 model."""
import numpy as np
import pytest
import torch

from gpu_util import DEV, rel_err
from test_oracle_forward_golden import FC, GOLD, load_case

pytestmark = pytest.mark.gpu


def _model(name, dtype):
    from pointtransformerv3_amd import PointTransformerV3
    kw, (grid, coord, feat, offset), sd, perms = load_case(name)
    torch.manual_seed(0)
    model = PointTransformerV3(**kw).eval()
    model.load_state_dict(sd)          # strict: the state_dict names and shapes are the reference's own
    model = model.to(DEV, dtype)
    data = dict(feat=torch.from_numpy(feat).to(DEV, dtype), coord=torch.from_numpy(coord).to(DEV),
                grid_coord=torch.from_numpy(grid).to(DEV), offset=torch.from_numpy(offset).to(DEV))
    return model, data, kw


def _levels(point):
    chain = [point]
    while "pooling_parent" in chain[-1]:
        chain.append(chain[-1]["pooling_parent"])
    return chain[::-1]


@pytest.mark.parametrize("name", list(FC.CASES))
def test_float_model_matches_reference_run(name):
    model, data, kw = _model(name, torch.float32)
    torch.manual_seed(FC.case_seed(name))
    with torch.inference_mode():
        point = model(data)
    pre = name + "/"
    want = GOLD[pre + "out"]
    assert tuple(point.feat.shape) == want.shape
    assert rel_err(point.feat, want) < (2e-3 if kw["enable_flash"] else 1e-4)
    # the levels still reachable from the result: level 0 for a full model, the whole chain in cls_mode
    levels = _levels(point)
    assert len(levels) == (5 if kw.get("cls_mode") else 1)
    for li, lv in enumerate(levels):
        lp = pre + f"level{li}/"
        assert int(GOLD[lp + "depth"]) == lv.serialized_depth
        for key, ref in (("serialized_code", "code"), ("serialized_order", "order"), ("serialized_inverse", "inverse"),
                         ("grid_coord", "grid_coord"), ("batch", "batch")):
            assert np.array_equal(lv[key].cpu().numpy(), GOLD[lp + ref]), (li, key)
        if "pooling_inverse" in lv:
            assert np.array_equal(lv["pooling_inverse"].cpu().numpy(), GOLD[lp + "cluster"]), li
        if lp + "pad" in GOLD.files and "pad" in lv:
            assert np.array_equal(lv["pad"].cpu().numpy(), GOLD[lp + "pad"])
            assert np.array_equal(lv["unpad"].cpu().numpy(), GOLD[lp + "unpad"])
            assert np.array_equal(lv["cu_seqlens_key"].cpu().numpy(), GOLD[lp + "cu_seqlens"])


@pytest.mark.parametrize("name", [n for n in FC.CASES if FC.CASES[n][0].get("enable_flash", True)])
def test_half_model_matches_reference_run(name):
    model, data, kw = _model(name, torch.float16)
    torch.manual_seed(FC.case_seed(name))
    with torch.inference_mode():
        point = model(data)
    assert point.feat.dtype == torch.float16
    assert rel_err(point.feat, GOLD[name + "/out"]) < 2e-2


def test_stage_features_match_reference_run():
    """Every stage of the fused-path case, through forward hooks on the product's modules (the same prefixes
    the reference's modules have)."""
    name = "flash_shuffle"
    model, data, kw = _model(name, torch.float32)
    seen = {}
    for prefix, module in model.named_modules():
        if name + "/trace/" + prefix in GOLD.files:
            module.register_forward_hook(lambda m, a, r, prefix=prefix: seen.__setitem__(prefix, r.feat.detach().clone()))
    torch.manual_seed(FC.case_seed(name))
    with torch.inference_mode():
        model(data)
    stages = [k.split("/trace/")[1] for k in GOLD.files if k.startswith(name + "/trace/")]
    assert len(stages) == 25 and set(stages) == set(seen)
    for st in stages:
        assert rel_err(seen[st], GOLD[name + "/trace/" + st]) < (1e-4 if st.startswith("embedding") else 2e-3), st


def test_parameter_gradients_match_reference_run():
    """Backward of the product (float master weights, fused path in fp16 like the reference) against the
    gradients autograd gave through the reference's classes."""
    for name in [n for n in FC.CASES if FC.CASES[n][2]["grads"]]:
        model, data, kw = _model(name, torch.float32)
        for m in model.modules():
            if hasattr(m, "drop_prob"):
                m.drop_prob = 0.0
        torch.manual_seed(FC.case_seed(name))
        out = model(data).feat
        probe = torch.randn(out.shape, generator=torch.Generator().manual_seed(FC.case_seed(name) + 1))
        (out.float() * probe.to(DEV)).sum().backward()
        pre = name + "/"
        names = bytes(GOLD[pre + "grad_names"]).decode().split("\n")
        heads, sums = GOLD[pre + "grad_head"], GOLD[pre + "grad_sums"]
        params = dict(model.named_parameters())
        assert list(params) == names
        scale = float(np.abs(heads).max())
        tol = 2e-2 if kw["enable_flash"] else 1e-3
        for i, n in enumerate(names):
            g = params[n].grad.float().reshape(-1).cpu()
            k = min(64, g.numel())
            ref_scale = max(float(np.abs(heads[i]).max()), 1e-3 * scale)
            assert float(np.abs(g[:k].numpy() - heads[i][:k]).max()) <= tol * ref_scale, (name, n)
            assert abs(float(g.double().abs().sum()) - sums[i][1]) <= tol * max(sums[i][1], 1e-3 * scale), (name, n)


def test_decoder_patch_smaller_than_the_cached_tables_is_refused():
    """The encoder's padding tables stay on the Point (model.py:384-391); a decoder layer with a smaller patch
    size would run sequences longer than the max_seqlen it declares (model.py:479). The product raises instead
    of staging more keys than it sized its on-chip buffers for."""
    from pointtransformerv3_amd import PointTransformerV3
    from pointtransformerv3_amd._lib import Ptv3Error
    kw, (grid, coord, feat, offset), sd, perms = load_case("dec_patch_larger")
    kw = dict(kw, enc_patch_size=(64,) * 5, dec_patch_size=(32,) * 4)
    model = PointTransformerV3(**kw).eval()
    model.load_state_dict(sd)
    model = model.to(DEV).half()
    data = dict(feat=torch.from_numpy(feat).to(DEV).half(), grid_coord=torch.from_numpy(grid).to(DEV),
                offset=torch.from_numpy(offset).to(DEV))
    with torch.inference_mode(), pytest.raises(Ptv3Error, match="patch"):
        model(data)
