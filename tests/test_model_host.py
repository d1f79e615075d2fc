"""Host-side checks of the drop-in interface that need no GPU."""
import inspect

import pytest
import torch


def test_constructor_signature_and_defaults():
    from pointtransformerv3_amd import PointTransformerV3
    sig = inspect.signature(PointTransformerV3.__init__)
    want = dict(in_channels=6, order=("z", "z-trans", "hilbert", "hilbert-trans"), stride=(2, 2, 2, 2),
                enc_depths=(2, 2, 2, 6, 2), enc_channels=(32, 64, 128, 256, 512), enc_num_head=(2, 4, 8, 16, 32),
                enc_patch_size=(1024,) * 5, dec_depths=(2, 2, 2, 2), dec_channels=(64, 64, 128, 256),
                dec_num_head=(4, 4, 8, 16), dec_patch_size=(1024,) * 4, mlp_ratio=4, qkv_bias=True, qk_scale=None,
                attn_drop=0.0, proj_drop=0.0, drop_path=0.3, pre_norm=True, shuffle_orders=True, enable_rpe=False,
                enable_flash=True, upcast_attention=False, upcast_softmax=False, cls_mode=False, pdnorm_bn=False,
                pdnorm_ln=False, pdnorm_decouple=True, pdnorm_adaptive=False, pdnorm_affine=True,
                pdnorm_conditions=("ScanNet", "S3DIS", "Structured3D"))
    got = {k: v.default for k, v in sig.parameters.items() if k != "self"}
    assert got == want
    assert list(got) == list(want)   # positional order too


def test_state_dict_names_and_shapes():
    from pointtransformerv3_amd import PointTransformerV3
    sd = PointTransformerV3().state_dict()
    assert sd["embedding.stem.conv.weight"].shape == (32, 5, 5, 5, 6)
    assert "embedding.stem.conv.bias" not in sd
    assert sd["embedding.stem.norm.running_var"].shape == (32,)
    assert sd["enc.enc1.down.proj.weight"].shape == (64, 32)
    assert sd["enc.enc1.down.norm.0.weight"].shape == (64,)
    assert sd["enc.enc3.block5.cpe.0.weight"].shape == (256, 3, 3, 3, 256)
    assert sd["enc.enc3.block5.cpe.0.bias"].shape == (256,)
    assert sd["enc.enc3.block5.cpe.1.weight"].shape == (256, 256)
    assert sd["enc.enc3.block5.cpe.2.bias"].shape == (256,)
    assert sd["enc.enc4.block1.attn.qkv.weight"].shape == (1536, 512)
    assert sd["enc.enc4.block1.attn.proj.bias"].shape == (512,)
    assert sd["enc.enc4.block1.norm1.0.weight"].shape == (512,)
    assert sd["enc.enc4.block1.mlp.0.fc1.weight"].shape == (2048, 512)
    assert sd["dec.dec0.up.proj.0.weight"].shape == (64, 64)
    assert sd["dec.dec3.up.proj.0.weight"].shape == (256, 512)
    assert sd["dec.dec3.up.proj_skip.0.weight"].shape == (256, 256)
    assert sd["dec.dec3.up.proj.1.running_mean"].shape == (256,)
    assert sd["dec.dec0.block1.mlp.0.fc2.weight"].shape == (64, 256)
    n_param = sum(v.numel() for k, v in sd.items() if "num_batches" not in k and "running" not in k)
    assert 46.0e6 < n_param < 46.3e6   # "46.2M" in the PTv3 paper
    assert not [k for k in sd if k.startswith("enc.enc0.down")]
    cls = PointTransformerV3(cls_mode=True)
    assert not hasattr(cls, "dec")


def test_block_order_index_and_drop_path_schedule():
    from pointtransformerv3_amd import PointTransformerV3
    m = PointTransformerV3()
    assert [m.enc.enc3[i + 1].attn.order_index for i in range(6)] == [0, 1, 2, 3, 0, 1]
    rates = []
    for s in range(5):
        stage = getattr(m.enc, f"enc{s}")
        for name, blk in stage.named_children():
            if name.startswith("block"):
                rates.append(getattr(blk.drop_path[0], "drop_prob", 0.0))
    want = torch.linspace(0, 0.3, 14).tolist()
    assert rates == pytest.approx(want)
    # decoder: rates laid out per stage over sum(dec_depths) and reversed inside a stage
    dr = torch.linspace(0, 0.3, 8).tolist()
    assert m.dec.dec3.block0.drop_path[0].drop_prob == pytest.approx(dr[7])
    assert m.dec.dec3.block1.drop_path[0].drop_prob == pytest.approx(dr[6])
    assert getattr(m.dec.dec0.block1.drop_path[0], "drop_prob", 0.0) == pytest.approx(0.0)


def test_point_batch_offset_roundtrip_and_attribute_access():
    from pointtransformerv3_amd import Point, batch2offset, offset2batch, offset2bincount
    off = torch.tensor([3, 3, 7])
    assert offset2bincount(off).tolist() == [3, 0, 4]
    assert offset2batch(off).tolist() == [0, 0, 0, 2, 2, 2, 2]
    assert batch2offset(torch.tensor([0, 0, 1, 1, 1])).tolist() == [2, 5]
    p = Point(offset=torch.tensor([2, 5]), feat=torch.zeros(5, 3))
    assert p.batch.tolist() == [0, 0, 1, 1, 1] and "batch" in p.keys()
    p.foo = 1
    assert p["foo"] == 1
    q = Point({"batch": torch.tensor([0, 1, 1])})
    assert q.offset.tolist() == [1, 3]
    with pytest.raises(AttributeError):
        _ = p.missing


def test_flash_flag_assertions_match_reference():
    from pointtransformerv3_amd import SerializedAttention
    with pytest.raises(AssertionError):
        SerializedAttention(64, 4, 1024, enable_flash=True, upcast_attention=True, upcast_softmax=False)
    with pytest.raises(AssertionError):
        SerializedAttention(60, 7, 1024)
    a = SerializedAttention(64, 4, 1024, enable_flash=False)
    assert a.patch_size == 0 and a.patch_size_max == 1024 and a.scale == 0.25


def test_forward_on_cpu_tensors_fails_loudly():
    from pointtransformerv3_amd import PointTransformerV3
    from pointtransformerv3_amd._lib import Ptv3Error
    m = PointTransformerV3(enc_depths=(1, 1, 1, 1, 1), dec_depths=(1, 1, 1, 1)).eval()
    data = dict(feat=torch.zeros(10, 6), grid_coord=torch.arange(30).reshape(10, 3).int(), offset=torch.tensor([10]))
    with pytest.raises(Ptv3Error):
        m(data)


def test_overlapped_prologue_is_opt_in_and_takes_no_cpu_tensors():
    from pointtransformerv3_amd import PointTransformerV3
    from pointtransformerv3_amd._lib import Ptv3Error
    m = PointTransformerV3(enc_depths=(1, 1, 1, 1, 1), dec_depths=(1, 1, 1, 1)).eval()
    assert m.overlap_index_prologue is False
    m.overlap_index_prologue = True
    data = dict(feat=torch.zeros(10, 6), grid_coord=torch.arange(30).reshape(10, 3).int(), offset=torch.tensor([10]))
    with torch.inference_mode(), pytest.raises(Ptv3Error):
        m(data)                       # the plain schedule, and its loud failure, for tensors that are not on the GPU
    assert m._prologue_state is None


def test_cast_of_cpu_parameters_is_computed_not_remembered():
    """Off the GPU a parameter is converted on every call (there is nothing to launch for it): the layouts are
    the ones the GPU kernel writes."""
    import torch
    from pointtransformerv3_amd import ops
    p = torch.nn.Parameter(torch.arange(24, dtype=torch.float32).reshape(2, 4, 3))
    assert ops.cast_cached(p, torch.float32) is p
    assert torch.equal(ops.cast_cached(p, torch.bfloat16).float(), p.detach())
    m = ops.cast_cached(p, torch.bfloat16, "mirror")
    assert m.shape == (3, 4, 2) and m.is_contiguous()
    assert all(float(m[k, 3 - j, i]) == float(p[i, j, k]) for i in range(2) for j in range(4) for k in range(3))
    w = torch.nn.Parameter(torch.arange(6, dtype=torch.float32).reshape(2, 3))
    assert torch.equal(ops.cast_cached(w, torch.float16, "transpose").float(), w.detach().t())
