"""Full PointTransformerV3 forward on the GPU vs the functional CPU oracle.
Tolerance: max-abs error relative to max-abs reference < 1e-4 (fp32) / 2e-2 (fp16)."""
import numpy as np
import pytest
import torch

from oracle.forward import ptv3_forward
from gpu_util import DEV, rel_err

pytestmark = pytest.mark.gpu


def _data(n_per_scene, n_scenes, grid=0.05, seed=10, lidar=False):
    from pointtransformerv3_amd import synthetic
    if lidar:
        scenes = [synthetic.lidar_scene(seed + i, grid) for i in range(n_scenes)]
        d = synthetic.collate(scenes)
        feat = synthetic.lidar_features(d["coord"], seed)
    else:
        scenes = [synthetic.room_scene(n_per_scene, seed + i, grid) for i in range(n_scenes)]
        d = synthetic.collate(scenes)
        feat = synthetic.room_features(d["coord"], seed)
    return d, feat


def _draw_perms(seed, shuffle_first, n_pool=4, k=4):
    """The row permutations a forward will draw from torch's CPU generator after
    torch.manual_seed(seed): one in Point.serialization when the model shuffles, then one per
    pooling stage — SerializedPooling is built without shuffle_orders (model.py:881-887), so it
    always shuffles. Re-seeds so the forward that follows draws the same sequence."""
    torch.manual_seed(seed)
    perms = [torch.randperm(k).numpy() if shuffle_first else None]
    perms += [torch.randperm(k).numpy() for _ in range(n_pool)]
    torch.manual_seed(seed)
    return perms


def _run(model, d, feat, dtype):
    data = dict(feat=torch.from_numpy(feat).to(DEV, dtype), grid_coord=torch.from_numpy(d["grid_coord"]).to(DEV),
                coord=torch.from_numpy(d["coord"]).to(DEV), offset=torch.from_numpy(d["offset"]).to(DEV))
    with torch.inference_mode():
        return model(data)


def test_forward_fp32_no_flash_small_patches():
    from pointtransformerv3_amd import PointTransformerV3
    kw = dict(enc_depths=(1, 1, 1, 2, 1), dec_depths=(1, 1, 1, 1), enc_patch_size=(512,) * 5, dec_patch_size=(512,) * 4)
    torch.manual_seed(0)
    model = PointTransformerV3(shuffle_orders=False, enable_flash=False, **kw).eval()
    d, feat = _data(3000, 2)
    perms = _draw_perms(5, False)
    want = ptv3_forward(model.state_dict(), d["grid_coord"], feat, d["offset"], enable_flash=False, perms=perms, **kw)
    point = _run(model.to(DEV), d, feat, torch.float32)
    assert point.feat.shape == want.shape
    assert rel_err(point.feat, want) < 1e-4


@pytest.mark.parametrize("shuffle", [False, True])
def test_forward_fp16_default_model(shuffle):
    from pointtransformerv3_amd import PointTransformerV3
    torch.manual_seed(1)
    model = PointTransformerV3(shuffle_orders=shuffle).eval().half()
    d, feat = _data(20000, 2, grid=0.02)
    perms = _draw_perms(77, shuffle)
    sd = {k: v.float() for k, v in model.state_dict().items()}   # the fp16-rounded weights, in fp32
    point = _run(model.to(DEV), d, feat.astype(np.float16).astype(np.float32), torch.float16)
    want = ptv3_forward(sd, d["grid_coord"], feat.astype(np.float16).astype(np.float32), d["offset"], perms=perms)
    assert point.feat.dtype == torch.float16
    assert torch.isfinite(point.feat.float()).all()
    assert rel_err(point.feat, want) < 2e-2
    # the Point carries the keys of the reference
    for key in ("serialized_code", "serialized_order", "serialized_inverse", "serialized_depth",
                "sparse_shape", "sparse_conv_feat", "pad", "unpad", "cu_seqlens_key", "offset", "batch"):
        assert key in point, key
    assert point.serialized_depth == int(d["grid_coord"].max()).bit_length()


def test_forward_lidar_4dim_fp16():
    from pointtransformerv3_amd import PointTransformerV3
    torch.manual_seed(2)
    kw = dict(enc_depths=(1, 1, 1, 1, 1), dec_depths=(1, 1, 1, 1))
    model = PointTransformerV3(in_channels=4, shuffle_orders=False, **kw).eval().half()
    d, feat = _data(0, 1, grid=0.05, seed=5000, lidar=True)
    feat = feat.astype(np.float16).astype(np.float32)
    sd = {k: v.float() for k, v in model.state_dict().items()}
    perms = _draw_perms(3, False)
    point = _run(model.to(DEV), d, feat, torch.float16)
    want = ptv3_forward(sd, d["grid_coord"], feat, d["offset"], perms=perms, **kw)
    assert point.serialized_depth == 12
    assert rel_err(point.feat, want) < 2e-2


def test_serialization_method_matches_oracle():
    from oracle import serialization as OS
    from pointtransformerv3_amd import Point
    d, feat = _data(5000, 3)
    p = Point(grid_coord=torch.from_numpy(d["grid_coord"]).to(DEV), offset=torch.from_numpy(d["offset"]).to(DEV),
              feat=torch.from_numpy(feat).to(DEV))
    p.serialization(order=list(OS.ORDERS))
    depth, code, order, inverse = OS.serialize(d["grid_coord"], d["batch"])
    assert p.serialized_depth == depth
    assert np.array_equal(p.serialized_code.cpu().numpy(), code)
    assert np.array_equal(p.serialized_order.cpu().numpy(), order)
    assert np.array_equal(p.serialized_inverse.cpu().numpy(), inverse)
    p.serialization(order="hilbert", depth=16)
    assert np.array_equal(p.serialized_code.cpu().numpy()[0], OS.encode(d["grid_coord"], d["batch"], 16, "hilbert"))
    p.sparsify()
    assert p.sparse_shape == [int(v) + 96 for v in d["grid_coord"].max(0)]
    assert p.sparse_conv_feat.indices.dtype == torch.int32 and p.sparse_conv_feat.batch_size == 3


def _full_size_inputs(lidar):
    if lidar:
        d, feat = _data(0, 2, grid=0.05, seed=5000, lidar=True)     # baseline config 5: two ~120k-point sweeps
    else:
        d, feat = _data(106_000, 4, grid=0.02, seed=4000)           # baseline config 4: four ~100k-point rooms
    return d, feat.astype(np.float16).astype(np.float32)


@pytest.mark.parametrize("lidar", [False, True])
def test_full_size_forward_properties(lidar):
    """Baseline configs 4 and 5 at full size, where the CPU oracle takes minutes: properties that do
    not depend on the size. (a) The order in which the points are stored is immaterial: every step
    of the model is defined on coordinates (curve codes, voxel neighbours, grid clusters), so a
    forward over shuffled rows gives the shuffled result. (b) Scenes of a batch do not interact in
    inference (the scene id tops every code, patches and voxel neighbourhoods stay inside a
    scene): scene 0 alone gives the rows of scene 0. (c) Two runs agree bit for bit. (d) The rows of scene 0 in the
    full batch agree with the CPU oracle run on scene 0 alone, which by (b) is the oracle's answer for the batch."""
    from pointtransformerv3_amd import PointTransformerV3
    torch.manual_seed(4)
    model = PointTransformerV3(in_channels=4 if lidar else 6, shuffle_orders=False).eval().half().to(DEV)
    d, feat = _full_size_inputs(lidar)
    n = len(feat)
    assert n > 150_000

    def run(dd, ff):
        _draw_perms(11, False)   # same pooling row shuffles in every run
        return _run(model, dd, ff, torch.float16).feat.float().cpu()

    base = run(d, feat)
    assert base.shape == (n, 64) and torch.isfinite(base).all()
    assert torch.equal(run(d, feat), base)                                   # (c)
    # (a) shuffle the rows inside every scene
    rng = np.random.default_rng(1)
    starts = np.concatenate([[0], d["offset"][:-1]])
    perm = np.concatenate([s + rng.permutation(e - s) for s, e in zip(starts, d["offset"])])
    dp = dict(d, grid_coord=d["grid_coord"][perm], coord=d["coord"][perm])
    got = run(dp, feat[perm])
    scale = float(base.abs().max())
    assert float((got - base[perm]).abs().max()) / scale < 2e-2
    # (b) the first scene alone
    n0 = int(d["offset"][0])
    d0 = dict(grid_coord=d["grid_coord"][:n0], coord=d["coord"][:n0], offset=d["offset"][:1])
    alone = run(d0, feat[:n0])
    assert float((alone - base[:n0]).abs().max()) / scale < 2e-2
    # (d) the CPU oracle on that scene alone (seconds at this size), against its rows of the full batch
    perms = _draw_perms(11, False)
    sd = {k: v.float().cpu() for k, v in model.state_dict().items()}
    want = ptv3_forward(sd, d0["grid_coord"], feat[:n0], d0["offset"], perms=perms)
    assert rel_err(base[:n0], want) < 2e-2


def test_forward_fp32_with_relative_position_bias():
    """enable_rpe=True on the non-fused attention path (model.py:297-316, :468-469): every block owns a
    table `attn.rpe.rpe_table`; the whole forward against the CPU oracle."""
    from pointtransformerv3_amd import PointTransformerV3
    kw = dict(enc_depths=(1, 1, 1, 1, 1), dec_depths=(1, 1, 1, 1), enc_patch_size=(256,) * 5, dec_patch_size=(256,) * 4)
    torch.manual_seed(6)
    model = PointTransformerV3(shuffle_orders=False, enable_flash=False, enable_rpe=True, upcast_attention=True,
                               upcast_softmax=True, **kw).eval()
    sd = model.state_dict()
    assert "enc.enc0.block0.attn.rpe.rpe_table" in sd and "dec.dec3.block0.attn.rpe.rpe_table" in sd
    with torch.no_grad():
        for k, v in sd.items():
            if k.endswith("rpe_table"):
                v.mul_(60.0)     # the initial std of 0.02 would hide the bias below the tolerance
    d, feat = _data(2500, 2)
    perms = _draw_perms(9, False)
    want = ptv3_forward(model.state_dict(), d["grid_coord"], feat, d["offset"], enable_flash=False, perms=perms, **kw)
    without = ptv3_forward({k: v for k, v in model.state_dict().items() if not k.endswith("rpe_table")},
                           d["grid_coord"], feat, d["offset"], enable_flash=False, perms=perms, **kw)
    assert float((want - without).abs().max() / want.abs().max()) > 1e-2     # the bias matters in this test
    _draw_perms(9, False)
    point = _run(model.to(DEV), d, feat, torch.float32)
    assert rel_err(point.feat, want) < 1e-4


def test_forward_cls_mode_encoder_only_fp16():
    """cls_mode (model.py:817, :976-981) stops after the encoder: the pooled points of the last stage."""
    from pointtransformerv3_amd import PointTransformerV3
    torch.manual_seed(4)
    model = PointTransformerV3(cls_mode=True, shuffle_orders=False).eval().half()
    d, feat = _data(9000, 2, grid=0.03)
    f16 = feat.astype(np.float16).astype(np.float32)
    perms = _draw_perms(21, False)
    sd = {k: v.float() for k, v in model.state_dict().items()}
    point = _run(model.to(DEV), d, f16, torch.float16)
    want = ptv3_forward(sd, d["grid_coord"], f16, d["offset"], perms=perms, cls_mode=True)
    assert point.feat.shape == want.shape and point.feat.shape[1] == 512
    assert rel_err(point.feat, want) < 2e-2
    assert "pooling_parent" in point   # the decoder never ran


def test_forward_pdnorm_picks_the_conditions_norms():
    """PDNorm (model.py:255-294) with decoupled norms is the plain model carrying that condition's norm
    parameters: same forward, bit for bit, through whichever kernels each of them takes."""
    from pointtransformerv3_amd import PointTransformerV3
    kw = dict(enc_depths=(1, 1, 1, 1, 1), dec_depths=(1, 1, 1, 1), shuffle_orders=False)
    torch.manual_seed(5)
    pd = PointTransformerV3(pdnorm_bn=True, pdnorm_ln=True, **kw).eval()
    for name, buf in pd.named_buffers():   # distinct statistics per condition
        if name.endswith("running_mean"):
            buf.normal_(0, 0.2)
        elif name.endswith("running_var"):
            buf.uniform_(0.6, 1.6)
    plain = PointTransformerV3(**kw).eval()
    cond = "S3DIS"
    idx = pd.embedding.stem.norm.conditions.index(cond) if hasattr(pd.embedding.stem, "norm") else 1
    pd_sd = pd.state_dict()
    sd = {}
    for key in plain.state_dict():
        if key in pd_sd:
            sd[key] = pd_sd[key]
            continue
        head, leaf = key.rsplit(".", 1)
        cand = f"{head}.norm.{idx}.{leaf}"
        assert cand in pd_sd, (key, cand)
        sd[key] = pd_sd[cand]
    plain.load_state_dict(sd)
    d, feat = _data(5000, 2, grid=0.04)
    f16 = feat.astype(np.float16).astype(np.float32)

    def run(model, extra):
        data = dict(feat=torch.from_numpy(f16).to(DEV, torch.float16), grid_coord=torch.from_numpy(d["grid_coord"]).to(DEV),
                    coord=torch.from_numpy(d["coord"]).to(DEV), offset=torch.from_numpy(d["offset"]).to(DEV), **extra)
        with torch.inference_mode():
            return model(data).feat
    got = run(pd.half().to(DEV), dict(condition=cond))
    want = run(plain.half().to(DEV), {})
    assert torch.isfinite(got.float()).all()
    # PDNorm modules run in torch, the plain model's norms in the fused kernels: same math, other rounding points
    assert rel_err(got, want.float().cpu()) < 2e-2
    other = run(pd, dict(condition="ScanNet"))
    assert rel_err(other, want.float().cpu()) > 1e-3   # another condition's statistics do change the result


def test_raw_points_through_grid_sample_and_forward():
    """Raw, unvoxelised scenes -> device voxelisation -> forward: the same output as handing the model
    the host-voxelised batch (the scene generator keeps the same first points)."""
    from pointtransformerv3_amd import PointTransformerV3, synthetic, voxelize
    grid = 0.04
    raw = [synthetic.room_points(15_000, 50 + i).astype(np.float32) for i in range(2)]
    coord = torch.from_numpy(np.concatenate(raw)).to(DEV)
    offset = torch.from_numpy(np.cumsum([len(r) for r in raw])).to(DEV)
    rng = np.random.default_rng(8)
    feat = torch.from_numpy(rng.random((len(coord), 6)).astype(np.float32)).to(DEV).half()
    batch = voxelize.grid_sample(coord, offset, grid, feat=feat)
    # host path: voxelize every scene with numpy, concatenate
    parts = [synthetic.voxelize_unique(r, np.float32(grid)) for r in raw]
    g_host = np.concatenate([p[0] for p in parts])
    starts = np.concatenate([[0], np.cumsum([len(r) for r in raw])[:-1]])
    keep = np.concatenate([p[1] + s for p, s in zip(parts, starts)])
    assert np.array_equal(batch["grid_coord"].cpu().numpy(), g_host) and np.array_equal(batch["index"].cpu().numpy(), keep)
    torch.manual_seed(6)
    model = PointTransformerV3(enc_depths=(1, 1, 1, 1, 1), dec_depths=(1, 1, 1, 1), shuffle_orders=False).eval().half().to(DEV)
    host = dict(feat=feat[torch.from_numpy(keep).to(DEV)], grid_coord=torch.from_numpy(g_host).to(DEV),
                coord=coord[torch.from_numpy(keep).to(DEV)], offset=torch.from_numpy(np.cumsum([len(p[1]) for p in parts])).to(DEV))
    with torch.inference_mode():
        torch.manual_seed(9); a = model({k: batch[k] for k in ("feat", "grid_coord", "coord", "offset")}).feat
        torch.manual_seed(9); b = model(host).feat
    assert a.shape[0] == len(keep) and torch.equal(a, b)


def test_forward_bf16_default_model():
    """The whole forward in bf16 (8 mantissa bits per stored activation) stays inside the same bound."""
    from pointtransformerv3_amd import PointTransformerV3
    torch.manual_seed(1)
    model = PointTransformerV3(shuffle_orders=False).eval().to(torch.bfloat16)
    d, feat = _data(20000, 2, grid=0.02)
    f = torch.from_numpy(feat).to(torch.bfloat16).float().numpy()
    perms = _draw_perms(77, False)
    sd = {k: v.float() for k, v in model.state_dict().items()}
    point = _run(model.to(DEV), d, f, torch.bfloat16)
    want = ptv3_forward(sd, d["grid_coord"], f, d["offset"], perms=perms)
    assert point.feat.dtype == torch.bfloat16
    assert rel_err(point.feat, want) < 2e-2


def test_forward_other_pooling_strides_fp32():
    """Strides 4 and 1 among the poolings (model.py:640-651: two levels at once, and none): the clusters
    started ahead of the pooling module and the pair lists of the coarser levels follow the stride."""
    from pointtransformerv3_amd import PointTransformerV3
    kw = dict(stride=(2, 4, 1, 2), enc_depths=(1, 1, 1, 1, 1), dec_depths=(1, 1, 1, 1),
              enc_patch_size=(256,) * 5, dec_patch_size=(256,) * 4)
    torch.manual_seed(12)
    model = PointTransformerV3(shuffle_orders=False, enable_flash=False, **kw).eval()
    d, feat = _data(6000, 2, grid=0.02)
    perms = _draw_perms(31, False)
    want = ptv3_forward(model.state_dict(), d["grid_coord"], feat, d["offset"], enable_flash=False, perms=perms, **kw)
    point = _run(model.to(DEV), d, feat, torch.float32)
    assert point.feat.shape == want.shape
    assert rel_err(point.feat, want) < 1e-4


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_forward_with_head_dim_32(dtype):
    """Half as many heads as the default (model.py:441-443: head dim = channels // num_heads = 32 everywhere):
    the attention then runs on the thread-per-query kernel, fp32 and half precision alike."""
    from pointtransformerv3_amd import PointTransformerV3
    kw = dict(enc_depths=(1, 1, 1, 1, 1), dec_depths=(1, 1, 1, 1), enc_num_head=(1, 2, 4, 8, 16), dec_num_head=(2, 2, 4, 8),
              enc_patch_size=(256,) * 5, dec_patch_size=(256,) * 4)
    torch.manual_seed(4)
    model = PointTransformerV3(shuffle_orders=False, enable_flash=dtype != torch.float32, **kw).eval()
    d, feat = _data(5000, 2, grid=0.02)
    perms = _draw_perms(41, False)
    x = feat.astype(np.float16).astype(np.float32)
    want = ptv3_forward(model.state_dict(), d["grid_coord"], x, d["offset"], enable_flash=dtype != torch.float32,
                        perms=perms, **kw)
    point = _run(model.to(DEV).to(dtype), d, x, dtype)
    assert point.feat.shape == want.shape
    assert rel_err(point.feat, want) < (1e-4 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("sizes", [[50], [1, 3000], [200, 2, 70]])
def test_forward_tiny_and_ragged_scenes_fp32(sizes):
    """Scenes smaller than a patch, single-point scenes, very unequal scenes in one batch."""
    from pointtransformerv3_amd import PointTransformerV3, synthetic
    kw = dict(enc_depths=(1, 1, 1, 1, 1), dec_depths=(1, 1, 1, 1), enc_patch_size=(128,) * 5, dec_patch_size=(128,) * 4)
    torch.manual_seed(0)
    model = PointTransformerV3(shuffle_orders=False, enable_flash=False, **kw).eval()
    scenes = []
    for i, n in enumerate(sizes):
        sc = synthetic.room_scene(max(n * 2, 4), 100 + i, 0.05)
        scenes.append(dict(coord=sc["coord"][:n], grid_coord=sc["grid_coord"][:n]))
    d = synthetic.collate(scenes)
    assert [len(s["grid_coord"]) for s in scenes] == sizes
    feat = synthetic.room_features(d["coord"], 1)
    perms = _draw_perms(3, False)
    want = ptv3_forward(model.state_dict(), d["grid_coord"], feat, d["offset"], enable_flash=False, perms=perms, **kw)
    point = _run(model.to(DEV), d, feat, torch.float32)
    assert rel_err(point.feat, want) < 1e-4


@pytest.mark.parametrize("separate", [False, True])
def test_forward_fp16_fused_and_separate_mlp_layers(separate):
    """The default forward runs the fused MLP at every width. With fc1 + GELU and fc2 as separate layers from 256
    channels on (fc2 and the 512 -> 1536 qkv on the package's tiled GEMM) the result is held to the same bar."""
    from pointtransformerv3_amd import PointTransformerV3, ops
    torch.manual_seed(1)
    model = PointTransformerV3(shuffle_orders=False).eval().half()
    d, feat = _data(20000, 2, grid=0.02)
    perms = _draw_perms(78, False)
    sd = {k: v.float() for k, v in model.state_dict().items()}
    x = feat.astype(np.float16).astype(np.float32)
    assert ops.MLP_ONLY_FUSED_PAYS == ops.MLP_ONLY_FUSED_CHANNELS
    old = ops.MLP_ONLY_FUSED_PAYS
    if separate:
        ops.MLP_ONLY_FUSED_PAYS = (32, 64, 128)
    try:
        point = _run(model.to(DEV), d, x, torch.float16)
    finally:
        ops.MLP_ONLY_FUSED_PAYS = old
    want = ptv3_forward(sd, d["grid_coord"], x, d["offset"], perms=perms)
    assert rel_err(point.feat, want) < 2e-2


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.float16, 2e-3), (torch.bfloat16, 1.6e-2)])
@pytest.mark.parametrize("n,k,nout", [(1000, 48, 144), (513, 6, 32), (77, 200, 50), (4096, 1024, 256), (1, 1, 1)])
def test_linear_any_matches_torch(dtype, tol, n, k, nout):
    """ptv3_linear_any_fwd (every Linear of an fp32 model, odd widths in half precision) against float64 torch:
    plain, with the exact GELU, and accumulating onto a residual in place."""
    from pointtransformerv3_amd import ops
    g = torch.Generator().manual_seed(n + k)
    x = torch.randn(n, k, generator=g).to(dtype)
    w = (torch.randn(nout, k, generator=g) / k ** 0.5).to(dtype)
    b = torch.randn(nout, generator=g).to(dtype)
    res = torch.randn(n, nout, generator=g).to(dtype)
    ref = x.double() @ w.double().t() + b.double()
    got = ops.linear_any(x.to(DEV), w.to(DEV), b.to(DEV))
    assert got.dtype == dtype and rel_err(got, ref) < tol
    got = ops.linear_any(x.to(DEV), w.to(DEV), b.to(DEV), gelu=True)
    assert rel_err(got, torch.nn.functional.gelu(ref)) < tol
    acc = res.to(DEV).clone()
    got = ops.linear_any(x.to(DEV), w.to(DEV), None, resid=acc)
    assert got.data_ptr() == acc.data_ptr()
    assert rel_err(got, res.double() + x.double() @ w.double().t()) < tol
    # leading dimensions are kept
    if n % 2 == 0:
        got = ops.linear_any(x.to(DEV).reshape(2, n // 2, k), w.to(DEV), b.to(DEV))
        assert got.shape == (2, n // 2, nout) and rel_err(got.reshape(n, nout), ref) < tol


def test_forward_widths_outside_the_mfma_kernels_fp16():
    """Channel widths the MFMA Linear kernels do not take (48, 96, ...: not 32 * 2^j) run through the general
    Linear kernel, never through a library, and meet the bar."""
    from pointtransformerv3_amd import PointTransformerV3
    kw = dict(enc_depths=(1, 1, 1), enc_channels=(48, 96, 192), enc_num_head=(3, 6, 12), enc_patch_size=(128,) * 3,
              dec_depths=(1, 1), dec_channels=(48, 96), dec_num_head=(3, 6), dec_patch_size=(128,) * 2,
              stride=(2, 2), in_channels=6)
    torch.manual_seed(5)
    model = PointTransformerV3(shuffle_orders=False, **kw).eval().half()
    d, feat = _data(3000, 2, grid=0.04)
    perms = _draw_perms(79, False, n_pool=2)
    sd = {k: v.float() for k, v in model.state_dict().items()}
    x = feat.astype(np.float16).astype(np.float32)
    point = _run(model.to(DEV), d, x, torch.float16)
    want = ptv3_forward(sd, d["grid_coord"], x, d["offset"], perms=perms, **kw)
    assert rel_err(point.feat, want) < 2e-2


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_eval_forward_follows_parameters_written_through_data(dtype):
    """A write through .data leaves no trace on a parameter's version counter; the derived copies (packed weights of
    the tile convolutions in a half model, half copies of float masters under autocast) are redone at every forward,
    so an evaluation forward after such a write computes with the new values."""
    from pointtransformerv3_amd import PointTransformerV3
    torch.manual_seed(3)
    model = PointTransformerV3(shuffle_orders=False).eval().to(DEV)
    if dtype == torch.float16:
        model = model.half()
    d, feat = _data(20000, 1, grid=0.02)
    x = feat.astype(np.float16).astype(np.float32)

    def run():
        torch.manual_seed(11)   # the pooling layers draw their order permutations from torch's CPU generator
        with torch.autocast("cuda", dtype=torch.float16, enabled=dtype == torch.float32):
            return _run(model, d, x, dtype).feat.float().clone()

    first = run()
    assert torch.equal(run(), first)
    # a 64-channel xCPE convolution (tile form in half precision) and a Linear weight
    conv = model.enc.enc1.block0.cpe[0]
    assert conv.in_channels == 64
    saved = conv.weight.data.clone()
    with torch.no_grad():
        version = conv.weight._version
        conv.weight.data.mul_(2.0)
        assert conv.weight._version == version          # nothing for a version check to see
        changed = run()
        assert not torch.equal(changed, first)
        conv.weight.data.copy_(saved)
        assert torch.equal(run(), first)
        fc = model.enc.enc2.block1.mlp[0].fc1
        fc.weight.data.mul_(0.5)
        assert not torch.equal(run(), first)
