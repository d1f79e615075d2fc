"""PointTransformerV3.overlap_index_prologue: the index work of every level of a forward first, on a stream of its
own, beside the forward before it. The schedule must not change a bit of any output, whatever the sequence of inputs."""
import numpy as np
import pytest
import torch

from gpu_util import DEV

pytestmark = pytest.mark.gpu


def _inputs(seed, n_scenes, pts):
    from pointtransformerv3_amd import synthetic
    scenes = [synthetic.room_scene(pts + 137 * i, seed + i, 0.04) for i in range(n_scenes)]
    d = synthetic.collate(scenes)
    feat = synthetic.room_features(d["coord"], seed)
    return dict(feat=torch.from_numpy(feat).to(DEV).half(), grid_coord=torch.from_numpy(d["grid_coord"]).to(DEV),
                offset=torch.from_numpy(d["offset"]).to(DEV))


@pytest.mark.parametrize("cls_mode", [False, True])
def test_overlapped_prologue_changes_no_bit_over_a_sequence_of_different_inputs(cls_mode):
    from pointtransformerv3_amd import PointTransformerV3
    torch.manual_seed(3)
    kw = dict(enc_depths=(1, 1, 2, 1, 1), dec_depths=(1, 1, 1, 1), enc_patch_size=(256,) * 5, dec_patch_size=(256,) * 4)
    model = PointTransformerV3(cls_mode=cls_mode, **kw).eval().half().to(DEV)
    assert model.overlap_index_prologue is False
    datas = [_inputs(11, 2, 9000), _inputs(23, 3, 4000), _inputs(37, 1, 15000)]
    torch.cuda.synchronize()     # the inputs are complete: what the option asks of its caller
    seq = [0, 1, 2, 2, 0, 1, 0, 0, 2, 1]

    def run(flag, keep):
        model.overlap_index_prologue = flag
        outs = []
        with torch.inference_mode():
            for k, i in enumerate(seq):
                torch.manual_seed(100 + k)          # the pooling stages shuffle their rows from the CPU generator
                out = model(dict(datas[i]))
                outs.append((out.feat.clone(), out.serialized_order.clone()) if not keep else (out.feat, out.serialized_order))
                del out                              # dropped at once: its index tensors go back to their pool
        torch.cuda.synchronize()
        return outs

    want = run(False, keep=True)
    for keep in (False, True):
        got = run(True, keep)
        for (f0, o0), (f1, o1) in zip(want, got):
            assert torch.equal(f0, f1) and torch.equal(o0, o1)
    # back to the plain schedule on the same model
    again = run(False, keep=True)
    assert all(torch.equal(a[0], b[0]) for a, b in zip(want, again))


def test_overlap_is_left_alone_in_training_mode_and_under_autograd():
    from pointtransformerv3_amd import PointTransformerV3
    torch.manual_seed(5)
    kw = dict(enc_depths=(1, 1, 1, 1, 1), dec_depths=(1, 1, 1, 1), enc_patch_size=(128,) * 5, dec_patch_size=(128,) * 4)
    model = PointTransformerV3(drop_path=0.0, **kw).half().to(DEV)
    model.overlap_index_prologue = True
    data = _inputs(5, 2, 3000)
    model.eval()
    out = model(dict(data)).feat                      # grad mode on: plain schedule
    assert model._prologue_state is None and torch.isfinite(out.float()).all()
    with torch.inference_mode():
        model(dict(data))
    assert model._prologue_state is not None


def test_packed_copies_are_refreshed_while_the_host_waits_and_once_per_epoch():
    """ops.refresh_derived_copies: the packed weight copies of modules that have been used before are redone when a
    read-back finds its value still on the way, once per invalidate_casts() epoch, never under autograd and never
    inside the overlapped prologue's scope (whose allocations are recycled)."""
    from pointtransformerv3_amd import ops
    from pointtransformerv3_amd.modules import MLP
    torch.manual_seed(9)
    mlp = MLP(128, 512).half().to(DEV)
    x = torch.randn(300, 128, device=DEV).half()
    with torch.inference_mode():
        first = ops.mlp_fused_module(x, x, mlp)                 # registers the module, packs its weights
        held = mlp._packed_stream[torch.float16]
        mlp.fc1.weight.data.mul_(2.0)                           # behind autograd's back: only the epoch tells
        ops.invalidate_casts()
        calls = []
        ops._IDLE_WORK.append(lambda: calls.append(1))
        try:
            with torch.enable_grad():
                ops.refresh_derived_copies()
            assert calls == [] and mlp._packed_stream[torch.float16][0] == held[0]      # not under autograd
            scope = ops.PrologueOverlap(torch.device(DEV))
            with scope.scope():
                assert ops.IDLE_WORK_ALLOWED is False
                before = len(calls)
                ops.refresh_derived_copies()
                assert len(calls) == before                      # not inside the scope (it ran on entering it)
            assert len(calls) == 1 and ops.IDLE_WORK_ALLOWED is True
            assert mlp._packed_stream[torch.float16][0] != held[0] and mlp._packed_stream[torch.float16][1] is held[1]
            ops.refresh_derived_copies()
            assert len(calls) == 1                               # once per epoch
            second = ops.mlp_fused_module(x, x, mlp)
            assert not torch.equal(first, second)
            assert torch.equal(second, ops.mlp_fused(x, x, mlp.fc1.weight, mlp.fc1.bias, mlp.fc2.weight, mlp.fc2.bias))
            ops.invalidate_casts()
            big = torch.randn(1 << 24, device=DEV)
            for _ in range(20):
                big = big * 1.0001                               # keeps the stream busy: the read-back has to wait
            assert ops.Readback(big[:4]).get() is not None
            assert len(calls) == 2                               # the waiting host did the work
        finally:
            ops._IDLE_WORK.pop()
