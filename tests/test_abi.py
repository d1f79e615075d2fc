"""CPU-side checks of the C ABI: the library loads, exports every symbol the header
declares, and rejects bad arguments without touching a device."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "ptv3_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ptv3_\w+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    from pointtransformerv3_amd import _lib
    names = _declared()
    assert len(names) >= 18
    assert sorted(_lib.SIGNATURES) == names
    lib = _lib.load()
    for n in names:
        assert hasattr(lib, n), n
    assert lib.ptv3_version() >= 1


def test_argument_errors_without_a_device():
    from pointtransformerv3_amd import _lib
    lib = _lib.load()
    ids = (ctypes.c_int32 * 1)(0)
    assert lib.ptv3_encode(None, None, 10, 17, ids, 1, None, None) == -2      # depth > 16 (model.py:108)
    assert lib.ptv3_encode(None, None, 10, 0, ids, 1, None, None) == -2
    assert lib.ptv3_encode(None, None, 10, 8, ids, 1, None, None) == -1       # null pointers
    assert lib.ptv3_encode(None, None, 0, 8, ids, 1, None, None) == 0         # empty input is fine
    bad = (ctypes.c_int32 * 1)(7)
    assert lib.ptv3_encode(None, None, 0, 8, bad, 1, None, None) == -1        # unknown order
    assert lib.ptv3_decode(None, 10, 17, 0, None, None, None) == -2
    assert lib.ptv3_decode(None, 10, 8, 4, None, None, None) == -1            # unknown order
    assert lib.ptv3_decode(None, 10, 8, 0, None, None, None) == -1            # null pointers
    assert lib.ptv3_decode(None, 0, 8, 2, None, None, None) == 0
    assert lib.ptv3_argsort(None, 10, 4, 64, None, None, None, 0, None) == -2  # > 63 bits (model.py:103)
    assert lib.ptv3_argsort(None, 0, 4, 30, None, None, None, 0, None) == 0
    assert lib.ptv3_patch_attn_fwd(None, 1, 10, 48, 2, None, None, None, 1, 1024, 0.25, None, None) == -4   # head dim 24
    assert lib.ptv3_patch_attn_fwd(None, 1, 10, 64, 2, None, None, None, 1, 1024, 0.25, None, None) == -1   # 32: taken; null pointers
    assert lib.ptv3_kmap_build(None, 10, 4, 0, None, None, 0, None) == -4
    assert lib.ptv3_subm_conv_fwd(None, 9, 10, 16, None, 27, 0, None, None, 16, None, None) == -1
    assert b"workspace" in lib.ptv3_strerror(-3)
    # the block halves at 128 / 256 channels: other widths and dtypes are not theirs, empty input is fine, null pointers
    tail = lambda dtype, n, c: lib.ptv3_block_tail_wide(None, None, None, None, None, None, 1e-5, None, None, None,
                                                        dtype, n, c, None, None)
    head = lambda dtype, n, c: lib.ptv3_block_head_wide(None, None, None, None, None, None, 1e-5, None, None, 1e-5, None,
                                                        dtype, n, c, None, None, None)
    for call in (tail, head):
        assert call(1, 10, 512) == -4 and call(1, 10, 64) == -4 and call(0, 10, 128) == -4   # width, width, fp32
        assert call(1, 0, 128) == 0 and call(2, 0, 256) == 0
        assert call(1, 10, 128) == -1 and call(1, -1, 128) == -1
    assert lib.ptv3_linear_pack_weights_blocks(128) == 8 and lib.ptv3_linear_pack_weights_blocks(96) == 0


def test_argument_errors_of_the_training_entry_points():
    """Shape and pointer checks come before any launch, so they can be exercised without a GPU."""
    from pointtransformerv3_amd import _lib
    lib = _lib.load()
    # Linear + GELU: fp16 / bf16 only, 32 ... 512 inputs, outputs in 32s; empty input is fine; null pointers
    assert lib.ptv3_linear_gelu_fwd(None, None, None, 0, 10, 64, 256, None, None, None) == -4
    assert lib.ptv3_linear_gelu_fwd(None, None, None, 1, 10, 48, 256, None, None, None) == -4
    assert lib.ptv3_linear_gelu_fwd(None, None, None, 1, 10, 64, 250, None, None, None) == -4
    assert lib.ptv3_linear_gelu_fwd(None, None, None, 1, 0, 64, 256, None, None, None) == 0
    assert lib.ptv3_linear_gelu_fwd(None, None, None, 1, 10, 64, 256, None, None, None) == -1
    assert lib.ptv3_linear_gelu_bwd(None, None, None, 2, 10, 64, 256, None, None) == -1
    assert lib.ptv3_linear_gelu_bwd(None, None, None, 2, 10, 1024, 256, None, None) == -4
    # mixed-dtype residual add: channels in 8s, known dtype codes
    assert lib.ptv3_scaled_add(None, 0, None, 2, None, 0, 10, 12, None, 0, None) == -4
    assert lib.ptv3_scaled_add(None, 0, None, 7, None, 0, 10, 16, None, 0, None) == -1
    assert lib.ptv3_scaled_add(None, 0, None, 2, None, 0, 0, 16, None, 0, None) == 0
    assert lib.ptv3_scaled_add(None, 0, None, 2, None, 0, 10, 16, None, 0, None) == -1
    # parameter casts: block counts of the two job kinds, empty tables, unknown dtype
    assert lib.ptv3_cast_params_blocks(1, 1, 4096, 0) == 1 and lib.ptv3_cast_params_blocks(1, 1, 4097, 0) == 2
    assert lib.ptv3_cast_params_blocks(65, 27, 64, 1) == 27 * 2 * 1 and lib.ptv3_cast_params_blocks(0, 3, 3, 1) == 0
    assert lib.ptv3_cast_params(None, 0, 0, 1, None) == 0
    assert lib.ptv3_cast_params(None, 3, 5, 1, None) == -1
    assert lib.ptv3_cast_params(None, -1, 5, 1, None) == -1
    # weight gradient from pair lists: matrix-core shapes only, every list needed
    assert lib.ptv3_subm_conv_wgrad_pairs(None, None, 0, 10, 64, 64, None, None, None, 27, None, None, None, 0, None) == -4
    assert lib.ptv3_subm_conv_wgrad_pairs(None, None, 1, 10, 60, 64, None, None, None, 27, None, None, None, 0, None) == -4
    assert lib.ptv3_subm_conv_wgrad_pairs(None, None, 1, 10, 64, 64, None, None, None, 27, None, None, None, 0, None) == -1
    assert lib.ptv3_conv_plan_pair_out(None, None, 0, 0, None, None) == 0
    assert lib.ptv3_conv_plan_pair_out(None, None, 5, 9, None, None) == -1


def test_pad_sizes_host_arithmetic():
    from pointtransformerv3_amd import ops
    assert ops.pad_sizes([2500], 1024) == (3072, 3)
    assert ops.pad_sizes([700], 1024) == (700, 1)
    assert ops.pad_sizes([1300, 2000, 4049], 512) == (1536 + 1024 + 2560, 3 + 2 + 5)
    assert ops.pad_sizes([5, 5, 45], 16) == (5 + 0 + 48, 1 + 0 + 3)


def test_workspace_queries():
    from pointtransformerv3_amd import _lib
    lib = _lib.load()
    assert lib.ptv3_argsort_workspace_bytes(400_000, 4) >= 4 * 400_000 * 24
    assert lib.ptv3_kmap_workspace_bytes(200_000) >= 2 * 200_000 * 12
    assert lib.ptv3_pool_clusters_workspace_bytes(1000) >= 16


def test_ops_reject_cpu_tensors():
    import torch
    from pointtransformerv3_amd import _lib, ops
    with pytest.raises(_lib.Ptv3Error):
        ops.encode_orders(torch.zeros(4, 3, dtype=torch.int32), None, 8, ["z"])
    with pytest.raises(_lib.Ptv3Error):
        ops.kmap_build(torch.zeros(4, 4, dtype=torch.int32), 3)


def test_static_entry_point_refuses_more_points_than_its_buffer_holds():
    """The size check comes before anything touches a device."""
    from pointtransformerv3_amd import _lib
    lib = _lib.load()
    limit = lib.ptv3_pool_clusters_static_max_points()
    assert limit == 1 << 24
    rc = lib.ptv3_pool_clusters_static(None, None, limit + 1, 3, None, 0, None, None, None, None, None)
    assert rc == -5 and b"fixed" in lib.ptv3_strerror(rc)
