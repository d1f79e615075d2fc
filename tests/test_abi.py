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
    assert lib.ptv3_argsort(None, 10, 4, 64, None, None, None, 0, None) == -2  # > 63 bits (model.py:103)
    assert lib.ptv3_argsort(None, 0, 4, 30, None, None, None, 0, None) == 0
    assert lib.ptv3_patch_attn_fwd(None, 1, 10, 64, 2, None, None, None, 1, 1024, 0.25, None, None) == -4
    assert lib.ptv3_kmap_build(None, 10, 4, 0, None, None, 0, None) == -4
    assert lib.ptv3_subm_conv_fwd(None, 9, 10, 16, None, 27, 0, None, None, 16, None, None) == -1
    assert b"workspace" in lib.ptv3_strerror(-3)


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
