"""ctypes access to the scalar C restatement (oracle/ptv3_oracle.c). TEST INFRASTRUCTURE."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libptv3_oracle.so")
_lib = None


def build():
    subprocess.run(["make", "-C", _HERE, "-s", "-B"], check=True)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.orc_encode.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64,
                                    ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
        _lib.orc_encode.restype = ctypes.c_int
        _lib.orc_kmap.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int,
                                  ctypes.c_void_p]
        _lib.orc_kmap.restype = ctypes.c_int
    return _lib


def encode(grid_coord, batch, depth, order_id):
    g = np.ascontiguousarray(grid_coord, dtype=np.int32)
    b = None if batch is None else np.ascontiguousarray(batch, dtype=np.int64)
    out = np.empty(g.shape[0], dtype=np.int64)
    rc = lib().orc_encode(g.ctypes.data, None if b is None else b.ctypes.data, g.shape[0],
                          depth, order_id, out.ctypes.data)
    if rc != 0:
        raise ValueError(f"orc_encode failed: {rc}")
    return out


def kmap(indices, ks):
    idx = np.ascontiguousarray(indices, dtype=np.int32)
    out = np.empty((idx.shape[0], ks ** 3), dtype=np.int32)
    rc = lib().orc_kmap(idx.ctypes.data, idx.shape[0], ks, out.ctypes.data)
    if rc != 0:
        raise ValueError(f"orc_kmap failed: {rc}")
    return out
