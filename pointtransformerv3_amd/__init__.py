"""MI355X-native Point Transformer V3 forward path.

Hand-written gfx950 HIP kernels (libptv3_hip.so, plain C ABI declared in include/ptv3_hip.h)
behind the Point / PointTransformerV3 Python interface of Pointcept's PTv3.
"""
from . import ops  # noqa: F401
from .serialization import encode  # noqa: F401

__all__ = ["ops", "encode"]


def __getattr__(name):
    # model classes import torch.nn machinery; load them on first use
    if name in ("Point", "PointModule", "PointSequential", "PointTransformerV3",
                "SerializedAttention", "SerializedPooling", "SerializedUnpooling", "Block",
                "Embedding", "MLP", "SubMConv3d", "SparseConvTensor", "DropPath",
                "offset2bincount", "offset2batch", "batch2offset"):
        from . import model
        return getattr(model, name)
    raise AttributeError(name)
