import torch

from .. import ops

ORDERS = ("z", "z-trans", "hilbert", "hilbert-trans")


@torch.inference_mode()
def encode(grid_coord, batch=None, depth=16, order="z"):
    """Code of every point along one space-filling curve: (N,) int64.

    Same arguments and result as serialization/default.py:8-24 of the reference. For several
    orders at once use ops.encode_orders, which reads the coordinates a single time."""
    assert order in ORDERS
    return ops.encode_orders(grid_coord, batch, depth, [order])[0]
