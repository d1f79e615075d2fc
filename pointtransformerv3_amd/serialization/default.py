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


@torch.inference_mode()
def decode(code, depth=16, order="z"):
    """(grid_coord (N,3) int64, batch (N,) int64) of codes made by encode: serialization/default.py:27-39
    of the reference, which like this function takes only the two untransposed orders.

    The reference's order="z" branch cannot return (its z_order_decode unpacks the four values of
    z_order.py:104-126 into three names, default.py:47); here it returns what that lookup-table
    decode computes."""
    assert order in {"z", "hilbert"}
    return ops.decode_order(code, depth, order)


def z_order_encode(grid_coord, depth=16):
    """serialization/default.py:42-46: the Morton code without a batch index."""
    return ops.encode_orders(grid_coord, None, depth, ["z"])[0]


def z_order_decode(code, depth):
    """serialization/default.py:49-52 (as z_order.py:104-126 computes it): (N,3) int64. Bits above
    3 * depth are ignored."""
    return ops.decode_order(code, depth, "z", with_batch=False)[0]


def hilbert_encode(grid_coord, depth=16):
    """serialization/default.py:55-56."""
    return ops.encode_orders(grid_coord, None, depth, ["hilbert"])[0]


def hilbert_decode(code, depth=16):
    """serialization/default.py:59-60 -> hilbert.py:201-303: (N,3) int64. Bits above 3 * depth are ignored
    (the reference keeps the low 3 * depth bits, hilbert.py:262)."""
    return ops.decode_order(code, depth, "hilbert", with_batch=False)[0]
