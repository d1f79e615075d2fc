"""CPU oracle for point-cloud serialization (TEST INFRASTRUCTURE, not product code).

Only tests, the smoke check and the CPU-baseline leg of the benchmark may import this
module; the shipped package never does.

numpy restatement of the space-filling-curve codes of the reference:

* z-order        -> serialization/z_order.py:40-50 (loop form), :66-101 (LUT form, masks)
* Hilbert        -> serialization/hilbert.py:91-198 (Skilling 2004, per-bit tensors)
* order dispatch -> serialization/default.py:8-24 ("-trans" swaps x/y, batch goes above
                    bit 3*depth)
* argsort + inverse permutation -> model.py:119-126

Everything is written on packed uint64 words instead of the reference's per-bit uint8
tensors, so a transcription slip cannot be shared with it.
"""
import numpy as np

ORDERS = ("z", "z-trans", "hilbert", "hilbert-trans")
ORDER_ID = {name: i for i, name in enumerate(ORDERS)}


def _as_u64_xyz(grid_coord, depth):
    """(N,3) integer coords -> three uint64 arrays truncated to `depth` low bits.

    The reference masks instead of range-checking (z_order.py:90-94) and keeps the last
    `depth` bits of the 64-bit two's-complement word (hilbert.py:143-152)."""
    g = np.asarray(grid_coord).astype(np.int64)
    assert g.ndim == 2 and g.shape[1] == 3
    mask = np.uint64((1 << depth) - 1)
    x = g[:, 0].view(np.uint64) & mask
    y = g[:, 1].view(np.uint64) & mask
    z = g[:, 2].view(np.uint64) & mask
    return x, y, z


def z_order_code(grid_coord, depth=16):
    """Morton code: bit i of x -> bit 3i+2, of y -> 3i+1, of z -> 3i (z_order.py:40-50)."""
    assert 0 < depth <= 16
    x, y, z = _as_u64_xyz(grid_coord, depth)
    key = np.zeros_like(x)
    one = np.uint64(1)
    for i in range(depth):
        s = np.uint64(i)
        key |= ((x >> s) & one) << np.uint64(3 * i + 2)
        key |= ((y >> s) & one) << np.uint64(3 * i + 1)
        key |= ((z >> s) & one) << np.uint64(3 * i)
    return key.view(np.int64)


def hilbert_code(grid_coord, depth=16):
    """Skilling's axes->transpose followed by Gray decoding (hilbert.py:154-181).

    Bit index 0 of the reference's bit tensors is the MSB of the `depth`-bit coordinate
    (hilbert.py:146-152 keeps the trailing `depth` bits of an MSB-first expansion), so
    its `for bit in range(num_bits)` walks q = depth-1 .. 0 here."""
    assert 0 < depth and 3 * depth <= 63
    X = list(_as_u64_xyz(grid_coord, depth))
    for q in range(depth - 1, -1, -1):
        Q = np.uint64(1 << q)
        P = np.uint64((1 << q) - 1)
        for i in range(3):
            on = (X[i] & Q) != 0
            # bit set: invert the lower bits of axis 0 (hilbert.py:160-165)
            inv = np.where(on, P, np.uint64(0))
            # bit clear: exchange the lower bits of axis 0 and axis i (hilbert.py:168-175)
            t = np.where(on, np.uint64(0), (X[0] ^ X[i]) & P)
            X[0] = X[0] ^ inv ^ t
            if i != 0:
                X[i] = X[i] ^ t
    # interleave: level b of axis i lands on bit 3b + (2 - i) (hilbert.py:178)
    g = np.zeros_like(X[0])
    one = np.uint64(1)
    for b in range(depth):
        s = np.uint64(b)
        for i in range(3):
            g |= ((X[i] >> s) & one) << np.uint64(3 * b + 2 - i)
    # Gray -> binary: prefix XOR from the MSB (hilbert.py:69-88, :181)
    h = g.copy()
    shift = 1
    while shift < 64:
        h ^= h >> np.uint64(shift)
        shift *= 2
    return h.view(np.int64)


def encode(grid_coord, batch=None, depth=16, order="z"):
    """serialization/default.py:8-24."""
    assert order in ORDER_ID
    g = np.asarray(grid_coord)
    if order.endswith("-trans"):
        g = g[:, [1, 0, 2]]
    code = z_order_code(g, depth) if order.startswith("z") else hilbert_code(g, depth)
    if batch is not None:
        b = np.asarray(batch).astype(np.int64)
        code = (b << np.int64(3 * depth)) | code
    return code


def z_order_decode(code, depth=16):
    """Inverse of z_order_code; the reference's own inverse is z_order.py:104-126."""
    c = np.asarray(code).astype(np.int64).view(np.uint64)
    one = np.uint64(1)
    out = np.zeros((c.shape[0], 3), dtype=np.int64)
    for i in range(depth):
        for a in range(3):
            bit = (c >> np.uint64(3 * i + 2 - a)) & one
            out[:, a] |= (bit << np.uint64(i)).astype(np.int64)
    return out


def hilbert_decode(code, depth=16):
    """Inverse of hilbert_code (Skilling transpose->axes); the reference's is
    hilbert.py:201-303. Used only for round-trip checks."""
    h = np.asarray(code).astype(np.int64).view(np.uint64)
    g = h ^ (h >> np.uint64(1))
    one = np.uint64(1)
    X = [np.zeros_like(g) for _ in range(3)]
    for b in range(depth):
        for i in range(3):
            X[i] |= ((g >> np.uint64(3 * b + 2 - i)) & one) << np.uint64(b)
    for q in range(depth):
        Q = np.uint64(1 << q)
        P = np.uint64((1 << q) - 1)
        for i in (2, 1, 0):
            on = (X[i] & Q) != 0
            inv = np.where(on, P, np.uint64(0))
            t = np.where(on, np.uint64(0), (X[0] ^ X[i]) & P)
            X[0] = X[0] ^ inv ^ t
            if i != 0:
                X[i] = X[i] ^ t
    return np.stack([x.view(np.int64) for x in X], axis=1)


def serialized_depth(grid_coord):
    """Adaptive depth: bit length of the largest coordinate (model.py:98-101)."""
    return int(np.asarray(grid_coord).max()).bit_length()


def serialize(grid_coord, batch, orders=ORDERS, depth=None):
    """model.py:98-126 without the optional row shuffle: returns (depth, code, order,
    inverse), each (k, N) int64. The argsort is stable, which is the unique answer when
    all codes of a row are distinct (one point per voxel)."""
    if depth is None:
        depth = serialized_depth(grid_coord)
    nb = int(np.asarray(batch).max()) + 1 if len(batch) else 1
    assert depth * 3 + nb.bit_length() <= 63 and depth <= 16  # model.py:103,108
    code = np.stack([encode(grid_coord, batch, depth, o) for o in orders])
    order = np.argsort(code, axis=1, kind="stable").astype(np.int64)
    inverse = np.empty_like(order)
    n = code.shape[1]
    for r in range(code.shape[0]):
        inverse[r, order[r]] = np.arange(n, dtype=np.int64)
    return depth, code, order, inverse
