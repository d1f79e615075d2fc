"""Pins the serialization oracle: golden vectors from the reference's Hilbert encoder,
closed forms, exhaustive invariants on small cubes, and agreement of the two independent
restatements (numpy on packed words, scalar C)."""
import os

import numpy as np
import pytest

from oracle import cnative
from oracle import serialization as S

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "hilbert_golden.npz"))


def _all_cells(d):
    r = np.arange(1 << d)
    return np.stack(np.meshgrid(r, r, r, indexing="ij"), -1).reshape(-1, 3).astype(np.int32)


@pytest.mark.parametrize("name", sorted(k[:-3] for k in GOLD.files if k.endswith("_in")))
def test_hilbert_matches_reference_golden(name):
    depth = int(name.split("_d")[1])
    pts, want = GOLD[name + "_in"], GOLD[name + "_out"]
    assert np.array_equal(S.hilbert_code(pts, depth), want)
    assert np.array_equal(cnative.encode(pts, None, depth, 2), want)


def test_hilbert_depth1_known_answers():
    # prefix-XOR of the bits (x,y,z): derived by hand, no reference involved
    kat = {(0, 0, 0): 0, (0, 0, 1): 1, (0, 1, 1): 2, (0, 1, 0): 3,
           (1, 1, 0): 4, (1, 1, 1): 5, (1, 0, 1): 6, (1, 0, 0): 7}
    pts = np.array(list(kat), dtype=np.int32)
    assert S.hilbert_code(pts, 1).tolist() == list(kat.values())


@pytest.mark.parametrize("d", [1, 2, 3, 4, 5])
def test_hilbert_is_a_hilbert_curve(d):
    cells = _all_cells(d)
    code = S.hilbert_code(cells, d)
    # bijection onto [0, 8^d)
    assert np.array_equal(np.sort(code), np.arange(8 ** d))
    # consecutive codes are face neighbours
    walk = cells[np.argsort(code)].astype(np.int64)
    assert np.all(np.abs(np.diff(walk, axis=0)).sum(1) == 1)
    # octree hierarchy: dropping a level == coding the parent cell one level up
    if d > 1:
        assert np.array_equal(code >> 3, S.hilbert_code(cells >> 1, d - 1))


@pytest.mark.parametrize("d", [1, 2, 3, 4])
def test_z_order_exhaustive_closed_form(d):
    cells = _all_cells(d)
    code = S.z_order_code(cells, d)
    want = np.zeros(len(cells), dtype=np.int64)
    for n, (x, y, z) in enumerate(cells.tolist()):
        for i in range(d):
            want[n] |= ((x >> i) & 1) << (3 * i + 2) | ((y >> i) & 1) << (3 * i + 1) | ((z >> i) & 1) << (3 * i)
    assert np.array_equal(code, want)
    assert np.array_equal(np.sort(code), np.arange(8 ** d))
    if d > 1:
        assert np.array_equal(code >> 3, S.z_order_code(cells >> 1, d - 1))


def test_z_order_known_answers():
    pts = np.array([[1, 0, 0], [0, 1, 0], [0, 0, 1], [3, 0, 0], [255, 255, 255], [256, 0, 0]], dtype=np.int32)
    assert S.z_order_code(pts, 16).tolist() == [4, 2, 1, 36, (1 << 24) - 1, 1 << 26]


def test_z_order_matches_byte_lut_form():
    # the reference evaluates the code through 256-entry tables on the low and high byte
    # (z_order.py:87-95); that form must equal the bit loop for every depth
    rng = np.random.default_rng(7)
    tab = np.arange(256, dtype=np.int64)
    zero = np.zeros(256, dtype=np.int32)
    ex = S.z_order_code(np.stack([tab, zero, zero], 1), 8)
    ey = S.z_order_code(np.stack([zero, tab, zero], 1), 8)
    ez = S.z_order_code(np.stack([zero, zero, tab], 1), 8)
    for depth in range(1, 17):
        p = rng.integers(0, 1 << 16, size=(2000, 3)).astype(np.int64)
        m = 255 if depth > 8 else (1 << depth) - 1
        key = ex[p[:, 0] & m] | ey[p[:, 1] & m] | ez[p[:, 2] & m]
        if depth > 8:
            m2 = (1 << (depth - 8)) - 1
            hi = ex[(p[:, 0] >> 8) & m2] | ey[(p[:, 1] >> 8) & m2] | ez[(p[:, 2] >> 8) & m2]
            key = hi << 24 | key
        assert np.array_equal(S.z_order_code(p.astype(np.int32), depth), key)


def test_hilbert_decode_inverts_reference_golden():
    """hilbert_decode on the codes the reference's own hilbert.py wrote for the fixture's points."""
    import os
    gold = np.load(os.path.join(os.path.dirname(__file__), "golden", "hilbert_golden.npz"))
    names = sorted(k[:-3] for k in gold.files if k.endswith("_in"))
    assert names
    for name in names:
        depth = int(name.split("_d")[1])
        # ("trunc" holds coordinates past the depth: encode keeps their low bits, decode returns those)
        assert np.array_equal(S.hilbert_decode(gold[name + "_out"], depth), gold[name + "_in"] & ((1 << depth) - 1)), name


def test_z_order_decode_hand_cases():
    """Bit 3i+2 is x's bit i, 3i+1 y's, 3i z's (z_order.py:66-101 read backwards)."""
    code = np.array([0b100, 0b010, 0b001, 0b100100, 1 << 26, (1 << 48) - 1], np.int64)
    want = [[1, 0, 0], [0, 1, 0], [0, 0, 1], [3, 0, 0], [256, 0, 0], [65535, 65535, 65535]]
    assert S.z_order_decode(code, 16).tolist() == want


@pytest.mark.parametrize("depth", [1, 5, 8, 9, 12, 16])
def test_roundtrip_and_c_agreement(depth):
    rng = np.random.default_rng(depth)
    p = rng.integers(0, 1 << depth, size=(5000, 3)).astype(np.int32)
    b = rng.integers(0, 4, size=5000).astype(np.int64)
    assert np.array_equal(S.z_order_decode(S.z_order_code(p, depth), depth), p)
    assert np.array_equal(S.hilbert_decode(S.hilbert_code(p, depth), depth), p)
    for oid, name in enumerate(S.ORDERS):
        assert np.array_equal(S.encode(p, b, depth, name), cnative.encode(p, b, depth, oid)), name
        assert np.array_equal(S.encode(p, None, depth, name), cnative.encode(p, None, depth, oid)), name


def test_batch_pack_and_trans_closed_form():
    p = np.array([[5, 9, 2]], dtype=np.int32)
    assert S.encode(np.array([[0, 0, 5]], np.int32), [3], 16, "z")[0] == (3 << 48) | S.z_order_code(np.array([[0, 0, 5]], np.int32), 16)[0]
    assert S.encode(p, [2], 9, "z-trans")[0] == (2 << 27) | S.z_order_code(np.array([[9, 5, 2]], np.int32), 9)[0]
    assert S.encode(p, [2], 9, "hilbert-trans")[0] == (2 << 27) | S.hilbert_code(np.array([[9, 5, 2]], np.int32), 9)[0]


def test_hilbert_depends_on_depth_z_does_not():
    p = np.array([[3, 1, 2], [7, 7, 0]], dtype=np.int32)
    assert np.array_equal(S.z_order_code(p, 3), S.z_order_code(p, 7))
    assert not np.array_equal(S.hilbert_code(p, 3), S.hilbert_code(p, 4))


def test_adaptive_depth():
    for mx, d in ((249, 8), (399, 9), (2999, 12)):
        assert S.serialized_depth(np.array([[0, mx, 1]])) == d


def test_serialize_order_inverse():
    rng = np.random.default_rng(3)
    cells = _all_cells(5)
    pick = rng.permutation(len(cells))[:4000]
    g = cells[pick]
    batch = np.sort(rng.integers(0, 3, size=len(g))).astype(np.int64)
    depth, code, order, inverse = S.serialize(g, batch)
    assert depth == 5 and code.shape == (4, 4000)
    for r in range(4):
        assert np.all(np.diff(code[r][order[r]]) > 0)
        assert np.array_equal(inverse[r][order[r]], np.arange(4000))
        # scenes never interleave: the batch id sits above the position bits
        assert np.all(np.diff(batch[order[r]]) >= 0)
