"""Pins of oracle/hilbert_ref.py: the properties that make the curve a Hilbert curve."""
import numpy as np

from oracle import hilbert_ref as R


def _cube(bits, n=3):
    g = np.stack(np.meshgrid(*[np.arange(1 << bits)] * n, indexing="ij"), -1).reshape(-1, n)
    return g


def test_textbook_2d_order_1():
    pts = np.array([[0, 0], [0, 1], [1, 1], [1, 0]])
    assert R.hilbert_distance(pts, 1).tolist() == [0, 1, 2, 3]


def test_bijection_unit_steps_and_origin():
    for bits in (1, 2, 3, 4):
        g = _cube(bits)
        h = R.hilbert_distance(g, bits)
        assert sorted(h.tolist()) == list(range(8 ** bits))          # a bijection onto 0 .. 8**bits - 1
        walk = g[np.argsort(h)]
        assert (walk[0] == 0).all()                                   # starts at the origin
        assert (np.abs(np.diff(walk, axis=0)).sum(1) == 1).all()      # consecutive positions are grid neighbours
    g2 = _cube(5, 2)
    walk = g2[np.argsort(R.hilbert_distance(g2, 5))]
    assert (np.abs(np.diff(walk, axis=0)).sum(1) == 1).all()


def test_nested_refinement():
    # the order-(b+1) curve visits the 8 children of a cell of the order-b curve consecutively, cells in order-b order
    g = _cube(3)
    fine = R.hilbert_distance(g, 3)
    coarse = R.hilbert_distance(g >> 1, 2)
    assert (fine >> 3 == coarse).all()


def test_grid_coords_and_serialize():
    rng = np.random.default_rng(0)
    pts = rng.uniform(-3, 9, size=(2, 50, 3)).astype(np.float32)
    pts[0, 0] = pts[0].min(0) + np.float32(20.0)       # 1000 cells: clamped to 511
    g = R.grid_coords(pts)
    for b in range(2):
        for i in range(50):
            want = np.minimum(np.trunc((pts[b, i] - pts[b].min(0)) / np.float32(0.02)).astype(np.int64), 511)
            assert (g[b, i] == want).all()
    assert g[0, 0].max() == 511
    code, idx, inv = R.serialize(pts, "yxz")
    assert (code == R.hilbert_distance(g[..., [1, 0, 2]], 9)).all()
    for b in range(2):
        assert (np.diff(code[b][idx[b]]) >= 0).all()
        assert (idx[b][inv[b]] == np.arange(50)).all()
