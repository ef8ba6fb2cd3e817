"""CPU oracle for the space-filling-curve serialization of the key points.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this module.  Plain numpy.

What it restates: models/dest_module.py:307-356 (``Serialization.forward`` / ``encode``): points are quantised
to a 2 cm grid relative to the per-sample minimum, clamped to 2**bit - 1, the three grid coordinates are permuted
by the order string, mapped to a position on a 3-D Hilbert curve, and argsorted.  The reference reads the curve
from a lookup table ``utils/hilbert/curve_template_3d_rank_9.pth`` that is not part of the repository, so the curve
itself cannot be compared: ``hilbert_distance`` is Skilling's transpose algorithm (J. Skilling, "Programming the
Hilbert curve", AIP Conf. Proc. 707, 2004), first coordinate most significant, the construction such templates are
usually generated with.  PARITY UNPINNED against the reference for the curve; pinned here are the properties that
make it a Hilbert curve (tests/test_oracle_hilbert.py): it is a bijection of the cube onto 0 .. 8**bit - 1,
consecutive positions are grid neighbours (unit steps), it starts at the origin, and the 2-D order-1 curve is the
textbook (0,0) (0,1) (1,1) (1,0).  ``grid_coords`` and ``serialize`` are pinned by direct evaluation.
"""
from __future__ import annotations

import numpy as np

ORDERS = {"xyz": (0, 1, 2), "xzy": (0, 2, 1), "yxz": (1, 0, 2), "yzx": (1, 2, 0), "zxy": (2, 0, 1), "zyx": (2, 1, 0)}


def hilbert_distance(coords, bits):
    """coords (..., n) non-negative integers < 2**bits -> position along the n-dimensional Hilbert curve."""
    X = [np.asarray(coords[..., i], dtype=np.int64).copy() for i in range(coords.shape[-1])]
    n = len(X)
    M = 1 << (bits - 1)
    Q = M
    while Q > 1:
        P = Q - 1
        for i in range(n):
            hit = (X[i] & Q) != 0
            X[0] = np.where(hit, X[0] ^ P, X[0])
            t = np.where(hit, 0, (X[0] ^ X[i]) & P)
            X[0] ^= t
            X[i] ^= t
        Q >>= 1
    for i in range(1, n):
        X[i] ^= X[i - 1]
    t = np.zeros_like(X[0])
    Q = M
    while Q > 1:
        t = np.where((X[n - 1] & Q) != 0, t ^ (Q - 1), t)
        Q >>= 1
    for i in range(n):
        X[i] ^= t
    h = np.zeros_like(X[0])
    for b in range(bits - 1, -1, -1):
        for i in range(n):
            h = (h << 1) | ((X[i] >> b) & 1)
    return h


def grid_coords(points, bits=9, cell=1.0 / 50.0):
    """points (B, N, 3) float32 -> int grid coordinates relative to the per-sample minimum, clamped to 2**bits - 1."""
    p = np.asarray(points, np.float32)
    g = np.trunc((p - p.min(axis=1, keepdims=True)) / np.float32(cell)).astype(np.int64)
    return np.minimum(g, (1 << bits) - 1)


def serialize(points, order="xyz", bits=9):
    """-> (codes (B, N), index (B, N) sorting the points along the curve, inverse index)."""
    g = grid_coords(points, bits)[..., list(ORDERS[order])]
    code = hilbert_distance(g, bits)
    idx = np.argsort(code, axis=-1, kind="stable")
    return code, idx, np.argsort(idx, axis=-1, kind="stable")
