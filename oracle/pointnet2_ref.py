"""CPU oracle for the point-set operators of the PointNet++ backbone.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this module.  Plain numpy; distances are
evaluated in float32 steps -- (dx*dx + dy*dy) + dz*dz with every operation rounded -- so that index choices are
well defined.

What each function restates (paths relative to the reference checkout; the definitions, not the thread layouts):

* ``furthest_point_sampling``  pointnet2/_ext_src/src/sampling_gpu.cu:84-180 with sampling.cpp:70-91: start at point
                               0, running minimum distance initialised to 1e10, points with |p|^2 <= 1e-3 skipped,
                               next = argmax.  Equal maxima go to the smaller index here; the reference's choice
                               among *exactly* equal distances depends on its block size (PARITY UNPINNED for such ties)
* ``ball_query``               ball_query_gpu.cu:20-44: first nsample hits in index order, the rest repeat the
                               first hit, zeros when there is none
* ``group_points`` / ``gather_points`` and their gradients   group_points_gpu.cu:10-78, sampling_gpu.cu:10-60
* ``three_nn``                 interpolate_gpu.cu:10-70: three smallest squared distances, strict comparisons in
                               index order (ties to the smaller index)
* ``three_interpolate`` and its gradient   interpolate_gpu.cu:72-157

Pinning status (tests/test_oracle_pointnet2.py): every function against an independent formulation -- sampling
against a set-based max-min loop in float64 on well separated points plus its defining property; ball query
against a sorted-hits formulation; 3-NN against a full argsort; grouping / gathering / interpolation against fancy
indexing and the gradients against finite differences of the forward (they are linear maps).
"""
from __future__ import annotations

import numpy as np


def _d2(a, b):
    """squared distance, float32 steps; a (..., 3), b (..., 3) broadcastable."""
    a = np.asarray(a, np.float32)
    b = np.asarray(b, np.float32)
    d = a - b
    return (d[..., 0] * d[..., 0] + d[..., 1] * d[..., 1]) + d[..., 2] * d[..., 2]


def furthest_point_sampling(xyz, npoint):
    xyz = np.asarray(xyz, np.float32)
    B, N, _ = xyz.shape
    out = np.zeros((B, npoint), np.int32)
    for b in range(B):
        p = xyz[b]
        live = _d2(p, np.zeros(3, np.float32)) > np.float32(1e-3)
        temp = np.full(N, 1e10, np.float32)
        old = 0
        for s in range(1, npoint):
            d = _d2(p, p[old])
            temp = np.where(live, np.minimum(temp, d), temp)
            cand = np.where(live, temp, np.float32(-1.0))
            old = int(np.argmax(cand)) if cand.max() > -1.0 else 0   # argmax returns the first maximum
            out[b, s] = old
    return out


def ball_query(radius, nsample, xyz, new_xyz):
    xyz = np.asarray(xyz, np.float32)
    new_xyz = np.asarray(new_xyz, np.float32)
    B, M, _ = new_xyz.shape
    out = np.zeros((B, M, nsample), np.int32)
    r2 = np.float32(radius) * np.float32(radius)
    for b in range(B):
        for j in range(M):
            hits = np.nonzero(_d2(xyz[b], new_xyz[b, j]) < r2)[0]
            if len(hits):
                out[b, j, :] = hits[0]
                k = min(nsample, len(hits))
                out[b, j, :k] = hits[:k]
    return out


def group_points(points, idx):
    """points (B, C, N), idx (B, M, S) -> (B, C, M, S)."""
    points = np.asarray(points)
    idx = np.asarray(idx)
    return np.stack([points[b][:, idx[b]] for b in range(points.shape[0])])


def group_points_grad(grad_out, idx, n):
    grad_out = np.asarray(grad_out, np.float64)
    B, C = grad_out.shape[:2]
    out = np.zeros((B, C, n))
    for b in range(B):
        for c in range(C):
            np.add.at(out[b, c], np.asarray(idx[b]).ravel(), grad_out[b, c].ravel())
    return out


def gather_points(points, idx):
    return group_points(points, np.asarray(idx)[:, :, None])[..., 0]


def gather_points_grad(grad_out, idx, n):
    return group_points_grad(np.asarray(grad_out)[..., None], np.asarray(idx)[:, :, None], n)


def three_nn(unknown, known):
    unknown = np.asarray(unknown, np.float32)
    known = np.asarray(known, np.float32)
    B, n, _ = unknown.shape
    dist2 = np.full((B, n, 3), np.inf, np.float32)
    idx = np.zeros((B, n, 3), np.int32)
    for b in range(B):
        d = _d2(unknown[b][:, None, :], known[b][None, :, :])       # (n, m)
        order = np.argsort(d, axis=1, kind="stable")[:, :3]          # stable: ties to the smaller index
        k = order.shape[1]
        dist2[b, :, :k] = np.take_along_axis(d, order, axis=1)
        idx[b, :, :k] = order
    return dist2, idx


def three_interpolate(points, idx, weight):
    """points (B, c, m), idx / weight (B, n, 3) -> (B, c, n)."""
    points = np.asarray(points, np.float64)
    out = np.zeros((points.shape[0], points.shape[1], idx.shape[1]))
    for b in range(points.shape[0]):
        for k in range(3):
            out[b] += points[b][:, idx[b, :, k]] * np.asarray(weight, np.float64)[b, :, k][None, :]
    return out


def three_interpolate_grad(grad_out, idx, weight, m):
    grad_out = np.asarray(grad_out, np.float64)
    B, c, n = grad_out.shape
    out = np.zeros((B, c, m))
    for b in range(B):
        for k in range(3):
            contrib = grad_out[b] * np.asarray(weight, np.float64)[b, :, k][None, :]
            for ch in range(c):
                np.add.at(out[b, ch], idx[b, :, k], contrib[ch])
    return out
