"""CPU oracle for the box-to-point distance encoding and the locality weight that feed the scan.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this module; tests/ use it as the
checker.  Plain numpy, fp64, written from the formulas and never importing the reference.

What each function restates (paths relative to the reference checkout):

* ``box_corners``        models/dest_module.py:26-103 (flip_axis_to_camera_tensor, get_3d_box_batch_tensor,
                         roty_batch_tensor, convert_corners_camera2lidar composed): the 8 corners of a box in the
                         input ("lidar") frame, corner order as in get_3d_box_batch_tensor
* ``corner_deltas``      models/dest_module.py:178-190: corner - key, the axis juggling around the rotation (which
                         composes to a rotation in the x-y plane), the signed log scale and the division by
                         max_value.  The rotation applied to flattened corner j = q*8 + c uses the angle of query
                         j mod nQ, because the reference tiles the angles with ``repeat((1, 8))``; this is restated
                         as it is (DEST always passes zero angles here, dest_module.py:284)
* ``grid_sample_trilinear``  torch.nn.functional.grid_sample for a 5-D input, mode "bilinear", padding "zeros",
                         align_corners=False, as BoxDistFun calls it (dest_module.py:193)
* ``box_dist``           models/dest_module.py:174-195 (BoxDistFun.forward): sum over the 8 corners, output
                         (B, nP, nQ, C)
* ``box_dist_table_grad``  the gradient of ``box_dist`` with respect to the table (what autograd of grid_sample
                         accumulates)
* ``local_weight``       models/dest_module.py:240-249

Pinning status (tests/test_oracle_boxdist.py): ``grid_sample_trilinear`` against torch's own grid_sample on the
CPU, at grid nodes (returns the table entry), and outside the volume (zero); ``box_corners`` against a hand
evaluation for axis-aligned boxes and a quarter turn; ``corner_deltas`` against a direct x-y rotation;
``box_dist_table_grad`` against finite differences; ``local_weight`` against a loop.  The reference holds no
golden vectors for these functions.
"""
from __future__ import annotations

import numpy as np

# corner sign patterns of get_3d_box_batch_tensor (dest_module.py:62-70): x uses l, y uses h, z uses w (camera frame)
_SX = np.array([1, 1, -1, -1, 1, 1, -1, -1], dtype=np.float64)
_SY = np.array([1, 1, 1, 1, -1, -1, -1, -1], dtype=np.float64)
_SZ = np.array([1, -1, -1, 1, 1, -1, -1, 1], dtype=np.float64)


def box_corners(center, size, angle):
    """center (..., 3), size (..., 3) = (l, w, h), angle (...) -> corners (..., 8, 3) in the input frame."""
    center = np.asarray(center, np.float64)
    size = np.asarray(size, np.float64)
    angle = np.asarray(angle, np.float64)
    # camera frame: (x, -z, y)
    cx, cy, cz = center[..., 0], -center[..., 2], center[..., 1]
    lx = size[..., 0:1] / 2 * _SX
    hy = size[..., 2:3] / 2 * _SY
    wz = size[..., 1:2] / 2 * _SZ
    c, s = np.cos(angle)[..., None], np.sin(angle)[..., None]
    # corners @ R^T with R = roty(angle) = [[c, 0, s], [0, 1, 0], [-s, 0, c]]
    X = lx * c + wz * s + cx[..., None]
    Y = hy + cy[..., None]
    Z = -lx * s + wz * c + cz[..., None]
    # back to the input frame: (X, Z, -Y)
    return np.stack([X, Z, -Y], axis=-1)


def corner_deltas(corners, key_xyz, angle, log_scale=512.0, max_value=4.0):
    """corners (B, nQ, 8, 3), key_xyz (B, nP, 3), angle (B, nQ) -> normalised deltas (B, nQ, 8, nP, 3)."""
    corners = np.asarray(corners, np.float64)
    key_xyz = np.asarray(key_xyz, np.float64)
    angle = np.asarray(angle, np.float64)
    B, nQ = corners.shape[:2]
    d = corners.reshape(B, nQ * 8, 1, 3) - key_xyz[:, None, :, :]
    # (x, y, z) -> (x, -z, y)
    d = np.stack([d[..., 0], -d[..., 2], d[..., 1]], axis=-1)
    ang = np.tile(angle, (1, 8))  # flattened corner j uses the angle of query j mod nQ
    c, s = np.cos(ang)[:, :, None], np.sin(ang)[:, :, None]
    # d @ R
    r0 = d[..., 0] * c - d[..., 2] * s
    r1 = d[..., 1]
    r2 = d[..., 0] * s + d[..., 2] * c
    # (X, -Z, Y) -> (X, Y, Z): negate component 1, swap components 1 and 2
    d = np.stack([r0, r2, -r1], axis=-1)
    d = np.sign(d) * np.log2(np.abs(d) * log_scale + 1.0) / np.log2(8.0)
    return (d / max_value).reshape(B, nQ, 8, -1, 3)


def _trilinear_terms(pts, D, H, W):
    """For points (N, 3) in grid_sample's (x, y, z) convention: 8 (flat index, weight, valid) triples."""
    x = ((pts[:, 0] + 1.0) * W - 1.0) / 2.0
    y = ((pts[:, 1] + 1.0) * H - 1.0) / 2.0
    z = ((pts[:, 2] + 1.0) * D - 1.0) / 2.0
    x0, y0, z0 = np.floor(x), np.floor(y), np.floor(z)
    out = []
    for dz in (0, 1):
        for dy in (0, 1):
            for dx in (0, 1):
                ix, iy, iz = x0 + dx, y0 + dy, z0 + dz
                w = (1 - np.abs(x - ix)) * (1 - np.abs(y - iy)) * (1 - np.abs(z - iz))
                ok = (ix >= 0) & (ix < W) & (iy >= 0) & (iy < H) & (iz >= 0) & (iz < D)
                flat = (np.clip(iz, 0, D - 1) * H + np.clip(iy, 0, H - 1)) * W + np.clip(ix, 0, W - 1)
                out.append((flat.astype(np.int64), np.where(ok, w, 0.0)))
    return out


def grid_sample_trilinear(table, pts):
    """table (C, D, H, W), pts (N, 3) as (x, y, z) in [-1, 1] -> (N, C)."""
    table = np.asarray(table, np.float64)
    pts = np.asarray(pts, np.float64)
    C, D, H, W = table.shape
    flat = table.reshape(C, -1)
    out = np.zeros((pts.shape[0], C))
    for idx, w in _trilinear_terms(pts, D, H, W):
        out += flat[:, idx].T * w[:, None]
    return out


def box_dist(key_xyz, query_xyz, query_size, query_angle, table, log_scale=512.0, max_value=4.0):
    """-> dist (B, nP, nQ, C): sum over the 8 corners of the table sampled at the corner-to-point deltas."""
    corners = box_corners(query_xyz, query_size, query_angle)
    delta = corner_deltas(corners, key_xyz, query_angle, log_scale, max_value)  # (B, nQ, 8, nP, 3)
    B, nQ, _, nP, _ = delta.shape
    s = grid_sample_trilinear(table, delta.reshape(-1, 3)).reshape(B, nQ, 8, nP, -1)
    return s.sum(axis=2).transpose(0, 2, 1, 3)


def box_dist_table_grad(key_xyz, query_xyz, query_size, query_angle, table_shape, ddist, log_scale=512.0,
                        max_value=4.0):
    """d(sum(dist * ddist)) / d table, ddist (B, nP, nQ, C) -> (C, D, H, W)."""
    C, D, H, W = table_shape
    corners = box_corners(query_xyz, query_size, query_angle)
    delta = corner_deltas(corners, key_xyz, query_angle, log_scale, max_value)
    B, nQ, _, nP, _ = delta.shape
    g = np.broadcast_to(np.asarray(ddist, np.float64).transpose(0, 2, 1, 3)[:, :, None], (B, nQ, 8, nP, C))
    g = g.reshape(-1, C)
    out = np.zeros((D * H * W, C))
    for idx, w in _trilinear_terms(delta.reshape(-1, 3), D, H, W):
        np.add.at(out, idx, g * w[:, None])
    return out.T.reshape(C, D, H, W)


def local_weight(key_xyz, query_pos, weight_dist=15.0, min_radius=0.64):
    """key_xyz (B, nP, 3), query_pos (B, nQ, 6) = centre + size -> (B, nP, nQ):
    exp(weight_dist * min(radius - |key - centre|, 0)), radius = max(|size|, min_radius)."""
    key_xyz = np.asarray(key_xyz, np.float64)
    query_pos = np.asarray(query_pos, np.float64)
    radius = np.maximum(np.sqrt((query_pos[:, :, 3:] ** 2).sum(-1)), min_radius)
    d = np.sqrt(((key_xyz[:, :, None, :] - query_pos[:, None, :, :3]) ** 2).sum(-1))
    return np.exp(weight_dist * np.minimum(radius[:, None, :] - d, 0.0))
