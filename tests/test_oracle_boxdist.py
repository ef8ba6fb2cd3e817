"""Pins of oracle/boxdist_ref.py (CPU): torch's grid_sample as the library routine, hand-evaluated boxes,
a direct x-y rotation, exact linearity in the table, and a loop for the locality weight."""
import numpy as np
import torch
import torch.nn.functional as F

from oracle import boxdist_ref as R


def test_grid_sample_matches_torch_library_routine():
    rng = np.random.default_rng(0)
    table = rng.standard_normal((5, 4, 6, 7))           # unequal D, H, W: an axis mix-up cannot cancel
    pts = rng.uniform(-1.35, 1.35, size=(4000, 3))
    got = R.grid_sample_trilinear(table, pts)
    ref = F.grid_sample(torch.from_numpy(table)[None], torch.from_numpy(pts).view(1, 1, 1, -1, 3), mode="bilinear",
                        padding_mode="zeros", align_corners=False)[0, :, 0, 0].T.numpy()
    assert np.abs(got - ref).max() < 1e-12


def test_grid_sample_at_nodes_and_outside():
    rng = np.random.default_rng(1)
    table = rng.standard_normal((3, 4, 5, 6))
    C, D, H, W = table.shape
    iz, iy, ix = np.meshgrid(np.arange(D), np.arange(H), np.arange(W), indexing="ij")
    pts = np.stack([(2 * ix + 1) / W - 1, (2 * iy + 1) / H - 1, (2 * iz + 1) / D - 1], -1).reshape(-1, 3)
    got = R.grid_sample_trilinear(table, pts)
    assert np.abs(got - table.reshape(C, -1).T).max() < 1e-12
    far = np.array([[1.5, 0.0, 0.0], [0.0, -1.6, 0.0], [0.2, 0.1, 1.41]])
    assert np.abs(R.grid_sample_trilinear(table, far)).max() == 0.0


def test_box_corners_by_hand():
    c = R.box_corners([1.0, 2.0, 3.0], [2.0, 4.0, 6.0], 0.0)
    # corner 0: +l/2 along x, +w/2 along y, and +h/2 along camera-y which is -z
    assert np.allclose(c[0], [2.0, 4.0, 0.0])
    assert np.allclose(c[6], [0.0, 0.0, 6.0])
    want = {(1 + sx, 2 + 2 * sy, 3 + 3 * sz) for sx in (-1, 1) for sy in (-1, 1) for sz in (-1, 1)}
    assert {tuple(np.round(v, 12)) for v in c} == want
    # quarter turn: camera roty maps local (lx, wz) to (wz, -lx) in the x-y plane
    q = R.box_corners([1.0, 2.0, 3.0], [2.0, 4.0, 6.0], np.pi / 2)
    assert np.allclose(q[0], [1 + 2.0, 2 - 1.0, 0.0])
    # a batch keeps its leading shape
    b = R.box_corners(np.zeros((2, 5, 3)), np.ones((2, 5, 3)), np.zeros((2, 5)))
    assert b.shape == (2, 5, 8, 3)


def test_corner_deltas_is_xy_rotation_then_signed_log():
    rng = np.random.default_rng(2)
    B, nQ, nP, ang = 2, 3, 7, 0.7
    corners = rng.uniform(-3, 3, size=(B, nQ, 8, 3))
    key = rng.uniform(-3, 3, size=(B, nP, 3))
    got = R.corner_deltas(corners, key, np.full((B, nQ), ang))
    d = corners[:, :, :, None, :] - key[:, None, None, :, :]
    rot = np.stack([d[..., 0] * np.cos(ang) - d[..., 1] * np.sin(ang),
                    d[..., 0] * np.sin(ang) + d[..., 1] * np.cos(ang), d[..., 2]], -1)
    want = np.sign(rot) * np.log(np.abs(rot) * 512 + 1) / np.log(8) / 4
    assert np.abs(got - want).max() < 1e-12
    zero = R.corner_deltas(corners, key, np.zeros((B, nQ)))
    assert np.abs(zero - np.sign(d) * np.log(np.abs(d) * 512 + 1) / np.log(8) / 4).max() < 1e-12


def test_box_dist_shape_and_linearity_in_table():
    rng = np.random.default_rng(3)
    B, nQ, nP, C = 2, 3, 5, 4
    key = rng.uniform(-2, 2, size=(B, nP, 3))
    qxyz = rng.uniform(-2, 2, size=(B, nQ, 3))
    qsize = rng.uniform(0.2, 2, size=(B, nQ, 3))
    ang = np.zeros((B, nQ))
    table = rng.standard_normal((C, 6, 6, 6))
    dist = R.box_dist(key, qxyz, qsize, ang, table)
    assert dist.shape == (B, nP, nQ, C)
    # a constant table samples to 8 * constant wherever all corners fall inside the volume
    ones = R.box_dist(key * 0.01, qxyz * 0.01, qsize * 0.01, ang, np.ones((1, 6, 6, 6)))
    assert np.abs(ones - 8.0).max() < 1e-12
    # gradient with respect to the table: dist is linear in it, so a unit perturbation gives the exact derivative
    ddist = rng.standard_normal(dist.shape)
    grad = R.box_dist_table_grad(key, qxyz, qsize, ang, table.shape, ddist)
    for _ in range(6):
        idx = tuple(rng.integers(0, s) for s in table.shape)
        e = np.zeros_like(table)
        e[idx] = 1.0
        assert abs((R.box_dist(key, qxyz, qsize, ang, e) * ddist).sum() - grad[idx]) < 1e-10


def test_local_weight_against_a_loop():
    rng = np.random.default_rng(4)
    key = rng.uniform(-2, 2, size=(2, 6, 3))
    qpos = np.concatenate([rng.uniform(-2, 2, size=(2, 4, 3)), rng.uniform(0.05, 1.5, size=(2, 4, 3))], -1)
    got = R.local_weight(key, qpos, 15.0)
    for b in range(2):
        for p in range(6):
            for q in range(4):
                r = max(np.linalg.norm(qpos[b, q, 3:]), 0.64)
                d = np.linalg.norm(key[b, p] - qpos[b, q, :3])
                assert abs(got[b, p, q] - np.exp(15.0 * min(r - d, 0.0))) < 1e-14
