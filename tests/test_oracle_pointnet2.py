"""Pins of oracle/pointnet2_ref.py: every operator against an independent formulation."""
import numpy as np

from oracle import pointnet2_ref as R


def test_fps_is_greedy_max_min():
    rng = np.random.default_rng(0)
    xyz = rng.uniform(1, 5, size=(2, 60, 3)).astype(np.float32)      # away from the origin: nothing skipped
    idx = R.furthest_point_sampling(xyz, 12)
    for b in range(2):
        p = xyz[b].astype(np.float64)
        chosen = [0]
        for s in range(1, 12):
            dmin = np.min(((p[:, None, :] - p[chosen][None, :, :]) ** 2).sum(-1), axis=1)
            chosen.append(int(np.argmax(dmin)))
        assert idx[b].tolist() == chosen
    assert len(set(idx[0].tolist())) == 12


def test_fps_skips_points_at_the_origin():
    xyz = np.array([[[1, 0, 0], [0, 0, 0], [0.01, 0.01, 0.01], [3, 0, 0], [-2, 0, 0]]], np.float32)
    idx = R.furthest_point_sampling(xyz, 3)[0].tolist()
    assert idx == [0, 4, 3]                       # 1 and 2 (|p|^2 <= 1e-3) are never drawn


def test_ball_query_definition():
    rng = np.random.default_rng(1)
    xyz = rng.uniform(-1, 1, size=(2, 80, 3)).astype(np.float32)
    q = rng.uniform(-1, 1, size=(2, 9, 3)).astype(np.float32)
    q[0, 0] = 50.0                                # no neighbour at all
    idx = R.ball_query(0.5, 6, xyz, q)
    assert (idx[0, 0] == 0).all()
    for b in range(2):
        for j in range(9):
            d = np.sqrt(((xyz[b].astype(np.float64) - q[b, j]) ** 2).sum(-1))
            hits = [k for k in range(80) if d[k] < 0.5 - 1e-6]
            sure = [k for k in range(80) if d[k] < 0.5 + 1e-6]
            got = idx[b, j].tolist()
            if not sure:
                continue
            want = (hits + [hits[0]] * 6)[:6] if hits else None
            if hits == sure:
                assert got == want


def test_three_nn_against_full_sort():
    rng = np.random.default_rng(2)
    u = rng.uniform(-1, 1, size=(2, 30, 3)).astype(np.float32)
    k = rng.uniform(-1, 1, size=(2, 50, 3)).astype(np.float32)
    d2, idx = R.three_nn(u, k)
    for b in range(2):
        full = ((u[b].astype(np.float64)[:, None] - k[b].astype(np.float64)[None]) ** 2).sum(-1)
        assert (np.argsort(full, axis=1)[:, :3] == idx[b]).all()
        assert np.allclose(np.sort(full, axis=1)[:, :3], d2[b], rtol=1e-5)
    d2, idx = R.three_nn(u[:, :4], k[:, :2])      # fewer than 3 known points: the missing ones are +inf
    assert np.isinf(d2[..., 2]).all() and (idx[..., 2] == 0).all()


def test_group_gather_interpolate_and_their_gradients():
    rng = np.random.default_rng(3)
    B, C, N, M, S = 2, 3, 11, 5, 4
    pts = rng.standard_normal((B, C, N))
    idx = rng.integers(0, N, size=(B, M, S)).astype(np.int32)
    g = R.group_points(pts, idx)
    for b in range(B):
        for c in range(C):
            for j in range(M):
                for s in range(S):
                    assert g[b, c, j, s] == pts[b, c, idx[b, j, s]]
    assert (R.gather_points(pts, idx[:, :, 0]) == g[..., 0]).all()
    # the gradients are the transposes of linear maps: <grad(gy), x> == <gy, forward(x)>
    gy = rng.standard_normal(g.shape)
    assert abs((R.group_points_grad(gy, idx, N) * pts).sum() - (gy * g).sum()) < 1e-10
    gy1 = rng.standard_normal((B, C, M))
    assert abs((R.gather_points_grad(gy1, idx[:, :, 0], N) * pts).sum() - (gy1 * g[..., 0]).sum()) < 1e-10
    n = 7
    i3 = rng.integers(0, N, size=(B, n, 3)).astype(np.int32)
    w3 = rng.uniform(0, 1, size=(B, n, 3))
    y = R.three_interpolate(pts, i3, w3)
    for b in range(B):
        for c in range(C):
            for j in range(n):
                assert abs(y[b, c, j] - sum(w3[b, j, k] * pts[b, c, i3[b, j, k]] for k in range(3))) < 1e-12
    gy2 = rng.standard_normal(y.shape)
    assert abs((R.three_interpolate_grad(gy2, i3, w3, N) * pts).sum() - (gy2 * y).sum()) < 1e-10
