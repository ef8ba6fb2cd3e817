"""Point-set operators (libissm_hip.so, issm_pn2_*) against the numpy oracle: indices exactly, values to fp32
rounding (the gradients are float-atomic sums: 1e-5 relative)."""
import numpy as np
import pytest
import torch

from oracle import pointnet2_ref as R

pytestmark = pytest.mark.gpu


def _cuda(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("shape", [(2, 700, 64), (1, 5000, 256), (3, 37, 37), (1, 1, 1)])
def test_furthest_point_sampling(shape):
    from dest3d_amd.pointnet2_utils import furthest_point_sample
    B, N, npoint = shape
    rng = np.random.default_rng(N)
    xyz = rng.uniform(-4, 4, size=(B, N, 3)).astype(np.float32)
    if N > 10:
        xyz[0, 3] = 0.0            # padding point at the origin: never drawn
        xyz[0, 7] = xyz[0, 5]      # a duplicate
    idx = furthest_point_sample(_cuda(xyz), npoint)
    assert idx.dtype == torch.int32 and idx.shape == (B, npoint)
    assert (idx.cpu().numpy() == R.furthest_point_sampling(xyz, npoint)).all()


def test_furthest_point_sampling_beyond_the_register_path():
    from dest3d_amd.pointnet2_utils import furthest_point_sample
    rng = np.random.default_rng(9)
    xyz = rng.uniform(-4, 4, size=(1, 50000, 3)).astype(np.float32)
    idx = furthest_point_sample(_cuda(xyz), 48).cpu().numpy()
    assert (idx == R.furthest_point_sampling(xyz, 48)).all()


@pytest.mark.parametrize("seed,npoint", [(3, 1024), (8, 1024), (54, 1024)])
def test_furthest_point_sampling_near_ties_go_the_way_of_plain_fp32_steps(seed, npoint):
    """Clouds in which two candidates' running minimum distances come within one unit in the last place of each other
    (draws 960, 885 and 874 of these seeds): a squared distance evaluated with a fused multiply-add, fma(dz, dz,
    fma(dy, dy, dx dx)), rounds the other way there and draws another point from then on.  The kernel evaluates
    (dx dx + dy dy) + dz dz with every operation rounded, like the oracle."""
    from dest3d_amd.pointnet2_utils import furthest_point_sample
    xyz = np.random.default_rng(seed).uniform(-2, 2, size=(1, 4096, 3)).astype(np.float32)
    idx = furthest_point_sample(_cuda(xyz), npoint).cpu().numpy()
    assert (idx == R.furthest_point_sampling(xyz, npoint)).all()


@pytest.mark.parametrize("shape", [(2, 3000, 128, 0.6, 16), (1, 100, 7, 0.3, 64), (2, 65, 5, 10.0, 3), (1, 40, 4, 1e-3, 8)])
def test_ball_query(shape):
    from dest3d_amd.pointnet2_utils import ball_query
    B, N, M, radius, nsample = shape
    rng = np.random.default_rng(N + M)
    xyz = rng.uniform(-2, 2, size=(B, N, 3)).astype(np.float32)
    q = xyz[:, rng.integers(0, N, size=M)] + rng.normal(0, 0.05, size=(B, M, 3)).astype(np.float32)
    q[0, 0] = 100.0
    idx = ball_query(radius, nsample, _cuda(xyz), _cuda(q.astype(np.float32)))
    assert idx.dtype == torch.int32
    assert (idx.cpu().numpy() == R.ball_query(radius, nsample, xyz, q.astype(np.float32))).all()


def test_three_nn_and_interpolate():
    from dest3d_amd.pointnet2_utils import three_interpolate, three_nn
    rng = np.random.default_rng(5)
    B, n, m, c = 2, 777, 300, 19
    u = rng.uniform(-2, 2, size=(B, n, 3)).astype(np.float32)
    k = rng.uniform(-2, 2, size=(B, m, 3)).astype(np.float32)
    dist, idx = three_nn(_cuda(u), _cuda(k))
    d2_ref, idx_ref = R.three_nn(u, k)
    assert (idx.cpu().numpy() == idx_ref).all()
    assert np.allclose(dist.cpu().numpy(), np.sqrt(d2_ref), rtol=1e-6, atol=0)
    feats = rng.standard_normal((B, c, m)).astype(np.float32)
    w = (1.0 / (np.sqrt(d2_ref) + 1e-8))
    w = (w / w.sum(-1, keepdims=True)).astype(np.float32)
    f = _cuda(feats).requires_grad_()
    y = three_interpolate(f, idx, _cuda(w))
    ref = R.three_interpolate(feats, idx_ref, w)
    assert np.abs(y.detach().cpu().numpy() - ref).max() <= 1e-5 * np.abs(ref).max()
    gy = rng.standard_normal(ref.shape).astype(np.float32)
    y.backward(_cuda(gy))
    gref = R.three_interpolate_grad(gy, idx_ref, w, m)
    assert np.abs(f.grad.cpu().numpy() - gref).max() <= 1e-5 * np.abs(gref).max()
    # fewer than three known points
    dist, idx = three_nn(_cuda(u[:, :5]), _cuda(k[:, :2]))
    assert torch.isinf(dist[..., 2]).all() and (idx[..., 2] == 0).all()


def test_group_and_gather_with_gradients():
    from dest3d_amd.pointnet2_utils import gather_operation, grouping_operation
    rng = np.random.default_rng(6)
    B, C, N, M, S = 2, 13, 500, 60, 16
    pts = rng.standard_normal((B, C, N)).astype(np.float32)
    idx = rng.integers(0, N, size=(B, M, S)).astype(np.int32)
    idx[0, 0, :] = 7                                  # many duplicates: the gradient accumulates
    f = _cuda(pts).requires_grad_()
    g = grouping_operation(f, _cuda(idx))
    assert (g.detach().cpu().numpy() == R.group_points(pts, idx)).all()
    gy = rng.standard_normal(g.shape).astype(np.float32)
    g.backward(_cuda(gy))
    gref = R.group_points_grad(gy, idx, N)
    assert np.abs(f.grad.cpu().numpy() - gref).max() <= 1e-5 * np.abs(gref).max()
    f2 = _cuda(pts).requires_grad_()
    y = gather_operation(f2, _cuda(idx[:, :, 0].copy()))
    assert (y.detach().cpu().numpy() == R.gather_points(pts, idx[:, :, 0])).all()
    gy1 = rng.standard_normal(y.shape).astype(np.float32)
    y.backward(_cuda(gy1))
    g1 = R.gather_points_grad(gy1, idx[:, :, 0], N)
    assert np.abs(f2.grad.cpu().numpy() - g1).max() <= 1e-5 * np.abs(g1).max()


def test_reference_layout_gradient_entry_points():
    """issm_pn2_group_points_grad / issm_pn2_three_interpolate_grad write the (b, c, n) layout directly (the Python
    wrappers use the channel-last variants): called here through the C ABI."""
    from dest3d_amd import _lib as L
    lib = L.load()
    rng = np.random.default_rng(12)
    B, C, N, M, S, n3 = 2, 70, 90, 11, 5, 33
    idx = rng.integers(0, N, size=(B, M, S)).astype(np.int32)
    gy = rng.standard_normal((B, C, M, S)).astype(np.float32)
    tg, ti = _cuda(gy), _cuda(idx)
    out = torch.zeros(B, C, N, device="cuda")
    st = L.current_stream_ptr(out.device)
    L.check(lib.issm_pn2_group_points_grad(B, C, N, M, S, tg.data_ptr(), ti.data_ptr(), out.data_ptr(), st), "group grad")
    ref = R.group_points_grad(gy, idx, N)
    assert np.abs(out.cpu().numpy() - ref).max() <= 1e-5 * np.abs(ref).max()
    out_cl = torch.zeros(B, N, C, device="cuda")
    L.check(lib.issm_pn2_group_points_grad_cl(B, C, N, M, S, tg.data_ptr(), ti.data_ptr(), out_cl.data_ptr(), st), "group grad cl")
    assert np.abs(out_cl.transpose(1, 2).cpu().numpy() - ref).max() <= 1e-5 * np.abs(ref).max()
    i3 = rng.integers(0, N, size=(B, n3, 3)).astype(np.int32)
    w3 = rng.uniform(0, 1, size=(B, n3, 3)).astype(np.float32)
    g3 = rng.standard_normal((B, C, n3)).astype(np.float32)
    out3 = torch.zeros(B, C, N, device="cuda")
    tg3, ti3, tw3 = _cuda(g3), _cuda(i3), _cuda(w3)     # kept alive until the kernel has run
    L.check(lib.issm_pn2_three_interpolate_grad(B, C, n3, N, tg3.data_ptr(), ti3.data_ptr(), tw3.data_ptr(),
                                                out3.data_ptr(), st), "interp grad")
    torch.cuda.synchronize()
    ref3 = R.three_interpolate_grad(g3, i3, w3, N)
    assert np.abs(out3.cpu().numpy() - ref3).max() <= 1e-5 * np.abs(ref3).max()


def test_query_and_group_module():
    from dest3d_amd.pointnet2_utils import GroupAll, QueryAndGroup, furthest_point_sample, gather_operation
    rng = np.random.default_rng(8)
    B, N, C, M, S = 2, 400, 5, 32, 8
    xyz = rng.uniform(-1, 1, size=(B, N, 3)).astype(np.float32)
    feats = rng.standard_normal((B, C, N)).astype(np.float32)
    txyz, tf = _cuda(xyz), _cuda(feats)
    fps = furthest_point_sample(txyz, M)
    new_xyz = gather_operation(txyz.transpose(1, 2).contiguous(), fps).transpose(1, 2).contiguous()
    out, gxyz = QueryAndGroup(0.4, S, use_xyz=True, ret_grouped_xyz=True, normalize_xyz=True)(txyz, new_xyz, tf)
    assert out.shape == (B, 3 + C, M, S) and gxyz.shape == (B, 3, M, S)
    idx = R.ball_query(0.4, S, xyz, new_xyz.cpu().numpy())
    want_xyz = (R.group_points(xyz.transpose(0, 2, 1), idx) - new_xyz.cpu().numpy().transpose(0, 2, 1)[..., None]) / 0.4
    assert np.allclose(gxyz.cpu().numpy(), want_xyz, atol=1e-6)
    assert (out[:, 3:].cpu().numpy() == R.group_points(feats, idx)).all()
    assert GroupAll()(txyz, None, tf).shape == (B, 3 + C, 1, N)


def test_error_codes():
    from dest3d_amd import _lib as L
    lib = L.load()
    assert lib.issm_pn2_furthest_point_sampling(1, 10, 4, None, None, None, None) == -1
    assert lib.issm_pn2_furthest_point_sampling(1, 0, 4, None, None, None, None) == -2
    assert lib.issm_pn2_ball_query(-1, 10, 4, 0.5, 8, None, None, None, None) == -2
    assert lib.issm_pn2_group_points(1, 2, 0, 4, 4, None, None, None, None) == -2
    assert lib.issm_pn2_three_nn(0, 5, 5, None, None, None, None, None) == 0
