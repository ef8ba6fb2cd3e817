"""Hilbert serialization codes (libissm_hip.so) against the numpy oracle: integer results, compared exactly."""
import numpy as np
import pytest
import torch

from oracle import hilbert_ref as R

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("order", ["xyz", "yxz", "zxy"])
@pytest.mark.parametrize("bit", [9, 4])
def test_codes_match_oracle(order, bit):
    from dest3d_amd.serialization import hilbert_codes
    rng = np.random.default_rng(7)
    pts = rng.uniform(-4, 4, size=(3, 2000, 3)).astype(np.float32)
    pts[1] *= 0.1                                     # many points per cell: ties
    pts[2, 5] = pts[2].min(0) + np.float32(30.0)      # beyond the grid: clamped
    code = hilbert_codes(torch.from_numpy(pts).cuda(), order, bit).cpu().numpy()
    g = R.grid_coords(pts, bit)[..., list(R.ORDERS[order])]
    assert (code == R.hilbert_distance(g, bit)).all()


def test_whole_cube_is_a_unit_step_walk():
    from dest3d_amd.serialization import Serialization
    s = Serialization(order=["xyz"], bit=4)
    g = np.stack(np.meshgrid(*[np.arange(16)] * 3, indexing="ij"), -1).reshape(-1, 3)
    code = s.encode(torch.from_numpy(g).cuda()).cpu().numpy()
    assert sorted(code.tolist()) == list(range(4096))
    walk = g[np.argsort(code)]
    assert (np.abs(np.diff(walk, axis=0)).sum(1) == 1).all()


def test_module_reorders_and_restores():
    from dest3d_amd.serialization import Serialization
    torch.manual_seed(0)
    pts = (8 * torch.rand(2, 1024, 3)).cuda()
    feat = torch.randn(2, 1024, 7).cuda()
    s = Serialization(order=["xyz", "yxz"], bit=9)
    s(pts)
    assert len(s.index_list) == 2 and s.index_list[0].shape == (2, 1024)
    for i in (0, 1):
        ordered = s.reorder_points(feat, i)
        assert torch.equal(s.reversed_reorder_points(ordered), feat)
        _, idx, inv = R.serialize(pts.cpu().numpy(), s.order[i], 9)
        assert (s.index_list[i].cpu().numpy() == idx).all() and (s.reversed_index_list[i].cpu().numpy() == inv).all()
    # neighbours along the curve are neighbours in space: far closer than random pairs
    walk = s.reorder_points(pts, 0)
    step = (walk[:, 1:] - walk[:, :-1]).norm(dim=-1).median().item()
    rand = (pts[:, 1:] - pts[:, :-1]).norm(dim=-1).median().item()
    assert step < 0.25 * rand


def test_rejects_bad_arguments():
    import ctypes as C
    from dest3d_amd import _lib as L
    lib = L.load()
    a = L.HilbertArgs()
    a.batch, a.npoint, a.bits, a.cell = 1, 4, 25, 0.02
    for i in range(3):
        a.order[i] = i
    assert lib.issm_hilbert_codes(C.byref(a)) == -5
    a.bits = 9
    a.order[2] = 1
    assert lib.issm_hilbert_codes(C.byref(a)) == -2
    a.order[2] = 2
    assert lib.issm_hilbert_codes(C.byref(a)) == -1
