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


def test_points_on_cell_boundaries_land_where_the_host_division_puts_them():
    """Points whose offset from the sample minimum is the float nearest to k * cell: the quotient is then within an
    ulp of the integer k, and whether trunc gives k or k - 1 depends on the division being correctly rounded.  The
    kernel must agree with torch.div(..., rounding_mode="trunc") on the CPU for every one of them
    (models/dest_module.py:326-329)."""
    from dest3d_amd.serialization import hilbert_codes
    cell = np.float32(1.0 / 50.0)
    k = np.arange(512, dtype=np.float32)
    pts = np.zeros((1, 3 * 512 + 1, 3), np.float32)           # row 0 stays at the origin: the sample minimum
    for ax in range(3):
        pts[0, 1 + ax * 512:1 + (ax + 1) * 512, ax] = k * cell
    t = torch.from_numpy(pts)
    want_grid = torch.div(t - t.min(1, keepdim=True)[0], float(cell), rounding_mode="trunc").long().clamp_max(511).numpy()
    assert (R.grid_coords(pts, 9) == want_grid).all()        # the oracle is the host division
    code = hilbert_codes(t.cuda(), "xyz", 9).cpu().numpy()
    assert (code == R.hilbert_distance(want_grid, 9)).all()
    # the case is not vacuous: some quotients do fall short of their integer
    assert (want_grid[0, 1:513, 0] != np.arange(512)).any()


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


@pytest.mark.parametrize("n", [1, 2, 5, 300, 1000, 1024, 1025, 4096])
def test_one_launch_order_equals_codes_and_stable_sorts(n):
    """issm_hilbert_order (minimum corner, positions, stable sort, inverse permutation of every order in one launch)
    against the separate steps: issm_hilbert_codes and torch's stable argsort, twice.  Many points share a cell (a
    coarse second half), so the order inside ties is tested too."""
    from dest3d_amd.serialization import ORDERS, hilbert_codes, hilbert_order
    print(f"[case] hilbert order n={n}", flush=True)
    g = torch.Generator().manual_seed(40 + n)
    pts = 8 * torch.rand(3, n, 3, generator=g)
    pts[:, n // 2:] = torch.round(pts[:, n // 2:] * 2) / 2      # a 0.5 m lattice: dozens of points per 2 cm cell
    pts[1, 0] = -3.0                                             # every sample has its own minimum corner
    pts = pts.cuda()
    orders = list(ORDERS)
    idx, inv = hilbert_order(pts, orders, 9)
    assert idx.shape == inv.shape == (6, 3, n) and idx.dtype == torch.int64
    for j, o in enumerate(orders):
        want = torch.argsort(hilbert_codes(pts, o, 9), dim=-1, stable=True)
        assert torch.equal(idx[j], want), o
        assert torch.equal(inv[j], torch.argsort(want, dim=-1)), o


@pytest.mark.parametrize("bad", [float("nan"), float("inf"), float("-inf")])
def test_non_finite_coordinates_sort_alike_in_the_one_launch_kernel_and_in_the_separate_steps(bad):
    """A NaN or infinite coordinate (a corrupt point): no conversion of NaN to an integer, and the one-launch kernel
    agrees with issm_hilbert_codes + a stable argsort -- the path longer samples take -- on index and inverse.  The
    minimum corner keeps a NaN the way torch.amin does, so both see the same cells; the result is a permutation."""
    from dest3d_amd.serialization import ORDERS, hilbert_codes, hilbert_order
    print(f"[case] hilbert order with a {bad} coordinate", flush=True)
    g = torch.Generator().manual_seed(7)
    pts = 8 * torch.rand(3, 500, 3, generator=g)
    pts[0, 17, 1] = bad                    # sample 0: one bad coordinate; sample 1: a whole bad point; sample 2: clean
    pts[1, 250] = bad
    pts = pts.cuda()
    orders = list(ORDERS)
    idx, inv = hilbert_order(pts, orders, 9)
    for j, o in enumerate(orders):
        want = torch.argsort(hilbert_codes(pts, o, 9), dim=-1, stable=True)
        assert torch.equal(idx[j], want), o
        assert torch.equal(inv[j], torch.argsort(want, dim=-1)), o
        assert torch.equal(torch.sort(idx[j], dim=-1).values, torch.arange(500, device="cuda").expand(3, 500))


def test_order_rejects_what_it_does_not_hold():
    import ctypes as C
    from dest3d_amd import _lib as L
    from dest3d_amd.serialization import Serialization
    lib = L.load()
    a = L.HilbertOrderArgs()
    a.batch, a.npoint, a.bits, a.norder, a.cell = 1, 5000, 9, 1, 0.02
    for i in range(3):
        a.order[0][i] = i
    assert lib.issm_hilbert_order(C.byref(a)) == -5 and b"4096" in lib.issm_last_error()
    a.npoint, a.bits = 100, 18
    assert lib.issm_hilbert_order(C.byref(a)) == -5
    a.bits, a.norder = 9, 7
    assert lib.issm_hilbert_order(C.byref(a)) == -2
    a.norder = 1
    assert lib.issm_hilbert_order(C.byref(a)) == -1            # no pointers
    # the module falls back to codes + library sorts above the limit, with the same result as the oracle
    torch.manual_seed(1)
    pts = (8 * torch.rand(1, 5000, 3)).cuda()
    s = Serialization(order=["zyx"], bit=9)
    s(pts)
    _, idx, inv = R.serialize(pts.cpu().numpy(), "zyx", 9)
    assert (s.index_list[0].cpu().numpy() == idx).all() and (s.reversed_index_list[0].cpu().numpy() == inv).all()
