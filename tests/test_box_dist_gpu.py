"""Box distance encoding + locality weight (libissm_hip.so) against the fp64 numpy oracle (itself pinned by torch's
grid_sample, tests/test_oracle_boxdist.py).  fp32: rel. error <= 1e-4 forward and table gradient (the sampling
position goes through a hardware log2; the table gradient is summed with LDS atomics); bf16 output: <= 1e-2."""
import numpy as np
import pytest
import torch

from oracle import boxdist_ref as R

pytestmark = pytest.mark.gpu


def _rel(a, b):
    a = np.asarray(a, np.float64)
    return np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30)


def _inputs(B, nP, nQ, seed, angles):
    rng = np.random.default_rng(seed)
    key = rng.uniform(-4, 4, size=(B, nP, 3)).astype(np.float32)
    qxyz = rng.uniform(-4, 4, size=(B, nQ, 3)).astype(np.float32)
    qsize = rng.uniform(0.1, 2.5, size=(B, nQ, 3)).astype(np.float32)
    ang = (rng.uniform(-3, 3, size=(B, nQ)) if angles else np.zeros((B, nQ))).astype(np.float32)
    return key, qxyz, qsize, ang


# the table gradient scatters with LDS atomics below 65536 (point, box) pairs and sorts by window above: both sizes
CASES = [(2, 37, 256, False, (10, 10, 10)), (1, 5, 300, True, (10, 10, 10)), (2, 64, 19, True, (4, 6, 7)),
         (1, 1, 1, False, (10, 10, 10)), (2, 160, 256, False, (10, 10, 10)), (1, 230, 300, True, (10, 10, 10)),
         (1, 1100, 64, True, (4, 6, 7)), (1, 1500, 43, True, (10, 10, 10))]   # two point segments, ragged box group


@pytest.mark.parametrize("case", CASES, ids=lambda c: "B%d_P%d_Q%d_ang%d_%dx%dx%d" % (*c[:3], int(c[3]), *c[4]))
def test_box_dist_forward_and_table_gradient(case):
    from dest3d_amd.box_dist import box_dist, box_parametrization_to_corners
    B, nP, nQ, angles, dims = case
    key, qxyz, qsize, ang = _inputs(B, nP, nQ, 11 + nP + nQ, angles)
    rng = np.random.default_rng(3)
    table = rng.standard_normal((16, *dims)).astype(np.float32)
    t = torch.from_numpy(table).cuda().requires_grad_()
    tk, tq, ts, ta = (torch.from_numpy(x).cuda() for x in (key, qxyz, qsize, ang))
    corners = box_parametrization_to_corners(tq, ts, ta)
    assert np.abs(corners.cpu().numpy() - R.box_corners(qxyz, qsize, ang)).max() < 1e-5
    dist = box_dist(t, tk, corners, ta if angles else None)
    ref = R.box_dist(key, qxyz, qsize, ang, table)
    assert dist.shape == (B, nP, nQ, 16) and dist.is_contiguous()
    e_fwd = _rel(dist.detach().cpu().numpy(), ref)
    assert e_fwd <= 2e-5
    g = rng.standard_normal(ref.shape).astype(np.float32)
    dist.backward(torch.from_numpy(g).cuda())
    gref = R.box_dist_table_grad(key, qxyz, qsize, ang, table.shape, g)
    e_bwd = _rel(t.grad.cpu().numpy(), gref)
    print(f"    pairs {B * nP * nQ}: dist err {e_fwd:.2e}, table gradient err {e_bwd:.2e}", flush=True)
    assert e_bwd <= 2e-5
    # bf16 output
    dist_bf = box_dist(t.detach(), tk, corners, ta if angles else None, out_dtype=torch.bfloat16)
    assert dist_bf.dtype == torch.bfloat16
    assert _rel(dist_bf.float().cpu().numpy(), ref) <= 1e-2


def test_local_weight_and_fused_module_call():
    from dest3d_amd.box_dist import BoxDistFun, local_weight
    B, nP, nQ = 2, 50, 256
    key, qxyz, qsize, ang = _inputs(B, nP, nQ, 5, False)
    qpos = np.concatenate([qxyz, qsize], -1)
    tk, tpos = torch.from_numpy(key).cuda(), torch.from_numpy(qpos).cuda()
    w = local_weight(tk, tpos, 15.0)
    wref = R.local_weight(key, qpos, 15.0)
    assert w.shape == (B, nP, nQ) and w.dtype == torch.float32
    assert np.abs(w.cpu().numpy() - wref).max() <= 1e-4      # values in [0, 1]; exp of up to -15 * 10
    torch.manual_seed(0)
    m = BoxDistFun(out_dim=16).cuda()
    assert set(m.state_dict()) == {"relative_coords_table", "cpb_mlps.0.weight", "cpb_mlps.0.bias", "cpb_mlps.2.weight"}
    dist, w2 = m(tk, tpos[..., :3], tpos[..., 3:], torch.zeros(B, nQ, device="cuda"), weight_query_pos=tpos)
    table = m.rpe_table().detach().double().cpu().numpy()
    ref = R.box_dist(key, qxyz, qsize, ang, table)
    assert _rel(dist.detach().cpu().numpy(), ref) <= 1e-4
    # the fused call derives centre and radius from the boxes inside the kernel: equal up to the rounding of the radius
    assert torch.allclose(w2, w, rtol=2e-4, atol=1e-7)
    dist.square().sum().backward()
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in m.parameters())
    # gradient of the MLP through the table: against autograd of the same MLP fed the oracle's table gradient
    gtab = R.box_dist_table_grad(key, qxyz, qsize, ang, table.shape, 2 * ref)
    m2 = BoxDistFun(out_dim=16).double()
    m2.load_state_dict({k: v.double().cpu() for k, v in m.state_dict().items()})
    (m2.rpe_table() * torch.from_numpy(gtab)).sum().backward()
    for (n, p), p2 in zip(m.named_parameters(), m2.parameters()):
        assert _rel(p.grad.cpu().numpy(), p2.grad.numpy()) <= 2e-3, n


def test_table_gradient_is_bit_reproducible():
    """The gradient is accumulated in 64-bit fixed point: the order of the adds cannot change it."""
    from dest3d_amd.box_dist import box_dist, box_parametrization_to_corners
    key, qxyz, qsize, ang = _inputs(2, 200, 256, 21, False)
    tk, tq, ts, ta = (torch.from_numpy(x).cuda() for x in (key, qxyz, qsize, ang))
    corners = box_parametrization_to_corners(tq, ts, ta)
    g = torch.randn(2, 200, 256, 16, generator=torch.Generator().manual_seed(1)).cuda()
    grads = []
    for _ in range(3):
        t = torch.randn(16, 10, 10, 10, generator=torch.Generator().manual_seed(2)).cuda().requires_grad_()
        box_dist(t, tk, corners).backward(g)
        grads.append(t.grad.clone())
    assert torch.equal(grads[0], grads[1]) and torch.equal(grads[0], grads[2])
    # a zero upstream gradient gives an exactly zero table gradient
    t = torch.randn(16, 10, 10, 10, generator=torch.Generator().manual_seed(2)).cuda().requires_grad_()
    box_dist(t, tk, corners).backward(torch.zeros_like(g))
    assert t.grad.abs().max().item() == 0.0
    # the fixed point is scaled to max|ddist|: upstream gradients of any magnitude give the same relative result,
    # vanishing ones a finite (zero) one; both sides of the 65536-pair switch between the two accumulation paths
    for npts in (200, 20):
        gs = g[:, :npts].contiguous()
        ref = None
        for scale in (1.0, 1e30, 1e-25, 1e-37):
            t = torch.randn(16, 10, 10, 10, generator=torch.Generator().manual_seed(2)).cuda().requires_grad_()
            box_dist(t, tk[:, :npts].contiguous(), corners).backward(gs * scale)
            assert torch.isfinite(t.grad).all()
            if ref is None:
                ref = t.grad.double()
            elif scale > 1e-30:
                assert _rel((t.grad.double() / scale).cpu().numpy(), ref.cpu().numpy()) <= 1e-6, (npts, scale)
            else:
                assert t.grad.abs().max().item() <= 1e-30


def test_box_dist_rejects_unbuilt_shapes():
    import ctypes as C
    from dest3d_amd import _lib as L
    lib = L.load()
    a = L.BoxDistArgs()
    a.batch, a.seqlen, a.nquery, a.D, a.H, a.W = 1, 4, 4, 11, 10, 10
    assert lib.issm_box_dist_fwd(C.byref(a)) == -5
    a.D = 10
    assert lib.issm_box_dist_fwd(C.byref(a)) == -1
