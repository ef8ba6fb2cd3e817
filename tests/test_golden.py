"""Golden vectors under tests/golden/ (written by tests/golden/make_fixtures.py from the fp64 oracle).

CPU: the stored outputs are re-derived by an independent scalar numpy loop, and the oracle still
reproduces its stored outputs and gradients.  GPU: the HIP operator reproduces them through the C ABI
(fp32: forward <= 1e-4, gradients <= 1e-3, both as ||a-b||_2/||b||_2 and max|a-b|/max|b|)."""
import glob
import math
import os

import numpy as np
import pytest
import torch

from oracle import issm_ref as R

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
SCANS = sorted(glob.glob(os.path.join(HERE, "scan_*.npz")))
NORMS = sorted(glob.glob(os.path.join(HERE, "rmsnorm_*.npz")))
LAYERNORMS = sorted(glob.glob(os.path.join(HERE, "layernorm_*.npz")))
FWD32, BWD32 = 1e-4, 1e-3


def _load(path):
    with np.load(path, allow_pickle=False) as f:
        return {k: f[k] for k in f.files}


def _scalar_scan(f):
    """Token-by-token recurrence with scalar loops, written without the oracle's helpers."""
    x, dt, A, B, C, D, h0 = (f["in_" + k] for k in ("x", "dt", "A", "B", "C", "D", "h0"))
    bias = f.get("in_dt_bias")
    z = f.get("in_z")
    lo, hi = f["dt_limit"]
    seq = f.get("seq_idx")   # packed rows: no state is carried over a change of id
    Bsz, L, H, P = x.shape
    N, G = dt.shape[-1], B.shape[2]
    y = np.zeros_like(x)
    fin = np.zeros_like(h0)
    for b in range(Bsz):
        for h in range(H):
            g = h // (H // G)
            for n in range(N):
                d = dt[b, :, h, n] + (bias[h, n] if bias is not None else 0.0)
                if bool(f["softplus"]):
                    d = np.where(d <= 20.0, np.log1p(np.exp(np.minimum(d, 20.0))), d)
                d = np.clip(d, lo, hi)
                for p in range(P):
                    s = h0[b, h, p, n]
                    for t in range(L):
                        if seq is not None and t > 0 and seq[b, t] != seq[b, t - 1]:
                            s = 0.0
                        s = math.exp(d[t] * A[h, n]) * s + d[t] * B[b, t, g, n] * x[b, t, h, p]
                        y[b, t, h, p] += C[b, t, g, n] * s
                    fin[b, h, p, n] = s
    y += D[None, None, :, None] * x
    if z is not None:
        y *= z / (1.0 + np.exp(-z))
    return y, fin


def test_fixtures_exist():
    assert len(SCANS) == 3 and len(NORMS) == 2 and len(LAYERNORMS) == 2


@pytest.mark.parametrize("path", SCANS, ids=os.path.basename)
def test_scan_fixture_matches_scalar_loop_and_oracle(path):
    f = _load(path)
    y, fin = _scalar_scan(f)
    np.testing.assert_allclose(f["y"], y, rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(f["final"], fin, rtol=1e-11, atol=1e-12)
    t = lambda k: None if ("in_" + k) not in f else torch.from_numpy(f["in_" + k]).requires_grad_()
    ins = {k: t(k) for k in ("x", "dt", "A", "B", "C", "D", "z", "dt_bias", "h0")}
    seq = None if "seq_idx" not in f else torch.from_numpy(f["seq_idx"])
    yo, fo = R.issm_scan_sequential(ins["x"], ins["dt"], ins["A"], ins["B"], ins["C"], D=ins["D"], z=ins["z"],
                                    dt_bias=ins["dt_bias"], initial_states=ins["h0"],
                                    dt_softplus=bool(f["softplus"]), dt_limit=tuple(f["dt_limit"]), seq_idx=seq)
    ((yo * torch.from_numpy(f["dy"])).sum() + (fo * torch.from_numpy(f["dfinal"])).sum()).backward()
    np.testing.assert_allclose(yo.detach().numpy(), f["y"], rtol=1e-12, atol=1e-13)
    for k, v in ins.items():
        if v is not None:
            np.testing.assert_allclose(v.grad.numpy(), f["grad_" + k], rtol=1e-10, atol=1e-12)
    # the chunked closed-form backward reproduces the stored gradients too
    gr = R.issm_bwd_closed_form(ins["x"].detach(), ins["dt"].detach(), ins["A"].detach(), ins["B"].detach(),
                                ins["C"].detach(), 16, torch.from_numpy(f["dy"]), dfinal=torch.from_numpy(f["dfinal"]),
                                D=ins["D"].detach(), dt_bias=None if ins["dt_bias"] is None else ins["dt_bias"].detach(),
                                initial_states=ins["h0"].detach(), dt_softplus=bool(f["softplus"]),
                                dt_limit=tuple(f["dt_limit"])) if ins["z"] is None and seq is None else None
    if gr is not None:
        for k in ("x", "dt", "A", "B", "C"):
            np.testing.assert_allclose(gr["d" + k].numpy(), f["grad_" + k], rtol=1e-8, atol=1e-10)


@pytest.mark.parametrize("path", NORMS, ids=os.path.basename)
def test_rmsnorm_fixture_matches_formula(path):
    f = _load(path)
    x, z, w = f["x"], f["z"], f["w"]
    gs, before = int(f["group"]), bool(f["before_gate"])
    silu = z / (1.0 + np.exp(-z))
    v = x if before else x * silu
    vg = v.reshape(v.shape[0], -1, gs)
    yn = (vg / np.sqrt((vg ** 2).mean(-1, keepdims=True) + 1e-5)).reshape(v.shape) * w
    np.testing.assert_allclose(f["y"], yn * silu if before else yn, rtol=1e-12, atol=1e-13)


@pytest.mark.parametrize("path", LAYERNORMS, ids=os.path.basename)
def test_layernorm_fixture_matches_formula(path):
    f = _load(path)
    x, z, w, b = f["x"], f["z"], f["w"], f["b"]
    gs, before = int(f["group"]), bool(f["before_gate"])
    silu = z / (1.0 + np.exp(-z))
    v = x if before else x * silu
    vg = v.reshape(v.shape[0], -1, gs)
    vg = vg - vg.mean(-1, keepdims=True)
    yn = (vg / np.sqrt((vg ** 2).mean(-1, keepdims=True) + 1e-5)).reshape(v.shape) * w + b
    np.testing.assert_allclose(f["y"], yn * silu if before else yn, rtol=1e-12, atol=1e-13)
    # the bias gradient is the column sum of the gradient that reaches the norm's output
    dy = f["dy"] * silu if before else f["dy"]
    np.testing.assert_allclose(f["db"], dy.sum(0), rtol=1e-12, atol=1e-13)


def _rel(a, b):
    a, b = a.detach().double().cpu(), torch.as_tensor(b).double()
    return max(((a - b).norm() / b.norm()).item(), ((a - b).abs().max() / b.abs().max()).item())


@pytest.mark.gpu
@pytest.mark.parametrize("path", SCANS, ids=os.path.basename)
def test_hip_scan_reproduces_fixture(path):
    from dest3d_amd import ISSM_chunk_scan_combined
    print(f"[case] golden {os.path.basename(path)}", flush=True)
    f = _load(path)
    t = lambda k: None if ("in_" + k) not in f else torch.from_numpy(f["in_" + k]).float().cuda().requires_grad_()
    ins = {k: t(k) for k in ("x", "dt", "A", "B", "C", "D", "z", "dt_bias", "h0")}
    seq = None if "seq_idx" not in f else torch.from_numpy(f["seq_idx"]).cuda()
    y, fin = ISSM_chunk_scan_combined(ins["x"], ins["dt"], ins["A"], ins["B"], ins["C"], 8, D=ins["D"], z=ins["z"],
                                      dt_bias=ins["dt_bias"], initial_states=ins["h0"], seq_idx=seq,
                                      dt_softplus=bool(f["softplus"]),
                                      dt_limit=(float(f["dt_limit"][0]), float(f["dt_limit"][1])),
                                      return_final_states=True)
    ((y * torch.from_numpy(f["dy"]).float().cuda()).sum()
     + (fin * torch.from_numpy(f["dfinal"]).float().cuda()).sum()).backward()
    torch.cuda.synchronize()
    assert _rel(y, f["y"]) <= FWD32 and _rel(fin, f["final"]) <= FWD32
    for k, v in ins.items():
        if v is not None:
            e = _rel(v.grad, f["grad_" + k])
            print(f"    d{k}: {e:.3e}", flush=True)
            assert e <= BWD32, (k, e)


@pytest.mark.gpu
@pytest.mark.parametrize("path", NORMS, ids=os.path.basename)
def test_hip_rmsnorm_reproduces_fixture(path):
    from dest3d_amd import rmsnorm_fn
    print(f"[case] golden {os.path.basename(path)}", flush=True)
    f = _load(path)
    x, z, w = (torch.from_numpy(f[k]).float().cuda().requires_grad_() for k in ("x", "z", "w"))
    y = rmsnorm_fn(x, w, None, z=z, eps=1e-5, group_size=int(f["group"]), norm_before_gate=bool(f["before_gate"]))
    (y * torch.from_numpy(f["dy"]).float().cuda()).sum().backward()
    torch.cuda.synchronize()
    assert _rel(y, f["y"]) <= FWD32
    for k, v in (("dx", x), ("dz", z), ("dw", w)):
        assert _rel(v.grad, f[k]) <= BWD32, k


@pytest.mark.gpu
@pytest.mark.parametrize("path", LAYERNORMS, ids=os.path.basename)
def test_hip_layernorm_reproduces_fixture(path):
    from dest3d_amd import layernorm_fn
    print(f"[case] golden {os.path.basename(path)}", flush=True)
    f = _load(path)
    x, z, w, b = (torch.from_numpy(f[k]).float().cuda().requires_grad_() for k in ("x", "z", "w", "b"))
    y = layernorm_fn(x, w, b, z=z, eps=1e-5, group_size=int(f["group"]), norm_before_gate=bool(f["before_gate"]))
    (y * torch.from_numpy(f["dy"]).float().cuda()).sum().backward()
    torch.cuda.synchronize()
    assert _rel(y, f["y"]) <= FWD32
    for k, v in (("dx", x), ("dz", z), ("dw", w), ("db", b)):
        assert _rel(v.grad, f[k]) <= BWD32, k
