"""Gated RMSNorm kernels (through the C ABI) against the fp64 oracle; tolerances as in
test_issm_gpu.py (fp32 fwd 1e-4 / grads 1e-3, bf16 fwd 2e-2 / grads 5e-2)."""
import pytest
import torch

from oracle import issm_ref as R
from tests.test_issm_gpu import _check, _say, FWD32, BWD32, FWD16, BWD16

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape,gs,nbg,use_z,dtype", [
    ((8, 1024, 256), None, False, True, torch.float32),     # what DEST uses (dest_module.py:512)
    ((3, 77, 288), None, False, True, torch.float32),
    ((5, 33, 288), 96, True, True, torch.float32),
    ((4, 50, 100), None, True, False, torch.float32),
    ((8, 256, 256), None, False, True, torch.bfloat16),
])
def test_gated_rmsnorm_fwd_bwd(shape, gs, nbg, use_z, dtype):
    from dest3d_amd import RMSNorm
    _say(f"rmsnorm {shape} gs={gs} nbg={nbg} z={use_z} {dtype}")
    g = torch.Generator().manual_seed(shape[1])
    x = torch.randn(*shape, generator=g).to(dtype)
    z = torch.randn(*shape, generator=g).to(dtype) if use_z else None
    w = torch.randn(shape[-1], generator=g) * 0.5 + 1.0
    dy = torch.randn(*shape, generator=g).to(dtype)
    ins = [t.double().clone().requires_grad_() for t in (x, w) + ((z,) if use_z else ())]
    yr = R.gated_rmsnorm_ref(ins[0], ins[1], z=ins[2] if use_z else None, eps=1e-5, norm_before_gate=nbg, group_size=gs)
    (yr * dy.double()).sum().backward()
    m = RMSNorm(shape[-1], eps=1e-5, group_size=gs, norm_before_gate=nbg, device="cuda")
    with torch.no_grad():
        m.weight.copy_(w)
    xg = x.cuda().requires_grad_()
    zg = z.cuda().requires_grad_() if use_z else None
    y = m(xg, zg)
    assert y.dtype == dtype and y.shape == x.shape
    (y.float() * dy.cuda().float()).sum().backward()
    torch.cuda.synchronize()
    ft, bt = (FWD32, BWD32) if dtype == torch.float32 else (FWD16, BWD16)
    _check("y", y, yr, ft)
    _check("dx", xg.grad, ins[0].grad, bt)
    _check("dw", m.weight.grad, ins[1].grad, bt)
    if use_z:
        _check("dz", zg.grad, ins[2].grad, bt)


def test_rmsnorm_strided_rows_and_import_shim():
    from issm_triton.layernorm_gated import RMSNorm as Shim
    from issm_triton.issm_combined import ISSM_chunk_scan_combined  # noqa: F401
    _say("rmsnorm strided rows")
    big = torch.randn(64, 600, device="cuda")
    x, z = big[:, :288], big[:, 300:588]           # row stride 600, as after torch.split of a projection
    m = Shim(288, eps=1e-5, norm_before_gate=False, device="cuda")
    y = m(x, z)
    yr = R.gated_rmsnorm_ref(x.cpu(), m.weight.detach().cpu(), z=z.cpu(), eps=1e-5, norm_before_gate=False)
    _check("y", y, yr, FWD32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm_rows_at_odd_element_offsets(dtype):
    """Rows that start at odd element offsets of a wider row with an odd stride (2-byte aligned in bf16, 4-byte in
    fp32): the 8 / 16-byte accesses of the fast path promise element alignment only.  Forward and backward."""
    from dest3d_amd import RMSNorm
    _say(f"rmsnorm rows at odd offsets, stride 601, {dtype}")
    g = torch.Generator().manual_seed(3)
    big = torch.randn(40, 601, generator=g).to(dtype)
    w = torch.randn(288, generator=g) * 0.5 + 1.0
    dy = torch.randn(40, 288, generator=g).to(dtype)
    xs, zs = slice(1, 289), slice(301, 589)
    ins = [big[:, xs].double().clone().requires_grad_(), w.double().clone().requires_grad_(),
           big[:, zs].double().clone().requires_grad_()]
    yr = R.gated_rmsnorm_ref(ins[0], ins[1], z=ins[2], eps=1e-5, norm_before_gate=False)
    (yr * dy.double()).sum().backward()
    m = RMSNorm(288, eps=1e-5, norm_before_gate=False, device="cuda")
    with torch.no_grad():
        m.weight.copy_(w)
    bg = big.cuda().requires_grad_()
    y = m(bg[:, xs], bg[:, zs])
    (y.float() * dy.cuda().float()).sum().backward()
    torch.cuda.synchronize()
    ft, bt = (FWD32, BWD32) if dtype == torch.float32 else (FWD16, BWD16)
    _check("y", y, yr, ft)
    _check("dx", bg.grad[:, xs], ins[0].grad, bt)
    _check("dz", bg.grad[:, zs], ins[2].grad, bt)
    _check("dw", m.weight.grad, ins[1].grad, bt)
