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


@pytest.mark.parametrize("shape,gs,nbg,use_z,rms,use_b,dtype", [
    ((8, 128, 288), None, False, True, False, True, torch.float32),    # LayerNorm module, gate before the norm
    ((3, 77, 288), None, True, True, False, True, torch.float32),      # gate after the norm: dz sees the bias
    ((5, 33, 288), 96, True, True, False, True, torch.float32),        # several groups per row (generic kernels)
    ((5, 33, 288), 96, False, True, True, True, torch.float32),        # RMS statistics with a bias, groups
    ((4, 50, 100), None, True, False, False, False, torch.float32),    # no gate, no bias, mean subtracted
    ((2, 9, 1500), None, False, True, False, True, torch.float32),     # rows wider than the register-resident form
    ((4, 64, 256), None, True, True, True, True, torch.float32),       # RMS statistics with a bias, one group
    ((8, 256, 256), None, False, True, False, True, torch.bfloat16),
    ((8, 64, 512), 128, True, True, False, True, torch.bfloat16),
])
def test_gated_layernorm_and_bias_fwd_bwd(shape, gs, nbg, use_z, rms, use_b, dtype):
    """LayerNorm statistics and the bias of layernorm_gated.py:35-97 / 145-260 (layernorm_fn, rmsnorm_fn with a bias),
    forward and all four gradients against the fp64 oracle."""
    from dest3d_amd import layernorm_fn
    _say(f"layernorm {shape} gs={gs} nbg={nbg} z={use_z} rms={rms} bias={use_b} {dtype}")
    g = torch.Generator().manual_seed(shape[1] + 1)
    x = (torch.randn(*shape, generator=g) + 0.7).to(dtype)      # a mean that is not zero
    z = torch.randn(*shape, generator=g).to(dtype) if use_z else None
    w = torch.randn(shape[-1], generator=g) * 0.5 + 1.0
    b = torch.randn(shape[-1], generator=g) * 0.5 if use_b else None
    dy = torch.randn(*shape, generator=g).to(dtype)
    leaf = lambda t: None if t is None else t.double().clone().requires_grad_()
    xr, wr, br, zr = leaf(x), leaf(w), leaf(b), leaf(z)
    yr = R.gated_rmsnorm_ref(xr, wr, z=zr, eps=1e-5, norm_before_gate=nbg, group_size=gs, bias=br, layer_norm=not rms)
    (yr * dy.double()).sum().backward()
    dev = lambda t: None if t is None else t.cuda().requires_grad_()
    xg, wg, bg, zg = dev(x), dev(w), dev(b), dev(z)
    y = layernorm_fn(xg, wg, bg, z=zg, eps=1e-5, group_size=gs, norm_before_gate=nbg, is_rms_norm=rms)
    assert y.dtype == dtype and y.shape == x.shape
    (y.float() * dy.cuda().float()).sum().backward()
    torch.cuda.synchronize()
    ft, bt = (FWD32, BWD32) if dtype == torch.float32 else (FWD16, BWD16)
    _check("y", y, yr, ft)
    _check("dx", xg.grad, xr.grad, bt)
    _check("dw", wg.grad, wr.grad, bt)
    if use_b:
        _check("db", bg.grad, br.grad, bt)
    if use_z:
        _check("dz", zg.grad, zr.grad, bt)


def test_bias_in_another_dtype_than_the_weight_is_not_rounded():
    """A bf16 weight with an fp32 bias (layernorm_gated.py:77-80 widens each to fp32 on its own): the bias must enter
    with all its fp32 bits.  The bias here is 1 + 2^-12 per column, which bf16 would round to 1; x = 0 and no gate make
    the output the bias itself."""
    from dest3d_amd import layernorm_fn
    _say("layernorm bf16 weight, fp32 bias")
    x = torch.zeros(4, 256, device="cuda")
    w = torch.ones(256, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    b = torch.full((256,), 1.0 + 2.0 ** -12, device="cuda", requires_grad=True)
    y = layernorm_fn(x, w, b, None, 1e-5, None, True, False)
    assert torch.equal(y, b.detach().expand(4, 256))
    y.sum().backward()
    assert w.grad.dtype == torch.bfloat16 and b.grad.dtype == torch.float32
    assert torch.equal(b.grad, torch.full((256,), 4.0, device="cuda"))


def test_forward_with_a_bias_has_no_column_limit_of_the_backward():
    """9000 columns with a bias: the forward runs (it stages nothing in LDS); only a backward would be refused."""
    from dest3d_amd import layernorm_fn
    _say("layernorm forward 9000 columns with bias")
    g = torch.Generator().manual_seed(3)
    x = torch.randn(3, 9000, generator=g)
    w = torch.randn(9000, generator=g)
    b = torch.randn(9000, generator=g)
    with torch.no_grad():
        y = layernorm_fn(x.cuda(), w.cuda(), b.cuda(), None, 1e-5, None, True, False)
    ref = torch.nn.functional.layer_norm(x.double(), (9000,), w.double(), b.double(), 1e-5)
    _check("y", y, ref, FWD32)


def test_layernorm_module_matches_torch_layer_norm():
    """The LayerNorm module without a gate is torch's own layer_norm (the library routine), forward and backward."""
    from issm_triton.layernorm_gated import LayerNorm
    _say("LayerNorm module against torch.nn.functional.layer_norm")
    torch.manual_seed(5)
    m = LayerNorm(288, eps=1e-5, device="cuda")
    with torch.no_grad():
        m.weight.normal_(1.0, 0.3)
        m.bias.normal_(0.0, 0.3)
    x = (torch.randn(40, 17, 288, device="cuda") * 2 + 1).requires_grad_()
    dy = torch.randn(40, 17, 288, device="cuda")
    y = m(x)
    (y * dy).sum().backward()
    got = (y.detach(), x.grad.clone(), m.weight.grad.clone(), m.bias.grad.clone())
    x.grad = None
    m.zero_grad()
    yr = torch.nn.functional.layer_norm(x.double(), (288,), m.weight.double(), m.bias.double(), eps=1e-5)
    gx, gw, gb = torch.autograd.grad((yr * dy.double()).sum(), (x, m.weight, m.bias))
    for name, a, b_, tol in zip(("y", "dx", "dw", "db"), got, (yr, gx, gw, gb), (FWD32, BWD32, BWD32, BWD32)):
        _check(name, a, b_, tol)


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
