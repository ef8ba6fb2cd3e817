"""Depthwise conv7 + SiLU on (B, L, C) (libissm_hip.so) against torch's Conv1d + SiLU in fp64 on the CPU
(the formulation of models/dest_module.py:400-423).  fp32: rel. error <= 1e-5 forward, 1e-4 gradients;
bf16: <= 1e-2 / 3e-2 (the convolution output is rounded to bf16 before SiLU, as a bf16 Conv1d module's is)."""
import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu


def _ref(u, ws, bs):
    C = u.shape[-1]
    return [F.silu(F.conv1d(u.transpose(1, 2), w.reshape(C, 1, 7), b, padding=3, groups=C)).transpose(1, 2)
            for w, b in zip(ws, bs)]


def _rel(a, b):
    return ((a.double().cpu() - b.double()).norm() / b.double().norm().clamp_min(1e-30)).item()


CASES = [
    # B, L, C, nsets, dtype, strided input
    (2, 100, 290, 2, torch.float32, True),
    (1, 5, 33, 1, torch.float32, False),
    (3, 16, 64, 2, torch.float32, False),
    (2, 1, 8, 2, torch.float32, False),
    (2, 257, 290, 2, torch.bfloat16, True),
    (1, 40, 130, 1, torch.bfloat16, False),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "B%d_L%d_C%d_S%d_%s_%s" % (*c[:4], str(c[4])[6:], "view" if c[5] else "dense"))
def test_dwconv_silu_matches_fp64(case):
    from dest3d_amd.dwconv import dwconv_silu
    B, L, C, S, dtype, strided = case
    g = torch.Generator().manual_seed(77 + L + C)
    full = torch.randn(B, L, C + 24, generator=g).to(dtype)
    base = full.cuda().requires_grad_()
    u = base[..., 8:8 + C] if strided else base[..., :C].contiguous()
    ws = [(0.4 * torch.randn(C, 1, 7, generator=g)).cuda().requires_grad_() for _ in range(S)]
    bs = [(0.2 * torch.randn(C, generator=g)).cuda().requires_grad_() for _ in range(S)]
    ys = dwconv_silu(u, ws, bs)
    u64 = (full[..., 8:8 + C] if strided else full[..., :C]).double().requires_grad_()
    w64 = [w.detach().double().cpu().requires_grad_() for w in ws]
    b64 = [b.detach().double().cpu().requires_grad_() for b in bs]
    refs = _ref(u64, w64, b64)
    ftol, gtol = (1e-5, 1e-4) if dtype == torch.float32 else (1e-2, 3e-2)
    assert len(ys) == S
    for y, r in zip(ys, refs):
        assert y.shape == (B, L, C) and y.dtype == dtype
        assert _rel(y, r) <= ftol
    gy = [torch.randn(B, L, C, generator=g).to(dtype) for _ in range(S)]
    torch.autograd.backward(list(ys), [t.cuda() for t in gy])
    torch.autograd.backward(refs, [t.double() for t in gy])
    got_du = base.grad[..., 8:8 + C] if strided else base.grad[..., :C]
    assert _rel(got_du, u64.grad) <= gtol
    for s in range(S):
        assert ws[s].grad.shape == (C, 1, 7)
        assert _rel(ws[s].grad, w64[s].grad) <= gtol
        assert _rel(bs[s].grad, b64[s].grad) <= gtol


CHAIN_CASES = [
    # B, L, C, dtype, strided input
    (2, 100, 290, torch.float32, True),
    (3, 16, 64, torch.float32, False),
    (2, 1, 8, torch.float32, False),
    (1, 5, 33, torch.float32, False),
    (1, 23, 40, torch.float32, False),
    (2, 257, 290, torch.bfloat16, True),
]


@pytest.mark.parametrize("case", CHAIN_CASES, ids=lambda c: "B%d_L%d_C%d_%s_%s" % (*c[:3], str(c[3])[6:], "view" if c[4] else "dense"))
def test_dwconv_chain_matches_fp64(case):
    """chain=True: the second set convolves the first set's result (models/dest_module.py:530,534), forward and every
    gradient -- du and the first set's weight gradient collect what flows back through the second convolution."""
    from dest3d_amd.dwconv import dwconv_silu
    B, L, C, dtype, strided = case
    print(f"[case] dwconv chain B={B} L={L} C={C} {dtype}", flush=True)
    g = torch.Generator().manual_seed(91 + L + C)
    full = torch.randn(B, L, C + 24, generator=g).to(dtype)
    base = full.cuda().requires_grad_()
    u = base[..., 8:8 + C] if strided else base[..., :C].contiguous()
    ws = [(0.4 * torch.randn(C, 1, 7, generator=g)).cuda().requires_grad_() for _ in range(2)]
    bs = [(0.2 * torch.randn(C, generator=g)).cuda().requires_grad_() for _ in range(2)]
    ys = dwconv_silu(u, ws, bs, chain=True)
    u64 = (full[..., 8:8 + C] if strided else full[..., :C]).double().requires_grad_()
    w64 = [w.detach().double().cpu().requires_grad_() for w in ws]
    b64 = [b.detach().double().cpu().requires_grad_() for b in bs]
    r0 = _ref(u64, w64[:1], b64[:1])[0]
    r1 = _ref(r0, w64[1:], b64[1:])[0]
    ftol, gtol = (1e-5, 1e-4) if dtype == torch.float32 else (1.5e-2, 4e-2)
    for y, r in zip(ys, (r0, r1)):
        assert y.shape == (B, L, C) and y.dtype == dtype
        assert _rel(y, r) <= ftol
    gy = [torch.randn(B, L, C, generator=g).to(dtype) for _ in range(2)]
    torch.autograd.backward(list(ys), [t.cuda() for t in gy])
    torch.autograd.backward([r0, r1], [t.double() for t in gy])
    got_du = base.grad[..., 8:8 + C] if strided else base.grad[..., :C]
    assert _rel(got_du, u64.grad) <= gtol
    for s in range(2):
        assert _rel(ws[s].grad, w64[s].grad) <= gtol
        assert _rel(bs[s].grad, b64[s].grad) <= gtol


def test_dwconv_chain_only_second_gradient():
    """Only the second output has a gradient: it still reaches u and the first set's parameters through the chain."""
    from dest3d_amd.dwconv import dwconv_silu
    g = torch.Generator().manual_seed(6)
    u = torch.randn(2, 50, 40, generator=g).cuda().requires_grad_()
    ws = [(0.4 * torch.randn(40, 7, generator=g)).cuda().requires_grad_() for _ in range(2)]
    bs = [(0.2 * torch.randn(40, generator=g)).cuda().requires_grad_() for _ in range(2)]
    _, y1 = dwconv_silu(u, ws, bs, chain=True)
    y1.sum().backward()
    u64 = u.detach().double().cpu().requires_grad_()
    w64 = [w.detach().double().cpu().requires_grad_() for w in ws]
    b64 = [b.detach().double().cpu().requires_grad_() for b in bs]
    r1 = _ref(_ref(u64, w64[:1], b64[:1])[0], w64[1:], b64[1:])[0]
    r1.sum().backward()
    assert _rel(u.grad, u64.grad) <= 1e-4
    assert _rel(ws[0].grad, w64[0].grad.reshape(40, 7)) <= 1e-4 and _rel(bs[0].grad, b64[0].grad) <= 1e-4


def test_dwconv_one_absent_gradient():
    from dest3d_amd.dwconv import dwconv_silu
    g = torch.Generator().manual_seed(5)
    u = torch.randn(2, 50, 40, generator=g).cuda().requires_grad_()
    ws = [torch.randn(40, 7, generator=g).cuda().requires_grad_() for _ in range(2)]
    bs = [torch.randn(40, generator=g).cuda().requires_grad_() for _ in range(2)]
    y0, y1 = dwconv_silu(u, ws, bs)
    y0.sum().backward()
    assert ws[1].grad.abs().max().item() == 0.0 and bs[1].grad.abs().max().item() == 0.0
    u64 = u.detach().double().cpu().requires_grad_()
    r = _ref(u64, [ws[0].detach().double().cpu()], [bs[0].detach().double().cpu()])[0]
    r.sum().backward()
    assert _rel(u.grad, u64.grad) <= 1e-4


def test_dwconv_rejects_unbuilt_shapes():
    import ctypes as C
    from dest3d_amd import _lib as L
    lib = L.load()
    a = L.DwConvArgs()
    a.batch, a.seqlen, a.channels, a.nsets, a.taps = 1, 8, 8, 1, 5
    assert lib.issm_dwconv_silu_fwd(C.byref(a)) == -5
    a.taps, a.nsets = 7, 3
    assert lib.issm_dwconv_silu_fwd(C.byref(a)) == -5
    a.nsets = 1
    assert lib.issm_dwconv_silu_fwd(C.byref(a)) == -1
    a.chain = 1                               # a chain needs two sets
    assert lib.issm_dwconv_silu_fwd(C.byref(a)) == -2


def test_dwconv_split_outputs_equal_the_slices():
    """With `split` the forward writes channels [0, split) and [split, C) as two dense tensors and the backward
    takes the gradient in the same two pieces: identical to slicing / concatenating around the unsplit call."""
    import ctypes as C
    from dest3d_amd import _lib as L
    from dest3d_amd import dwconv as D
    lib = L.load()
    g = torch.Generator().manual_seed(3)
    B, Ln, Cn, split = 2, 45, 38, 32
    u = torch.randn(B, Ln, Cn, generator=g).cuda()
    w = torch.randn(2, Cn, 7, generator=g).cuda()
    b = torch.randn(2, Cn, generator=g).cuda()
    dy = torch.randn(2, B, Ln, Cn, generator=g).cuda()

    def run(split_at):
        y = torch.empty(2, B, Ln, Cn if not split_at else split_at, device="cuda")
        tail = torch.empty(2, B, Ln, Cn - split_at, device="cuda") if split_at else None
        pre = torch.empty(2, B, Ln, Cn, device="cuda")
        a = D._args(u, 2)
        a.w, a.bias, a.y, a.pre = w.data_ptr(), b.data_ptr(), y.data_ptr(), pre.data_ptr()
        keep = []
        if split_at:
            a.split, a.y_tail = split_at, tail.data_ptr()
        L.check(lib.issm_dwconv_silu_fwd(C.byref(a)), "fwd")
        du = torch.empty(B, Ln, Cn, device="cuda")
        part = torch.empty(lib.issm_dwconv_partial_rows(B, Ln), 2, 8, Cn, device="cuda")
        dw, db = torch.empty(2, Cn, 7, device="cuda"), torch.empty(2, Cn, device="cuda")
        a.du, a.partial, a.dw, a.dbias = du.data_ptr(), part.data_ptr(), dw.data_ptr(), db.data_ptr()
        for s in range(2):
            if split_at:
                keep += [dy[s, ..., :split_at].contiguous(), dy[s, ..., split_at:].contiguous()]
                a.dy[s], a.dy_tail[s] = keep[-2].data_ptr(), keep[-1].data_ptr()
            else:
                a.dy[s] = dy[s].data_ptr()
        L.check(lib.issm_dwconv_silu_bwd(C.byref(a)), "bwd")
        torch.cuda.synchronize()
        return y, tail, du, dw, db

    y0, _, du0, dw0, db0 = run(0)
    y1, t1, du1, dw1, db1 = run(split)
    assert torch.equal(y1, y0[..., :split]) and torch.equal(t1, y0[..., split:])
    assert torch.equal(du1, du0) and torch.equal(dw1, dw0) and torch.equal(db1, db0)
