"""Generation of dt / B / C from the distance encoding (libissm_hip.so) against an fp64 evaluation of the
reference's formulas (models/dest_module.py:541-553): two Linear layers over dist, transposes, broadcast
biases.  fp32: rel. error <= 1e-5 forward, 1e-4 gradients; bf16: <= 1e-2 / 2e-2 (outputs are rounded to
bf16; sums run in fp32)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _ref(dist, W, bias, H, G, has_back):
    base = torch.einsum("rm,blkm->blrk", W, dist)
    R0 = H + 2 * G
    main = base + bias[..., :R0].unsqueeze(-1)
    outs = [main[:, :, :H], main[:, :, H:H + G], main[:, :, H + G:]]
    if has_back:
        outs.append(base[:, :, H:H + G] + bias[..., R0:R0 + G].unsqueeze(-1))
        outs.append(base[:, :, H + G:] + bias[..., R0 + G:].unsqueeze(-1))
    return outs


def _rel(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm().clamp_min(1e-30)).item()


CASES = [
    # B, L, K, H, G, back, dtype
    (2, 37, 256, 8, 1, True, torch.float32),
    (1, 16, 256, 8, 2, True, torch.float32),
    (3, 5, 100, 4, 1, False, torch.float32),
    (1, 33, 300, 2, 2, True, torch.float32),
    (2, 64, 256, 8, 1, True, torch.bfloat16),
    (1, 19, 77, 3, 1, False, torch.bfloat16),
    (1, 11, 50, 3, 1, True, torch.bfloat16),     # K even, not a multiple of 4
    (2, 6, 77, 2, 1, False, torch.float32),      # K odd
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "B%d_L%d_K%d_H%d_G%d_back%d_%s" % (*c[:5], int(c[5]), str(c[6])[6:]))
def test_scan_params_match_fp64(case):
    from dest3d_amd.param_gen import scan_params
    B, L, K, H, G, back, dtype = case
    g = torch.Generator().manual_seed(1234 + L + K)
    M, R0 = 16, H + 2 * G
    R = R0 + (2 * G if back else 0)
    dist = torch.randn(B, L, K, M, generator=g).to(dtype).cuda().requires_grad_()
    W = (0.3 * torch.randn(R0, M, generator=g)).cuda().requires_grad_()
    bias = torch.randn(B, L, R, generator=g).cuda().requires_grad_()
    outs = scan_params(dist, W, bias, H, G, back)
    d64, W64, b64 = (t.detach().double().requires_grad_() for t in (dist, W, bias))
    refs = _ref(d64, W64, b64, H, G, back)
    assert len(outs) == len(refs)
    ftol, gtol = (1e-5, 1e-4) if dtype == torch.float32 else (1e-2, 2e-2)
    for o, r in zip(outs, refs):
        assert o.shape == r.shape and o.dtype == dtype and o.is_contiguous()
        assert _rel(o, r) <= ftol
    # the last output gets no gradient: absent gradients count as zero
    gouts = [torch.randn(o.shape, generator=g).to(dtype).cuda() for o in outs[:-1]]
    torch.autograd.backward(list(outs[:-1]), gouts)
    torch.autograd.backward(refs[:-1], [t.double() for t in gouts])
    assert _rel(dist.grad, d64.grad) <= gtol
    assert _rel(W.grad, W64.grad) <= gtol
    assert _rel(bias.grad, b64.grad) <= gtol
    if back:
        assert bias.grad[..., -G:].abs().max().item() == 0.0


WCASES = [
    (2, 21, 256, 8, 1, True, torch.float32),
    (1, 9, 100, 4, 2, False, torch.float32),
    (2, 33, 128, 8, 1, True, torch.bfloat16),
    (1, 7, 52, 3, 1, True, torch.bfloat16),
    (1, 5, 50, 2, 1, True, torch.bfloat16),
    (1, 4, 33, 2, 1, False, torch.float32),
]


@pytest.mark.parametrize("case", WCASES, ids=lambda c: "B%d_L%d_K%d_H%d_G%d_back%d_%s" % (*c[:5], int(c[5]), str(c[6])[6:]))
def test_scan_params_with_locality_weights(case):
    """dt = softplus(raw) * weights (models/dest_module.py:553-557), gradients of dist, W, bias and weights."""
    import torch.nn.functional as F
    from dest3d_amd.param_gen import scan_params
    B, L, K, H, G, back, dtype = case
    g = torch.Generator().manual_seed(99 + L + K)
    M, R0 = 16, H + 2 * G
    R = R0 + (2 * G if back else 0)
    dist = torch.randn(B, L, K, M, generator=g).to(dtype).cuda().requires_grad_()
    W = (0.6 * torch.randn(R0, M, generator=g)).cuda().requires_grad_()
    bias = (2.0 * torch.randn(B, L, R, generator=g)).cuda().requires_grad_()
    bias.data[0, 0, 0] = 40.0   # softplus above torch's threshold
    wts = torch.rand(B, L, K, generator=g)
    wts[0, :, ::7] = 0.0        # dropped entries
    wts = wts.cuda().requires_grad_()
    outs = scan_params(dist, W, bias, H, G, back, weights=wts)
    d64, W64, b64, w64 = (t.detach().double().requires_grad_() for t in (dist, W, bias, wts))
    refs = _ref(d64, W64, b64, H, G, back)
    raw = refs[0]
    if dtype == torch.bfloat16:   # the saved raw value is rounded to the I/O dtype before softplus, as a bf16 module's is
        raw = raw + (raw.detach().float().bfloat16().double() - raw.detach())
    refs[0] = F.softplus(raw) * w64.unsqueeze(2)
    ftol, gtol = (1e-5, 2e-4) if dtype == torch.float32 else (1e-2, 3e-2)
    for o, r in zip(outs, refs):
        assert o.shape == r.shape and o.dtype == dtype
        assert _rel(o, r) <= ftol
    gouts = [torch.randn(o.shape, generator=g).to(dtype).cuda() for o in outs]
    torch.autograd.backward(list(outs), gouts)
    torch.autograd.backward(refs, [t.double() for t in gouts])
    assert _rel(dist.grad, d64.grad) <= gtol
    assert _rel(W.grad, W64.grad) <= gtol
    assert _rel(bias.grad, b64.grad) <= gtol
    assert _rel(wts.grad, w64.grad) <= gtol


def test_scan_params_rejects_unbuilt_shapes():
    from dest3d_amd import _lib as L
    import ctypes as C
    lib = L.load()
    a = L.PGenArgs()
    a.tokens, a.K, a.M, a.H, a.G = 4, 8, 8, 2, 1
    assert lib.issm_param_gen_fwd(C.byref(a)) == -5
    a.M, a.H = 16, 12
    assert lib.issm_param_gen_fwd(C.byref(a)) == -5
    a.H = 2
    assert lib.issm_param_gen_fwd(C.byref(a)) == -1
