"""The host-side mirror of DEST's MultiHeadISSMScan against a pure-PyTorch fp64 evaluation of the
reference module's forward (models/dest_module.py:515-612) that uses the oracle for the scan and the
gated RMSNorm, on the same state_dict.  Error measure and tolerances as in test_issm_gpu.py."""
import sys

import pytest
import torch

pytestmark = pytest.mark.gpu
FWD32, BWD32, FWD16 = 1e-4, 1e-3, 2e-2


def _err(a, b):
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    assert torch.isfinite(a).all()
    return max(((a - b).norm() / b.norm().clamp_min(1e-300)).item(),
               ((a - b).abs().max() / b.abs().max().clamp_min(1e-300)).item())


def _check(name, a, b, tol):
    e = _err(a, b)
    print(f"    {name:28s} err={e:.3e} (tol {tol:g})", flush=True)
    assert e <= tol, f"{name}: {e:.3e} > {tol:g}"


def _module_ref(sd, cfg, in_key, in_query, dist, mask):
    """dest_module.py:528-585 in the reference's own order of operations (oracle/module_ref.py; the order of the two
    convolutions is pinned in tests/test_module_cpu.py)."""
    from oracle.module_ref import multi_head_issm_scan_ref
    return multi_head_issm_scan_ref(sd, cfg, in_key, in_query, dist, mask)


@pytest.mark.parametrize("biscan,mask_kind", [(True, None), (True, "float"), (True, "bool"), (False, "bool"), (False, "float")])
def test_module_matches_fp64_evaluation(biscan, mask_kind):
    from dest3d_amd.scan_module import MultiHeadISSMScan
    print(f"[case] module mirror biscan={biscan} mask={mask_kind}", flush=True)
    sys.stdout.flush()
    torch.manual_seed(7)
    Bsz, L, K, D, M, H = 2, 130, 48, 72, 16, 2                       # headdim 36 as in the detector
    m = MultiHeadISSMScan(d_model=D, d_state=K, d_dist=M, chunk_size=256, nheads=H, expand=1, use_biscan=biscan)
    with torch.no_grad():                                            # make every parameter matter
        m.D.normal_()
        m.key_norm.weight.add_(0.1 * torch.randn(D))
        m.query_norm.bias.normal_(std=0.1)
    g = torch.Generator().manual_seed(8)
    ins = dict(in_key=torch.randn(Bsz, L, D, generator=g), in_query=torch.randn(Bsz, K, D, generator=g),
               dist=0.5 * torch.randn(Bsz, L, K, M, generator=g))
    mask = None
    if mask_kind == "float":
        mask = torch.rand(Bsz, L, K, generator=g)
    elif mask_kind == "bool":
        mask = torch.rand(Bsz, L, K, generator=g) < 0.2
    w_key, w_query = torch.randn(Bsz, L, D, generator=g), torch.randn(Bsz, K, D, generator=g)

    sd = {k: v.detach().double().clone().requires_grad_() for k, v in m.state_dict().items()}
    rin = {k: v.double().clone().requires_grad_() for k, v in ins.items()}
    cfg = dict(nheads=H, ngroups=1, d_inner=D, d_state=K, use_biscan=biscan)
    ok_ref, oq_ref = _module_ref(sd, cfg, rin["in_key"], rin["in_query"], rin["dist"], mask)
    ((ok_ref * w_key.double()).sum() + (oq_ref * w_query.double()).sum()).backward()

    m = m.cuda()
    gin = {k: v.cuda().requires_grad_() for k, v in ins.items()}
    ok, oq = m(gin["in_key"], gin["in_query"], gin["dist"], None, mask=None if mask is None else mask.cuda())
    ((ok * w_key.cuda()).sum() + (oq * w_query.cuda()).sum()).backward()
    torch.cuda.synchronize()
    _check("out_key", ok, ok_ref, FWD32)
    _check("out_query", oq, oq_ref, FWD32)
    for k in ins:
        _check("d" + k, gin[k].grad, rin[k].grad, BWD32)
    for k, p in m.named_parameters():
        _check("d" + k, p.grad, sd[k].grad, BWD32)


def test_token_linear_under_autocast():
    """The projections' autograd node under torch.autocast: forward in bf16, and the backward's products see operands
    of one dtype (fp32 parameters and input, bf16 output gradient)."""
    from dest3d_amd.scan_module import _LinearTokens
    print("[case] _LinearTokens under autocast", flush=True)
    g = torch.Generator().manual_seed(2)
    x = torch.randn(2048, 72, generator=g).cuda().requires_grad_()
    w = (0.1 * torch.randn(40, 72, generator=g)).cuda().requires_grad_()
    with torch.autocast("cuda", dtype=torch.bfloat16):
        y = _LinearTokens.apply(x, w)
        assert y.dtype == torch.bfloat16
        y.float().square().mean().backward()
    x64, w64 = x.detach().double().cpu().requires_grad_(), w.detach().double().cpu().requires_grad_()
    (x64 @ w64.T).square().mean().backward()
    assert x.grad.dtype == torch.float32 and w.grad.dtype == torch.float32
    _check("dx", x.grad, x64.grad, 3e-2)
    _check("dw", w.grad, w64.grad, 3e-2)


def test_six_layer_stack_bf16_at_detector_shape():
    """Six mirror layers at the detector's decoder shape (d_model 288, 8 heads of 36, K = 256 queries,
    L = 1024 keys, batch 8, d_dist 16), bf16 forward + backward, against the same stack in fp32 on the
    bf16-rounded weights and inputs.  The fp32 stack is pinned by test_module_matches_fp64_evaluation."""
    from dest3d_amd.scan_module import MultiHeadISSMScan
    print("[case] six-layer bf16 stack B=8 L=1024 K=256 d_model=288", flush=True)
    torch.manual_seed(11)
    layers = torch.nn.ModuleList(MultiHeadISSMScan(d_model=288, d_state=256, d_dist=16, chunk_size=256, nheads=8,
                                                   expand=1) for _ in range(6)).cuda().bfloat16()
    ref = torch.nn.ModuleList(MultiHeadISSMScan(d_model=288, d_state=256, d_dist=16, chunk_size=256, nheads=8,
                                                expand=1) for _ in range(6)).cuda()
    ref.load_state_dict({k: v.float() for k, v in layers.state_dict().items()})
    g = torch.Generator().manual_seed(12)
    key = torch.randn(8, 1024, 288, generator=g).bfloat16().cuda()
    query = torch.randn(8, 256, 288, generator=g).bfloat16().cuda()
    dist = (0.5 * torch.randn(8, 1024, 256, 16, generator=g)).bfloat16().cuda()

    def run(stack, k, q, d):
        k, q = k.clone().requires_grad_(), q.clone().requires_grad_()
        hk, hq = k, q
        for layer in stack:                                   # residual stack, as the decoder layers chain
            ok, oq = layer(hk, hq, d, None)
            hk, hq = hk + ok, hq + oq
        (hk.float().square().mean() + hq.float().square().mean()).backward()
        return hk, hq, k.grad, q.grad

    o16 = run(layers, key, query, dist)
    o32 = run(ref, key.float(), query.float(), dist.float())
    torch.cuda.synchronize()
    for name, a, b in zip(("out_key", "out_query", "d in_key", "d in_query"), o16, o32):
        _check(name, a, b, 5e-2)


def test_layer_step_as_hip_graph_replays_match_eager():
    """Forward + backward of one layer recorded into a HIP graph (the library allocates nothing and records no memset,
    so the whole step is capturable) and replayed three times on new input contents, with eager steps and
    synchronisations in between; every replay must reproduce the eager step's outputs and gradients (same kernels,
    same fixed-order reductions: measured bit-identical; the bound only leaves room for the GEMM library)."""
    from dest3d_amd.scan_module import MultiHeadISSMScan
    print("[case] layer forward+backward as a HIP graph", flush=True)
    torch.manual_seed(21)
    m = MultiHeadISSMScan(d_model=72, d_state=48, d_dist=16, chunk_size=256, nheads=2, expand=1).cuda()
    key = torch.randn(2, 130, 72, device="cuda", requires_grad=True)
    query = torch.randn(2, 48, 72, device="cuda", requires_grad=True)
    dist = (0.5 * torch.randn(2, 130, 48, 16, device="cuda")).requires_grad_()
    weights = torch.rand(2, 130, 48, device="cuda")
    leaves = (key, query, dist)

    def step():
        ok, oq = m(key, query, dist, None, weights)
        (ok.square().mean() + oq.square().mean()).backward()
        return ok, oq

    def clear():
        m.zero_grad(set_to_none=True)
        for t in leaves:
            t.grad = None

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            clear()
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    clear()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        g_out = step()
    g_grads = [t.grad for t in leaves] + [p.grad for p in m.parameters()]
    assert all(g is not None for g in g_grads)
    for rep in range(3):
        with torch.no_grad():
            for t in leaves:
                t.copy_(torch.randn_like(t) * (0.5 if t is dist else 1.0))
            weights.copy_(torch.rand_like(weights))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in g_out] + [g.clone() for g in g_grads]
        for t, g in zip(list(leaves) + list(m.parameters()), g_grads):
            t.grad = None                                      # eager step writes fresh gradient tensors
        want_out = step()
        torch.cuda.synchronize()
        want = list(want_out) + [t.grad for t in leaves] + [p.grad for p in m.parameters()]
        for i, (a, b) in enumerate(zip(got, want)):                 # same kernels: equal up to a library GEMM's choice
            assert torch.allclose(a, b, rtol=1e-5, atol=1e-6 * float(b.abs().max())), \
                f"replay {rep}: tensor {i} differs from the eager step"
        for t, g in zip(list(leaves) + list(m.parameters()), g_grads):
            t.grad = g                                         # the graph's static gradient buffers again
