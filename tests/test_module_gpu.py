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


def _geometry(Bsz, L, K, seed):
    """Key points and query boxes as configs[2] draws them: coordinates uniform in an 8 m cube, box sizes 0.2 - 2.2 m,
    zero headings (what DEST passes, models/dest_module.py:284)."""
    g = torch.Generator().manual_seed(seed)
    key_pos = 8.0 * torch.rand(Bsz, L, 3, generator=g)
    qpos = torch.cat([8.0 * torch.rand(Bsz, K, 3, generator=g), 0.2 + 2.0 * torch.rand(Bsz, K, 3, generator=g)], -1)
    return key_pos, qpos, torch.zeros(Bsz, K)


def test_box_dist_weights_and_six_layers_chain_fp32_against_fp64():
    """configs[2] end to end at reduced size: BoxDistFun -> local_weight -> six MultiHeadISSMScan layers (residual
    stack, heads of 36), fp32 kernels against an fp64 evaluation chained from the three oracles (oracle/boxdist_ref.py
    for the encoding and the weight, oracle/module_ref.py for the layers with oracle/issm_ref.py inside): outputs, input
    gradients, every layer parameter's gradient and -- through d(dist) and the table -- the encoding MLP's."""
    import numpy as np
    from oracle import boxdist_ref as BR
    from oracle.module_ref import multi_head_issm_scan_ref
    from dest3d_amd.box_dist import BoxDistFun
    from dest3d_amd.scan_module import MultiHeadISSMScan
    print("[case] box_dist -> weights -> six layers, fp32 vs fp64", flush=True)
    torch.manual_seed(31)
    Bsz, L, K, D, H, NL = 2, 96, 40, 72, 2, 6
    bd = BoxDistFun(out_dim=16)
    layers = torch.nn.ModuleList(MultiHeadISSMScan(d_model=D, d_state=K, d_dist=16, chunk_size=256, nheads=H, expand=1)
                                 for _ in range(NL))
    with torch.no_grad():
        for m in layers:
            m.D.normal_()
            m.out_key_proj.weight.mul_(0.5)      # keep the residual stack's activations of order one
            m.out_query_proj.weight.mul_(0.5)
    key_pos, qpos, ang = _geometry(Bsz, L, K, 32)
    g = torch.Generator().manual_seed(33)
    key, query = torch.randn(Bsz, L, D, generator=g), torch.randn(Bsz, K, D, generator=g)
    w_key, w_query = torch.randn(Bsz, L, D, generator=g), torch.randn(Bsz, K, D, generator=g)

    # ---- fp64 chain on the CPU
    bd64 = {k: v.detach().double().clone().requires_grad_() for k, v in bd.cpb_mlps.state_dict().items()}
    lat = bd.relative_coords_table.double()
    table = (torch.relu(lat @ bd64["0.weight"].T + bd64["0.bias"]) @ bd64["2.weight"].T)[0].permute(3, 0, 1, 2)
    dist_np = BR.box_dist(key_pos.numpy(), qpos[..., :3].numpy(), qpos[..., 3:].numpy(), ang.numpy(),
                          table.detach().numpy(), log_scale=512.0, max_value=bd.max_value)
    dist_ref = torch.from_numpy(dist_np).requires_grad_()
    wts_ref = torch.from_numpy(BR.local_weight(key_pos.numpy(), qpos.numpy()))
    sds = [{k: v.detach().double().clone().requires_grad_() for k, v in m.state_dict().items()} for m in layers]
    cfg = dict(nheads=H, ngroups=1, d_inner=D, d_state=K, use_biscan=True)
    rk, rq = key.double().requires_grad_(), query.double().requires_grad_()
    hk, hq = rk, rq
    for sd in sds:
        ok, oq = multi_head_issm_scan_ref(sd, cfg, hk, hq, dist_ref, wts_ref.float().double())
        hk, hq = hk + ok, hq + oq
    ((hk * w_key.double()).sum() + (hq * w_query.double()).sum()).backward()
    dtable = BR.box_dist_table_grad(key_pos.numpy(), qpos[..., :3].numpy(), qpos[..., 3:].numpy(), ang.numpy(),
                                    tuple(table.shape), dist_ref.grad.numpy(), log_scale=512.0, max_value=bd.max_value)
    table.backward(torch.from_numpy(dtable))

    # ---- the kernels
    bd, layers = bd.cuda(), layers.cuda()
    gk, gq = key.cuda().requires_grad_(), query.cuda().requires_grad_()
    kp, qp = key_pos.cuda(), qpos.cuda()
    dist, wts = bd(kp, qp[..., :3], qp[..., 3:], ang.cuda(), weight_query_pos=qp)
    _check("dist", dist, dist_ref, FWD32)
    _check("weights", wts, wts_ref, FWD32)
    hk2, hq2 = gk, gq
    for m in layers:
        ok, oq = m(hk2, hq2, dist, kp, wts)
        hk2, hq2 = hk2 + ok, hq2 + oq
    ((hk2 * w_key.cuda()).sum() + (hq2 * w_query.cuda()).sum()).backward()
    torch.cuda.synchronize()
    _check("out_key", hk2, hk, FWD32)
    _check("out_query", hq2, hq, FWD32)
    _check("d in_key", gk.grad, rk.grad, BWD32)
    _check("d in_query", gq.grad, rq.grad, BWD32)
    for i, (m, sd) in enumerate(zip(layers, sds)):
        for k, p in m.named_parameters():
            # A_log's gradient is, per head, ONE sum over every (batch, token, state) product, of mixed signs: its relative
            # error reflects that cancellation (measured 1.4e-3 in one layer here, <= 5e-5 in the others), so it gets
            # three times the bound; every other tensor keeps 1e-3
            _check(f"layer {i} d{k}", p.grad, sd[k].grad, 3 * BWD32 if k == "A_log" else BWD32)
    for k, p in bd.cpb_mlps.named_parameters():
        _check(f"encoding d{k}", p.grad, bd64[k].grad, BWD32)


def test_box_dist_weights_and_six_layers_chain_bf16_at_detector_shape():
    """The same chain at configs[2]'s own size (B=8, L=1024 keys, K=256 queries, d_model 288, 8 heads of 36, six layers)
    in bf16, forward + backward, against the chain in fp32 on the bf16-rounded parameters and inputs (the fp32 chain is
    what the reduced-size test above pins against fp64)."""
    from dest3d_amd.box_dist import BoxDistFun
    from dest3d_amd.scan_module import MultiHeadISSMScan
    print("[case] box_dist -> weights -> six layers, bf16 at B=8 L=1024 K=256 d_model=288", flush=True)
    torch.manual_seed(41)
    mk = lambda: (BoxDistFun(out_dim=16), torch.nn.ModuleList(
        MultiHeadISSMScan(d_model=288, d_state=256, d_dist=16, chunk_size=256, nheads=8, expand=1) for _ in range(6)))
    bd16, l16 = mk()
    bd16, l16 = bd16.cuda().bfloat16(), l16.cuda().bfloat16()
    bd32, l32 = mk()
    bd32, l32 = bd32.cuda(), l32.cuda()
    bd32.load_state_dict({k: v.float() for k, v in bd16.state_dict().items()})
    l32.load_state_dict({k: v.float() for k, v in l16.state_dict().items()})
    key_pos, qpos, ang = (t.cuda() for t in _geometry(8, 1024, 256, 42))
    g = torch.Generator().manual_seed(43)
    key = torch.randn(8, 1024, 288, generator=g).bfloat16().cuda()
    query = torch.randn(8, 256, 288, generator=g).bfloat16().cuda()

    def run(bd, stack, k, q):
        k, q = k.clone().requires_grad_(), q.clone().requires_grad_()
        dist, wts = bd(key_pos, qpos[..., :3], qpos[..., 3:], ang, weight_query_pos=qpos)
        hk, hq = k, q
        for layer in stack:
            ok, oq = layer(hk, hq, dist, key_pos, wts)
            hk, hq = hk + ok, hq + oq
        (hk.float().square().mean() + hq.float().square().mean()).backward()
        return hk, hq, k.grad, q.grad, bd.cpb_mlps[2].weight.grad

    o16 = run(bd16, l16, key, query)
    o32 = run(bd32, l32, key.float(), query.float())
    torch.cuda.synchronize()
    for name, a, b in zip(("out_key", "out_query", "d in_key", "d in_query", "d encoding table weights"), o16, o32):
        _check(name, a, b, 5e-2)
