"""Pins the CPU oracle (oracle/issm_ref.py) without the reference: brute-force loops,
closed forms, invariances and gradcheck.  A dropped term, wrong sign/index or a
transposed operand in the oracle fails at least one of these."""
import math

import numpy as np
import pytest
import torch

from oracle import issm_ref as R

torch.manual_seed(0)


def _rand_problem(Bsz=2, L=12, H=4, P=3, N=5, G=2, seed=0, h0=True):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    x = r(Bsz, L, H, P)
    dt = torch.rand(Bsz, L, H, N, generator=g, dtype=torch.float64) * 0.5
    A = -torch.exp(torch.rand(H, N, generator=g, dtype=torch.float64) * 2.0)
    B = r(Bsz, L, G, N)
    C = r(Bsz, L, G, N)
    D = r(H)
    h = r(Bsz, H, P, N) if h0 else None
    return x, dt, A, B, C, D, h


def _brute_numpy(x, dt, A, B, C, D, h0):
    """Independent statement of the recurrence with scalar loops only."""
    x, dt, A, B, C = (t.numpy() for t in (x, dt, A, B, C))
    Bsz, L, H, P = x.shape
    N = dt.shape[-1]
    G = B.shape[2]
    y = np.zeros((Bsz, L, H, P))
    fin = np.zeros((Bsz, H, P, N))
    for b in range(Bsz):
        for h in range(H):
            g = h // (H // G)
            for p in range(P):
                for n in range(N):
                    s = 0.0 if h0 is None else float(h0[b, h, p, n])
                    for t in range(L):
                        s = math.exp(dt[b, t, h, n] * A[h, n]) * s + dt[b, t, h, n] * B[b, t, g, n] * x[b, t, h, p]
                        y[b, t, h, p] += C[b, t, g, n] * s
                    fin[b, h, p, n] = s
    if D is not None:
        y += D.numpy()[None, None, :, None] * x
    return y, fin


def test_sequential_matches_bruteforce_loops():
    x, dt, A, B, C, D, h0 = _rand_problem()
    y, fin = R.issm_scan_sequential(x, dt, A, B, C, D=D, initial_states=h0)
    yb, fb = _brute_numpy(x, dt, A, B, C, D, h0)
    np.testing.assert_allclose(y.numpy(), yb, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(fin.numpy(), fb, rtol=1e-12, atol=1e-12)


def test_scalar_case_by_hand():
    # N=P=H=B=1, two steps, written out by hand
    x = torch.tensor([2.0, -1.0], dtype=torch.float64).reshape(1, 2, 1, 1)
    dt = torch.tensor([0.5, 0.25], dtype=torch.float64).reshape(1, 2, 1, 1)
    A = torch.tensor([[-2.0]], dtype=torch.float64)
    B = torch.tensor([3.0, 4.0], dtype=torch.float64).reshape(1, 2, 1, 1)
    C = torch.tensor([5.0, 6.0], dtype=torch.float64).reshape(1, 2, 1, 1)
    h0 = torch.tensor(7.0, dtype=torch.float64).reshape(1, 1, 1, 1)
    D = torch.tensor([0.5], dtype=torch.float64)
    h1 = math.exp(-1.0) * 7.0 + 0.5 * 3.0 * 2.0
    h2 = math.exp(-0.5) * h1 + 0.25 * 4.0 * (-1.0)
    y, fin = R.issm_scan_sequential(x, dt, A, B, C, D=D, initial_states=h0)
    assert y.flatten().tolist() == pytest.approx([5.0 * h1 + 1.0, 6.0 * h2 - 0.5], rel=1e-14)
    assert fin.item() == pytest.approx(h2, rel=1e-14)


def test_closed_form_A_zero_is_prefix_sum():
    x, dt, A, B, C, D, h0 = _rand_problem(G=1)
    A = torch.zeros_like(A)
    y, fin = R.issm_scan_sequential(x, dt, A, B, C, initial_states=h0)
    inj = (dt * B.expand(-1, -1, x.shape[2], -1))[:, :, :, None, :] * x[..., None]   # (B,L,H,P,N)
    hs = h0[:, None] + torch.cumsum(inj, dim=1)
    y_ref = torch.einsum("blhpn,bln->blhp", hs, C[:, :, 0])
    torch.testing.assert_close(y, y_ref, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(fin, hs[:, -1], rtol=1e-12, atol=1e-12)


def test_closed_form_dt_zero_and_B_zero():
    x, dt, A, B, C, D, h0 = _rand_problem(G=1)
    y, fin = R.issm_scan_sequential(x, torch.zeros_like(dt), A, B, C, D=D, initial_states=h0)
    y_ref = torch.einsum("bhpn,bln->blhp", h0, C[:, :, 0]) + D[None, None, :, None] * x
    torch.testing.assert_close(y, y_ref, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(fin, h0, rtol=0, atol=0)
    # B = 0: pure decay h_t = exp(cumsum(dt*A)) * h0
    y, fin = R.issm_scan_sequential(x, dt, A, torch.zeros_like(B), C, initial_states=h0)
    dec = torch.exp(torch.cumsum(dt * A[None, None], dim=1))                      # (B,L,H,N)
    y_ref = torch.einsum("bhpn,blhn,bln->blhp", h0, dec, C[:, :, 0])
    torch.testing.assert_close(y, y_ref, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(fin, h0 * dec[:, -1][:, :, None, :], rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("chunk", [1, 2, 3, 4, 6, 12])
def test_chunked_equals_sequential_any_chunk(chunk):
    x, dt, A, B, C, D, h0 = _rand_problem()
    y, fin = R.issm_scan_sequential(x, dt, A, B, C, initial_states=h0)
    yc, fc = R.issm_scan_chunked(x, dt, A, B, C, chunk, initial_states=h0)
    torch.testing.assert_close(yc, y, rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(fc, fin, rtol=1e-10, atol=1e-10)


def test_chunked_no_initial_state_and_positive_A():
    x, dt, A, B, C, D, _ = _rand_problem(h0=False)
    A = A.clone()
    A[0] = 0.3            # growing modes are legal for the math
    y, fin = R.issm_scan_sequential(x, dt, A, B, C)
    yc, fc = R.issm_scan_chunked(x, dt, A, B, C, 4)
    torch.testing.assert_close(yc, y, rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(fc, fin, rtol=1e-10, atol=1e-10)


def test_softplus_and_clamp_semantics():
    v = torch.tensor([-30.0, -1.0, 0.0, 5.0, 20.0, 20.5, 40.0], dtype=torch.float64)
    torch.testing.assert_close(R.softplus_ref(v), torch.nn.functional.softplus(v, threshold=20.0), rtol=1e-14, atol=0)
    assert R.softplus_ref(v)[-1].item() == 40.0
    dt = torch.tensor([-0.2, 0.05, 0.7], dtype=torch.float64).reshape(1, 3, 1, 1)
    out = R.dt_transform(dt, dt_bias=torch.tensor([[0.1]], dtype=torch.float64), dt_limit=(0.0, 0.5))
    assert out.flatten().tolist() == pytest.approx([0.0, 0.15, 0.5])
    # order is bias -> softplus -> clamp
    out = R.dt_transform(dt, dt_bias=torch.tensor([[0.1]], dtype=torch.float64), dt_softplus=True, dt_limit=(0.0, 0.72))
    exp = [min(math.log1p(math.exp(t + 0.1)), 0.72) for t in (-0.2, 0.05, 0.7)]
    assert out.flatten().tolist() == pytest.approx(exp)


def test_D_with_hdim_and_z_gate_order():
    x, dt, A, B, C, D, h0 = _rand_problem()
    D2 = torch.randn(x.shape[2], x.shape[3], dtype=torch.float64)
    z = torch.randn_like(x)
    y0, _ = R.issm_scan_sequential(x, dt, A, B, C, initial_states=h0)
    y1, _ = R.issm_scan_sequential(x, dt, A, B, C, D=D2, z=z, initial_states=h0)
    # gate applies to y + D*x (issm_chunk_scan.py:196-210)
    torch.testing.assert_close(y1, (y0 + D2[None, None] * x) * torch.nn.functional.silu(z), rtol=1e-12, atol=1e-12)


def test_time_reversal_symmetry_of_biscan():
    x, dt, A, B, C, D, h0 = _rand_problem()
    xb, Bb, Cb = torch.randn_like(x), torch.randn_like(B), torch.randn_like(C)
    yf, yb, lf, lb = R.issm_biscan_ref(x, xb, dt, A, B, Bb, C, Cb, D=D, initial_states=h0)
    y2, l2 = R.issm_scan_sequential(x, dt, A, B, C, D=D, initial_states=h0)
    torch.testing.assert_close(yf, y2, rtol=0, atol=0)
    # backward direction by explicit index reversal in a loop
    yb_np, lb_np = _brute_numpy(xb.flip(1), dt.flip(1), A, Bb.flip(1), Cb.flip(1), D, h0)
    np.testing.assert_allclose(yb.numpy(), yb_np[:, ::-1], rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(lb.numpy(), lb_np, rtol=1e-12, atol=1e-12)


def test_gradcheck_sequential_tiny():
    x, dt, A, B, C, D, h0 = _rand_problem(Bsz=1, L=4, H=2, P=2, N=3, G=1)
    ins = [t.clone().requires_grad_() for t in (x, dt, A, B, C, D, h0)]

    def f(x, dt, A, B, C, D, h0):
        return R.issm_scan_sequential(x, dt, A, B, C, D=D, initial_states=h0)

    assert torch.autograd.gradcheck(f, ins, eps=1e-6, atol=1e-7, rtol=1e-5)


@pytest.mark.parametrize("L,chunk,softplus", [(12, 4, False), (10, 4, True), (7, 8, True)])
def test_closed_form_backward_matches_autograd(L, chunk, softplus):
    x, dt, A, B, C, D, h0 = _rand_problem(L=L, seed=3)
    if softplus:
        dt = dt * 8.0 - 3.0                     # pre-softplus values, some negative
    dt_bias = torch.randn(A.shape, dtype=torch.float64) * 0.1
    lim = (0.05, 1.5) if softplus else (0.0, R.INF)
    dy = torch.randn_like(x)
    dfin = torch.randn_like(h0)
    ins = [t.clone().requires_grad_() for t in (x, dt, A, B, C, D, dt_bias, h0)]
    y, fin = R.issm_scan_sequential(ins[0], ins[1], ins[2], ins[3], ins[4], D=ins[5], dt_bias=ins[6],
                                    initial_states=ins[7], dt_softplus=softplus, dt_limit=lim)
    (y * dy).sum().add((fin * dfin).sum()).backward()
    g = R.issm_bwd_closed_form(x, dt, A, B, C, chunk, dy, dfinal=dfin, D=D, dt_bias=dt_bias,
                               initial_states=h0, dt_softplus=softplus, dt_limit=lim)
    names = ["dx", "ddt", "dA", "dB", "dC", "dD", "ddt_bias", "dinitial_states"]
    for name, t in zip(names, ins):
        torch.testing.assert_close(g[name], t.grad, rtol=1e-9, atol=1e-9, msg=lambda m: f"{name}: {m}")
    # invariant: dA = sum_{b,t} da * dt'  is implied by ddt/dA agreeing; also clamp mask zeros exist
    if softplus:
        assert (g["ddt"] == 0).any()


def test_closed_form_intermediates_against_chunk_by_chunk_autograd():
    """The per-chunk quantities that issm_bwd_closed_form(intermediates=True) returns -- and that the GPU stage tests
    compare the kernels with -- derived independently: the sequence is scanned chunk by chunk with the token-by-token
    recurrence, each chunk started from the previous chunk's final state, with a zero "extra log-decay" leaf eps_c[n]
    multiplying the state handed to the next chunk.  Then, by autograd alone,
      states[c]  = state entering chunk c              S[c]   = final state of chunk c scanned from a zero state
      y          = concatenated chunk outputs          dS[c]  = dL / d(state handed over after chunk c)
      dH[c]      = dL / d(state entering chunk c) holding later states fixed  (= grad through chunk c's outputs only)
      g_next[c]  = dL / d eps_c   (= sum_p dS[c] * states[c + 1]: what reaches the chunk's total decay via the states)
    and M, dM from their definitions with scalar loops."""
    chunk, L = 4, 11                                     # ragged last chunk
    x, dt, A, B, C, D, h0 = _rand_problem(L=L, seed=11)
    Bsz, _, H, P = x.shape
    N = dt.shape[-1]
    dy, dfin = torch.randn_like(x), torch.randn_like(h0)
    out = R.issm_bwd_closed_form(x, dt, A, B, C, chunk, dy, dfinal=dfin, D=None, initial_states=h0, intermediates=True)
    nc = math.ceil(L / chunk)
    states, eps, ys, handed = [h0.clone().requires_grad_()], [], [], []
    for c in range(nc):
        sl = slice(c * chunk, min(L, (c + 1) * chunk))
        y_c, fin_c = R.issm_scan_sequential(x[:, sl], dt[:, sl], A, B[:, sl], C[:, sl], initial_states=states[-1])
        e = torch.zeros(Bsz, H, N, dtype=torch.float64, requires_grad=True)
        nxt = fin_c * torch.exp(e)[:, :, None, :]
        nxt.retain_grad()
        eps.append(e); ys.append(y_c); handed.append(nxt)
        states.append(nxt)
    y = torch.cat(ys, dim=1)
    ((y * dy).sum() + (states[-1] * dfin).sum()).backward()
    close = lambda a, b, name: torch.testing.assert_close(a, b, rtol=1e-9, atol=1e-10, msg=lambda m: f"{name}: {m}")
    close(out["y"], y.detach(), "y")
    close(out["states"], torch.stack([t.detach() for t in states], dim=1), "states")
    close(out["dS"], torch.stack([t.grad for t in handed], dim=1), "dS")
    close(out["g_next"], torch.stack([e.grad for e in eps], dim=1), "g_next")
    close(out["dinitial_states"], states[0].grad, "dh0")
    for c in range(nc):
        sl = slice(c * chunk, min(L, (c + 1) * chunk))
        # chunk-local end state: the chunk scanned from nothing
        _, s_c = R.issm_scan_sequential(x[:, sl], dt[:, sl], A, B[:, sl], C[:, sl])
        close(out["S"][:, c], s_c, f"S[{c}]")
        # dH[c]: gradient of this chunk's outputs alone with respect to its entry state
        hin = states[c].detach().clone().requires_grad_()
        y_c, _ = R.issm_scan_sequential(x[:, sl], dt[:, sl], A, B[:, sl], C[:, sl], initial_states=hin)
        (y_c * dy[:, sl]).sum().backward()
        close(out["dH"][:, c], hin.grad, f"dH[{c}]")
    # M[l][s] = sum_n C[l,n] B[s,n] dt[s,n] exp(sum_{s<k<=l} dt[k,n] A[n]) and dM = tril(dy x^T), scalar loops on (b=1, h=2)
    b, h, g = 1, 2, 2 // (H // B.shape[2])
    a = (dt * A[None, None]).numpy()
    for c in range(nc):
        lo, hi = c * chunk, min(L, (c + 1) * chunk)
        for l in range(lo, hi):
            for s_ in range(lo, l + 1):
                m = sum(C[b, l, g, n].item() * B[b, s_, g, n].item() * dt[b, s_, h, n].item()
                        * math.exp(a[b, s_ + 1:l + 1, h, n].sum()) for n in range(N))
                assert abs(out["M"][b, c, h, l - lo, s_ - lo].item() - m) < 1e-10
                dm = sum(dy[b, l, h, p].item() * x[b, s_, h, p].item() for p in range(P))
                assert abs(out["dM"][b, c, h, l - lo, s_ - lo].item() - dm) < 1e-10


def test_gated_rmsnorm_closed_form_and_grad():
    x = torch.randn(3, 5, 8, dtype=torch.float64)
    z = torch.randn(3, 5, 8, dtype=torch.float64)
    w = torch.randn(8, dtype=torch.float64)
    y = R.gated_rmsnorm_ref(x, w, z=z, eps=1e-5, norm_before_gate=False)
    u = x * z * torch.sigmoid(z)
    exp = u / torch.sqrt((u * u).mean(-1, keepdim=True) + 1e-5) * w
    torch.testing.assert_close(y, exp, rtol=1e-13, atol=1e-13)
    y2 = R.gated_rmsnorm_ref(x, w, z=z, eps=1e-5, norm_before_gate=True)
    exp2 = x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-5) * w * z * torch.sigmoid(z)
    torch.testing.assert_close(y2, exp2, rtol=1e-13, atol=1e-13)
    # scale invariance of rmsnorm without gate (eps -> 0)
    y3 = R.gated_rmsnorm_ref(x, w, eps=0.0)
    torch.testing.assert_close(R.gated_rmsnorm_ref(3.0 * x, w, eps=0.0), y3, rtol=1e-12, atol=1e-12)
    # each row of y3/w has unit mean square
    torch.testing.assert_close(((y3 / w) ** 2).mean(-1), torch.ones(3, 5, dtype=torch.float64), rtol=1e-12, atol=1e-12)
    ins = [t.clone().requires_grad_() for t in (x[:1, :2], w, z[:1, :2])]
    assert torch.autograd.gradcheck(lambda a, b, c: R.gated_rmsnorm_ref(a, b, z=c), ins, eps=1e-6, atol=1e-7)


def test_layernorm_form_against_the_library_routines():
    """layer_norm=True / bias: torch's own layer_norm (one group) and group_norm (several groups per row) are the
    library routines; the gate is the plain product on either side; shift invariance and the bias as closed forms."""
    F = torch.nn.functional
    x = torch.randn(6, 24, dtype=torch.float64)
    z = torch.randn(6, 24, dtype=torch.float64)
    w = torch.randn(24, dtype=torch.float64)
    b = torch.randn(24, dtype=torch.float64)
    y = R.gated_rmsnorm_ref(x, w, eps=1e-5, bias=b, layer_norm=True)
    torch.testing.assert_close(y, F.layer_norm(x, (24,), w, b, eps=1e-5), rtol=1e-12, atol=1e-12)
    yg = R.gated_rmsnorm_ref(x, w, eps=1e-5, bias=b, layer_norm=True, group_size=8)
    torch.testing.assert_close(yg, F.group_norm(x, 3, w, b, eps=1e-5), rtol=1e-12, atol=1e-12)
    # gate after the norm multiplies the biased output; gate before the norm replaces the input
    y1 = R.gated_rmsnorm_ref(x, w, z=z, eps=1e-5, bias=b, layer_norm=True, norm_before_gate=True)
    torch.testing.assert_close(y1, F.layer_norm(x, (24,), w, b, eps=1e-5) * F.silu(z), rtol=1e-12, atol=1e-12)
    y0 = R.gated_rmsnorm_ref(x, w, z=z, eps=1e-5, bias=b, layer_norm=True, norm_before_gate=False)
    torch.testing.assert_close(y0, F.layer_norm(x * F.silu(z), (24,), w, b, eps=1e-5), rtol=1e-12, atol=1e-12)
    # a constant added to a row changes nothing with the mean subtracted, and does change the RMS form
    torch.testing.assert_close(R.gated_rmsnorm_ref(x + 3.0, w, layer_norm=True), R.gated_rmsnorm_ref(x, w, layer_norm=True),
                               rtol=1e-10, atol=1e-10)
    assert (R.gated_rmsnorm_ref(x + 3.0, w) - R.gated_rmsnorm_ref(x, w)).abs().max() > 0.1
    # the bias of the RMS form is a plain addition
    torch.testing.assert_close(R.gated_rmsnorm_ref(x, w, bias=b), R.gated_rmsnorm_ref(x, w) + b, rtol=1e-13, atol=1e-13)


@pytest.mark.parametrize("first_id", [0, 4])
def test_packed_sequences_are_independent_runs(first_id):
    """seq_idx: a row that packs three sequences gives, segment by segment, what three separate runs give -- outputs,
    final state and gradients.  The initial states count as id 0 (issm_chunk_scan.py:123, issm_state_passing.py:91):
    they feed the first sequence when its id is 0 and nothing when the ids start higher."""
    torch.manual_seed(3)
    Bsz, L, H, P, N = 1, 11, 2, 3, 4
    x = torch.randn(Bsz, L, H, P, dtype=torch.float64, requires_grad=True)
    dt = (torch.rand(Bsz, L, H, N, dtype=torch.float64) * 0.5).requires_grad_()
    A = -torch.rand(H, N, dtype=torch.float64) * 3
    Bm = torch.randn(Bsz, L, 1, N, dtype=torch.float64)
    Cm = torch.randn(Bsz, L, 1, N, dtype=torch.float64)
    h0 = torch.randn(Bsz, H, P, N, dtype=torch.float64, requires_grad=True)
    seq = torch.tensor([[0, 0, 0, 3, 3, 3, 3, 3, 5, 5, 5]]) + first_id
    y, fin = R.issm_scan_sequential(x, dt, A, Bm, Cm, initial_states=h0, seq_idx=seq)
    w = torch.randn_like(y)
    gx, gdt, gh0 = torch.autograd.grad((y * w).sum() + fin.sum(), (x, dt, h0))
    ys, gxs, gdts = [], [], []
    for lo, hi in ((0, 3), (3, 8), (8, 11)):
        xs = x.detach()[:, lo:hi].clone().requires_grad_()
        dts = dt.detach()[:, lo:hi].clone().requires_grad_()
        h0s = h0.detach().clone().requires_grad_()
        yi, fi = R.issm_scan_sequential(xs, dts, A, Bm[:, lo:hi], Cm[:, lo:hi],
                                        initial_states=h0s if lo == 0 and first_id == 0 else None)
        loss = (yi * w[:, lo:hi]).sum() + (fi.sum() if hi == L else 0.0)
        a, b = torch.autograd.grad(loss, (xs, dts), retain_graph=True)
        if lo == 0:
            gh0s = torch.autograd.grad(loss, h0s)[0] if first_id == 0 else torch.zeros_like(h0)
        ys.append(yi.detach()); gxs.append(a); gdts.append(b)
    torch.testing.assert_close(y.detach(), torch.cat(ys, 1), rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(fin.detach(), fi.detach(), rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(gx, torch.cat(gxs, 1), rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(gdt, torch.cat(gdts, 1), rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(gh0, gh0s, rtol=1e-12, atol=1e-12)


def test_packed_sequences_match_the_id_equality_masks_of_the_reference_kernels():
    """The reference has no reset: each of its kernels multiplies a decay by [id == id'] -- token pairs inside a chunk
    (issm_cabt_bmm.py:146-148), a token against the id before its chunk for the incoming state, with 0 before the first
    chunk (issm_chunk_scan.py:123,133), and chunk ends against each other in the state passing (issm_state_passing.py:
    91-99).  For ids that never decrease all of these say "same sequence", so  y_l = sum_{s<=l} [id_l == id_s] C_l
    decay(l,s) dt_s B_s x_s + [id_l == 0 == every id before l] C_l decay(l,-1) h0,  evaluated here pair by pair."""
    torch.manual_seed(5)
    L, P, N = 9, 2, 3
    x = torch.randn(1, L, 1, P, dtype=torch.float64)
    dt = torch.rand(1, L, 1, N, dtype=torch.float64) * 0.5
    A = -torch.rand(1, N, dtype=torch.float64) * 2
    Bm = torch.randn(1, L, 1, N, dtype=torch.float64)
    Cm = torch.randn(1, L, 1, N, dtype=torch.float64)
    h0 = torch.randn(1, 1, P, N, dtype=torch.float64)
    for ids in ([0, 0, 0, 1, 1, 2, 2, 2, 2], [1, 1, 1, 1, 2, 2, 2, 3, 3], [0] * 9, [2] * 9):
        y, _ = R.issm_scan_sequential(x, dt, A, Bm, Cm, initial_states=h0, seq_idx=torch.tensor([ids]))
        a = dt[0, :, 0] * A[0]                                       # (L, N)
        for l in range(L):
            for p_ in range(P):
                acc = 0.0
                for n in range(N):
                    for s_ in range(l + 1):
                        if ids[l] == ids[s_]:
                            acc += (Cm[0, l, 0, n] * torch.exp(a[s_ + 1:l + 1, n].sum()) * dt[0, s_, 0, n]
                                    * Bm[0, s_, 0, n] * x[0, s_, 0, p_]).item()
                    if ids[l] == 0:
                        acc += (Cm[0, l, 0, n] * torch.exp(a[:l + 1, n].sum()) * h0[0, 0, p_, n]).item()
                assert abs(acc - y[0, l, 0, p_].item()) < 1e-12, (ids, l, p_)


def test_make_inputs_is_deterministic_and_in_range():
    a = R.make_inputs(1, 8, 2, 4, 8, seed=7)
    b = R.make_inputs(1, 8, 2, 4, 8, seed=7)
    for k in a:
        assert torch.equal(a[k], b[k])
    assert a["dt_raw"].min() >= -4 and a["dt_raw"].max() <= -1
    assert (a["A"] <= -1).all() and (a["A"] >= -16).all()
    assert (a["A"][:, :1] == a["A"]).all()


def test_bench_generator_draws_the_same_problem_as_the_tests_generator():
    """bench.py carries its own copy of the generator (it may not import this package's checker outside its CPU
    baseline): a seed must name the same tensors in both."""
    import bench
    a = R.make_inputs(2, 24, 3, 4, 8, G=1, seed=1235, h0_std=0.1)
    b = bench.synthetic_inputs(torch, 2, 24, 3, 4, 8, G=1, seed=1235, h0_std=0.1)
    for k in b:
        assert torch.equal(a[k], b[k]), k


def test_clamp_limits_are_the_fp32_roundings_the_kernels_receive():
    """A dt that an fp32 caller clamped to 0.02 equals float32(0.02) = 0.0199999995529...: it sits on the limit the
    reference's kernels compare with (their dt_min is an fp32 scalar) and keeps its gradient; against the double 0.02
    it would count as clamped.  One element below and one above for contrast."""
    import numpy as np
    lim = float(np.float32(0.02))
    dt = torch.tensor([lim, float(np.nextafter(np.float32(0.02), np.float32(0))), 0.05], dtype=torch.float64).reshape(1, 3, 1, 1)
    dt.requires_grad_()
    out = R.dt_transform(dt, None, False, (0.02, 0.3))
    out.sum().backward()
    assert out.flatten().tolist() == [lim, lim, 0.05]
    assert dt.grad.flatten().tolist() == [1.0, 0.0, 1.0]
    x = torch.randn(1, 3, 1, 2, dtype=torch.float64)
    A, B, C = -torch.ones(1, 1, dtype=torch.float64), torch.ones(1, 3, 1, 1, dtype=torch.float64), torch.ones(1, 3, 1, 1, dtype=torch.float64)
    g = R.issm_bwd_closed_form(x, dt.detach(), A, B, C, 4, torch.ones_like(x), dt_limit=(0.02, 0.3))
    assert g["ddt"].flatten()[0] != 0 and g["ddt"].flatten()[1] == 0
