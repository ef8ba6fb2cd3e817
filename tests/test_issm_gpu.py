"""Parity of the HIP path (through the C ABI) with the CPU oracle on identical seeded inputs.

Error measure, stated once: for every tensor we check BOTH
    rel_l2  = ||a-b||_2 / ||b||_2      and      rel_inf = max|a-b| / max|b|
against the fp64 oracle.  Tolerances are the ones the task names: fp32 forward <= 1e-4,
fp32 gradients <= 1e-3; bf16 forward <= 2e-2, bf16 gradients <= 5e-2.
"""
import ctypes as C
import math
import sys

import pytest
import torch

from oracle import issm_ref as R

pytestmark = pytest.mark.gpu

FWD32, BWD32, FWD16, BWD16 = 1e-4, 1e-3, 2e-2, 5e-2


def _say(msg):
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


def _err(a, b):
    a = a.detach().double().cpu()
    b = b.detach().double().cpu()
    assert a.shape == b.shape, (a.shape, b.shape)
    assert torch.isfinite(a).all(), "non-finite values in kernel output"
    l2 = ((a - b).norm() / b.norm().clamp_min(1e-300)).item()
    li = ((a - b).abs().max() / b.abs().max().clamp_min(1e-300)).item()
    return l2, li


def _check(name, a, b, tol):
    l2, li = _err(a, b)
    print(f"    {name:18s} rel_l2={l2:.3e} rel_inf={li:.3e} (tol {tol:g})", flush=True)
    assert l2 <= tol and li <= tol, f"{name}: rel_l2={l2:.3e} rel_inf={li:.3e} > {tol:g}"


def _problem(Bsz, L, H, P, N, G, seed, h0=True, softplus=True, D="h", z=False, bias=True):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g)
    u = lambda *s: torch.rand(*s, generator=g)
    d = dict(x=r(Bsz, L, H, P), A=-torch.exp(u(H, N) * math.log(16.0)), B=r(Bsz, L, G, N) / math.sqrt(N),
             C=r(Bsz, L, G, N) / math.sqrt(N))
    if softplus:
        d["dt"] = u(Bsz, L, H, N) * 3.0 - 4.0
        d["dt_bias"] = r(H, N) * 0.2 if bias else None
        d["dt_limit"] = (0.03, 0.25)           # both clamp sides active
    else:
        d["dt"] = torch.nn.functional.softplus(u(Bsz, L, H, N) * 3.0 - 4.0)
        d["dt"][0, 0, 0, :3] = -0.1            # negative dt is clamped to 0 by the default limit
        d["dt_bias"] = None
        d["dt_limit"] = (0.0, float("inf"))
    d["softplus"] = softplus
    d["D"] = None if D is None else (r(H) if D == "h" else r(H, P))
    d["z"] = r(Bsz, L, H, P) if z else None
    d["h0"] = r(Bsz, H, P, N) * 0.5 if h0 else None
    d["dy"] = r(Bsz, L, H, P)
    d["dfinal"] = r(Bsz, H, P, N)
    return d


def _oracle(d, names):
    ins = {k: d[k].double().clone().requires_grad_() for k in names if d[k] is not None}
    y, fin = R.issm_scan_sequential(ins["x"], ins["dt"], ins["A"], ins["B"], ins["C"], D=ins.get("D"),
                                    z=ins.get("z"), dt_bias=ins.get("dt_bias"), initial_states=ins.get("h0"),
                                    dt_softplus=d["softplus"], dt_limit=d["dt_limit"])
    ((y * d["dy"].double()).sum() + (fin * d["dfinal"].double()).sum()).backward()
    return y.detach(), fin.detach(), {k: v.grad for k, v in ins.items()}


GRAD_NAMES = ["x", "dt", "A", "B", "C", "D", "z", "dt_bias", "h0"]


def _run_operator(d, dtype, chunk_size=64):
    from dest3d_amd import ISSM_chunk_scan_combined
    dev = "cuda"
    cast = lambda t, dt_=dtype: None if t is None else t.to(dev, dt_).requires_grad_()
    ins = dict(x=cast(d["x"]), dt=cast(d["dt"]), A=cast(d["A"], torch.float32), B=cast(d["B"]), C=cast(d["C"]),
               D=cast(d["D"], torch.float32), z=cast(d["z"]), dt_bias=cast(d["dt_bias"], torch.float32),
               h0=cast(d["h0"], torch.float32))
    y, fin = ISSM_chunk_scan_combined(ins["x"], ins["dt"], ins["A"], ins["B"], ins["C"], chunk_size, D=ins["D"],
                                      z=ins["z"], dt_bias=ins["dt_bias"], initial_states=ins["h0"],
                                      dt_softplus=d["softplus"], dt_limit=d["dt_limit"], return_final_states=True)
    assert y.dtype == dtype and fin.dtype == torch.float32
    loss = (y.float() * d["dy"].to(dev)).sum() + (fin * d["dfinal"].to(dev)).sum()
    loss.backward()
    torch.cuda.synchronize()
    return y, fin, {k: (None if v is None else v.grad) for k, v in ins.items()}, ins


CASES = [
    # Bsz, L, H, P, N, G, kwargs
    (2, 64, 2, 32, 64, 1, dict()),
    (2, 150, 4, 32, 96, 2, dict(D="hp")),
    (1, 200, 2, 16, 40, 1, dict(z=True)),
    (1, 130, 2, 36, 128, 1, dict(softplus=False, D="h")),
    (1, 96, 2, 64, 64, 2, dict(h0=False, bias=False, D=None)),
    (1, 320, 8, 32, 256, 1, dict(softplus=False)),
    (1, 70, 2, 20, 30, 1, dict(D="hp", z=True)),         # N not a multiple of 4, P not a multiple of 16
    (1, 1, 1, 8, 16, 1, dict()),                          # a single token
    (1, 128, 2, 36, 64, 1, dict(D="hp", z=True)),        # complete chunks / slices, ragged head dimension
    (2, 64, 2, 20, 128, 2, dict(softplus=False)),
    (1, 192, 1, 64, 64, 1, dict()),                       # complete tiles, widest head dimension
    # state passing: 32-column slices with stand-in rows, 37 chunks (six register slots, a last batch of one step)
    (1, 64 * 37, 2, 20, 64, 1, dict()),
    (1, 64 * 7 - 5, 1, 40, 96, 1, dict(D="hp")),          # two rows per thread, four slots, ragged last chunk
    (4, 64 * 5, 8, 36, 256, 1, dict(softplus=False)),    # 64-column slices, three slots, 5 chunks, P = 36
    (16, 70, 8, 16, 96, 1, dict()),                      # many workgroups, N a multiple of 32 but not of 64
    # state passing, few workgroups and many chunks (column sums of several steps added up together): 35 chunks
    # leave a last batch of five steps with one row per thread, of three with two rows per thread
    (1, 64 * 35, 1, 32, 32, 1, dict(softplus=False)),
    (1, 64 * 35 - 9, 1, 40, 32, 1, dict(D="h")),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: f"B{c[0]}L{c[1]}H{c[2]}P{c[3]}N{c[4]}G{c[5]}" + "".join(
    f"_{k}{v}" for k, v in c[6].items()))
def test_operator_fp32_matches_oracle(case):
    Bsz, L, H, P, N, G, kw = case
    _say(f"operator fp32 {case}")
    d = _problem(Bsz, L, H, P, N, G, seed=11 + L, **kw)
    y_ref, fin_ref, g_ref = _oracle(d, GRAD_NAMES)
    y, fin, g, _ = _run_operator(d, torch.float32, chunk_size=64 if L % 2 else 256)
    _check("out", y, y_ref, FWD32)
    _check("final_states", fin, fin_ref, FWD32)
    for k in GRAD_NAMES:
        if d[k] is None:
            assert g[k] is None
            continue
        _check("d" + k, g[k], g_ref[k], BWD32)


@pytest.mark.parametrize("P", [128, 96, 67])
def test_head_dimension_above_the_tile_limit(P):
    """Heads wider than the kernels' 64 run as several narrower heads that share dt, A, dt_bias and the group's B, C
    (128 -> 2 x 64, 96 -> 2 x 48, the prime 67 -> 67 x 1); every gradient, the repeated parameters' included."""
    _say(f"operator fp32 headdim {P}")
    d = _problem(1, 100, 2, P, 48, 1, seed=P, D="hp", z=True)
    y_ref, fin_ref, g_ref = _oracle(d, GRAD_NAMES)
    y, fin, g, _ = _run_operator(d, torch.float32)
    _check("out", y, y_ref, FWD32)
    _check("final_states", fin, fin_ref, FWD32)
    for k in GRAD_NAMES:
        _check("d" + k, g[k], g_ref[k], BWD32)
    if P == 128:
        from dest3d_amd import ISSM_biscan_combined, ISSM_chunk_scan_combined
        cu = lambda t: t.cuda()
        x2 = torch.randn(1, 100, 2, P, generator=torch.Generator().manual_seed(1))
        args = (cu(d["dt"]), cu(d["A"]), cu(d["B"]), cu(d["B"]), cu(d["C"]), cu(d["C"]))
        yf, yb, lf, lb = ISSM_biscan_combined(cu(d["x"]), cu(x2), *args, 64, D=cu(d["D"]), dt_bias=cu(d["dt_bias"]),
                                              dt_softplus=True, dt_limit=d["dt_limit"])
        flip = lambda t: t.flip(1)
        yb1, lb1 = ISSM_chunk_scan_combined(flip(cu(x2)), flip(args[0]), args[1], flip(args[2]), flip(args[4]), 64,
                                            D=cu(d["D"]), dt_bias=cu(d["dt_bias"]), dt_softplus=True,
                                            dt_limit=d["dt_limit"], return_final_states=True)
        assert yb.shape == (1, 100, 2, P) and lb.shape == (1, 2, P, 48)
        assert torch.equal(yb, flip(yb1)) and torch.equal(lb, lb1)


def _seq_ids(Bsz, L, cuts):
    """(Bsz, L) ids that go up by one at the given token positions (row b uses cuts[b])."""
    s = torch.zeros(Bsz, L, dtype=torch.int32)
    for b in range(Bsz):
        for c in cuts[b]:
            s[b, c:] += 1
    return s


@pytest.mark.parametrize("first_id", [0, 1])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_packed_sequences_match_oracle(dtype, first_id):
    """seq_idx (issm_combined.py:29): several sequences packed into a batch row; no state crosses a change of id.
    Changes inside a chunk, at a chunk's first row, at its last row, in adjacent rows and in the ragged last chunk;
    row 1 of the batch has no change at all.  Every gradient against the oracle's recurrence with resets.
    first_id = 1: the ids of batch row 0 start at 1, so its initial states (which count as id 0,
    issm_chunk_scan.py:123) reach no token and receive a zero gradient; batch row 1 still starts at 0."""
    _say(f"operator with seq_idx {dtype} first id {first_id}")
    L_ = 64 * 3 + 21
    d = _problem(2, L_, 2, 32, 96, 1, seed=77, D="h", z=True)
    if dtype == torch.bfloat16:
        for k in ("x", "dt", "B", "C", "z"):
            d[k] = d[k].bfloat16().float()
    seq = _seq_ids(2, L_, [[5, 40, 41, 64, 127, 130, 200], []])
    seq[0] += first_id
    ins = {k: d[k].double().clone().requires_grad_() for k in GRAD_NAMES if d[k] is not None}
    y_ref, fin_ref = R.issm_scan_sequential(ins["x"], ins["dt"], ins["A"], ins["B"], ins["C"], D=ins["D"], z=ins["z"],
                                            dt_bias=ins["dt_bias"], initial_states=ins["h0"],
                                            dt_softplus=d["softplus"], dt_limit=d["dt_limit"], seq_idx=seq)
    ((y_ref * d["dy"].double()).sum() + (fin_ref * d["dfinal"].double()).sum()).backward()
    from dest3d_amd import ISSM_chunk_scan_combined
    cast = lambda t, dt_=dtype: None if t is None else t.to("cuda", dt_).requires_grad_()
    g = dict(x=cast(d["x"]), dt=cast(d["dt"]), A=cast(d["A"], torch.float32), B=cast(d["B"]), C=cast(d["C"]),
             D=cast(d["D"], torch.float32), z=cast(d["z"]), dt_bias=cast(d["dt_bias"], torch.float32),
             h0=cast(d["h0"], torch.float32))
    y, fin = ISSM_chunk_scan_combined(g["x"], g["dt"], g["A"], g["B"], g["C"], 64, D=g["D"], z=g["z"],
                                      dt_bias=g["dt_bias"], initial_states=g["h0"], seq_idx=seq.cuda().long(),
                                      dt_softplus=d["softplus"], dt_limit=d["dt_limit"], return_final_states=True)
    ((y.float() * d["dy"].cuda()).sum() + (fin * d["dfinal"].cuda()).sum()).backward()
    torch.cuda.synchronize()
    ft, bt = (FWD32, BWD32) if dtype == torch.float32 else (FWD16, BWD16)
    _check("out", y, y_ref.detach(), ft)
    _check("final_states", fin, fin_ref.detach(), ft)
    for k in GRAD_NAMES:
        if d[k] is not None:
            _check("d" + k, g[k].grad, ins[k].grad, bt)
    if first_id:
        # the kernels multiply a decay across a change of id by 2^-128 where the reference multiplies by 0
        assert ins["h0"].grad[0].abs().max() == 0 and g["h0"].grad[0].abs().max() < 1e-30


def test_dt_already_clamped_by_an_fp32_caller_keeps_its_gradient():
    """dt = clamp(x, 0.02, 0.3) computed in fp32 and passed with dt_limit = (0.02, 0.3): a third of the entries sit
    exactly on float32(0.02) or float32(0.3).  They are not *outside* the limits, so their gradient passes, in the
    kernels (fp32 compare, as in the reference) and in the oracle (limits rounded to fp32)."""
    _say("dt on the clamp limits")
    d = _problem(2, 100, 2, 16, 64, 1, seed=31, softplus=False)
    d["dt"] = torch.clamp(torch.rand(2, 100, 2, 64, generator=torch.Generator().manual_seed(5)) * 0.45 - 0.05, 0.02, 0.3)
    d["dt_limit"] = (0.02, 0.3)
    on_limit = ((d["dt"] == d["dt"].min()) | (d["dt"] == d["dt"].max())).float().mean().item()
    assert on_limit > 0.3
    y_ref, fin_ref, g_ref = _oracle(d, GRAD_NAMES)
    assert (g_ref["dt"][d["dt"] == d["dt"].min()] != 0).any()
    y, fin, g, _ = _run_operator(d, torch.float32)
    _check("out", y, y_ref, FWD32)
    for k in GRAD_NAMES:
        if d[k] is not None:
            _check("d" + k, g[k], g_ref[k], BWD32)


def test_packed_sequences_randomised():
    """Seeded draws of shapes, options and change points (up to five per batch row, anywhere, repeats allowed) in fp32
    and bf16 against the oracle's recurrence with resets."""
    from dest3d_amd import ISSM_chunk_scan_combined
    rng = torch.Generator().manual_seed(606)
    pick = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=rng))
    flip = lambda: bool(torch.randint(0, 2, (1,), generator=rng))
    for trial in range(8):
        dtype = torch.bfloat16 if trial % 4 == 3 else torch.float32
        G = pick(1, 2)
        H = G * pick(1, 2)
        Bsz, L_, P, N = pick(1, 3), [pick(2, 200), 64 * pick(1, 4)][trial % 2], pick(1, 64), [pick(1, 200), 64, 128][trial % 3]
        kw = dict(h0=flip(), softplus=flip(), D=[None, "h", "hp"][pick(0, 2)], z=flip(), bias=flip())
        case = (Bsz, L_, H, P, N, G, kw, str(dtype))
        _say(f"randomised seq_idx {trial}: {case}")
        d = _problem(Bsz, L_, H, P, N, G, seed=700 + trial, **kw)
        if dtype == torch.bfloat16:
            for k in ("x", "dt", "B", "C", "z"):
                d[k] = None if d[k] is None else d[k].bfloat16().float()
        seq = _seq_ids(Bsz, L_, [[pick(0, L_ - 1) for _ in range(pick(0, 5))] for _ in range(Bsz)])
        ins = {k: d[k].double().clone().requires_grad_() for k in GRAD_NAMES if d[k] is not None}
        y_ref, fin_ref = R.issm_scan_sequential(ins["x"], ins["dt"], ins["A"], ins["B"], ins["C"], D=ins.get("D"),
                                                z=ins.get("z"), dt_bias=ins.get("dt_bias"), initial_states=ins.get("h0"),
                                                dt_softplus=d["softplus"], dt_limit=d["dt_limit"], seq_idx=seq)
        ((y_ref * d["dy"].double()).sum() + (fin_ref * d["dfinal"].double()).sum()).backward()
        cast = lambda t, dt_=dtype: None if t is None else t.to("cuda", dt_).requires_grad_()
        g = dict(x=cast(d["x"]), dt=cast(d["dt"]), A=cast(d["A"], torch.float32), B=cast(d["B"]), C=cast(d["C"]),
                 D=cast(d["D"], torch.float32), z=cast(d["z"]), dt_bias=cast(d["dt_bias"], torch.float32),
                 h0=cast(d["h0"], torch.float32))
        y, fin = ISSM_chunk_scan_combined(g["x"], g["dt"], g["A"], g["B"], g["C"], 64, D=g["D"], z=g["z"],
                                          dt_bias=g["dt_bias"], initial_states=g["h0"], seq_idx=seq.cuda(),
                                          dt_softplus=d["softplus"], dt_limit=d["dt_limit"], return_final_states=True)
        ((y.float() * d["dy"].cuda()).sum() + (fin * d["dfinal"].cuda()).sum()).backward()
        torch.cuda.synchronize()
        ft, bt = (FWD32, BWD32) if dtype == torch.float32 else (FWD16, BWD16)
        _check(f"out {case}", y, y_ref.detach(), ft)
        _check(f"final_states {case}", fin, fin_ref.detach(), ft)
        for k in GRAD_NAMES:
            if d[k] is not None:
                _check(f"d{k} {case}", g[k].grad, ins[k].grad, bt)


def test_packed_sequences_equal_separate_calls():
    """Two sequences packed into one row give what two calls give, the second without an initial state; a constant
    seq_idx changes nothing (to rounding: a call with seq_idx runs the general kernel variants for every chunk, a call
    without it the complete-tile variants for the complete chunks)."""
    from dest3d_amd import ISSM_chunk_scan_combined
    _say("seq_idx: packed = separate")
    d = _problem(1, 150, 2, 32, 64, 1, seed=9, softplus=False)
    t = {k: d[k].cuda() for k in ("x", "dt", "A", "B", "C")}
    cut = 70
    seq = _seq_ids(1, 150, [[cut]]).cuda()
    y, fin = ISSM_chunk_scan_combined(t["x"], t["dt"], t["A"], t["B"], t["C"], 64, seq_idx=seq, return_final_states=True)
    part = lambda sl: ISSM_chunk_scan_combined(t["x"][:, sl], t["dt"][:, sl], t["A"], t["B"][:, sl], t["C"][:, sl], 64,
                                               return_final_states=True)
    y0, _ = part(slice(0, cut))
    y1, fin1 = part(slice(cut, 150))
    _check("first sequence", y[:, :cut], y0, FWD32)
    _check("second sequence", y[:, cut:], y1, FWD32)
    _check("final state", fin, fin1, FWD32)
    ya, fa = ISSM_chunk_scan_combined(t["x"], t["dt"], t["A"], t["B"], t["C"], 64, seq_idx=torch.zeros_like(seq),
                                      return_final_states=True)
    yb, fb = ISSM_chunk_scan_combined(t["x"], t["dt"], t["A"], t["B"], t["C"], 64, return_final_states=True)
    _check("constant ids: out", ya, yb, 1e-5)
    _check("constant ids: final state", fa, fb, 1e-5)


@pytest.mark.parametrize("L_", [192, 150])   # complete chunks; a ragged last chunk beside complete ones (one launch, two code paths)
def test_operator_bf16_matches_oracle(L_):
    _say(f"operator bf16 L={L_}")
    d = _problem(2, L_, 4, 32, 128, 1, seed=5)
    # the oracle sees the bf16-rounded inputs, so only kernel arithmetic is compared
    for k in ("x", "dt", "B", "C"):
        d[k] = d[k].bfloat16().float()
    y_ref, fin_ref, g_ref = _oracle(d, GRAD_NAMES)
    y, fin, g, _ = _run_operator(d, torch.bfloat16)
    _check("out", y, y_ref, FWD16)
    _check("final_states", fin, fin_ref, FWD16)
    for k in GRAD_NAMES:
        if d[k] is not None:
            assert g[k].dtype == (torch.bfloat16 if k in ("x", "dt", "B", "C") else torch.float32)
            _check("d" + k, g[k], g_ref[k], BWD16)


@pytest.mark.parametrize("P", [16, 32, 36])
def test_bf16_parameter_gradients_survive_the_cancellation_in_the_running_sum_gradient(P):
    """d/d(running sum of dt'A) of a row is a suffix sum in which every pair of rows enters twice with opposite signs;
    ddt_bias and dA add those sums up over all tokens, times A.  With bf16 operands the two entries of a pair must be
    the same rounded product (and the chunk state accurate beyond bf16), or the leftovers pile up with one sign:
    strongly decaying columns (|A| > 10) without an initial state showed up to 19 % of max|ddt_bias|.  Ten times
    below the bf16 bar here."""
    _say(f"bf16 ddt_bias / dA under cancellation, P={P}")
    d = _problem(3, 128, 6, P, 256, 2, seed=4242, h0=False)
    d["dt_limit"] = (0.0, float("inf"))
    for k in ("x", "dt", "B", "C"):
        d[k] = d[k].bfloat16().float()
    y_ref, fin_ref, g_ref = _oracle(d, GRAD_NAMES)
    y, fin, g, _ = _run_operator(d, torch.bfloat16)
    _check("out", y, y_ref, FWD16)
    _check("final_states", fin, fin_ref, 1e-4)     # the chunk states keep 16 significant bits per operand
    for k in ("dt_bias", "A"):
        _check("d" + k, g[k], g_ref[k], BWD16 / 10)
    for k in ("x", "dt", "B", "C", "D"):
        _check("d" + k, g[k], g_ref[k], BWD16)


def test_randomised_shapes_bf16_match_oracle():
    """Seeded draws of every dimension and option in bf16, one direction and the fused pair of directions, against the
    fp64 oracle on the bf16-rounded inputs."""
    from dest3d_amd import ISSM_biscan_combined
    rng = torch.Generator().manual_seed(4048)
    pick = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=rng))
    flip = lambda: bool(torch.randint(0, 2, (1,), generator=rng))
    for trial in range(10):
        G = pick(1, 2)
        H = G * pick(1, 3)
        Bsz, L, P, N = pick(1, 3), [pick(1, 210), 64 * pick(1, 4)][trial % 2], [pick(1, 64), 16, 48, 64][trial % 4], pick(1, 280)
        kw = dict(h0=flip(), softplus=flip(), D=[None, "h", "hp"][pick(0, 2)], z=False, bias=flip())
        bidir = trial % 3 == 2
        case = (Bsz, L, H, P, N, G, kw, "bidir" if bidir else "uni")
        _say(f"randomised bf16 {trial}: {case}")
        d = _problem(Bsz, L, H, P, N, G, seed=900 + trial, **kw)
        for k in ("x", "dt", "B", "C"):
            d[k] = d[k].bfloat16().float()
        if not bidir:
            y_ref, fin_ref, g_ref = _oracle(d, GRAD_NAMES)
            y, fin, g, _ = _run_operator(d, torch.bfloat16, chunk_size=[64, 128, 256][trial % 3])
            _check(f"out {case}", y, y_ref, FWD16)
            _check(f"final_states {case}", fin, fin_ref, FWD16)
            for k in GRAD_NAMES:
                if d[k] is not None:
                    _check(f"d{k} {case}", g[k], g_ref[k], BWD16)
            continue
        gen = torch.Generator().manual_seed(1900 + trial)
        d["x_b"] = torch.randn(d["x"].shape, generator=gen).bfloat16().float()
        d["B_b"] = (torch.randn(d["B"].shape, generator=gen) / math.sqrt(N)).bfloat16().float()
        d["C_b"] = (torch.randn(d["C"].shape, generator=gen) / math.sqrt(N)).bfloat16().float()
        dy_b, dl_b = torch.randn(d["x"].shape, generator=gen), torch.randn(d["dfinal"].shape, generator=gen)
        names = [k for k in ["x", "x_b", "dt", "A", "B", "B_b", "C", "C_b", "D", "dt_bias", "h0"] if d[k] is not None]
        ref = {k: d[k].double().clone().requires_grad_() for k in names}
        ro = R.issm_biscan_ref(ref["x"], ref["x_b"], ref["dt"], ref["A"], ref["B"], ref["B_b"], ref["C"], ref["C_b"],
                               D=ref.get("D"), dt_bias=ref.get("dt_bias"), initial_states=ref.get("h0"),
                               dt_softplus=d["softplus"], dt_limit=d["dt_limit"])
        ((ro[0] * d["dy"].double()).sum() + (ro[1] * dy_b.double()).sum() + (ro[2] * d["dfinal"].double()).sum()
         + (ro[3] * dl_b.double()).sum()).backward()
        io = ("x", "x_b", "dt", "B", "B_b", "C", "C_b")
        gi = {k: d[k].to("cuda", torch.bfloat16 if k in io else torch.float32).requires_grad_() for k in names}
        o = ISSM_biscan_combined(gi["x"], gi["x_b"], gi["dt"], gi["A"], gi["B"], gi["B_b"], gi["C"], gi["C_b"], 64,
                                 D=gi.get("D"), dt_bias=gi.get("dt_bias"), initial_states=gi.get("h0"),
                                 dt_softplus=d["softplus"], dt_limit=d["dt_limit"])
        ((o[0].float() * d["dy"].cuda()).sum() + (o[1].float() * dy_b.cuda()).sum() + (o[2] * d["dfinal"].cuda()).sum()
         + (o[3] * dl_b.cuda()).sum()).backward()
        torch.cuda.synchronize()
        for name, a, b in zip(("y_f", "y_b", "last_f", "last_b"), o, ro):
            _check(f"{name} {case}", a, b.detach(), FWD16)
        for k in names:
            _check(f"d{k} {case}", gi[k].grad, ref[k].grad, BWD16)


def test_biscan_matches_two_flipped_scans_and_oracle():
    from dest3d_amd import ISSM_biscan_combined, ISSM_chunk_scan_combined
    _say("bidirectional fused")
    d = _problem(2, 150, 4, 32, 96, 2, seed=3, softplus=False)
    g = torch.Generator().manual_seed(99)
    d["x_b"] = torch.randn(d["x"].shape, generator=g)
    d["B_b"] = torch.randn(d["B"].shape, generator=g) / math.sqrt(96)
    d["C_b"] = torch.randn(d["C"].shape, generator=g) / math.sqrt(96)
    dy_b = torch.randn(d["x"].shape, generator=g)
    dl_b = torch.randn(d["h0"].shape, generator=g)
    names = ["x", "x_b", "dt", "A", "B", "B_b", "C", "C_b", "D", "h0"]
    ref_in = {k: d[k].double().clone().requires_grad_() for k in names}
    yf, yb, lf, lb = R.issm_biscan_ref(ref_in["x"], ref_in["x_b"], ref_in["dt"], ref_in["A"], ref_in["B"],
                                       ref_in["B_b"], ref_in["C"], ref_in["C_b"], D=ref_in["D"],
                                       initial_states=ref_in["h0"])
    ((yf * d["dy"].double()).sum() + (yb * dy_b.double()).sum() + (lf * d["dfinal"].double()).sum()
     + (lb * dl_b.double()).sum()).backward()
    dev = "cuda"
    gi = {k: d[k].to(dev).requires_grad_() for k in names}
    o = ISSM_biscan_combined(gi["x"], gi["x_b"], gi["dt"], gi["A"], gi["B"], gi["B_b"], gi["C"], gi["C_b"], 64,
                             D=gi["D"], initial_states=gi["h0"])
    ((o[0] * d["dy"].to(dev)).sum() + (o[1] * dy_b.to(dev)).sum() + (o[2] * d["dfinal"].to(dev)).sum()
     + (o[3] * dl_b.to(dev)).sum()).backward()
    torch.cuda.synchronize()
    for name, a, b in zip(("y_f", "y_b", "last_f", "last_b"), o, (yf, yb, lf, lb)):
        _check(name, a, b, FWD32)
    for k in names:
        _check("d" + k, gi[k].grad, ref_in[k].grad, BWD32)
    # and bit-for-bit what the module would compute with flips and two single-direction calls
    fl = lambda t: torch.flip(t, dims=[1])
    with torch.no_grad():
        y2, l2 = ISSM_chunk_scan_combined(fl(gi["x_b"]).contiguous(), fl(gi["dt"]).contiguous(), gi["A"],
                                          fl(gi["B_b"]).contiguous(), fl(gi["C_b"]).contiguous(), 64, D=gi["D"],
                                          initial_states=gi["h0"], return_final_states=True)
    assert torch.equal(fl(y2), o[1]) and torch.equal(l2, o[3])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_heads_outside_the_tile_kernel_range_are_redone_by_the_level_kernel(dtype):
    """Complete tiles, both directions, four heads in two groups: head 1 decays by far more than 2^96 per 16 rows
    everywhere, head 3 only inside one stretch of tokens, heads 0 and 2 nowhere.  The chunk backward then runs partly in
    the tile-base kernel and partly in the level-hierarchy kernel -- per (workgroup, head), in either direction or both
    -- and the two write one ddt / dB / dC together; everything against the fp64 oracle, and the marks themselves
    through the stage entry point."""
    from dest3d_amd import ISSM_biscan_combined
    _say(f"heads in and out of the tile kernel's range, {dtype}")
    Bsz, L_, H, P, N, G = 2, 192, 4, 32, 128, 2
    d = _problem(Bsz, L_, H, P, N, G, seed=61, softplus=False)
    d["dt"] = d["dt"].abs()
    d["A"][1] = -80.0 * (1.0 + torch.rand(N, generator=torch.Generator().manual_seed(1)))
    d["dt"][:, 70:110, 3] *= 80.0
    g = torch.Generator().manual_seed(62)
    d["x_b"] = torch.randn(d["x"].shape, generator=g)
    d["B_b"] = torch.randn(d["B"].shape, generator=g) / math.sqrt(N)
    d["C_b"] = torch.randn(d["C"].shape, generator=g) / math.sqrt(N)
    dy_b = torch.randn(d["x"].shape, generator=g)
    dl_b = torch.randn(d["h0"].shape, generator=g)
    io = ("x", "x_b", "dt", "B", "B_b", "C", "C_b")
    names = list(io) + ["A", "D", "h0"]
    q = {k: (d[k].to(dtype).float() if k in io else d[k]) for k in names}     # what the kernels are handed
    ref_in = {k: q[k].double().clone().requires_grad_() for k in names}
    yf, yb, lf, lb = R.issm_biscan_ref(ref_in["x"], ref_in["x_b"], ref_in["dt"], ref_in["A"], ref_in["B"],
                                       ref_in["B_b"], ref_in["C"], ref_in["C_b"], D=ref_in["D"],
                                       initial_states=ref_in["h0"])
    ((yf * d["dy"].double()).sum() + (yb * dy_b.double()).sum() + (lf * d["dfinal"].double()).sum()
     + (lb * dl_b.double()).sum()).backward()
    dev = "cuda"
    gi = {k: q[k].to(dev, dtype if k in io else torch.float32).requires_grad_() for k in names}
    o = ISSM_biscan_combined(gi["x"], gi["x_b"], gi["dt"], gi["A"], gi["B"], gi["B_b"], gi["C"], gi["C_b"], 64,
                             D=gi["D"], initial_states=gi["h0"])
    ((o[0].float() * d["dy"].to(dev)).sum() + (o[1].float() * dy_b.to(dev)).sum() + (o[2] * d["dfinal"].to(dev)).sum()
     + (o[3] * dl_b.to(dev)).sum()).backward()
    torch.cuda.synchronize()
    # (fp32 bars as in test_extreme_decay_is_finite_and_accurate: running sums in the thousands cost fp32 exponent bits)
    fwd, bwd = (1e-3, 1e-2) if dtype == torch.float32 else (2e-2, 5e-2)
    for name, a, b in zip(("y_f", "y_b", "last_f", "last_b"), o, (yf, yb, lf, lb)):
        _check(name, a, b, fwd)
    for k in names:
        _check("d" + k, gi[k].grad, ref_in[k].grad, 5e-2 if k == "A" else bwd)
    # the marks: one direction through the stage entry point, on intermediates of the right shapes
    if dtype == torch.float32:
        dd = dict(d, z=None, dt_bias=None)
        L, prob, a = _stage_args(dd)
        lib = L.load()
        nc = L_ // 64
        f = lambda *s_: torch.zeros(s_, device=dev)
        states, dst, dm, gn = f(Bsz, nc + 1, H, P, N), f(Bsz, nc, H, P, N), f(Bsz, nc, H, 64, 64), f(Bsz, nc, H, N)
        ddt, dB, dC = f(Bsz, L_, H, N), f(Bsz, L_, G, N), f(Bsz, L_, G, N)
        pa, pb = f(Bsz * nc, H, N), f(Bsz * nc, H, N)
        dyd = d["dy"].to(dev)
        a.dout[0] = L.tensor_desc(dyd)
        a.ddt, a.dB[0], a.dC[0] = (L.tensor_desc(t) for t in (ddt, dB, dC))
        redo = torch.full((lib.issm_bwd_chunk_redo_ints(C.byref(a)),), -1, dtype=torch.int32, device=dev)
        L.check(lib.issm_stage_bwd_chunk(C.byref(a), 0, None, states.data_ptr(), dst.data_ptr(), dm.data_ptr(),
                                         gn.data_ptr(), pa.data_ptr(), pb.data_ptr(), redo.data_ptr()), "bwd_chunk")
        torch.cuda.synchronize()
        marks = redo.view(Bsz, nc, G, N // 64, H // G).cpu()      # (batch, chunk, group, slice, head of the group)
        assert set(marks.unique().tolist()) == {0, 1}
        assert bool((marks[..., 0] == 0).all()), "heads 0 and 2 stay in the tile-base kernel"
        assert bool((marks[:, :, 0, :, 1] == 1).all()), "head 1 is out of range everywhere"
        assert bool((marks[:, 1, 1, :, 1] == 1).all()) and bool((marks[:, 0, 1, :, 1] == 0).all()), \
            "head 3 is out of range only in the chunk that holds tokens 70..109"


def _stage_args(d, ndir=1):
    """ScanArgs + device tensors for direct stage calls (single direction, fp32)."""
    from dest3d_amd import _lib as L
    from dest3d_amd.issm_combined import _Problem
    dev = "cuda"
    t = {k: (None if d[k] is None else d[k].to(dev)) for k in ("x", "dt", "A", "B", "C", "D", "z", "dt_bias", "h0")}
    prob = _Problem([t["x"]], t["dt"], t["A"], [t["B"]], [t["C"]], 64, t["D"], [t["z"]], t["dt_bias"], t["h0"], None,
                    d["softplus"], d["dt_limit"])
    return L, prob, prob.args()


@pytest.mark.parametrize("shape", [
    (2, 150, 4, 32, 96, 2),
    # head dimensions that leave threads of the state-passing kernels without a row of their own (stand-ins that only
    # load): 20 of 32 rows and 40 of 64 with 32-column slices, 36 of 48 with 64-column slices and many workgroups
    (1, 150, 2, 20, 64, 1), (1, 150, 2, 40, 96, 1), (4, 130, 8, 36, 512, 1),
    # complete 64 x 64 tiles only: the kernels written for them (row-lane chunk_local, tile-base bwd_chunk)
    (2, 192, 4, 32, 128, 2), (1, 128, 2, 36, 64, 1), (1, 128, 2, 64, 192, 1),
], ids=lambda s: "B%dL%dH%dP%dN%dG%d" % s)
def test_stage_entry_points_match_oracle_intermediates(shape):
    """chunk_local -> state_passing -> chunk_scan and the backward stages, each against the
    explicit sums of the oracle (oracle.issm_bwd_closed_form(intermediates=True))."""
    _say(f"stage entry points {shape}")
    Bsz, L_, H, P, N, G = shape
    # (the seed is one for which no dt lands within fp32 rounding of a clamp limit: there the mask of the fp32 kernels
    # and of the fp64 oracle differ for that one element, and with it the element's whole ddt)
    d = _problem(Bsz, L_, H, P, N, G, seed=23, D="h")
    ref = R.issm_bwd_closed_form(d["x"], d["dt"], d["A"], d["B"], d["C"], 64, d["dy"], dfinal=d["dfinal"], D=d["D"],
                                 dt_bias=d["dt_bias"], initial_states=d["h0"], dt_softplus=True,
                                 dt_limit=d["dt_limit"], intermediates=True)
    L, prob, a = _stage_args(d)
    lib = L.load()
    dev = "cuda"
    nc = math.ceil(L_ / 64)
    f = lambda *s: torch.full(s, float("nan"), device=dev)
    states, cs_last, cabt = f(Bsz, nc + 1, H, P, N), f(Bsz, nc, H, N), f(Bsz, nc, H, 64, 64)
    L.check(lib.issm_stage_chunk_local(C.byref(a), states.data_ptr(), cs_last.data_ptr(), cabt.data_ptr()), "local")
    torch.cuda.synchronize()
    _check("S (chunk states)", states[:, :nc], ref["S"], FWD32)
    _check("cs_last", cs_last, ref["cs_last"], FWD32)
    _check("M (cabt, tril)", torch.tril(cabt), ref["M"], FWD32)
    fin = f(Bsz, H, P, N)
    a.final_states[0] = fin.data_ptr()
    L.check(lib.issm_stage_state_passing_fwd(C.byref(a), states.data_ptr(), cs_last.data_ptr()), "sp_fwd")
    torch.cuda.synchronize()
    _check("entry states", states, ref["states"], FWD32)
    _check("final", fin, ref["states"][:, -1], FWD32)
    out = f(Bsz, L_, H, P)
    a.out[0] = L.tensor_desc(out)
    L.check(lib.issm_stage_chunk_scan(C.byref(a), states.data_ptr(), cabt.data_ptr(), None), "scan")
    torch.cuda.synchronize()
    _check("y", out, ref["y"] + d["D"].double()[None, None, :, None] * d["x"].double(), FWD32)
    # backward stages
    dy = d["dy"].to(dev)
    dfin = d["dfinal"].to(dev)
    a.dout[0] = L.tensor_desc(dy)
    a.dfinal[0] = dfin.data_ptr()
    dst, dm = f(Bsz, nc, H, P, N), f(Bsz, nc, H, 64, 64)
    L.check(lib.issm_stage_bwd_dstates(C.byref(a), None, dst.data_ptr(), dm.data_ptr()), "dstates")
    torch.cuda.synchronize()
    _check("dH", dst, ref["dH"], BWD32)
    # dM leaves the kernel as a pair of symmetric bf16 matrices per unit, dM = hi + lo to 16 bits (include/issm.h)
    halves = dm.view(torch.bfloat16).reshape(Bsz, nc, H, 2, 64, 64).float()
    _check("dM", torch.tril(halves[:, :, :, 0] + halves[:, :, :, 1]), ref["dM"], BWD32)
    g_next, dh0d = f(Bsz, nc, H, N), f(1, Bsz, H, P, N)
    L.check(lib.issm_stage_state_passing_bwd(C.byref(a), states.data_ptr(), cs_last.data_ptr(), dst.data_ptr(),
                                             g_next.data_ptr(), dh0d.data_ptr()), "sp_bwd")
    torch.cuda.synchronize()
    _check("dS", dst, ref["dS"], BWD32)
    _check("g_next", g_next, ref["g_next"], BWD32)
    _check("dh0", dh0d[0], ref["dinitial_states"], BWD32)
    ddt, dB, dC, dx = f(Bsz, L_, H, N), f(Bsz, L_, G, N), f(Bsz, L_, G, N), f(Bsz, L_, H, P)
    pa, pb, pd = f(Bsz * nc, H, N), f(Bsz * nc, H, N), f(Bsz * nc * H, P)
    a.ddt, a.dB[0], a.dC[0], a.dx[0] = (L.tensor_desc(t) for t in (ddt, dB, dC, dx))
    redo = torch.full((lib.issm_bwd_chunk_redo_ints(C.byref(a)),), -1, dtype=torch.int32, device=dev)
    L.check(lib.issm_stage_bwd_chunk(C.byref(a), 0, None, states.data_ptr(), dst.data_ptr(), dm.data_ptr(),
                                     g_next.data_ptr(), pa.data_ptr(), pb.data_ptr(), redo.data_ptr()), "bwd_chunk")
    L.check(lib.issm_stage_bwd_dx(C.byref(a), None, dst.data_ptr(), cabt.data_ptr(), pd.data_ptr()), "bwd_dx")
    dA, dbias, dD, dh0 = f(H, N), f(H, N), f(H), f(Bsz, H, P, N)
    a.dA, a.ddt_bias, a.dD, a.dh0 = dA.data_ptr(), dbias.data_ptr(), dD.data_ptr(), dh0.data_ptr()
    L.check(lib.issm_stage_bwd_reduce(C.byref(a), pa.data_ptr(), pb.data_ptr(), pd.data_ptr(), dh0d.data_ptr()), "red")
    torch.cuda.synchronize()
    for name, t, k in (("ddt", ddt, "ddt"), ("dB", dB, "dB"), ("dC", dC, "dC"), ("dx", dx, "dx"), ("dA", dA, "dA"),
                       ("ddt_bias", dbias, "ddt_bias"), ("dD", dD, "dD"), ("dh0", dh0, "dinitial_states")):
        _check(name, t, ref[k], BWD32)


def test_inplace_edit_between_forward_and_backward_raises():
    """The operator saves its inputs for the backward as the reference does (issm_combined.py:42): changing one of them
    in place before backward must raise PyTorch's version-counter error, not return gradients of other data."""
    from dest3d_amd import ISSM_chunk_scan_combined
    from dest3d_amd.issm_combined import ISSM_biscan_combined
    print("[case] in-place edit of a saved input", flush=True)
    I = R.make_inputs(1, 70, 2, 16, 32, G=1, seed=3)
    for name in ("x", "dt_raw", "B", "C"):
        g = {k: I[k].cuda().requires_grad_() for k in ("x", "dt_raw", "A", "B", "C")}
        w = {k: v * 1.0 for k, v in g.items()}              # non-leaf copies that may be edited in place
        y = ISSM_chunk_scan_combined(w["x"], w["dt_raw"], w["A"], w["B"], w["C"], 64, dt_softplus=True)
        w[name].mul_(2.0)
        with pytest.raises(RuntimeError, match="modified by an inplace operation"):
            y.sum().backward()
    g = {k: I[k].cuda().requires_grad_() for k in ("x", "dt_raw", "A", "B", "C")}
    w = {k: v * 1.0 for k, v in g.items()}
    yf, yb, _, _ = ISSM_biscan_combined(w["x"], w["x"], w["dt_raw"], w["A"], w["B"], w["B"], w["C"], w["C"], 64,
                                        dt_softplus=True)
    w["dt_raw"].add_(1.0)
    with pytest.raises(RuntimeError, match="modified by an inplace operation"):
        (yf.sum() + yb.sum()).backward()


def test_error_codes_do_not_abort():
    from dest3d_amd import _lib as L
    _say("error codes")
    lib = L.load()
    d = _problem(1, 64, 2, 32, 64, 1, seed=1)
    _, prob, a = _stage_args(d)
    n = C.c_size_t()
    a.dims.headdim = 0
    assert lib.issm_fwd_workspace_bytes(C.byref(a), C.byref(n)) == -2
    a.dims.headdim = 128
    assert lib.issm_fwd_workspace_bytes(C.byref(a), C.byref(n)) == -5 and b"headdim" in lib.issm_last_error()
    a.dims.headdim = 32
    a.flags |= L.FLAG_SEQ_IDX
    assert lib.issm_scan_fwd(C.byref(a)) == -1 and b"seq_idx is NULL" in lib.issm_last_error()
    a.flags &= ~L.FLAG_SEQ_IDX
    a.dt_min = -1.0
    assert lib.issm_scan_fwd(C.byref(a)) == -5
    a.dt_min = 0.0
    assert lib.issm_scan_fwd(C.byref(a)) == -6           # no workspace
    a.io_dtype = 7
    assert lib.issm_scan_fwd(C.byref(a)) == -4
    from dest3d_amd import ISSM_chunk_scan_combined
    t = {k: d[k].cuda() for k in ("x", "dt", "A", "B", "C")}
    with pytest.raises(RuntimeError, match="dt_limit"):
        ISSM_chunk_scan_combined(t["x"], t["dt"], t["A"], t["B"], t["C"], 64, dt_limit=(-1.0, 1.0))
    with pytest.raises(RuntimeError, match="no CPU path"):
        ISSM_chunk_scan_combined(*(d[k] for k in ("x", "dt", "A", "B", "C")), 64)


def test_properties_at_benchmark_shape():
    """Size-independent checks at B=8, L=1024, H=8, P=32, N=256: chunk_size argument invariance,
    closed forms (dt=0; B=0), linearity in x, determinism, and the oracle on one batch element."""
    from dest3d_amd import ISSM_chunk_scan_combined as op
    _say("benchmark shape properties")
    I = R.make_inputs(8, 1024, 8, 32, 256, seed=1235)
    dev = "cuda"
    t = {k: v.to(dev) for k, v in I.items()}
    kw = dict(D=t["D"], dt_softplus=True, return_final_states=True)
    y, fin = op(t["x"], t["dt_raw"], t["A"], t["B"], t["C"], 64, **kw)
    y2, fin2 = op(t["x"], t["dt_raw"], t["A"], t["B"], t["C"], 256, **kw)
    assert torch.equal(y, y2) and torch.equal(fin, fin2)          # chunk_size is a no-op, runs are reproducible
    # linearity in x (h0 = 0, no gate): scan(2x) = 2 scan(x) exactly in binary floating point
    y3, fin3 = op(2 * t["x"], t["dt_raw"], t["A"], t["B"], t["C"], 64, **kw)
    assert torch.equal(y3, 2 * y) and torch.equal(fin3, 2 * fin)
    # dt' = 0 everywhere (clamped): y = C.h0 + D x, final = h0
    h0 = torch.randn(8, 8, 32, 256, device=dev)
    y4, fin4 = op(t["x"], -torch.ones_like(t["dt_raw"]), t["A"], t["B"], t["C"], 64, D=t["D"], initial_states=h0,
                  return_final_states=True)
    ref4 = torch.einsum("bhpn,bln->blhp", h0.double(), t["C"][:, :, 0].double()) + t["D"].double()[None, None, :, None] * t["x"].double()
    _check("dt=0: y", y4, ref4, FWD32)
    assert torch.equal(fin4, h0)
    # B = 0: pure decay of h0 (A scaled down so that 1024 steps of decay stay representable)
    A5 = t["A"] * 0.01
    y5, fin5 = op(t["x"], t["dt_raw"], A5, torch.zeros_like(t["B"]), t["C"], 64, initial_states=h0,
                  dt_softplus=True, return_final_states=True)
    dec = torch.exp(torch.cumsum(torch.nn.functional.softplus(t["dt_raw"].double()) * A5.double()[None, None], dim=1))
    _check("B=0: final", fin5, h0.double() * dec[:, -1][:, :, None, :], FWD32)
    _check("B=0: y", y5, torch.einsum("bhpn,blhn,bln->blhp", h0.double(), dec, t["C"][:, :, 0].double()), FWD32)
    # oracle on batch element 0, forward and all gradients
    sl = {k: (v[:1] if v.dim() == 4 and v.shape[0] == 8 else v) for k, v in I.items()}
    ins = {k: sl[k].double().clone().requires_grad_() for k in ("x", "dt_raw", "A", "B", "C", "D")}
    yr, fr = R.issm_scan_sequential(ins["x"], ins["dt_raw"], ins["A"], ins["B"], ins["C"], D=ins["D"], dt_softplus=True)
    ((yr * sl["dy"].double()).sum() + (fr * sl["dfinal"].double()).sum()).backward()
    gi = {k: sl[k].to(dev).requires_grad_() for k in ins}
    yg, fg = op(gi["x"], gi["dt_raw"], gi["A"], gi["B"], gi["C"], 64, D=gi["D"], dt_softplus=True, return_final_states=True)
    ((yg * sl["dy"].to(dev)).sum() + (fg * sl["dfinal"].to(dev)).sum()).backward()
    torch.cuda.synchronize()
    _check("y[0]", yg, yr, FWD32)
    _check("final[0]", fg, fr, FWD32)
    for k in ins:
        _check("d" + k, gi[k].grad, ins[k].grad, BWD32)


def test_forward_only_at_the_cpu_runnable_configuration():
    """The reference's own CPU-runnable case on the GPU: forward only, fp32, B=2, L=1024, H=8, P=32, N=256, G=1, the
    chunk size 64, dt through softplus with dt_bias inside the
    kernels, zero initial states, no autograd graph.  Both batch elements are checked against the sequential fp64 oracle
    and against the chunked restatement of the reference's formulation (oracle/issm_ref.py: issm_scan_chunked)."""
    from dest3d_amd import ISSM_chunk_scan_combined as op
    _say("config0 forward only B=2")
    I = R.make_inputs(2, 1024, 8, 32, 256, seed=77)
    dev = "cuda"
    t = {k: v.to(dev) for k, v in I.items()}
    bias = I["dt_bias"]
    h0 = torch.zeros(2, 8, 32, 256)
    with torch.no_grad():
        y, fin = op(t["x"], t["dt_raw"], t["A"], t["B"], t["C"], 64, D=t["D"], dt_bias=bias.to(dev),
                    initial_states=h0.to(dev), dt_softplus=True, return_final_states=True)
        torch.cuda.synchronize()
    assert not y.requires_grad and y.dtype == torch.float32
    dbl = {k: v.double() for k, v in I.items()}
    yr, fr = R.issm_scan_sequential(dbl["x"], dbl["dt_raw"], dbl["A"], dbl["B"], dbl["C"], D=dbl["D"],
                                    dt_bias=bias.double(), initial_states=h0.double(), dt_softplus=True)
    _check("y", y, yr, FWD32)
    _check("final", fin, fr, FWD32)
    yc, fc = R.issm_scan_chunked(dbl["x"], R.dt_transform(dbl["dt_raw"], bias.double(), True), dbl["A"], dbl["B"],
                                 dbl["C"], 64, initial_states=h0.double())
    yc = yc + dbl["D"][None, None, :, None] * dbl["x"]
    _check("y vs chunked", y, yc, FWD32)
    _check("final vs chunked", fin, fc, FWD32)


def test_benchmark_shape_bf16_bidirectional():
    """configs[1] with bf16 inputs (x, B, C, dt bf16; A, D fp32; fp32 states), both directions fused, at full size
    (B=8, L=1024, H=8, P=32, N=256): the fused call against two single-direction calls on flipped copies (outputs bit
    for bit; gradients as the sum of the parts), run-to-run reproducibility, and the fp64 oracle on one (batch, head)
    through the fused call -- forward and every gradient inside the bf16 tolerances."""
    from dest3d_amd import ISSM_biscan_combined, ISSM_chunk_scan_combined as op
    _say("benchmark shape bf16 bidirectional B=8 L=1024 H=8 P=32 N=256")
    dev = "cuda"
    I = R.make_inputs(8, 1024, 8, 32, 256, seed=1235, h0_std=0.1)
    g2 = torch.Generator().manual_seed(1236)
    bf = lambda v: v.to(dev, torch.bfloat16)
    t = dict(x=bf(I["x"]), x_b=bf(torch.randn(I["x"].shape, generator=g2)), dt=bf(I["dt_raw"]), B=bf(I["B"]),
             B_b=bf(torch.randn(I["B"].shape, generator=g2) / 16.0), C=bf(I["C"]),
             C_b=bf(torch.randn(I["C"].shape, generator=g2) / 16.0), A=I["A"].to(dev), D=I["D"].to(dev),
             h0=I["h0"].to(dev))
    dy, dy_b = I["dy"].to(dev), torch.randn(I["x"].shape, generator=g2).to(dev)
    df, df_b = I["dfinal"].to(dev), torch.randn(I["dfinal"].shape, generator=g2).to(dev)
    names = ("x", "x_b", "dt", "A", "B", "B_b", "C", "C_b", "D", "h0")

    def fused():
        g = {k: t[k].detach().clone().requires_grad_() for k in names}
        o = ISSM_biscan_combined(g["x"], g["x_b"], g["dt"], g["A"], g["B"], g["B_b"], g["C"], g["C_b"], 64, D=g["D"],
                                 initial_states=g["h0"], dt_softplus=True)
        ((o[0].float() * dy).sum() + (o[1].float() * dy_b).sum() + (o[2] * df).sum() + (o[3] * df_b).sum()).backward()
        torch.cuda.synchronize()
        return o, g

    o, g = fused()
    o2, g2_ = fused()
    for a, b in zip(o, o2):
        assert torch.equal(a, b)
    for k in names:
        assert torch.equal(g[k].grad, g2_[k].grad), f"d{k} differs between two runs"
    # two single-direction calls, the second on flipped copies
    fl = lambda v: torch.flip(v, dims=[1]).contiguous()
    a = {k: t[k].detach().clone().requires_grad_() for k in ("x", "dt", "A", "B", "C", "D", "h0")}
    y1, l1 = op(a["x"], a["dt"], a["A"], a["B"], a["C"], 64, D=a["D"], initial_states=a["h0"], dt_softplus=True,
                return_final_states=True)
    ((y1.float() * dy).sum() + (l1 * df).sum()).backward()
    r = {k: t[k].detach().clone().requires_grad_() for k in ("x_b", "dt", "A", "B_b", "C_b", "D", "h0")}
    y2, l2 = op(fl(r["x_b"]), fl(r["dt"]), r["A"], fl(r["B_b"]), fl(r["C_b"]), 64, D=r["D"], initial_states=r["h0"],
                dt_softplus=True, return_final_states=True)
    ((y2.float() * fl(dy_b)).sum() + (l2 * df_b).sum()).backward()
    torch.cuda.synchronize()
    assert torch.equal(o[0], y1) and torch.equal(o[2], l1)
    assert torch.equal(o[1], torch.flip(y2, dims=[1])) and torch.equal(o[3], l2)
    for k, part in (("x", a["x"]), ("B", a["B"]), ("C", a["C"]), ("x_b", r["x_b"])):
        assert torch.equal(g[k].grad, part.grad), f"d{k}: fused != single direction"
    # the reversed direction of the fused call adds up the heads of a group in the opposite order: equal to rounding
    for k, part in (("B_b", r["B_b"]), ("C_b", r["C_b"])):
        _check(f"d{k} fused vs single direction", g[k].grad, part.grad, 1e-2)
    for k in ("A", "D", "h0"):
        _check(f"d{k} fused vs sum of parts", g[k].grad, a[k].grad + r[k].grad, 1e-5)
    # ddt leaves in bf16: the fused call rounds the fp32 sum of the two directions once, the two calls round each part
    _check("ddt fused vs sum of parts", g["dt"].grad, a["dt"].grad.float() + r["dt"].grad.float(), 1e-2)
    del o2, g2_, a, r, y1, y2
    # oracle on (b, h) = (5, 3), both directions through the fused call on strided views
    b0, hh = 5, 3
    sl = {k: (t[k][b0:b0 + 1, :, hh:hh + 1] if k in ("x", "x_b", "dt") else
              t[k][hh:hh + 1] if k in ("A", "D") else
              t[k][b0:b0 + 1, hh:hh + 1] if k == "h0" else t[k][b0:b0 + 1]) for k in names}
    w = [v.double().cpu() for v in (dy[b0:b0 + 1, :, hh:hh + 1], dy_b[b0:b0 + 1, :, hh:hh + 1],
                                     df[b0:b0 + 1, hh:hh + 1], df_b[b0:b0 + 1, hh:hh + 1])]
    ref = {k: v.detach().double().cpu().clone().requires_grad_() for k, v in sl.items()}
    o_ref = R.issm_biscan_ref(ref["x"], ref["x_b"], ref["dt"], ref["A"], ref["B"], ref["B_b"], ref["C"], ref["C_b"],
                              D=ref["D"], initial_states=ref["h0"], dt_softplus=True)
    sum((oi * wi).sum() for oi, wi in zip(o_ref, w)).backward()
    gg = {k: v.detach().requires_grad_() for k, v in sl.items()}
    og = ISSM_biscan_combined(gg["x"], gg["x_b"], gg["dt"], gg["A"], gg["B"], gg["B_b"], gg["C"], gg["C_b"], 64,
                              D=gg["D"], initial_states=gg["h0"], dt_softplus=True)
    sum((oi.float() * wi.to(dev).float()).sum() for oi, wi in zip(og, w)).backward()
    torch.cuda.synchronize()
    for name, ai, bi in zip(("y_f", "y_b", "last_f", "last_b"), og, o_ref):
        _check(name, ai, bi, FWD16)
    for k in ref:
        _check("d" + k, gg[k].grad, ref[k].grad, BWD16)


def _split_sequence_check(t, dtype, Lh, tol_sum):
    """scan(whole sequence) must equal scan(first part) followed by scan(rest) started from the first part's
    final state, forward and backward (the backward chains d(initial_states) of the second call into
    d(final_states) of the first).  Both runs use the same chunk boundaries, so everything except the
    outputs agree bit for bit; gradients agree to rounding (the carried state gradient crosses the cut through
    a different but equivalent sequence of operations)."""
    from dest3d_amd import ISSM_chunk_scan_combined as op
    names = ("x", "dt", "A", "B", "C", "D", "h0")
    leaf = lambda: {k: t[k].detach().clone().requires_grad_() for k in names}
    kw = dict(dt_softplus=True, return_final_states=True)
    a = leaf()
    y, fin = op(a["x"], a["dt"], a["A"], a["B"], a["C"], 64, D=a["D"], initial_states=a["h0"], **kw)
    ((y.float() * t["dy"]).sum() + (fin * t["dfinal"]).sum()).backward()
    b = leaf()
    cut = lambda v, lo, hi: v[:, lo:hi]
    y1, f1 = op(cut(b["x"], 0, Lh), cut(b["dt"], 0, Lh), b["A"], cut(b["B"], 0, Lh), cut(b["C"], 0, Lh), 64,
                D=b["D"], initial_states=b["h0"], **kw)
    y2, f2 = op(cut(b["x"], Lh, None), cut(b["dt"], Lh, None), b["A"], cut(b["B"], Lh, None), cut(b["C"], Lh, None),
                64, D=b["D"], initial_states=f1, **kw)
    ((y1.float() * t["dy"][:, :Lh]).sum() + (y2.float() * t["dy"][:, Lh:]).sum() + (f2 * t["dfinal"]).sum()).backward()
    torch.cuda.synchronize()
    assert torch.equal(torch.cat([y1, y2], dim=1), y) and torch.equal(f2, fin)
    for k in names:
        _check(f"d{k} (split vs whole)", b[k].grad, a[k].grad, tol_sum)
    return y, fin, a


def test_long_sequence_bf16_shape():
    """B=2, L=16384 (256 chunks), H=8, P=32, N=256, bf16 inputs with fp32 states: split-sequence composition at
    full size, and the fp64 oracle on one (batch, head) over the whole length."""
    from dest3d_amd import ISSM_chunk_scan_combined as op
    _say("long sequence bf16 B=2 L=16384 H=8 P=32 N=256")
    dev = "cuda"
    I = R.make_inputs(2, 16384, 8, 32, 256, seed=1237, h0_std=0.1)
    bf = lambda v: v.to(dev, torch.bfloat16)
    t = dict(x=bf(I["x"]), dt=bf(I["dt_raw"]), B=bf(I["B"]), C=bf(I["C"]), A=I["A"].to(dev), D=I["D"].to(dev),
             h0=I["h0"].to(dev), dy=I["dy"].to(dev), dfinal=I["dfinal"].to(dev))
    _split_sequence_check(t, torch.bfloat16, 8192, 1e-2)
    # oracle on (b, h) = (1, 5): strided views of the big tensors go straight into the operator
    b0, h0 = 1, 5
    sl = dict(x=t["x"][b0:b0 + 1, :, h0:h0 + 1], dt=t["dt"][b0:b0 + 1, :, h0:h0 + 1], A=t["A"][h0:h0 + 1],
              B=t["B"][b0:b0 + 1], C=t["C"][b0:b0 + 1], D=t["D"][h0:h0 + 1], h0=t["h0"][b0:b0 + 1, h0:h0 + 1])
    dy, df = t["dy"][b0:b0 + 1, :, h0:h0 + 1], t["dfinal"][b0:b0 + 1, h0:h0 + 1]
    ref = {k: v.detach().double().cpu().clone().requires_grad_() for k, v in sl.items()}
    yr, fr = R.issm_scan_sequential(ref["x"], ref["dt"], ref["A"], ref["B"], ref["C"], D=ref["D"],
                                    initial_states=ref["h0"], dt_softplus=True)
    ((yr * dy.double().cpu()).sum() + (fr * df.double().cpu()).sum()).backward()
    g = {k: v.detach().requires_grad_() for k, v in sl.items()}      # keeps the strides of the views
    yg, fg = op(g["x"], g["dt"], g["A"], g["B"], g["C"], 64, D=g["D"], initial_states=g["h0"], dt_softplus=True,
                return_final_states=True)
    ((yg.float() * dy).sum() + (fg * df).sum()).backward()
    torch.cuda.synchronize()
    _check("y", yg, yr, FWD16)
    _check("final", fg, fr, FWD16)
    for k in ref:
        _check("d" + k, g[k].grad, ref[k].grad, BWD16)


def test_large_bidirectional_fp32_shape():
    """B=16, L=2048, H=16, P=64, N=512, fp32, both directions, h0 ~ N(0, 0.1): split-sequence composition of the
    single-direction operator at full size, the fused bidirectional call against two single-direction calls
    (bit-equal), and the fp64 oracle on one (batch, head)."""
    from dest3d_amd import ISSM_biscan_combined, ISSM_chunk_scan_combined as op
    _say("large bidirectional fp32 B=16 L=2048 H=16 P=64 N=512")
    dev = "cuda"
    I = R.make_inputs(16, 2048, 16, 64, 512, seed=1238, h0_std=0.1)
    t = dict(x=I["x"].to(dev), dt=I["dt_raw"].to(dev), B=I["B"].to(dev), C=I["C"].to(dev), A=I["A"].to(dev),
             D=I["D"].to(dev), h0=I["h0"].to(dev), dy=I["dy"].to(dev), dfinal=I["dfinal"].to(dev))
    del I
    y, fin, a = _split_sequence_check(t, torch.float32, 1024, 1e-5)
    # fused bidirectional call, direction 2 = same tensors read back to front
    names = ("x", "dt", "A", "B", "C", "D", "h0")
    g = {k: t[k].detach().clone().requires_grad_() for k in names}
    yf, yb, lf, lb = ISSM_biscan_combined(g["x"], g["x"], g["dt"], g["A"], g["B"], g["B"], g["C"], g["C"], 128,
                                          D=g["D"], initial_states=g["h0"], dt_softplus=True)
    assert torch.equal(yf, y) and torch.equal(lf, fin)
    fl = lambda v: torch.flip(v, dims=[1]).contiguous()
    r = {k: t[k].detach().clone().requires_grad_() for k in names}
    y2, l2 = op(fl(r["x"]), fl(r["dt"]), r["A"], fl(r["B"]), fl(r["C"]), 128, D=r["D"], initial_states=r["h0"],
                dt_softplus=True, return_final_states=True)
    assert torch.equal(torch.flip(y2, dims=[1]), yb) and torch.equal(l2, lb)
    dyb = torch.flip(t["dy"], dims=[1]) * 0.5
    ((yf * t["dy"]).sum() + (yb * dyb).sum() + (lf * t["dfinal"]).sum() + (lb * t["dfinal"]).sum()).backward()
    ((y2 * torch.flip(dyb, dims=[1])).sum() + (l2 * t["dfinal"]).sum()).backward()
    torch.cuda.synchronize()
    # d(fused) = d(direction 1 alone) + d(direction 2 alone): float addition of two bit-identical parts
    for k in ("x", "B", "C"):
        _check(f"d{k} fused vs sum of parts", g[k].grad, a[k].grad + r[k].grad, 1e-6)
    for k in ("dt", "A", "D", "h0"):
        _check(f"d{k} fused vs sum of parts", g[k].grad, a[k].grad + r[k].grad, 1e-5)
    del g, r, a, y2, yb, yf
    torch.cuda.empty_cache()
    # oracle on (b, h) = (3, 7), both directions through the fused call
    b0, hh = 3, 7
    sl = dict(x=t["x"][b0:b0 + 1, :, hh:hh + 1], dt=t["dt"][b0:b0 + 1, :, hh:hh + 1], A=t["A"][hh:hh + 1],
              B=t["B"][b0:b0 + 1], C=t["C"][b0:b0 + 1], D=t["D"][hh:hh + 1], h0=t["h0"][b0:b0 + 1, hh:hh + 1])
    dy, df = t["dy"][b0:b0 + 1, :, hh:hh + 1], t["dfinal"][b0:b0 + 1, hh:hh + 1]
    ref = {k: v.detach().double().cpu().clone().requires_grad_() for k, v in sl.items()}
    o_ref = R.issm_biscan_ref(ref["x"], ref["x"], ref["dt"], ref["A"], ref["B"], ref["B"], ref["C"], ref["C"],
                              D=ref["D"], initial_states=ref["h0"], dt_softplus=True)
    w = (dy.double().cpu(), 0.5 * dy.double().cpu(), df.double().cpu(), -df.double().cpu())
    sum((o * wi).sum() for o, wi in zip(o_ref, w)).backward()
    gg = {k: v.detach().requires_grad_() for k, v in sl.items()}     # keeps the strides of the views
    o = ISSM_biscan_combined(gg["x"], gg["x"], gg["dt"], gg["A"], gg["B"], gg["B"], gg["C"], gg["C"], 128,
                             D=gg["D"], initial_states=gg["h0"], dt_softplus=True)
    sum((oi * wi.to(dev).float()).sum() for oi, wi in zip(o, w)).backward()
    torch.cuda.synchronize()
    for name, ai, bi in zip(("y_f", "y_b", "last_f", "last_b"), o, o_ref):
        _check(name, ai, bi, FWD32)
    for k in ref:
        _check("d" + k, gg[k].grad, ref[k].grad, BWD32)


def test_extreme_decay_is_finite_and_accurate():
    """Decays that underflow within a few rows (|dt' A| up to ~3000 per step) and rows that do not decay at all
    (dt' = 0) in the same chunk: the level factors never exceed 1, so nothing may overflow (every head here is outside
    the tile-base kernel's range and falls to the level-hierarchy kernel).  Accuracy bar here: 1e-3 instead of
    1e-4 / 1e-3 -- with running sums of dt' A in the thousands, one fp32 ulp of the sum (the reference keeps it in fp32 as
    well, issm_chunk_state.py:84-104) is already ~5e-4 in the exponent.  dA is one sum per (head, state) over all tokens of
    terms of both signs that nearly cancel here (condition number ~5000 against the intra-chunk matrix dM = dy x^T): dM
    reaches the kernels with 16 significand bits, which alone is worth 2e-2 of max |dA| on this input (1.7e-3 with an
    fp32 dM), hence its own bar."""
    _say("extreme decay")
    d = _problem(1, 192, 2, 32, 64, 1, seed=21, softplus=False)
    g = torch.Generator().manual_seed(22)
    dt = torch.rand(1, 192, 2, 64, generator=g) * 3.0
    dt[:, ::5] = 0.0                                   # rows without decay or input
    dt[:, 7::11] *= 10.0                               # rows that wipe the state
    d["dt"] = dt
    d["A"] = -torch.exp(torch.rand(2, 64, generator=g) * math.log(100.0))
    y_ref, fin_ref, g_ref = _oracle(d, GRAD_NAMES)
    y, fin, gr, _ = _run_operator(d, torch.float32)
    _check("out", y, y_ref, 1e-3)
    _check("final_states", fin, fin_ref, 1e-3)
    for k in GRAD_NAMES:
        if d[k] is not None:
            _check("d" + k, gr[k], g_ref[k], 5e-2 if k == "A" else 1e-2 if k == "dt" else 1e-3)


def test_hip_graph_replays_match_eager():
    """The entry points allocate nothing and issue no memset, so a caller can capture them: a captured forward +
    backward step (bidirectional, fp32) replayed three times, with eager work and synchronisations between the
    replays, reproduces the eager results bit for bit every time."""
    import bench
    keep = dict(bench.SHAPE)
    bench.SHAPE.update(B=2, L=320, H=4, P=32, N=128, G=1)
    try:
        _say("hip graph capture: B2 L320 H4 P32 N128 bidirectional fp32")
        r = bench.Runner(torch, 2, torch.float32)
        r.step()
        torch.cuda.synchronize()
        outs = lambda: [t.clone() for t in (*r.out, *r.fin, *r.dx, *r.dB, *r.dC, r.ddt, r.dA, r.dD, r.dh0)]
        eager = outs()
        graph = r.capture()
        for i in range(3):
            for t in (*r.out, *r.fin, *r.dx, *r.dB, *r.dC, r.ddt, r.dA, r.dD, r.dh0):
                t.fill_(float("nan"))
            junk = torch.randn(512, 512, device="cuda") @ torch.randn(512, 512, device="cuda")   # eager work between replays
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            for a, b in zip(outs(), eager):
                assert torch.equal(a, b), f"replay {i} differs from the eager step"
            assert torch.isfinite(junk).all()
    finally:
        bench.SHAPE.clear()
        bench.SHAPE.update(keep)


def test_randomised_shapes_fp32_match_oracle():
    """Twelve seeded draws of every dimension and option (ragged lengths, head and state sizes that are not
    multiples of the tile sizes, grouped B / C, each optional input present or absent) against the fp64 oracle."""
    rng = torch.Generator().manual_seed(2024)
    pick = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=rng))
    flip = lambda: bool(torch.randint(0, 2, (1,), generator=rng))
    for trial in range(12):
        G = pick(1, 2)
        H = G * pick(1, 3)
        Bsz, L, P, N = pick(1, 3), pick(1, 210), pick(1, 64), pick(1, 280)
        kw = dict(h0=flip(), softplus=flip(), D=[None, "h", "hp"][pick(0, 2)], z=flip(), bias=flip())
        case = (Bsz, L, H, P, N, G, kw)
        _say(f"randomised fp32 {trial}: {case}")
        d = _problem(Bsz, L, H, P, N, G, seed=500 + trial, **kw)
        y_ref, fin_ref, g_ref = _oracle(d, GRAD_NAMES)
        y, fin, g, _ = _run_operator(d, torch.float32, chunk_size=[64, 128, 256][trial % 3])
        _check(f"out {case}", y, y_ref, FWD32)
        _check(f"final_states {case}", fin, fin_ref, FWD32)
        for k in GRAD_NAMES:
            if d[k] is None:
                assert g[k] is None
                continue
            _check(f"d{k} {case}", g[k], g_ref[k], BWD32)


@pytest.mark.parametrize("L_", [256, 230], ids=["complete_tiles", "ragged"])
def test_nearly_undamped_scan_keeps_the_parameter_gradients(L_):
    """dt' between 1e-6 and 5e-5 (what tiny locality weights make of it): every decay is within 1e-3 of 1, the scan is
    nearly a plain running sum, and dA, dB, dC are sums whose terms carry a factor dt'.

    (i) dt' handed over as it is (dt_softplus=False): every output and gradient at the usual fp32 bars.
    (ii) dt' made inside the kernels by softplus of pre-activations in [-14, -10].  The reference evaluates softplus as
    log(exp(x) + 1) in fp32 (softplus.py:9-11), and so do the kernels (with the hardware's exp2 / log2): for exp(x) near
    1e-5 the rounding of 1 + exp(x) alone is worth up to 1 % of the result, so dt' -- and with it dA, dB, dC and the final
    states, all proportional to dt' here -- differs from the exact softplus of the fp64 oracle by 1e-3 .. 1e-2.  That is
    a property of the formula, not of the scan (part (i) runs the same scan at 1e-5); the test states the bound.  The
    reference's module applies softplus in PyTorch and hands dt over as in (i) (dest_module.py:553-559)."""
    _say(f"nearly undamped scan L={L_}")
    g = torch.Generator().manual_seed(92)
    d = _problem(2, L_, 4, 32, 128, 1, seed=91, D="h", softplus=False, h0=False)
    d["dt"] = torch.rand(2, L_, 4, 128, generator=g) * 4.9e-5 + 1e-6
    d["dt_limit"] = (0.0, float("inf"))
    y_ref, fin_ref, g_ref = _oracle(d, GRAD_NAMES)
    y, fin, gk, _ = _run_operator(d, torch.float32)
    _check("out", y, y_ref, FWD32)
    _check("final_states", fin, fin_ref, FWD32)
    for k in GRAD_NAMES:
        if d[k] is not None:
            _check("d" + k, gk[k], g_ref[k], BWD32)
    # (ii)
    d = _problem(2, L_, 4, 32, 128, 1, seed=93, D="h", softplus=True, h0=False, bias=False)
    d["dt"] = torch.rand(2, L_, 4, 128, generator=g) * 4.0 - 14.0
    d["dt_limit"] = (0.0, float("inf"))
    y, fin, gk, _ = _run_operator(d, torch.float32)
    y_ref, fin_ref, g_exact = _oracle(d, GRAD_NAMES)
    _check("out | in-kernel softplus", y, y_ref, FWD32)          # dominated by D x
    _check("dx | in-kernel softplus", gk["x"], g_exact["x"], BWD32)
    worst = max(max(_err(gk[k], g_exact[k])) for k in ("A", "B", "C"))
    worst = max(worst, max(_err(fin, fin_ref)))
    print(f"    against the exact softplus: worst of final states, dA, dB, dC = {worst:.3e}", flush=True)
    assert 2e-4 < worst < 3e-2


def test_bidirectional_bf16_ddt_is_the_once_rounded_sum_of_the_two_directions():
    """ddt is shared by the two directions.  With a bf16 ddt the first direction's share travels in fp32 (through the
    backward workspace) and the second direction's launch writes bf16(share 1 + share 2): one rounding.  The fp32 share
    of direction 1 is read from the workspace of this call; the fp32 share of direction 2 from the workspace of a second
    call whose direction 1 is this call's direction 2 on flipped tokens (equal to fp32 rounding: another instantiation
    of the kernel).  The returned ddt must lie within half a bf16 unit in the last place of the fp32 sum of the two
    -- everywhere; rounding the first share to bf16 before the addition, as a shared bf16 ddt would, breaks that in a
    visible fraction of the elements (checked, so that the test is known to tell the two apart)."""
    import bench
    _say("bidirectional bf16 ddt: single rounding")
    shape = dict(B=2, L=192, H=2, P=32, N=128, G=1, cs=64)
    r1 = bench.Runner(torch, 2, torch.bfloat16, shape=shape, h0_std=0.1)
    r2 = bench.Runner(torch, 2, torch.bfloat16, shape=shape, h0_std=0.1)
    fl = lambda v: torch.flip(v, dims=[1])
    for k in ("x", "B", "C", "dy"):
        r2.t[k][0].copy_(fl(r1.t[k][1]))
        r2.t[k][1].copy_(fl(r1.t[k][0]))
    r2.t["dfinal"][0].copy_(r1.t["dfinal"][1])
    r2.t["dfinal"][1].copy_(r1.t["dfinal"][0])
    r2.t["dt"].copy_(fl(r1.t["dt"]))
    n = shape["B"] * shape["L"] * shape["H"] * shape["N"]
    share = []
    for r in (r1, r2):
        r.step()
        torch.cuda.synchronize()
        tail = r.bws.view(torch.float32)[-((n + 63) // 64 * 64):][:n]     # last region of the backward workspace
        share.append(tail.view(shape["B"], shape["L"], shape["H"], shape["N"]).clone())
    assert torch.isfinite(share[0]).all() and share[0].abs().max() > 0
    for ra, p_own, p_other in ((r1, share[0], fl(share[1])), (r2, share[1], fl(share[0]))):
        total = p_own.double() + p_other.double()
        got = ra.ddt.double()
        ulp = torch.exp2(torch.floor(torch.log2(got.abs().clamp_min(1e-30))) - 7)      # bf16: 8 significand bits
        slack = 0.5 * ulp * 1.001 + 4e-6 * (p_own.abs() + p_other.abs()).double()      # + the second share's fp32 noise
        once = (got - total).abs() <= slack
        assert once.all(), f"{(~once).sum().item()} of {n} elements are further than half a bf16 ulp from the fp32 sum"
        twice = (p_own.to(torch.bfloat16).float() + p_other).to(torch.bfloat16).double()  # what a shared bf16 ddt gives
        frac = ((twice - total).abs() > slack).double().mean().item()
        print(f"    rounded twice, {100 * frac:.1f} % of the elements would miss the bound", flush=True)
        assert frac > 0.01


@pytest.mark.parametrize("io_dtype,dt_dtype", [(torch.float32, torch.bfloat16), (torch.bfloat16, torch.float32)],
                         ids=["x_fp32_dt_bf16", "x_bf16_dt_fp32"])
@pytest.mark.parametrize("L_", [192, 150], ids=["complete_tiles", "ragged"])
def test_dt_of_another_dtype_than_x(io_dtype, dt_dtype, L_):
    """dt and x / B / C may have different element types (include/issm.h: io_dtype, dt_dtype): the complete-tile forward
    kernel reads each in its own type, the chunk backward falls back to the level-hierarchy kernel for the mix.  Inputs
    are rounded to the types they are passed in, so the oracle sees the same numbers."""
    _say(f"mixed dtypes x {io_dtype} dt {dt_dtype} L={L_}")
    d = _problem(2, L_, 4, 32, 128, 2, seed=61, D="h")
    for k in ("x", "B", "C"):
        d[k] = d[k].to(io_dtype).float()
    d["dt"] = d["dt"].to(dt_dtype).float()
    y_ref, fin_ref, g_ref = _oracle(d, GRAD_NAMES)
    from dest3d_amd import ISSM_chunk_scan_combined
    dev = "cuda"
    cast = lambda t, dt_: None if t is None else t.to(dev, dt_).requires_grad_()
    ins = dict(x=cast(d["x"], io_dtype), dt=cast(d["dt"], dt_dtype), A=cast(d["A"], torch.float32), B=cast(d["B"], io_dtype),
               C=cast(d["C"], io_dtype), D=cast(d["D"], torch.float32), dt_bias=cast(d["dt_bias"], torch.float32),
               h0=cast(d["h0"], torch.float32))
    y, fin = ISSM_chunk_scan_combined(ins["x"], ins["dt"], ins["A"], ins["B"], ins["C"], 64, D=ins["D"],
                                      dt_bias=ins["dt_bias"], initial_states=ins["h0"], dt_softplus=True,
                                      dt_limit=d["dt_limit"], return_final_states=True)
    assert y.dtype == io_dtype
    ((y.float() * d["dy"].to(dev)).sum() + (fin * d["dfinal"].to(dev)).sum()).backward()
    torch.cuda.synchronize()
    assert ins["dt"].grad.dtype == dt_dtype
    ft, bt = (FWD32, BWD32) if io_dtype == torch.float32 else (FWD16, BWD16)
    _check("out", y, y_ref, ft)
    _check("final_states", fin, fin_ref, ft)
    for k in ("x", "dt", "A", "B", "C", "D", "dt_bias", "h0"):
        # a bf16 ddt is rounded to 8 bits whatever the arithmetic behind it
        _check("d" + k, ins[k].grad, g_ref[k], BWD16 if (k == "dt" and dt_dtype == torch.bfloat16) else bt)
