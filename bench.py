#!/usr/bin/env python3
"""Benchmark of the ISSM chunked scan on one MI355X.

Workload (the configuration the headline metric is quoted on): B=8, L=1024, H=8, P=32, N=256, G=1, chunk=64, forward +
backward of the bidirectional pair of scans (second direction = reversed token order, same dt /
A / D / initial states), fp32 inputs, synthetic seeded data already resident in HBM.
One "step" = one forward + backward call of the operator.  `value` is microseconds per step.

Besides the driver's JSON contract the line carries
  roofline           the dominant kernel's achieved fraction of its bound (live HIP-event timing); `traffic` is read
                     from the committed rocprofv3 summary under profiles/
  cpu_baseline       the oracle's chunked pure-PyTorch formulation timed on the host cores (fwd+bwd sample scaled to
                     the workload, and configs[0]'s own forward-only B=2 figure)
  stages_us, stage_roofline, step_roofline   every kernel of the step against the roofline that bounds it, and the
                     whole step against its compulsory traffic and FLOPs
  variants_us        fwd+bwd time of the unidirectional fp32 / bf16 and bidirectional bf16 variants (also at the
                     detector's head dimension 36), of configs[3] (long sequence) and configs[4] (large state), and
                     of one whole detector layer around the scan
  variant_rooflines  the same per-kernel and whole-step rooflines for the bf16 headline variant, configs[3], configs[4]
`--workload NAME` runs one scan workload alone (the command the kernel traces under profiles/ are taken with).
"""
import argparse
import ctypes as C
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_BF16_MFMA_TFLOPS = 2500.0
PEAK_HBM_GBS = 8000.0

SHAPE = dict(B=8, L=1024, H=8, P=32, N=256, G=1, cs=64)


# The scan workloads this script can time: the headline (configs[1], fp32), its variants, and the baseline's other scan
# configurations (configs[3]: long sequence; configs[4]: large state).  shape overrides SHAPE.
# Unless a workload says `presoftplus`, dt is handed over raw with dt_softplus=True and a (H, N) dt_bias of zeros: bias,
# softplus and clamp run inside the kernels (issm_chunk_state.py:84-99).  `presoftplus` is the module's call pattern
# (models/dest_module.py:600-611): dt = softplus(dt_raw) computed by the caller, dt_softplus=False, no bias.
# `fwd_only` times the forward alone (configs[0], the reference's own forward-only harness test_issm.py:113-135).
# Every workload runs with the library's internal chunk of 64 tokens, whatever chunk_size the configuration names.
WORKLOADS = {
    "headline": dict(shape={}, ndir=2, dtype="float32"),
    "headline_module_call_pattern": dict(shape={}, ndir=2, dtype="float32", presoftplus=True),
    "config0_gpu_forward_only_B2": dict(shape=dict(B=2), ndir=1, dtype="float32", fwd_only=True),
    "uni_fp32": dict(shape={}, ndir=1, dtype="float32"),
    "uni_bf16": dict(shape={}, ndir=1, dtype="bfloat16"),
    "bidir_bf16": dict(shape={}, ndir=2, dtype="bfloat16"),
    "bidir_bf16_headdim36": dict(shape=dict(P=36), ndir=2, dtype="bfloat16"),   # the detector's head size
    "long_sequence_B2_L16384_uni_bf16": dict(shape=dict(B=2, L=16384), ndir=1, dtype="bfloat16"),
    "large_state_B16_L2048_H16_P64_N512_bidir_fp32": dict(shape=dict(B=16, L=2048, H=16, P=64, N=512), ndir=2,
                                                          dtype="float32", h0_std=0.1),
}


def synthetic_inputs(torch, Bsz, L, H, P, N, G=1, seed=1234, h0_std=0.0):
    """The benchmark configurations' synthetic inputs: generated on the CPU in fp32 in a fixed order (x, dt_raw, A, B,
    C, D, h0, dy, dfinal).  x ~ N(0,1); dt_raw ~ U(-4,-1) (to be softplus'ed); A = -exp(U(ln 1, ln 16)) per head,
    broadcast over N; B, C ~ N(0, 1/sqrt(N)); D ~ N(0,1); h0 = 0 or N(0, h0_std).  The same sequence of draws as the
    tests' generator, so a seed names the same problem in both (tests/test_oracle.py checks that)."""
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g)
    u = lambda *s: torch.rand(*s, generator=g)
    x = r(Bsz, L, H, P)
    dt_raw = u(Bsz, L, H, N) * 3.0 - 4.0
    A = -torch.exp(u(H) * math.log(16.0))[:, None].expand(H, N).contiguous()
    Bm = r(Bsz, L, G, N) / math.sqrt(N)
    Cm = r(Bsz, L, G, N) / math.sqrt(N)
    D = r(H)
    h0 = r(Bsz, H, P, N) * h0_std
    dy = r(Bsz, L, H, P)
    dfinal = r(Bsz, H, P, N)
    return dict(x=x, dt_raw=dt_raw, A=A, B=Bm, C=Cm, D=D, h0=h0, dy=dy, dfinal=dfinal)


def make_problem(torch, shape, ndir, dtype, seed=1235, h0_std=0.0, presoftplus=False):
    SHAPE = shape
    I = synthetic_inputs(torch, SHAPE["B"], SHAPE["L"], SHAPE["H"], SHAPE["P"], SHAPE["N"], SHAPE["G"], seed=seed,
                         h0_std=h0_std)
    g = torch.Generator().manual_seed(seed + 1)
    dev = "cuda"
    t = dict(x=[I["x"]], B=[I["B"]], C=[I["C"]], dy=[I["dy"]], dfinal=[I["dfinal"]])
    if ndir == 2:
        t["x"].append(torch.randn(I["x"].shape, generator=g))
        t["B"].append(torch.randn(I["B"].shape, generator=g) / math.sqrt(SHAPE["N"]))
        t["C"].append(torch.randn(I["C"].shape, generator=g) / math.sqrt(SHAPE["N"]))
        t["dy"].append(torch.randn(I["x"].shape, generator=g))
        t["dfinal"].append(torch.randn(I["dfinal"].shape, generator=g))
    out = {k: [v.to(dev, dtype if k in ("x", "B", "C", "dy") else torch.float32) for v in vs] for k, vs in t.items()}
    if presoftplus:   # module call pattern: dt already softplus'ed by the caller
        out["dt"] = torch.nn.functional.softplus(I["dt_raw"]).to(dev, dtype)
        out["dt_bias"] = None
    else:             # the kernels apply bias -> softplus -> clamp
        out["dt"] = I["dt_raw"].to(dev, dtype)
        out["dt_bias"] = torch.zeros(SHAPE["H"], SHAPE["N"], device=dev)
    out["A"] = I["A"].to(dev)
    out["D"] = I["D"].to(dev)
    out["h0"] = I["h0"].to(dev)
    return out


class Runner:
    """Forward + backward through the C ABI with preallocated buffers (no autograd, no allocation
    in the timed region): exactly the kernels ISSMChunkScanCombinedFn launches."""

    def __init__(self, torch, ndir, dtype, shape=None, h0_std=0.0, presoftplus=False, fwd_only=False):
        from dest3d_amd import _lib as L
        from dest3d_amd.issm_combined import _Problem
        self.torch, self.L, self.lib = torch, L, L.load()
        self.ndir = ndir
        SHAPE = self.shape = dict(globals()["SHAPE"], **(shape or {}))
        self.elt = 2 if dtype == torch.bfloat16 else 4
        self.fwd_only = fwd_only
        t = self.t = make_problem(torch, SHAPE, ndir, dtype, h0_std=h0_std, presoftplus=presoftplus)
        self.prob = _Problem(t["x"], t["dt"], t["A"], t["B"], t["C"], SHAPE["cs"], t["D"], [None] * ndir, t["dt_bias"],
                             t["h0"], None, not presoftplus, (0.0, float("inf")))
        a = self.a = self.prob.args()
        dev = "cuda"
        B_, L_, H, P, N, G = (SHAPE[k] for k in ("B", "L", "H", "P", "N", "G"))
        e = lambda *s, dt=torch.float32: torch.empty(*s, dtype=dt, device=dev)
        self.out = [e(B_, L_, H, P, dt=dtype) for _ in range(ndir)]
        self.fin = [e(B_, H, P, N) for _ in range(ndir)]
        self.dx = [e(B_, L_, H, P, dt=dtype) for _ in range(ndir)]
        self.dB = [e(B_, L_, G, N, dt=dtype) for _ in range(ndir)]
        self.dC = [e(B_, L_, G, N, dt=dtype) for _ in range(ndir)]
        self.ddt = e(B_, L_, H, N, dt=dtype)
        self.dA, self.dD, self.dh0 = e(H, N), e(H), e(B_, H, P, N)
        self.dbias = e(H, N) if t["dt_bias"] is not None else None
        self.ws = self.prob.workspace(a, bwd=False)
        self.bws = self.prob.workspace(a, bwd=True)
        for i in range(ndir):
            a.out[i] = L.tensor_desc(self.out[i])
            a.final_states[i] = self.fin[i].data_ptr()
            a.dout[i] = L.tensor_desc(t["dy"][i])
            a.dfinal[i] = t["dfinal"][i].data_ptr()
            a.dx[i], a.dB[i], a.dC[i] = (L.tensor_desc(v[i]) for v in (self.dx, self.dB, self.dC))
        a.ddt = L.tensor_desc(self.ddt)
        a.dA, a.dD, a.dh0 = self.dA.data_ptr(), self.dD.data_ptr(), self.dh0.data_ptr()
        a.ddt_bias = L.ptr(self.dbias)
        a.workspace, a.workspace_bytes = self.ws.data_ptr(), self.ws.numel()
        a.saved = self.ws.data_ptr()
        a.bwd_workspace, a.bwd_workspace_bytes = self.bws.data_ptr(), self.bws.numel()
        a.stream = L.current_stream_ptr(torch.device("cuda"))

    def step(self):
        self.L.check(self.lib.issm_scan_fwd(C.byref(self.a)), "fwd")
        if not self.fwd_only:
            self.L.check(self.lib.issm_scan_bwd(C.byref(self.a)), "bwd")

    RAMP_MS = 40.0

    def ramp(self):
        """Untimed: keep the card under this workload's load for RAMP_MS.  After an idle spell (allocations, host work,
        a fresh process) it runs below its steady clocks for 20 - 30 ms, whatever the number of warm-up steps asked for."""
        torch = self.torch
        t0 = time.perf_counter()
        while (time.perf_counter() - t0) * 1e3 < self.RAMP_MS:
            for _ in range(4):
                self.step()
            torch.cuda.synchronize()

    def time_steps(self, steps, warmup):
        torch = self.torch
        self.ramp()
        for _ in range(warmup):
            self.step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            self.step()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps * 1e6

    def capture(self):
        """Record one step (forward + backward, 9 kernel launches, no allocation, no memset) into a HIP graph on a side
        stream of default priority and return the graph."""
        torch = self.torch
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        keep = self.a.stream
        self.a.stream = side.cuda_stream
        with torch.cuda.stream(side):
            self.step()
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            self.step()
        self.a.stream = keep
        torch.cuda.current_stream().wait_stream(side)
        return graph

    def time_graph_replays(self, steps, warmup):
        torch = self.torch
        graph = self.capture()
        for _ in range(warmup):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            graph.replay()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps * 1e6

    def step_percentiles(self, steps):
        """p10 / p50 / p90 of single steps, each bracketed by HIP events on the launch stream (caches not flushed
        between steps: consecutive steps reuse the same buffers, as a training loop does)."""
        torch = self.torch
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
        for e0, e1 in ev:
            e0.record()
            self.step()
            e1.record()
        torch.cuda.synchronize()
        t = sorted(e0.elapsed_time(e1) * 1e3 for e0, e1 in ev)
        pick = lambda q: round(t[min(len(t) - 1, int(q * len(t)))], 2)
        return {"p10": pick(0.10), "p50": pick(0.50), "p90": pick(0.90)}

    def stage_times(self, reps=20):
        """Average duration of each kernel, HIP events on the launch stream around `reps`
        back-to-back launches of that kernel."""
        torch, lib, a = self.torch, self.lib, self.a
        nd = self.ndir
        B_, L_, H, P, N = (self.shape[k] for k in ("B", "L", "H", "P", "N"))
        nc = math.ceil(L_ / 64)
        Bt = B_ * nd
        f = lambda *s: torch.zeros(*s, device="cuda")
        st, csl, cabt = f(Bt, nc + 1, H, P, N), f(Bt, nc, H, N), f(Bt, nc, H, 64, 64)
        dst, dm, gn, dh0d = f(Bt, nc, H, P, N), f(Bt, nc, H, 64, 64), f(Bt, nc, H, N), f(nd, B_, H, P, N)
        pa, pb, pd = f(Bt * nc, H, N), f(Bt * nc, H, N), f(Bt * nc * H, P)
        redo = torch.zeros(lib.issm_bwd_chunk_redo_ints(C.byref(a)), dtype=torch.int32, device="cuda")
        p = lambda t: t.data_ptr()
        stages = [
            ("chunk_local", lambda: lib.issm_stage_chunk_local(C.byref(a), p(st), p(csl), p(cabt))),
            ("state_passing_fwd", lambda: lib.issm_stage_state_passing_fwd(C.byref(a), p(st), p(csl))),
            ("chunk_scan", lambda: lib.issm_stage_chunk_scan(C.byref(a), p(st), p(cabt), None)),
            ("bwd_dstates", lambda: lib.issm_stage_bwd_dstates(C.byref(a), None, p(dst), p(dm))),
            ("state_passing_bwd", lambda: lib.issm_stage_state_passing_bwd(C.byref(a), p(st), p(csl), p(dst), p(gn), p(dh0d))),
            ("bwd_chunk", lambda: [lib.issm_stage_bwd_chunk(C.byref(a), d, None, p(st), p(dst), p(dm), p(gn), p(pa), p(pb), p(redo))
                                   for d in range(nd)][-1]),
            ("bwd_dx", lambda: lib.issm_stage_bwd_dx(C.byref(a), None, p(dst), p(cabt), p(pd))),
            ("bwd_reduce", lambda: lib.issm_stage_bwd_reduce(C.byref(a), p(pa), p(pb), p(pd), p(dh0d))),
        ]
        res = {}
        for name, fn in stages:
            for _ in range(3):
                self.L.check(fn(), name)
            # (allocations and host work leave the card idle, and it then runs the next 20 ms below its steady clocks:
            # every stage is launched for about that long before it is timed)
            w0, w1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            w0.record()
            for _ in range(3):
                fn()
            w1.record()
            w1.synchronize()
            for _ in range(min(400, int(25e3 / max(w0.elapsed_time(w1) / 3 * 1e3, 1.0)))):
                fn()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(reps):
                fn()
            e1.record()
            e1.synchronize()
            res[name] = e0.elapsed_time(e1) / reps * 1e3
        return res


KERNEL_OF_STAGE = {"chunk_local": "k_local_tile", "state_passing_fwd": "k_state_fwd_full", "chunk_scan": "k_chunk_scan",
                   "bwd_dstates": "k_bwd_dstates", "state_passing_bwd": "k_state_bwd_full", "bwd_chunk": "k_bwd_tile",
                   "bwd_dx": "k_bwd_dx", "bwd_reduce": "k_bwd_reduce"}


def measured_traffic(stage):
    """HBM bytes of a stage's kernel launches at the headline workload, as the committed profile summary holds them
    (profiles/issm_fwd_bwd_bidir_fp32_hbm_traffic.md: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this script, scaled by
    the same counters on a plain copy; last column of the kernel's rows, added up over the stage's launches -- the chunk
    backward is launched once per direction, and its algorithmic bytes are counted the same way); None if the summary
    has no such row."""
    import re
    path = os.path.join(ROOT, "profiles", "issm_fwd_bwd_bidir_fp32_hbm_traffic.md")
    pat = re.compile(KERNEL_OF_STAGE.get(stage, stage) + r"\b")
    total = None
    try:
        for row in open(path):
            cells = [c.strip() for c in row.strip().strip("|").split("|")]
            if len(cells) >= 4 and pat.search(cells[0]):
                total = (total or 0.0) + float(cells[-1]) * 1e6
    except (OSError, ValueError):
        return None
    return total


def stage_work(ndir, shape=None, elt=4):
    """Algorithmic FLOPs (2*MAC; exps not counted) and algorithmic bytes (every operand read once, every result
    written once; caller tensors in their `elt`-byte type, intermediates fp32; dt counted once for both directions)
    per launch of each kernel, and the same for the whole step ("step": compulsory bytes only -- inputs read once in
    each pass, outputs and gradients written once)."""
    SHAPE_ = dict(SHAPE, **(shape or {}))
    B_, L_, H, P, N, G = (SHAPE_[k] for k in ("B", "L", "H", "P", "N", "G"))
    cs = 64
    U = B_ * ndir * H * math.ceil(L_ / cs)
    tri = cs * (cs + 1) // 2
    E_cs, E_st = U * P * N, B_ * ndir * H * P * N          # chunk states; initial / final states
    E_x, E_bc = ndir * B_ * L_ * H * P, ndir * B_ * L_ * G * N   # x / y / dy / dx; B, C and their gradients
    E_dt, E_m, E_v = B_ * L_ * H * N, U * cs * cs, U * N   # dt / ddt; intra-chunk matrix M / dM; per-chunk vectors
    s = elt
    w = {
        # reads dt, x, B, C; writes chunk-local end states S, M, the chunks' total decay
        "chunk_local": (2 * U * (cs * P * N + tri * N), s * (E_dt + E_x + 2 * E_bc) + 4 * (E_cs + E_m + E_v)),
        # reads dt, C, x, states H, M; writes y
        "chunk_scan": (2 * U * (cs * P * N + tri * P), s * (E_dt + E_bc + 2 * E_x) + 4 * (E_cs + E_m)),
        # reads dt, C, dy, x; writes dH, dM
        "bwd_dstates": (2 * U * (cs * P * N + tri * P), s * (E_dt + E_bc + 2 * E_x) + 4 * (E_cs + E_m)),
        # all launches: read dt, x, dy, B, C, H, dS, dM, g_last; write ddt, dB, dC, the dA / ddt_bias partials
        "bwd_chunk": (2 * U * (2 * cs * P * N + 2 * tri * N),
                      s * (2 * E_dt + 2 * E_x + 4 * E_bc) + 4 * (2 * E_cs + E_m + 3 * E_v)),
        # reads dt, B, dy, x, dS, M; writes dx
        "bwd_dx": (2 * U * (cs * P * N + tri * P), s * (E_dt + E_bc + 3 * E_x) + 4 * (E_cs + E_m)),
        "state_passing_fwd": (0, 4 * (2 * E_cs + U * N + 2 * E_st)),
        "state_passing_bwd": (0, 4 * (3 * E_cs + 2 * U * N + 2 * E_st)),
    }
    # whole step, compulsory traffic only: every caller tensor read once per pass, every output and gradient written
    # once, each direction counted with its own read of dt and initial states (a lower bound would share them)
    E_dtd = ndir * E_dt
    fwd_rd = s * (E_x + 2 * E_bc + E_dtd + E_st)
    fwd = fwd_rd + s * E_x + 4 * E_st
    bwd = fwd_rd + s * E_x + 4 * E_st + s * (E_x + 2 * E_bc + E_dtd + E_st)
    w["step"] = (sum(f for f, _ in w.values()), fwd + bwd)
    return w


def stage_bound(flops, nbytes, us, elt=4):
    """The roofline that bounds a stage is the one with the longer minimum time; returns (bound, achieved in the
    bound's unit, fraction of its peak, {mfma fraction, hbm fraction}).  The matrix peak is the one of the inputs' type:
    fp32 (157.3 TFLOP/s) for fp32 inputs, bf16 (2.5 PFLOP/s) for bf16 inputs -- with those every stage is HBM-bound."""
    t = us * 1e-6
    peak = PEAK_BF16_MFMA_TFLOPS if elt == 2 else PEAK_FP32_MFMA_TFLOPS
    f_mfma = flops / t / (peak * 1e12)
    f_hbm = nbytes / t / (PEAK_HBM_GBS * 1e9)
    both = {"mfma_frac": round(f_mfma, 4), "hbm_frac": round(f_hbm, 4)}
    if f_mfma >= f_hbm:
        return "mfma", flops / t / 1e12, f_mfma, both
    return "hbm", nbytes / t / 1e9, f_hbm, both


def workload_report(run, step_us, reps=20):
    """Per-kernel durations of a workload with the roofline that bounds each (the one with the longer minimum time:
    fp32 matrix peak for the FLOPs, HBM peak for the bytes), and the same for the whole step on its compulsory bytes."""
    stages = run.stage_times(reps)
    work = stage_work(run.ndir, run.shape, run.elt)
    per_stage = {}
    for k, (fl, nb) in work.items():
        if k == "step":
            continue
        b, _, fr, both = stage_bound(fl, nb, stages[k], run.elt)
        per_stage[k] = {"us": round(stages[k], 2), "bound": b, "frac": round(fr, 4), **both}
    b, ach, fr, both = stage_bound(*work["step"], step_us, run.elt)
    return {"stages_us": {k: round(v, 2) for k, v in stages.items()}, "stage_roofline": per_stage,
            "step_roofline": {"us": round(step_us, 2), "gflop": round(work["step"][0] / 1e9, 2),
                              "compulsory_mb": round(work["step"][1] / 1e6, 1), "bound": b, "frac": round(fr, 4), **both}}


def cpu_baseline(torch):
    """Chunked pure-PyTorch formulation (oracle.issm_scan_chunked after oracle.dt_transform, fp32, autograd backward)
    on the host cores, on a bounded sample: 2 of the 8 batch elements, one direction, 2 repetitions (about 15-30 s);
    scaled by 8 (= 4 x batch, 2 x directions) to the workload's unit.  Threads: the host share of one GPU on the
    measurement machines is 16 cores (OMP_NUM_THREADS there), so that many are used even where os.cpu_count() reports
    the whole machine; both numbers are in the record."""
    from oracle import issm_ref as R
    host = os.cpu_count() or 1
    try:
        host = min(host, len(os.sched_getaffinity(0)))
    except AttributeError:
        pass
    cores = min(host, int(os.environ.get("OMP_NUM_THREADS", "0") or 0) or host)
    torch.set_num_threads(cores)
    I = R.make_inputs(2, SHAPE["L"], SHAPE["H"], SHAPE["P"], SHAPE["N"], SHAPE["G"], seed=1235)
    bias = torch.zeros(SHAPE["H"], SHAPE["N"])
    ins = [I["x"].clone().requires_grad_(), I["dt_raw"].clone().requires_grad_(),
           I["A"].clone().requires_grad_(), I["B"].clone().requires_grad_(), I["C"].clone().requires_grad_()]

    def fwd(x, dt_raw, A, B, C_):
        return R.issm_scan_chunked(x, R.dt_transform(dt_raw, bias, True), A, B, C_, SHAPE["cs"])

    best = float("inf")
    for _ in range(2):
        for t in ins:
            t.grad = None
        t0 = time.perf_counter()
        y, fin = fwd(*ins)
        ((y * I["dy"]).sum() + (fin * I["dfinal"]).sum()).backward()
        best = min(best, time.perf_counter() - t0)
    # configs[0] as BASELINE.json states it: forward only, B=2, the same formulation, no gradient bookkeeping
    with torch.no_grad():
        f = float("inf")
        for _ in range(2):
            t0 = time.perf_counter()
            fwd(*[t.detach() for t in ins])
            f = min(f, time.perf_counter() - t0)
    return {"value": best * 8 * 1e6, "unit": "us/call", "cores": cores, "host_cpu_count": os.cpu_count(),
            "kind": "port",
            "sample": "B=2 of 8, one direction, fwd+bwd incl. bias/softplus/clamp of dt, fp32, best of 2; scaled x8 to "
                      "B=8 bidirectional",
            "config0_forward_only_B2_us": round(f * 1e6, 1)}


def time_box_dist_layer(torch, steps=10, warmup=15):
    """BoxDistFun + local_weight + MultiHeadISSMScan as ISSMDecoderLayer chains them (models/dest_module.py:283-290)
    at the configs[2] shape, bf16 module, forward + backward, microseconds.  Returns (whole, box_dist forward only)."""
    from dest3d_amd.box_dist import BoxDistFun
    from dest3d_amd.scan_module import MultiHeadISSMScan
    torch.manual_seed(0)
    m = MultiHeadISSMScan(d_model=288, d_state=256, d_dist=16, chunk_size=256, nheads=8, expand=1).cuda().bfloat16()
    bd = BoxDistFun(out_dim=16).cuda().bfloat16()
    key = torch.randn(8, 1024, 288, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    query = torch.randn(8, 256, 288, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    key_pos = 8.0 * torch.rand(8, 1024, 3, device="cuda")
    query_pos = torch.cat([8.0 * torch.rand(8, 256, 3, device="cuda"), 0.2 + 2.0 * torch.rand(8, 256, 3, device="cuda")], -1)
    zero_angle = torch.zeros(8, 256, device="cuda")
    g_key, g_query = torch.randn_like(key) / 64, torch.randn_like(query) / 64   # what the next layer hands back

    def encode():
        return bd(key_pos, query_pos[..., :3], query_pos[..., 3:], zero_angle, weight_query_pos=query_pos)

    def step():
        for mod in (m, bd):
            mod.zero_grad(set_to_none=True)   # as an optimizer step would: no accumulation into old gradients
        key.grad = query.grad = None
        dist, weights = encode()
        ok, oq = m(key, query, dist, key_pos, weights)
        torch.autograd.backward((ok, oq), (g_key, g_query))

    out = []
    for fn in (step, encode):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        out.append((time.perf_counter() - t0) / steps * 1e6)
    return out


def time_box_dist_vs_torch(torch, reps=3):
    """BoxDistFun at the layer shape: the library's kernels against the same formulas written with PyTorch ops
    (corner deltas, signed log, `grid_sample` on the (1, 16, 10, 10, 10) table, sum over corners -- the formulation of
    models/dest_module.py:174-195 with zero angles), forward and forward + backward, milliseconds; and their largest
    absolute difference."""
    import torch.nn.functional as F
    from dest3d_amd.box_dist import BoxDistFun, box_parametrization_to_corners
    torch.manual_seed(0)
    B, nP, nQ = 8, 1024, 256
    bd = BoxDistFun(out_dim=16).cuda()
    key_pos = 8.0 * torch.rand(B, nP, 3, device="cuda")
    qpos = torch.cat([8.0 * torch.rand(B, nQ, 3, device="cuda"), 0.2 + 2.0 * torch.rand(B, nQ, 3, device="cuda")], -1)
    ang = torch.zeros(B, nQ, device="cuda")

    def with_torch_ops():
        corners = box_parametrization_to_corners(qpos[..., :3], qpos[..., 3:], ang).detach()
        deltas = corners.reshape(B, -1, 3)[:, :, None, :] - key_pos[:, None, :, :]
        deltas = torch.sign(deltas) * torch.log2(torch.abs(deltas) * 512 + 1.0) / math.log2(8)
        rpe = F.grid_sample(bd.rpe_table()[None], (deltas / 4.0).view(1, 1, 1, -1, 3), mode="bilinear",
                            align_corners=False).reshape(-1, B, nQ, 8, nP)
        return rpe.sum(dim=-2).permute(1, 3, 2, 0)

    def with_kernels():
        return bd(key_pos, qpos[..., :3], qpos[..., 3:], ang)

    res = {}
    for name, fn in (("kernels", with_kernels), ("torch_ops", with_torch_ops)):
        for bw in (False, True):
            for i in range(reps + 1):
                if i == 1:
                    torch.cuda.synchronize()
                    t0 = time.perf_counter()
                bd.zero_grad(set_to_none=True)
                d = fn()
                if bw:
                    d.square().sum().backward()
            torch.cuda.synchronize()
            res[f"{name}_{'fwd_bwd' if bw else 'fwd'}_ms"] = round((time.perf_counter() - t0) / reps * 1e3, 3)
    with torch.no_grad():
        res["max_abs_difference"] = float((with_kernels() - with_torch_ops()).abs().max())
    return res


def time_pointnet2_ops(torch, reps=5):
    """The backbone's point-set operators at the detector's first set-abstraction shape (batch 8, 20000 points, 2048
    centres, 64 samples, 128 / 256 channels), milliseconds per call."""
    from dest3d_amd import pointnet2_utils as pn
    torch.manual_seed(0)
    B, N = 8, 20000
    xyz = (8 * torch.rand(B, N, 3)).cuda()
    feat = torch.randn(B, 128, N).cuda().requires_grad_()
    res = {}

    def t(name, fn):
        out = fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            out = fn()
        torch.cuda.synchronize()
        res[name] = round((time.perf_counter() - t0) / reps * 1e3, 3)
        return out

    fps = t("furthest_point_sample_2048_of_20000", lambda: pn.furthest_point_sample(xyz, 2048))
    new_xyz = pn.gather_operation(xyz.transpose(1, 2).contiguous(), fps).transpose(1, 2).contiguous()
    idx = t("ball_query_r0.2_64", lambda: pn.ball_query(0.2, 64, xyz, new_xyz))
    g = t("grouping_c128_fwd", lambda: pn.grouping_operation(feat, idx))
    gy = torch.randn_like(g)
    t("grouping_c128_fwd_bwd", lambda: torch.autograd.grad(pn.grouping_operation(feat, idx), feat, gy))
    d, i3 = t("three_nn_20000_x_2048", lambda: pn.three_nn(xyz, new_xyz))
    w = torch.softmax(-d, -1)
    f2 = torch.randn(B, 256, 2048).cuda().requires_grad_()
    y = t("three_interpolate_c256_fwd", lambda: pn.three_interpolate(f2, i3, w))
    gy2 = torch.randn_like(y)
    t("three_interpolate_c256_fwd_bwd", lambda: torch.autograd.grad(pn.three_interpolate(f2, i3, w), f2, gy2))
    return res


def time_serialization(torch, reps=50):
    """The Hilbert-curve order (models/dest_module.py:307-397) at the detector's sizes: the curve positions alone
    (`issm_hilbert_codes`, microseconds and bytes moved), the two orders with their sorts and inverse permutations
    (`Serialization.forward`), and the gather of the key features into curve order.  HIP events around each call."""
    from dest3d_amd.serialization import Serialization, hilbert_codes
    torch.manual_seed(0)
    res = {}

    def t(fn):
        fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return round(e0.elapsed_time(e1) / reps * 1e3, 2)

    for name, B, N, C_ in (("keys_8x1024", 8, 1024, 288), ("backbone_8x20000", 8, 20000, 256)):
        pts = (8 * torch.rand(B, N, 3)).cuda()
        feat = torch.randn(B, N, C_, device="cuda", dtype=torch.bfloat16)
        ser = Serialization(order=("xyz", "yxz"))
        ser(pts)
        r = {"hilbert_codes_us": t(lambda: hilbert_codes(pts, "xyz")),
             "codes_bytes": B * N * (12 + 8),   # three float coordinates in, one 64-bit position out
             "two_orders_with_sorts_us": t(lambda: ser(pts)),
             "gather_features_us": t(lambda: ser.reorder_points(feat, 0)),
             "gather_bytes": 2 * B * N * C_ * 2 + B * N * 8}
        res[name] = r
    return res


def layer_compulsory_bytes(nlayers=1, with_encoding=False, B=8, L=1024, K=256, d_model=288, d_dist=16, elt=2):
    """Compulsory HBM bytes of a forward + backward step through `nlayers` MultiHeadISSMScan layers at the configs[2]
    shape if nothing but the layer's own inputs, outputs and their gradients crossed HBM (dt, B, C and every scan
    intermediate staying on chip): per layer and pass, the distance encoding `dist` (B, L, K, 16) and the locality
    weights (B, L, K) fp32 are read once, key (B, L, d) and query (B, K, d) features are read and written once; the
    backward also reads the two output gradients, writes the two input gradients and writes d(dist).  With the
    encoding: BoxDistFun writes `dist` and the weights once and its backward reads the summed d(dist) once (positions
    and the table are negligible)."""
    e_dist, e_w = B * L * K * d_dist * elt, B * L * K * 4
    e_feat = (B * L + B * K) * d_model * elt
    fwd = e_dist + e_w + 2 * e_feat
    bwd = e_dist + e_w + 2 * e_feat + 2 * e_feat + e_dist
    total = nlayers * (fwd + bwd)
    if with_encoding:
        total += e_dist + e_w + e_dist
    return total


def time_layer_stack(torch, steps=5, warmup=4, nlayers=6):
    """configs[2] as a whole: BoxDistFun + local_weight once, then `nlayers` MultiHeadISSMScan layers as a residual
    stack (models/dest_detector.py:207-235 calls the decoder layers on one shared encoding), bf16, forward + backward
    from a scalar loss, eager; microseconds per step."""
    from dest3d_amd.box_dist import BoxDistFun
    from dest3d_amd.scan_module import MultiHeadISSMScan
    torch.manual_seed(0)
    bd = BoxDistFun(out_dim=16).cuda().bfloat16()
    stack = torch.nn.ModuleList(MultiHeadISSMScan(d_model=288, d_state=256, d_dist=16, chunk_size=256, nheads=8,
                                                  expand=1) for _ in range(nlayers)).cuda().bfloat16()
    key = torch.randn(8, 1024, 288, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    query = torch.randn(8, 256, 288, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    key_pos = 8.0 * torch.rand(8, 1024, 3, device="cuda")
    query_pos = torch.cat([8.0 * torch.rand(8, 256, 3, device="cuda"), 0.2 + 2.0 * torch.rand(8, 256, 3, device="cuda")], -1)
    zero_angle = torch.zeros(8, 256, device="cuda")
    g_key, g_query = torch.randn_like(key) / 64, torch.randn_like(query) / 64

    def step():
        for mod in (stack, bd):
            mod.zero_grad(set_to_none=True)
        key.grad = query.grad = None
        dist, weights = bd(key_pos, query_pos[..., :3], query_pos[..., 3:], zero_angle, weight_query_pos=query_pos)
        hk, hq = key, query
        for layer in stack:
            ok, oq = layer(hk, hq, dist, key_pos, weights)
            hk, hq = hk + ok, hq + oq
        torch.autograd.backward((hk, hq), (g_key, g_query))

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps * 1e6


def caller_rooflines(variants):
    """The caller-side timings against the HBM time of their compulsory bytes (layer_compulsory_bytes)."""
    rows = {"detector_layer_bf16_fwd_bwd": (1, False), "detector_layer_bf16_fwd_bwd_as_hip_graph": (1, False),
            "box_dist_plus_layer_bf16_fwd_bwd": (1, True), "detector_six_layers_plus_box_dist_bf16_fwd_bwd": (6, True)}
    out = {}
    for k, (nl, enc) in rows.items():
        if k in variants:
            nb = layer_compulsory_bytes(nl, enc)
            out[k] = {"us": variants[k], "compulsory_mb": round(nb / 1e6, 1), "bound": "hbm",
                      "frac": round(nb / (variants[k] * 1e-6) / (PEAK_HBM_GBS * 1e9), 4)}
    return out


def time_module_layer(torch, steps=10, warmup=25, dtype=None, as_graph=False):
    """One MultiHeadISSMScan-equivalent layer (configs[2]: d_model 288, 8 heads of 36, K = 256 queries, L = 1024
    keys, batch 8, d_dist 16, bf16 unless `dtype` says fp32, float locality weights as mask -- what DEST's decoder layer passes,
    models/dest_module.py:283-290), forward + backward through autograd from given output gradients (as inside a
    stack of layers: no loss is computed here), microseconds.  Includes the PyTorch projections and norms around the
    scan.  With `as_graph` the step is recorded once into a HIP graph (the pattern
    of torch.cuda.graphs for a whole training step) and the replays are timed: the GPU's time without the host's."""
    from dest3d_amd.scan_module import MultiHeadISSMScan
    torch.manual_seed(0)
    dtype = dtype or torch.bfloat16
    m = MultiHeadISSMScan(d_model=288, d_state=256, d_dist=16, chunk_size=256, nheads=8, expand=1).cuda().to(dtype)
    key = torch.randn(8, 1024, 288, device="cuda", dtype=dtype, requires_grad=True)
    query = torch.randn(8, 256, 288, device="cuda", dtype=dtype, requires_grad=True)
    dist = (0.5 * torch.randn(8, 1024, 256, 16, device="cuda")).to(dtype).requires_grad_()
    weights = torch.exp(-15.0 * (torch.rand(8, 1024, 256, device="cuda") - 0.5).clamp_min(0.0))

    g_key, g_query = torch.randn_like(key) / 64, torch.randn_like(query) / 64   # what the next layer hands back

    def step():
        m.zero_grad(set_to_none=True)   # as an optimizer step would: no accumulation into old gradients
        key.grad = query.grad = dist.grad = None
        ok, oq = m(key, query, dist, None, weights)
        torch.autograd.backward((ok, oq), (g_key, g_query))

    if as_graph:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        m.zero_grad(set_to_none=True)
        key.grad = query.grad = dist.grad = None
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            ok, oq = m(key, query, dist, None, weights)
            torch.autograd.backward((ok, oq), (g_key, g_query))
        step = graph.replay
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps * 1e6


def make_runner(torch, name):
    spec = WORKLOADS[name]
    return Runner(torch, spec["ndir"], getattr(torch, spec["dtype"]), spec["shape"], spec.get("h0_std", 0.0),
                  presoftplus=spec.get("presoftplus", False), fwd_only=spec.get("fwd_only", False))


def workload_text(name):
    """What a workload runs, in words (the `config.workload` of its JSON line)."""
    spec = WORKLOADS[name]
    sh = dict(SHAPE, **spec["shape"])
    return ("B={B} L={L} H={H} P={P} N={N} G={G}".format(**sh) + ", "
            + ("forward only" if spec.get("fwd_only") else "fwd+bwd") + ", "
            + ("bidirectional pair (fused)" if spec["ndir"] == 2 else "one direction") + ", "
            + ("fp32 I/O" if spec["dtype"] == "float32" else "bf16 I/O, fp32 states and accumulation") + ", "
            + ("dt pre-softplused by the caller (dt_softplus=False, no dt_bias)" if spec.get("presoftplus")
               else "dt_softplus=True (in-kernel), dt_bias (H,N) zeros, dt_limit (0, inf)")
            + ", internal chunk 64" + (", h0 ~ N(0, %g)" % spec["h0_std"] if spec.get("h0_std") else ", h0 = 0"))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    # After an idle spell the card needs about 20 ms of continuous load to reach its steady clocks (the first steps of a
    # run take 596 us, the 40th 535): Runner.ramp() covers that before the warm-up steps, whatever their number.
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-variants", action="store_true", help="time only the headline workload")
    ap.add_argument("--steps-only", action="store_true",
                    help="headline workload: the step loop and nothing else (for a kernel trace of the kernels as they run inside a step)")
    ap.add_argument("--only-layer", action="store_true",
                    help="time only the whole detector layer (module forward + backward) and print its JSON line")
    ap.add_argument("--only-box-dist", action="store_true",
                    help="time BoxDistFun: the kernels against the same formulas in PyTorch ops, and print the JSON line")
    ap.add_argument("--only-pointnet2", action="store_true",
                    help="time only the backbone's point-set operators and print their JSON line (ms per call)")
    ap.add_argument("--only-serialization", action="store_true",
                    help="time the Hilbert-curve order (codes, sorts, feature gather) at the detector's sizes")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also run a plain 256 MiB device copy (calibrates FETCH_SIZE / WRITE_SIZE under rocprofv3 --pmc)")
    ap.add_argument("--workload", choices=sorted(WORKLOADS), default=None,
                    help="run only this scan workload's forward + backward step loop and print its JSON line")
    ap.add_argument("--traffic", type=float, default=None,
                    help="measured HBM bytes per launch of the dominant kernel (from rocprofv3 --pmc), echoed into roofline.traffic")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one MI355X: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)

    if args.only_box_dist:
        print(json.dumps({"box_dist_8x1024x256": time_box_dist_vs_torch(torch)}))
        return
    if args.only_pointnet2:
        print(json.dumps({"pointnet2_ops_ms": time_pointnet2_ops(torch)}))
        return
    if args.only_serialization:
        print(json.dumps({"serialization": time_serialization(torch)}))
        return
    if args.only_layer:
        whole, enc = time_box_dist_layer(torch, args.steps, args.warmup)
        print(json.dumps({"detector_layer_bf16_fwd_bwd_us": round(time_module_layer(torch, args.steps, args.warmup), 2),
                          "detector_layer_bf16_fwd_bwd_as_hip_graph_us":
                              round(time_module_layer(torch, args.steps, args.warmup, as_graph=True), 2),
                          "box_dist_plus_layer_bf16_fwd_bwd_us": round(whole, 2),
                          "box_dist_and_weight_fwd_us": round(enc, 2), "steps": args.steps, "warmup": args.warmup}))
        return
    if args.calib_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
    if args.workload:
        # one workload's step loop only (what the profiles under profiles/ are taken from)
        r = make_runner(torch, args.workload)
        us = r.time_steps(args.steps, args.warmup)
        rep = {} if (args.no_variants or r.fwd_only) else workload_report(r, us)
        print(json.dumps({"workload": args.workload, "config": {"workload": workload_text(args.workload)},
                          "us_per_step": round(us, 2), "steps": args.steps, "warmup": args.warmup, **rep}))
        return
    run = make_runner(torch, "headline")
    us = run.time_steps(args.steps, args.warmup)
    if args.steps_only:
        print(json.dumps({"workload": "headline", "us_per_step": round(us, 2), "steps": args.steps, "warmup": args.warmup}))
        return
    pct = run.step_percentiles(max(args.steps, 20))
    rep = workload_report(run, us)
    stages, per_stage = rep["stages_us"], rep["stage_roofline"]
    work = stage_work(2)
    dom = max((k for k in stages if k in work), key=lambda k: stages[k])
    bound, achieved, frac, _ = stage_bound(*work[dom], stages[dom])
    roof = {"bound": bound, "achieved": achieved, "peak": PEAK_FP32_MFMA_TFLOPS if bound == "mfma" else PEAK_HBM_GBS,
            "unit": "TFLOP/s" if bound == "mfma" else "GB/s", "frac": frac, "traffic": None, "kernel": dom}
    roof["traffic"] = args.traffic if args.traffic is not None else measured_traffic(dom)
    variants, variant_rooflines = {}, {}
    if not args.no_variants:
        variants["headline_as_hip_graph_replay"] = round(run.time_graph_replays(args.steps, max(args.warmup, 40)), 2)
        del run
        for name, spec in WORKLOADS.items():
            if name == "headline":
                continue
            big = bool(spec["shape"].get("L", 0) > 4096 or spec["shape"].get("N", 0) > 256)
            r = make_runner(torch, name)
            v = r.time_steps(5 if big else max(args.steps // 2, 5), 2 if big else 5)
            variants[name] = round(v, 2)
            if name in ("headline_module_call_pattern", "bidir_bf16", "long_sequence_B2_L16384_uni_bf16",
                        "large_state_B16_L2048_H16_P64_N512_bidir_fp32"):
                variant_rooflines[name] = workload_report(r, v, reps=5 if big else 20)
            del r
            torch.cuda.empty_cache()
        variants["detector_layer_bf16_fwd_bwd"] = round(time_module_layer(torch), 2)
        variants["detector_layer_bf16_fwd_bwd_as_hip_graph"] = round(time_module_layer(torch, as_graph=True), 2)
        variants["detector_layer_fp32_fwd_bwd"] = round(time_module_layer(torch, dtype=torch.float32), 2)
        variants["box_dist_plus_layer_bf16_fwd_bwd"] = round(time_box_dist_layer(torch)[0], 2)
        variants["detector_six_layers_plus_box_dist_bf16_fwd_bwd"] = round(time_layer_stack(torch), 2)
    line = {
        "metric": "ISSM scan fwd+bwd us/call at B=8,L=1024,N=256", "value": round(us, 2), "unit": "us/call",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "clock_ramp_ms_before_warmup": Runner.RAMP_MS,
        "ms_per_step": round(us / 1e3, 5),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[1]: " + workload_text("headline"),
                   "variants": {k: workload_text(k) for k in WORKLOADS if k != "headline"}},
        "roofline": {k: (round(v, 4) if isinstance(v, float) else v) for k, v in roof.items()},
        "step_us_percentiles": pct,
        "stages_us": stages,
        "stage_roofline": per_stage,
        "step_roofline": rep["step_roofline"],
        "variants_us": variants,
        "variant_rooflines": variant_rooflines,
        "caller_rooflines": caller_rooflines(variants),
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(torch)
        line["cpu_baseline"]["value"] = round(line["cpu_baseline"]["value"], 1)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
