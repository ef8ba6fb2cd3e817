"""issm_gated_rmsnorm_bwd_noalloc (the entry point that allocates nothing: partial sums in a scratch array inside the
library) against issm_gated_rmsnorm_bwd with a caller buffer, through the C ABI.  Same kernels, fixed-order sums:
every output must be equal bit for bit -- on two calls in a row, the second on a smaller problem (the scratch array
then still holds the first call's partials)."""
import ctypes as C

import pytest
import torch

pytestmark = pytest.mark.gpu


def _run(lib, L, rows, ncols, dtype, gated, seed, noalloc, layer=False):
    from dest3d_amd import layernorm_gated as N
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, ncols, generator=g).to(dtype).cuda()
    z = torch.randn(rows, ncols, generator=g).to(dtype).cuda() if gated else None
    w = (1.0 + 0.1 * torch.randn(ncols, generator=g)).cuda()
    dy = torch.randn(rows, ncols, generator=g).to(dtype).cuda()
    b = (0.1 * torch.randn(ncols, generator=g)).cuda() if layer else None   # LayerNorm statistics and a bias
    y = torch.empty_like(x)
    rstd = torch.empty(rows, dtype=torch.float32, device="cuda")
    mean = torch.empty(rows, dtype=torch.float32, device="cuda")
    a = N._norm_args(x, z, w, 1e-5, None, False, b, layer)
    a.y, a.y_row_stride, a.rstd = y.data_ptr(), y.stride(0), rstd.data_ptr()
    if layer:
        a.mean = mean.data_ptr()
    L.check(lib.issm_gated_rmsnorm_fwd(C.byref(a)), "fwd")
    dx = torch.full_like(x, float("nan"))
    dz = torch.full_like(x, float("nan")) if gated else None
    dw = torch.full((ncols,), float("nan"), device="cuda")
    db = torch.full((ncols,), float("nan"), device="cuda") if layer else None
    a.dy, a.dy_row_stride = dy.data_ptr(), dy.stride(0)
    a.dx, a.dx_row_stride = dx.data_ptr(), dx.stride(0)
    if gated:
        a.dz, a.dz_row_stride = dz.data_ptr(), dz.stride(0)
    a.dw = dw.data_ptr()
    if layer:
        a.db = db.data_ptr()
    if noalloc:
        a.dw_partial = a.db_partial = None
        L.check(lib.issm_gated_rmsnorm_bwd_noalloc(C.byref(a)), "bwd_noalloc")
    else:
        part = torch.empty(2, lib.issm_rmsnorm_bwd_blocks(rows), ncols, dtype=torch.float32, device="cuda")
        a.dw_partial = part[0].data_ptr()
        if layer:
            a.db_partial = part[1].data_ptr()
        L.check(lib.issm_gated_rmsnorm_bwd(C.byref(a)), "bwd")
    torch.cuda.synchronize()
    return dx, dz, dw, db


def test_noalloc_rmsnorm_bwd_equals_the_buffered_entry_point_twice_in_a_row():
    from dest3d_amd import _lib as L
    lib = L.load()
    # first a large problem (all 2048 row blocks, the detector's 288 columns), then smaller ones on the used scratch;
    # also the generic (non-vector) path: 50 columns, and a gate-less call
    # and with LayerNorm statistics and a bias (the bias gradient's partial sums follow the weight's in the array)
    for rows, ncols, dtype, gated, layer in [(8192, 288, torch.bfloat16, True, False), (300, 288, torch.bfloat16, True, False),
                                             (4096, 1024, torch.float32, True, False), (7, 50, torch.float32, False, False),
                                             (4096, 512, torch.float32, True, True), (33, 288, torch.bfloat16, True, True),
                                             (1, 288, torch.float32, True, False),
                                             # a bias case, then a larger case without one: its weight partials cover
                                             # the part of the array where the bias partials of the call before lie
                                             (2048, 512, torch.float32, True, True), (4096, 1024, torch.float32, True, False)]:
        print(f"[case] rmsnorm bwd noalloc rows={rows} ncols={ncols} {dtype} gated={gated} layer={layer}", flush=True)
        got = _run(lib, L, rows, ncols, dtype, gated, 5 + rows, noalloc=True, layer=layer)
        want = _run(lib, L, rows, ncols, dtype, gated, 5 + rows, noalloc=False, layer=layer)
        for name, a, b in zip(("dx", "dz", "dw", "db"), got, want):
            if b is None:
                assert a is None
                continue
            assert torch.isfinite(b.float()).all(), name
            assert torch.equal(a, b), f"{name} differs at rows={rows} ncols={ncols}"


def test_noalloc_rmsnorm_bwd_rejects_what_does_not_fit():
    from dest3d_amd import _lib as L
    from dest3d_amd import layernorm_gated as N
    lib = L.load()
    rows, ncols = 4096, 2048                                  # 2048 blocks x 2048 columns > 2048 x 1024 floats
    x = torch.zeros(rows, ncols, device="cuda")
    w = torch.ones(ncols, device="cuda")
    rstd = torch.ones(rows, device="cuda")
    dw = torch.zeros(ncols, device="cuda")
    a = N._norm_args(x, None, w, 1e-5, None, False)
    a.rstd = rstd.data_ptr()
    a.dy, a.dy_row_stride, a.dx, a.dx_row_stride, a.dw = x.data_ptr(), ncols, x.data_ptr(), ncols, dw.data_ptr()
    assert lib.issm_gated_rmsnorm_bwd_noalloc(C.byref(a)) == -6
    assert b"scratch" in lib.issm_last_error()
    assert lib.issm_gated_rmsnorm_bwd_noalloc(None) == -1
    # 1024 columns always fit, whatever the row count
    assert lib.issm_rmsnorm_bwd_blocks(10 ** 7) * 1024 <= 2048 * 1024
    # with a bias the partial sums take twice the room: 4096 rows x 1024 columns no longer fit
    x1 = torch.zeros(4096, 1024, device="cuda")
    a = N._norm_args(x1, None, w[:1024].contiguous(), 1e-5, None, False, w[:1024].contiguous(), False)
    a.rstd = rstd.data_ptr()
    a.dy, a.dy_row_stride, a.dx, a.dx_row_stride, a.dw, a.db = x1.data_ptr(), 1024, x1.data_ptr(), 1024, dw.data_ptr(), dw.data_ptr()
    assert lib.issm_gated_rmsnorm_bwd_noalloc(C.byref(a)) == -6 and b"weight and bias" in lib.issm_last_error()


def _prepared(lib, L, rows, ncols, dtype, seed, layer):
    """Forward done, every backward buffer allocated: what is left is the backward call itself."""
    from dest3d_amd import layernorm_gated as N
    g = torch.Generator().manual_seed(seed)
    t = dict(x=torch.randn(rows, ncols, generator=g).to(dtype).cuda(), z=torch.randn(rows, ncols, generator=g).to(dtype).cuda(),
             w=(1.0 + 0.1 * torch.randn(ncols, generator=g)).cuda(), dy=torch.randn(rows, ncols, generator=g).to(dtype).cuda(),
             b=(0.1 * torch.randn(ncols, generator=g)).cuda() if layer else None)
    t["y"] = torch.empty_like(t["x"])
    t["rstd"] = torch.empty(rows, dtype=torch.float32, device="cuda")
    t["mean"] = torch.empty(rows, dtype=torch.float32, device="cuda")
    for k in ("dx", "dz"):
        t[k] = torch.full_like(t["x"], float("nan"))
    for k in ("dw", "db"):
        t[k] = torch.full((ncols,), float("nan"), device="cuda")
    t["part"] = torch.empty(2, lib.issm_rmsnorm_bwd_blocks(rows), ncols, dtype=torch.float32, device="cuda")

    def args():
        a = N._norm_args(t["x"], t["z"], t["w"], 1e-5, None, False, t["b"], layer)   # stream = torch's current one
        a.y, a.y_row_stride, a.rstd = t["y"].data_ptr(), t["y"].stride(0), t["rstd"].data_ptr()
        if layer:
            a.mean, a.db = t["mean"].data_ptr(), t["db"].data_ptr()
        a.dy, a.dy_row_stride = t["dy"].data_ptr(), t["dy"].stride(0)
        a.dx, a.dx_row_stride = t["dx"].data_ptr(), t["dx"].stride(0)
        a.dz, a.dz_row_stride = t["dz"].data_ptr(), t["dz"].stride(0)
        a.dw = t["dw"].data_ptr()
        return a
    L.check(lib.issm_gated_rmsnorm_fwd(C.byref(args())), "fwd")
    return t, args


def _buffered(lib, L, t, args, layer):
    a = args()
    a.dw_partial = t["part"][0].data_ptr()
    if layer:
        a.db_partial = t["part"][1].data_ptr()
    L.check(lib.issm_gated_rmsnorm_bwd(C.byref(a)), "bwd")
    torch.cuda.synchronize()
    return {k: t[k].clone() for k in ("dx", "dz", "dw") + (("db",) if layer else ())}


@pytest.mark.parametrize("layer", [False, True])
def test_noalloc_rmsnorm_bwd_allocates_nothing_and_takes_null_partial_buffers(layer):
    """What the entry point is for: between the state before and after the call neither the driver's free memory
    (which also sees allocations made behind torch's back) nor torch's own count moves, with dw_partial and
    db_partial both NULL."""
    from dest3d_amd import _lib as L
    lib = L.load()
    print(f"[case] rmsnorm bwd noalloc allocation check layer={layer}", flush=True)
    t, args = _prepared(lib, L, 3000, 288, torch.bfloat16, 41, layer)
    want = _buffered(lib, L, t, args, layer)
    a = args()
    a.dw_partial = a.db_partial = None
    L.check(lib.issm_gated_rmsnorm_bwd_noalloc(C.byref(a)), "warm-up")     # first call on the device resolves the address
    torch.cuda.synchronize()
    for k in ("dx", "dz", "dw", "db"):
        t[k].fill_(float("nan"))
    torch.cuda.synchronize()
    free0, alloc0, resv0 = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    L.check(lib.issm_gated_rmsnorm_bwd_noalloc(C.byref(a)), "bwd_noalloc")
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0
    assert torch.cuda.memory_allocated() == alloc0 and torch.cuda.memory_reserved() == resv0
    for k, v in want.items():
        assert torch.equal(t[k], v), k


def test_noalloc_rmsnorm_bwd_in_a_hip_graph_replays_like_eager():
    """The callers the entry point names record it into a graph.  After one eager call on the device (which resolves
    the scratch array's address; a first call under capture is refused), the call is captured and replayed three
    times on changed inputs, with eager work and synchronisations of the program's own between the replays; every
    replay must equal the buffered entry point on the same inputs bit for bit."""
    from dest3d_amd import _lib as L
    lib = L.load()
    print("[case] rmsnorm bwd noalloc under graph capture", flush=True)
    t, args = _prepared(lib, L, 2500, 288, torch.bfloat16, 43, True)
    a = args()
    a.dw_partial = a.db_partial = None
    L.check(lib.issm_gated_rmsnorm_bwd_noalloc(C.byref(a)), "warm-up")
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            ac = args()                                       # picks up the capturing stream
            ac.dw_partial = ac.db_partial = None
            L.check(lib.issm_gated_rmsnorm_bwd_noalloc(C.byref(ac)), "bwd_noalloc under capture")
    torch.cuda.current_stream().wait_stream(side)
    g = torch.Generator().manual_seed(99)
    for rep in range(3):
        t["dy"].copy_(torch.randn(t["dy"].shape, generator=g).to(t["dy"].dtype))
        want = _buffered(lib, L, t, args, True)             # eager work of the program's own, then a synchronisation
        for k in ("dx", "dz", "dw", "db"):
            t[k].fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for k, v in want.items():
            assert torch.equal(t[k], v), (rep, k)
