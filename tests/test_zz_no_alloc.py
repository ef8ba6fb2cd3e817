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
                                             (1, 288, torch.float32, True, False)]:
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
