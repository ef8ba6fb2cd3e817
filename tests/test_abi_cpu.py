"""CPU-side checks: the C-ABI library loads, exports every symbol include/issm.h declares,
its host-side validation returns status codes, and the Python operator refuses to run
without a GPU (there is no fallback path)."""
import ctypes as C
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    from dest3d_amd import _lib as L
    if not os.path.exists(L.LIB_PATH):
        from dest3d_amd.build import build
        build(verbose=False)
    return L.load()


def _declared():
    src = open(os.path.join(ROOT, "include", "issm.h")).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(issm_[a-z0-9_]+)\s*\(", src)))


def test_every_declared_symbol_is_exported(lib):
    from dest3d_amd import _lib as L
    names = _declared()
    assert len(names) >= 18
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/issm.h but not exported"
    assert sorted(L.EXPORTS) == names
    assert lib.issm_abi_version() == 5


def test_struct_layout_matches_header(lib):
    """ctypes mirrors must have the C sizes: a size query round-trips through the struct."""
    from dest3d_amd import _lib as L
    a = L.ScanArgs()
    d = a.dims
    d.batch, d.seqlen, d.nheads, d.headdim, d.dstate, d.ngroups, d.chunk_size, d.ndir = 8, 1024, 8, 32, 256, 1, 64, 1
    n = C.c_size_t()
    assert lib.issm_fwd_workspace_bytes(C.byref(a), C.byref(n)) == 0
    nc = 16
    exp = 4 * (8 * (nc + 1) * 8 * 32 * 256 + 8 * nc * 8 * 256 + 8 * nc * 8 * 64 * 64)
    assert n.value == exp
    # the last field of the struct is read where the header says it is
    a.z[0].ptr = 1
    assert lib.issm_fwd_workspace_bytes(C.byref(a), C.byref(n)) == 0
    assert n.value == exp + 4 * 8 * 1024 * 8 * 32
    d.ndir = 2
    a.z[0].ptr = None
    assert lib.issm_bwd_workspace_bytes(C.byref(a), C.byref(n)) == 0
    assert n.value > 2 * 4 * 8 * nc * 8 * 32 * 256


def test_status_codes(lib):
    from dest3d_amd import _lib as L
    a = L.ScanArgs()
    n = C.c_size_t()
    assert lib.issm_fwd_workspace_bytes(None, C.byref(n)) == -1
    assert lib.issm_fwd_workspace_bytes(C.byref(a), C.byref(n)) == -2
    assert b"non-positive" in lib.issm_last_error()
    d = a.dims
    d.batch, d.seqlen, d.nheads, d.headdim, d.dstate, d.ngroups, d.chunk_size, d.ndir = 1, 64, 3, 32, 64, 2, 64, 1
    assert lib.issm_fwd_workspace_bytes(C.byref(a), C.byref(n)) == -2 and b"divisible" in lib.issm_last_error()
    d.ngroups = 1
    d.ndir = 3
    assert lib.issm_fwd_workspace_bytes(C.byref(a), C.byref(n)) == -2
    d.ndir = 1
    d.chunk_size = 0
    assert lib.issm_fwd_workspace_bytes(C.byref(a), C.byref(n)) == -2
    d.chunk_size = 256
    d.headdim = 65
    assert lib.issm_fwd_workspace_bytes(C.byref(a), C.byref(n)) == -5
    d.headdim = 32
    assert lib.issm_scan_fwd(C.byref(a)) == -1          # A is NULL: validated before any launch
    # stride rules are checked on the host before any launch (the pointers are never dereferenced)
    fake = 0x1000
    a.A = fake
    for t in (a.dt, a.x[0], a.Bm[0], a.Cm[0]):
        t.ptr = fake
        t.stride[0], t.stride[1], t.stride[2] = 64 * 3 * 64, 3 * 64, 64
    a.dt.stride[1] = -1
    assert lib.issm_scan_fwd(C.byref(a)) == -3 and b"negative stride" in lib.issm_last_error()
    a.dt.stride[1] = 1 << 30
    assert lib.issm_scan_fwd(C.byref(a)) == -3 and b"32-bit" in lib.issm_last_error()
    a.dt.stride[1] = 3 * 64
    assert lib.issm_scan_fwd(C.byref(a)) == -6          # now only the workspace is missing
    # seq_idx: the flag without the array, and the array (the struct's last fields) with two directions
    a.flags |= L.FLAG_SEQ_IDX
    assert lib.issm_scan_fwd(C.byref(a)) == -1 and b"seq_idx is NULL" in lib.issm_last_error()
    a.seq_idx = fake
    a.seq_idx_stride[0], a.seq_idx_stride[1] = 64, 1
    assert lib.issm_scan_fwd(C.byref(a)) == -6
    a.dims.ndir = 2
    assert lib.issm_scan_fwd(C.byref(a)) == -5 and b"one direction" in lib.issm_last_error()
    a.dims.ndir = 1
    a.flags &= ~L.FLAG_SEQ_IDX
    na = L.NormArgs()
    assert lib.issm_gated_rmsnorm_fwd(C.byref(na)) == -2
    # the fields appended for LayerNorm statistics and the bias are read where the header puts them
    na.rows, na.ncols = 4, 8
    na.x = na.w = na.rstd = na.y = fake
    na.layer_norm = 1
    assert lib.issm_gated_rmsnorm_fwd(C.byref(na)) == -1 and b"mean is NULL" in lib.issm_last_error()
    na.layer_norm, na.bias = 0, fake
    na.dy = na.dx = na.dw_partial = na.dw = fake
    assert lib.issm_gated_rmsnorm_bwd(C.byref(na)) == -1 and b"db_partial" in lib.issm_last_error()
    assert lib.issm_rmsnorm_bwd_blocks(10) == 10 and lib.issm_rmsnorm_bwd_blocks(10 ** 6) == 2048


def test_operator_has_no_cpu_path():
    from dest3d_amd import ISSM_chunk_scan_combined, RMSNorm
    x = torch.randn(1, 64, 2, 32)
    dt = torch.rand(1, 64, 2, 64)
    A = -torch.rand(2, 64)
    Bm = torch.randn(1, 64, 1, 64)
    with pytest.raises(RuntimeError, match="no CPU path"):
        ISSM_chunk_scan_combined(x, dt, A, Bm, Bm, 64)
    with pytest.raises(RuntimeError, match="no CPU path"):
        RMSNorm(64)(torch.randn(4, 64))


def test_product_does_not_import_the_oracle():
    for dirpath, _, files in os.walk(os.path.join(ROOT, "dest3d_amd")):
        for f in files:
            if f.endswith(".py"):
                assert "oracle" not in open(os.path.join(dirpath, f)).read(), f


def test_bench_refuses_more_than_one_gpu_and_a_missing_gpu():
    """bench.py measures one GPU: `--gpus N` above 1 exits with a message that says so, before anything touches a
    device; without a GPU it exits with a message as well (there is nothing to fall back to)."""
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 2 and "one MI355X" in r.stderr and r.stdout.strip() == ""
    if not torch.cuda.is_available():
        r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py")], capture_output=True, text=True, timeout=300)
        assert r.returncode == 2 and "needs a GPU" in r.stderr
