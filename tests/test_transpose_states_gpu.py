"""issm_transpose_states (libissm_hip.so): out[b][c][r] = alpha * (in0[b][r][c] + in1[b][r][c]) with the dtype
conversion folded in -- the rearrangements between queries and scan states of models/dest_module.py:537-538, :575
and :582.  With fp32 in and out the result is bit-exact against the same arithmetic in torch (one add, one
multiply, no reassociation); a bf16 output is that fp32 value rounded to nearest-even, as torch's cast does."""
import ctypes as C

import pytest
import torch

pytestmark = pytest.mark.gpu

CASES = [
    # B, R, C, in dtype, out dtype, second input, alpha
    (2, 300, 256, torch.float32, torch.float32, False, 1.0),
    (2, 256, 300, torch.float32, torch.float32, True, 0.5),
    (1, 1, 1, torch.float32, torch.float32, True, 0.5),
    (3, 65, 63, torch.float32, torch.bfloat16, True, 0.5),
    (3, 63, 129, torch.bfloat16, torch.float32, False, 0.5),
    (2, 70, 64, torch.bfloat16, torch.bfloat16, True, 0.5),
    (1, 7, 200, torch.bfloat16, torch.bfloat16, False, 1.0),
]


def _call(in0, in1, alpha, out_dtype):
    from dest3d_amd import _lib as L
    lib = L.load()
    B, R, Cn = in0.shape
    out = torch.full((B, Cn, R), float("nan"), dtype=out_dtype, device=in0.device)
    a = L.TransposeArgs()
    a.batch, a.rows, a.cols = B, R, Cn
    a.in_dtype, a.out_dtype = L.dtype_code(in0.dtype), L.dtype_code(out_dtype)
    a.in0, a.in1, a.out = in0.data_ptr(), None if in1 is None else in1.data_ptr(), out.data_ptr()
    a.alpha = alpha
    a.stream = L.current_stream_ptr(in0.device)
    rc = lib.issm_transpose_states(C.byref(a))
    torch.cuda.synchronize()
    return rc, out


@pytest.mark.parametrize("case", CASES, ids=lambda c: "B%d_R%d_C%d_%s_%s_%s" % (*c[:3], str(c[3])[6:], str(c[4])[6:], "sum" if c[5] else "one"))
def test_transpose_states_matches_torch(case):
    B, R, Cn, idt, odt, two, alpha = case
    g = torch.Generator().manual_seed(5 + R * Cn)
    in0 = torch.randn(B, R, Cn, generator=g).to(idt).cuda()
    in1 = torch.randn(B, R, Cn, generator=g).to(idt).cuda() if two else None
    rc, out = _call(in0, in1, alpha, odt)
    assert rc == 0
    s = in0.float() if in1 is None else in0.float() + in1.float()
    want = (s * alpha).transpose(1, 2).to(odt)
    assert out.shape == want.shape and out.dtype == odt
    assert torch.equal(out, want)


def test_transpose_states_rejects_bad_arguments_and_accepts_empty():
    from dest3d_amd import _lib as L
    lib = L.load()
    assert lib.issm_transpose_states(None) != 0
    x = torch.zeros(1, 4, 4, device="cuda")
    a = L.TransposeArgs()
    a.batch, a.rows, a.cols, a.in_dtype, a.out_dtype = 1, 4, 4, 7, 0
    a.in0 = a.out = x.data_ptr()
    assert lib.issm_transpose_states(C.byref(a)) != 0
    a.in_dtype, a.in0 = 0, None
    assert lib.issm_transpose_states(C.byref(a)) != 0
    a.rows = 0
    assert lib.issm_transpose_states(C.byref(a)) == 0
    a.rows = -1
    assert lib.issm_transpose_states(C.byref(a)) != 0
