"""Operator API of the interactive-SSM chunked scan on MI355X.

Same Python surface as the reference's issm_triton/issm_combined.py:
``ISSM_chunk_scan_combined(x, dt, A, B, C, chunk_size, D=None, z=None, dt_bias=None,
initial_states=None, seq_idx=None, dt_softplus=False, dt_limit=(0, inf),
return_final_states=False)`` (issm_combined.py:16-34) backed by
``ISSMChunkScanCombinedFn`` (issm_combined.py:37-54) with the same 14 backward slots.
Host code only marshals pointers; all arithmetic runs in libissm_hip.so.

``ISSM_biscan_combined`` additionally runs the bidirectional pair of scans that
MultiHeadISSMScan issues (models/dest_module.py:565-575) in one call, reading the shared
dt backwards for the second direction instead of materialising flipped copies.
"""
from __future__ import annotations

import ctypes as C
import math
from typing import List, Optional, Sequence, Tuple

import torch

from . import _lib as L

INF = float("inf")


def _io_cast(t: Optional[torch.Tensor], dtype: torch.dtype) -> Optional[torch.Tensor]:
    if t is None:
        return None
    if t.dtype != dtype:
        t = t.to(dtype)
    if t.stride(-1) != 1:
        t = t.contiguous()
    return t


def _f32c(t: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    return None if t is None else t.detach().to(torch.float32).contiguous()


def _kernel_dtype(dt: torch.dtype) -> torch.dtype:
    return dt if dt in (torch.float32, torch.bfloat16) else torch.float32


class _Problem:
    """Validated, kernel-ready view of one call (1 or 2 directions)."""

    def __init__(self, xs, dt, A, Bs, Cs, chunk_size, D, zs, dt_bias, h0, seq_idx, dt_softplus, dt_limit):
        x0 = xs[0]
        L.require_gpu(x0, "x")
        if x0.dim() != 4:
            raise ValueError(f"x must be (batch, seqlen, nheads, headdim), got {tuple(x0.shape)}")
        self.batch, self.seqlen, self.nheads, self.headdim = x0.shape
        if Bs[0].dim() != 4:
            raise ValueError(f"B must be (batch, seqlen, ngroups, dstate), got {tuple(Bs[0].shape)}")
        self.ngroups, self.dstate = Bs[0].shape[2], Bs[0].shape[3]
        b, l, h, p, g, n = self.batch, self.seqlen, self.nheads, self.headdim, self.ngroups, self.dstate
        # shape rules of issm_combined.py:58-83
        assert h % g == 0, "nheads must be divisible by ngroups"
        for x_, B_, C_ in zip(xs, Bs, Cs):
            assert x_.shape == (b, l, h, p)
            assert B_.shape == (b, l, g, n)
            assert C_.shape == B_.shape
        assert dt.shape == (b, l, h, n)
        assert A.shape == (h, n)
        for z_ in zs:
            if z_ is not None:
                assert z_.shape == (b, l, h, p)
        if D is not None:
            assert D.shape == (h, p) or D.shape == (h,)
        if dt_bias is not None:
            assert dt_bias.shape == (h, n)
        if h0 is not None:
            assert h0.shape == (b, h, p, n)
        self.seq_idx = None
        if seq_idx is not None:
            assert seq_idx.shape == (b, l)                      # issm_combined.py:70-71
            if len(xs) != 1:
                raise NotImplementedError("seq_idx with the fused bidirectional scan")
            self.seq_idx = seq_idx.detach().to(torch.int32).contiguous()
        if not (isinstance(chunk_size, int) and chunk_size > 0):
            raise ValueError(f"chunk_size must be a positive int, got {chunk_size!r}")
        self.ndir = len(xs)
        self.chunk_size = chunk_size
        self.io_dtype = _kernel_dtype(x0.dtype)
        self.dt_dtype = _kernel_dtype(dt.dtype)
        self.xs = [_io_cast(t.detach(), self.io_dtype) for t in xs]
        self.Bs = [_io_cast(t.detach(), self.io_dtype) for t in Bs]
        self.Cs = [_io_cast(t.detach(), self.io_dtype) for t in Cs]
        self.zs = [_io_cast(None if t is None else t.detach(), self.io_dtype) for t in zs]
        self.dt = _io_cast(dt.detach(), self.dt_dtype)
        self.A = _f32c(A)
        self.D = _f32c(D)
        self.dt_bias = _f32c(dt_bias)
        if h0 is not None:
            self.h0 = _io_cast(h0.detach(), _kernel_dtype(h0.dtype))
        else:
            self.h0 = None
        self.dt_softplus = bool(dt_softplus)
        self.dt_limit = (float(dt_limit[0]), float(dt_limit[1]))
        self.device = x0.device
        self.nchunks = math.ceil(l / L.ISSM_CHUNK)

    def args(self) -> L.ScanArgs:
        a = L.ScanArgs()
        d = a.dims
        d.batch, d.seqlen, d.nheads, d.headdim = self.batch, self.seqlen, self.nheads, self.headdim
        d.dstate, d.ngroups, d.chunk_size, d.ndir = self.dstate, self.ngroups, self.chunk_size, self.ndir
        a.io_dtype = L.dtype_code(self.io_dtype)
        a.dt_dtype = L.dtype_code(self.dt_dtype)
        a.h0_dtype = L.dtype_code(self.h0.dtype) if self.h0 is not None else L.ISSM_F32
        a.flags = (L.FLAG_DT_SOFTPLUS if self.dt_softplus else 0) | \
                  (L.FLAG_D_HAS_HDIM if (self.D is not None and self.D.dim() == 2) else 0)
        if self.seq_idx is not None:
            a.flags |= L.FLAG_SEQ_IDX
            a.seq_idx = self.seq_idx.data_ptr()
            a.seq_idx_stride[0], a.seq_idx_stride[1] = self.seq_idx.stride(0), self.seq_idx.stride(1)
        a.dt_min = self.dt_limit[0]
        a.dt_max = min(self.dt_limit[1], 3.0e38)
        for i in range(self.ndir):
            a.x[i] = L.tensor_desc(self.xs[i])
            a.Bm[i] = L.tensor_desc(self.Bs[i])
            a.Cm[i] = L.tensor_desc(self.Cs[i])
            a.z[i] = L.tensor_desc(self.zs[i])
        a.dt = L.tensor_desc(self.dt)
        a.A = L.ptr(self.A)
        a.D = L.ptr(self.D)
        a.dt_bias = L.ptr(self.dt_bias)
        a.h0 = L.tensor_desc(self.h0)
        a.stream = L.current_stream_ptr(self.device)
        return a

    def workspace(self, a: L.ScanArgs, bwd: bool) -> torch.Tensor:
        lib = L.load()
        n = C.c_size_t(0)
        fn = lib.issm_bwd_workspace_bytes if bwd else lib.issm_fwd_workspace_bytes
        L.check(fn(C.byref(a), C.byref(n)), "workspace query")
        return torch.empty(max(n.value, 256), dtype=torch.uint8, device=self.device)


def _scan_fwd(prob: _Problem, want_final: bool):
    lib = L.load()
    with torch.cuda.device(prob.device):
        a = prob.args()
        outs = [torch.empty((prob.batch, prob.seqlen, prob.nheads, prob.headdim), dtype=prob.io_dtype,
                            device=prob.device) for _ in range(prob.ndir)]
        finals = [torch.empty((prob.batch, prob.nheads, prob.headdim, prob.dstate), dtype=torch.float32,
                              device=prob.device) if want_final else None for _ in range(prob.ndir)]
        ws = prob.workspace(a, bwd=False)
        for i in range(prob.ndir):
            a.out[i] = L.tensor_desc(outs[i])
            a.final_states[i] = L.ptr(finals[i])
        a.workspace = ws.data_ptr()
        a.workspace_bytes = ws.numel()
        L.check(lib.issm_scan_fwd(C.byref(a)), "issm_scan_fwd")
    return outs, finals, ws


def _scan_bwd(prob: _Problem, saved_ws: torch.Tensor, douts, dfinals, want_dz: bool):
    lib = L.load()
    dev = prob.device
    with torch.cuda.device(dev):
        a = prob.args()
        a.saved = saved_ws.data_ptr()
        douts = [_io_cast(t, prob.io_dtype) for t in douts]
        dfinals = [_f32c(t) for t in dfinals]
        dxs = [torch.empty_like(o, memory_format=torch.contiguous_format) for o in prob.xs]
        dBs = [torch.empty(prob.Bs[i].shape, dtype=prob.io_dtype, device=dev) for i in range(prob.ndir)]
        dCs = [torch.empty(prob.Cs[i].shape, dtype=prob.io_dtype, device=dev) for i in range(prob.ndir)]
        dzs = [torch.empty(prob.xs[i].shape, dtype=prob.io_dtype, device=dev) if (want_dz and prob.zs[i] is not None)
               else None for i in range(prob.ndir)]
        ddt = torch.empty(prob.dt.shape, dtype=prob.dt_dtype, device=dev)
        dA = torch.empty(prob.A.shape, dtype=torch.float32, device=dev)
        dD = torch.empty(prob.D.shape, dtype=torch.float32, device=dev) if prob.D is not None else None
        dbias = torch.empty(prob.dt_bias.shape, dtype=torch.float32, device=dev) if prob.dt_bias is not None else None
        dh0 = torch.empty((prob.batch, prob.nheads, prob.headdim, prob.dstate), dtype=torch.float32, device=dev)
        ws = prob.workspace(a, bwd=True)
        for i in range(prob.ndir):
            a.dout[i] = L.tensor_desc(douts[i])
            a.dfinal[i] = L.ptr(dfinals[i])
            a.dx[i] = L.tensor_desc(dxs[i])
            a.dB[i] = L.tensor_desc(dBs[i])
            a.dC[i] = L.tensor_desc(dCs[i])
            a.dz[i] = L.tensor_desc(dzs[i])
        a.ddt = L.tensor_desc(ddt)
        a.dA, a.dD, a.ddt_bias, a.dh0 = L.ptr(dA), L.ptr(dD), L.ptr(dbias), L.ptr(dh0)
        a.bwd_workspace = ws.data_ptr()
        a.bwd_workspace_bytes = ws.numel()
        L.check(lib.issm_scan_bwd(C.byref(a)), "issm_scan_bwd")
    return dxs, ddt, dA, dBs, dCs, dD, dzs, dbias, dh0


def _like(g: Optional[torch.Tensor], dtype: Optional[torch.dtype]) -> Optional[torch.Tensor]:
    """Gradient in the dtype of the input it belongs to (None if that input was absent)."""
    if g is None or dtype is None:
        return None
    return g if g.dtype == dtype else g.to(dtype)


def _dtypes(*ts):
    return tuple(None if t is None else t.dtype for t in ts)


class ISSMChunkScanCombinedFn(torch.autograd.Function):
    """Autograd contract of issm_combined.py:37-54 (14 inputs, grads for x, dt, A, B, C, D, z,
    dt_bias, initial_states; None for chunk_size, seq_idx, dt_softplus, dt_limit,
    return_final_states)."""

    @staticmethod
    def forward(ctx, x, dt, A, B, C, chunk_size, D=None, z=None, dt_bias=None, initial_states=None, seq_idx=None,
                dt_softplus=False, dt_limit=(0.0, INF), return_final_states=False):
        prob = _Problem([x], dt, A, [B], [C], chunk_size, D, [z], dt_bias, initial_states, seq_idx, dt_softplus,
                        dt_limit)
        outs, finals, ws = _scan_fwd(prob, return_final_states)
        # The caller's tensors go through save_for_backward (issm_combined.py:42 does the same): `prob` holds detached
        # views of the same storage, and reading ctx.saved_tensors in backward is what makes PyTorch raise when one of
        # them was modified in place between forward and backward instead of returning gradients of changed data.
        ctx.save_for_backward(x, dt, A, B, C, D, z, dt_bias, initial_states)
        ctx.prob = prob
        ctx.ws = ws
        ctx.return_final_states = return_final_states
        ctx.refs = _dtypes(x, dt, A, B, C, D, z, dt_bias, initial_states)
        out = outs[0] if outs[0].dtype == x.dtype else outs[0].to(x.dtype)
        return out if not return_final_states else (out, finals[0])

    @staticmethod
    def backward(ctx, dout, *args):
        ctx.saved_tensors  # version check of the inputs
        prob = ctx.prob
        x, dt, A, B, C, D, z, dt_bias, h0 = ctx.refs
        dfinal = args[0] if ctx.return_final_states else None
        dxs, ddt, dA, dBs, dCs, dD, dzs, dbias, dh0 = _scan_bwd(prob, ctx.ws, [dout], [dfinal], want_dz=z is not None)
        return (_like(dxs[0], x), _like(ddt, dt), _like(dA, A), _like(dBs[0], B), _like(dCs[0], C), None,
                _like(dD, D), _like(dzs[0], z), _like(dbias, dt_bias), _like(dh0, h0), None, None, None, None)


def ISSM_chunk_scan_combined(x, dt, A, B, C, chunk_size, D=None, z=None, dt_bias=None, initial_states=None,
                             seq_idx=None, dt_softplus=False, dt_limit=(0.0, INF), return_final_states=False):
    """
    Argument:
        x: (batch, seqlen, nheads, headdim)
        dt: (batch, seqlen, nheads, dstate)
        A: (nheads, dstate)
        B: (batch, seqlen, ngroups, dstate)
        C: (batch, seqlen, ngroups, dstate)
        chunk_size: int (accepted for parity; the result does not depend on it)
        D: (nheads, headdim) or (nheads,)
        z: (batch, seqlen, nheads, headdim)
        dt_bias: (nheads, dstate)
        initial_states: (batch, nheads, headdim, dstate)
        seq_idx: (batch, seqlen) integer ids of the sequences packed into a row, or None.  The ids of a row must
            not decrease.  initial_states count as id 0 (issm_chunk_scan.py:123): they feed the first sequence of a
            row whose ids start at 0 and nothing in a row whose ids start higher.  Every change of id is a cut
            (the reference's equality masks would reconnect a repeated id inside a chunk only; not reproduced).
        dt_softplus: whether to apply softplus to dt (+ dt_bias)
    Return:
        out: (batch, seqlen, nheads, headdim)  [, final_states (batch, nheads, headdim, dstate) fp32]
    """
    s = _head_split(x.shape[-1]) if x.dim() == 4 else 1
    if s > 1:
        x, dt, A, D, z, dt_bias, initial_states = _split_heads(s, x, dt, A, D, z, dt_bias, initial_states)
    res = ISSMChunkScanCombinedFn.apply(x, dt, A, B, C, chunk_size, D, z, dt_bias, initial_states, seq_idx,
                                        dt_softplus, dt_limit, return_final_states)
    if s == 1:
        return res
    if return_final_states:
        return _merge_heads(s, res[0]), _merge_heads(s, res[1], state=True)
    return _merge_heads(s, res)


MAX_HEADDIM = 64   # what one workgroup's tiles are built for (ISSM_E_UNSUPPORTED above it)


def _head_split(headdim: int) -> int:
    """The scan is independent across the head dimension, so a head wider than the kernels' 64 runs as `s` heads of
    headdim / s that share the head's dt, A and dt_bias (the reference has no such limit, issm_combined.py:58-83):
    the smallest s that divides headdim with headdim / s <= 64."""
    if headdim <= MAX_HEADDIM:
        return 1
    return next(s for s in range(2, headdim + 1) if headdim % s == 0 and headdim // s <= MAX_HEADDIM)


def _split_heads(s, x, dt, A, D, z, dt_bias, h0):
    """Views / repeats that turn (H, P) into (H s, P / s), head h -> heads h s .. h s + s - 1 (same group as h).
    Plain differentiable tensor operations: autograd sums the gradients of the repeated dt, A, dt_bias, D."""
    b, l, h, p = x.shape
    q = p // s
    rep = lambda t, dim: None if t is None else t.repeat_interleave(s, dim=dim)
    heads = lambda t: None if t is None else t.reshape(b, l, h * s, q)
    if D is not None:
        D = D.reshape(h * s, q) if D.dim() == 2 else D.repeat_interleave(s, dim=0)
    h0 = None if h0 is None else h0.reshape(b, h * s, q, h0.shape[-1])
    return heads(x), rep(dt, 2), rep(A, 0), D, heads(z), rep(dt_bias, 0), h0


def _merge_heads(s, t, state=False):
    if state:   # (B, H s, P / s, N) -> (B, H, P, N)
        return t.reshape(t.shape[0], t.shape[1] // s, t.shape[2] * s, t.shape[3])
    return t.reshape(t.shape[0], t.shape[1], t.shape[2] // s, t.shape[3] * s)


class ISSMBiScanFn(torch.autograd.Function):
    """Both directions of MultiHeadISSMScan's bidirectional scan in one operator call.
    Inputs are in natural time order; direction "b" is scanned from the last token to the
    first and its output is returned in natural order (what dest_module.py:568-573 obtains
    with four flips and a second operator call)."""

    @staticmethod
    def forward(ctx, x_f, x_b, dt, A, B_f, B_b, C_f, C_b, chunk_size, D, dt_bias, initial_states, dt_softplus,
                dt_limit):
        prob = _Problem([x_f, x_b], dt, A, [B_f, B_b], [C_f, C_b], chunk_size, D, [None, None], dt_bias,
                        initial_states, None, dt_softplus, dt_limit)
        outs, finals, ws = _scan_fwd(prob, True)
        ctx.save_for_backward(x_f, x_b, dt, A, B_f, B_b, C_f, C_b, D, dt_bias, initial_states)  # see ISSMChunkScanCombinedFn
        ctx.prob = prob
        ctx.ws = ws
        ctx.refs = _dtypes(x_f, x_b, dt, A, B_f, B_b, C_f, C_b, D, dt_bias, initial_states)
        cast = lambda o, r: o if o.dtype == r.dtype else o.to(r.dtype)
        return cast(outs[0], x_f), cast(outs[1], x_b), finals[0], finals[1]

    @staticmethod
    def backward(ctx, dy_f, dy_b, dl_f, dl_b):
        ctx.saved_tensors  # version check of the inputs
        prob = ctx.prob
        x_f, x_b, dt, A, B_f, B_b, C_f, C_b, D, dt_bias, h0 = ctx.refs
        dxs, ddt, dA, dBs, dCs, dD, _, dbias, dh0 = _scan_bwd(prob, ctx.ws, [dy_f, dy_b], [dl_f, dl_b], want_dz=False)
        return (_like(dxs[0], x_f), _like(dxs[1], x_b), _like(ddt, dt), _like(dA, A), _like(dBs[0], B_f),
                _like(dBs[1], B_b), _like(dCs[0], C_f), _like(dCs[1], C_b), None, _like(dD, D), _like(dbias, dt_bias),
                _like(dh0, h0), None, None)


def ISSM_biscan_combined(x_f, x_b, dt, A, B_f, B_b, C_f, C_b, chunk_size, D=None, dt_bias=None,
                         initial_states=None, dt_softplus=False, dt_limit=(0.0, INF)):
    """Returns (y_f, y_b, last_f, last_b), all in natural time order; see ISSMBiScanFn."""
    s = _head_split(x_f.shape[-1]) if x_f.dim() == 4 else 1
    if s > 1:
        x_b = x_b.reshape(x_b.shape[0], x_b.shape[1], x_b.shape[2] * s, x_b.shape[3] // s)
        x_f, dt, A, D, _, dt_bias, initial_states = _split_heads(s, x_f, dt, A, D, None, dt_bias, initial_states)
    res = ISSMBiScanFn.apply(x_f, x_b, dt, A, B_f, B_b, C_f, C_b, chunk_size, D, dt_bias, initial_states,
                             dt_softplus, dt_limit)
    if s == 1:
        return res
    return (_merge_heads(s, res[0]), _merge_heads(s, res[1]), _merge_heads(s, res[2], state=True),
            _merge_heads(s, res[3], state=True))
