"""Gated RMSNorm / LayerNorm on MI355X with the Python surface of the reference's
issm_triton/layernorm_gated.py: ``RMSNorm`` and ``LayerNorm`` modules (layernorm_gated.py:378-427),
``rmsnorm_fn`` / ``layernorm_fn`` (:370-375) and the autograd function behind them (``LayerNormFn``,
:328-367).  Arithmetic runs in libissm_hip.so."""
from __future__ import annotations

import ctypes as C
from typing import Optional

import torch

from . import _lib as L


def _rows(t: torch.Tensor) -> torch.Tensor:
    t = t.reshape(-1, t.shape[-1])
    return t if t.stride(-1) == 1 else t.contiguous()


def _norm_args(x2, z2, w, eps, group_size, norm_before_gate, bias=None, layer_norm=False) -> L.NormArgs:
    a = L.NormArgs()
    a.rows, a.ncols = x2.shape
    a.group_size = 0 if group_size is None else int(group_size)
    a.dtype = L.dtype_code(x2.dtype)
    a.weight_dtype = L.dtype_code(w.dtype)
    a.norm_before_gate = int(bool(norm_before_gate))
    a.eps = float(eps)
    a.x, a.w = x2.data_ptr(), w.data_ptr()
    a.x_row_stride = x2.stride(0)
    if z2 is not None:
        a.z = z2.data_ptr()
        a.z_row_stride = z2.stride(0)
    if bias is not None:
        a.bias = bias.data_ptr()
    a.layer_norm = int(bool(layer_norm))
    a.stream = L.current_stream_ptr(x2.device)
    return a


class LayerNormFn(torch.autograd.Function):
    """layernorm_gated.py:328-367: same arguments, same four gradients (x, weight, bias, z)."""

    @staticmethod
    def forward(ctx, x, weight, bias, z=None, eps=1e-6, group_size=None, norm_before_gate=True, is_rms_norm=False):
        L.require_gpu(x, "x")
        lib = L.load()
        shape = x.shape
        kdt = x.dtype if x.dtype in (torch.float32, torch.bfloat16) else torch.float32
        x2 = _rows(x.detach().to(kdt))
        z2 = None
        if z is not None:
            assert z.shape == shape
            z2 = _rows(z.detach().to(kdt))
        w = weight.detach()
        w = w if w.dtype in (torch.float32, torch.bfloat16) else w.float()
        assert w.shape == (shape[-1],)
        b = None
        if bias is not None:
            assert bias.shape == (shape[-1],)
            # The kernels read weight and bias in one dtype, the reference's widen each to fp32 on its own
            # (layernorm_gated.py:77-80): where the two differ both go to fp32, so that neither is rounded.
            if bias.dtype != w.dtype:
                w = w.float()
            b = bias.detach().to(w.dtype).contiguous()
        w = w.contiguous()
        gs = shape[-1] if group_size is None else group_size
        assert shape[-1] % gs == 0
        with torch.cuda.device(x.device):
            y = torch.empty_like(x2, memory_format=torch.contiguous_format)
            stats = torch.empty((2, (shape[-1] // gs) * x2.shape[0]), dtype=torch.float32, device=x.device)
            a = _norm_args(x2, z2, w, eps, group_size, norm_before_gate, b, not is_rms_norm)
            a.y, a.y_row_stride, a.rstd = y.data_ptr(), y.stride(0), stats[0].data_ptr()
            if not is_rms_norm:
                a.mean = stats[1].data_ptr()
            L.check(lib.issm_gated_rmsnorm_fwd(C.byref(a)), "issm_gated_rmsnorm_fwd")
        ctx.save_for_backward(x2, z2, w, b, stats)
        ctx.meta = (shape, eps, group_size, norm_before_gate, is_rms_norm, x.dtype, weight.dtype,
                    None if bias is None else bias.dtype, None if z is None else z.dtype)
        return y.reshape(shape).to(x.dtype)

    @staticmethod
    def backward(ctx, dy):
        lib = L.load()
        x2, z2, w, b, stats = ctx.saved_tensors
        shape, eps, group_size, nbg, is_rms, xdt, wdt, bdt, zdt = ctx.meta
        dy2 = _rows(dy.to(x2.dtype))
        with torch.cuda.device(x2.device):
            dx = torch.empty_like(x2)
            dz = torch.empty_like(z2) if z2 is not None else None
            nb = lib.issm_rmsnorm_bwd_blocks(x2.shape[0])
            nparam = 1 if b is None else 2
            part = torch.empty((nparam, nb, x2.shape[1]), dtype=torch.float32, device=x2.device)
            dwb = torch.empty((nparam, x2.shape[1]), dtype=torch.float32, device=x2.device)
            a = _norm_args(x2, z2, w, eps, group_size, nbg, b, not is_rms)
            a.rstd = stats[0].data_ptr()
            if not is_rms:
                a.mean = stats[1].data_ptr()
            a.dy, a.dy_row_stride = dy2.data_ptr(), dy2.stride(0)
            a.dx, a.dx_row_stride = dx.data_ptr(), dx.stride(0)
            if dz is not None:
                a.dz, a.dz_row_stride = dz.data_ptr(), dz.stride(0)
            a.dw_partial, a.dw = part[0].data_ptr(), dwb[0].data_ptr()
            if b is not None:
                a.db_partial, a.db = part[1].data_ptr(), dwb[1].data_ptr()
            L.check(lib.issm_gated_rmsnorm_bwd(C.byref(a)), "issm_gated_rmsnorm_bwd")
        return (dx.reshape(shape).to(xdt), dwb[0].to(wdt), None if b is None else dwb[1].to(bdt),
                None if dz is None else dz.reshape(shape).to(zdt), None, None, None, None)


def layernorm_fn(x, weight, bias, z=None, eps=1e-6, group_size=None, norm_before_gate=True, is_rms_norm=False):
    """layernorm_gated.py:370-371."""
    return LayerNormFn.apply(x, weight, bias, z, eps, group_size, norm_before_gate, is_rms_norm)


def rmsnorm_fn(x, weight, bias, z=None, eps=1e-6, group_size=None, norm_before_gate=True):
    """layernorm_gated.py:374-375."""
    return LayerNormFn.apply(x, weight, bias, z, eps, group_size, norm_before_gate, True)


class LayerNorm(torch.nn.Module):
    """Drop-in for issm_triton.layernorm_gated.LayerNorm (layernorm_gated.py:378-403)."""

    def __init__(self, hidden_size, eps=1e-5, group_size=None, norm_before_gate=True, device=None, dtype=None):
        """If group_size is not None, each group of group_size features is normalised on its own.
        group_size=None means a single group."""
        factory_kwargs = {"device": device, "dtype": dtype}
        super().__init__()
        self.eps = eps
        self.weight = torch.nn.Parameter(torch.empty(hidden_size, **factory_kwargs))
        self.bias = torch.nn.Parameter(torch.empty(hidden_size, **factory_kwargs))
        self.group_size = group_size
        self.norm_before_gate = norm_before_gate
        self.reset_parameters()

    def reset_parameters(self):
        torch.nn.init.ones_(self.weight)
        torch.nn.init.zeros_(self.bias)

    def forward(self, x, z=None):
        """norm(x) * silu(z) if norm_before_gate, else norm(x * silu(z)); z optional."""
        return layernorm_fn(x, self.weight, self.bias, z=z, group_size=self.group_size, eps=self.eps,
                            norm_before_gate=self.norm_before_gate)


class RMSNorm(torch.nn.Module):
    """Drop-in for issm_triton.layernorm_gated.RMSNorm (layernorm_gated.py:405-427)."""

    def __init__(self, hidden_size, eps=1e-5, group_size=None, norm_before_gate=True, device=None, dtype=None):
        """If group_size is not None, each group of group_size features is normalised on its own.
        group_size=None means a single group."""
        factory_kwargs = {"device": device, "dtype": dtype}
        super().__init__()
        self.eps = eps
        self.weight = torch.nn.Parameter(torch.empty(hidden_size, **factory_kwargs))
        self.register_parameter("bias", None)
        self.group_size = group_size
        self.norm_before_gate = norm_before_gate
        self.reset_parameters()

    def reset_parameters(self):
        torch.nn.init.ones_(self.weight)

    def forward(self, x, z=None):
        """norm(x) * silu(z) if norm_before_gate, else norm(x * silu(z)); z optional."""
        return rmsnorm_fn(x, self.weight, self.bias, z=z, eps=self.eps, group_size=self.group_size,
                          norm_before_gate=self.norm_before_gate)
