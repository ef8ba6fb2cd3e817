"""Depthwise 7-tap convolution along the token order + SiLU on (B, L, C) tensors, on MI355X.

The arithmetic of DEST's PointLiteConv (models/dest_module.py:400-423: ``nn.Conv1d(C, C, 7, padding=3,
groups=C)`` over ``feature.transpose(1, 2)``, then ``SiLU``), without the transposes: channels stay
innermost.  ``dwconv_silu`` applies one or two (weight, bias) sets in one pass: to the same input, or --
``chain=True`` -- the second set to the first set's output, which is MultiHeadISSMScan's pair
(dest_module.py:530 reassigns ``xbc = key_conv(xbc)``; :534 feeds that to ``key_conv_back``).
Runs in libissm_hip.so; there is no fallback path."""
from __future__ import annotations

import ctypes as C
from typing import Sequence

import torch

from . import _lib as L

TAPS = 7


def _args(u, nsets) -> L.DwConvArgs:
    a = L.DwConvArgs()
    a.batch, a.seqlen, a.channels = u.shape
    a.nsets, a.taps = nsets, TAPS
    a.dtype = L.dtype_code(u.dtype)
    a.u, a.u_batch_stride, a.u_token_stride = u.data_ptr(), u.stride(0), u.stride(1)
    a.stream = L.current_stream_ptr(u.device)
    return a


class DwConvSiLUFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, u, nsets, chain, *wb):
        """wb = weight_0, bias_0[, weight_1, bias_1]; weight (C, 1, 7) or (C, 7), bias (C,)."""
        L.require_gpu(u, "u")
        lib = L.load()
        Bsz, Ln, Cn = u.shape
        ud = u.detach()
        if ud.dtype not in (torch.float32, torch.bfloat16):
            ud = ud.float()
        if ud.stride(2) != 1 or ud.stride(1) < Cn:
            ud = ud.contiguous()
        w = torch.stack([wb[2 * s].detach().reshape(Cn, TAPS).float() for s in range(nsets)]).contiguous()
        b = torch.stack([wb[2 * s + 1].detach().float() for s in range(nsets)]).contiguous()
        with torch.cuda.device(ud.device):
            y = torch.empty((nsets, Bsz, Ln, Cn), dtype=ud.dtype, device=ud.device)
            pre = torch.empty_like(y)
            a = _args(ud, nsets)
            a.w, a.bias, a.y, a.pre = w.data_ptr(), b.data_ptr(), y.data_ptr(), pre.data_ptr()
            a.chain = int(chain)
            L.check(lib.issm_dwconv_silu_fwd(C.byref(a)), "issm_dwconv_silu_fwd")
        ctx.save_for_backward(ud, w, pre)
        ctx.meta = (nsets, u.dtype, [t.dtype for t in wb], [t.shape for t in wb], int(chain))
        return tuple(y[s].to(u.dtype) for s in range(nsets))

    @staticmethod
    def backward(ctx, *dys):
        lib = L.load()
        ud, w, pre = ctx.saved_tensors
        nsets, udt, wdts, wshapes, chain = ctx.meta
        Bsz, Ln, Cn = ud.shape
        g = [None if t is None else t.to(ud.dtype).contiguous() for t in dys]
        with torch.cuda.device(ud.device):
            du = torch.empty((Bsz, Ln, Cn), dtype=ud.dtype, device=ud.device) if ctx.needs_input_grad[0] else None
            rows = lib.issm_dwconv_partial_rows(Bsz, Ln)
            partial = torch.empty((max(rows, 1), nsets, 8, Cn), dtype=torch.float32, device=ud.device)
            dw = torch.zeros((nsets, Cn, TAPS), dtype=torch.float32, device=ud.device)
            db = torch.zeros((nsets, Cn), dtype=torch.float32, device=ud.device)
            a = _args(ud, nsets)
            a.w, a.pre = w.data_ptr(), pre.data_ptr()
            a.chain = chain
            for s in range(nsets):
                a.dy[s] = None if g[s] is None else g[s].data_ptr()
            a.du = None if du is None else du.data_ptr()
            a.partial, a.dw, a.dbias = partial.data_ptr(), dw.data_ptr(), db.data_ptr()
            L.check(lib.issm_dwconv_silu_bwd(C.byref(a)), "issm_dwconv_silu_bwd")
        grads = []
        for s in range(nsets):
            grads.append(dw[s].reshape(wshapes[2 * s]).to(wdts[2 * s]))
            grads.append(db[s].to(wdts[2 * s + 1]))
        return (None if du is None else du.to(udt), None, None, *grads)


def dwconv_silu(u: torch.Tensor, weights: Sequence[torch.Tensor], biases: Sequence[torch.Tensor], chain: bool = False):
    """silu(depthwise conv7(.) + bias) for each (weight, bias) set; u (B, L, C), channels contiguous.
    Every set reads u, or with ``chain`` (two sets) the second reads the first one's result.
    Returns a tuple of (B, L, C) tensors, one per set (one or two sets)."""
    assert len(weights) == len(biases) and 1 <= len(weights) <= 2
    assert not chain or len(weights) == 2
    wb = [t for pair in zip(weights, biases) for t in pair]
    return DwConvSiLUFn.apply(u, len(weights), bool(chain), *wb)
