"""dt / B / C of the interactive scan from the pairwise distance encoding, in one pass on MI355X.

MultiHeadISSMScan.forward (models/dest_module.py:541-553) builds these with two Linear layers over
``dist`` (B, L, K, M), two transposes and broadcast bias additions.  ``scan_params`` computes the same
values directly in the layout the scan reads -- (B, L, H|G, K), K contiguous -- and its backward returns
the gradients of ``dist``, of the stacked projection weight and of the per-token biases.  Arithmetic runs
in libissm_hip.so (fp32 accumulation; inputs and outputs fp32 or bf16)."""
from __future__ import annotations

import ctypes as C

import torch

from . import _lib as L

MAX_ROWS = 12   # H + 2G the kernels are built for
WIDTH = 16      # M the kernels are built for


def supported(dist: torch.Tensor, nheads: int, ngroups: int) -> bool:
    return (dist.is_cuda and dist.shape[-1] == WIDTH and nheads + 2 * ngroups <= MAX_ROWS
            and dist.dtype in (torch.float32, torch.bfloat16))


def _args(dist, W, H, G, has_back) -> L.PGenArgs:
    a = L.PGenArgs()
    a.tokens = dist.shape[0] * dist.shape[1]
    a.K, a.M, a.H, a.G = dist.shape[2], dist.shape[3], H, G
    a.dtype = L.dtype_code(dist.dtype)
    a.has_back = int(has_back)
    a.dist, a.W = dist.data_ptr(), W.data_ptr()
    a.stream = L.current_stream_ptr(dist.device)
    return a


class ScanParamsFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, dist, W, bias, weights, nheads, ngroups, has_back):
        L.require_gpu(dist, "dist")
        lib = L.load()
        H, G = nheads, ngroups
        Bsz, Ln, K, M = dist.shape
        R0 = H + 2 * G
        R = R0 + (2 * G if has_back else 0)
        assert W.shape == (R0, M) and bias.shape == (Bsz, Ln, R)
        d = dist.detach().contiguous()
        w = W.detach().float().contiguous()
        b = bias.detach().float().contiguous()
        wt = None
        if weights is not None:
            assert weights.shape == (Bsz, Ln, K)
            wt = weights.detach().float().contiguous()
        with torch.cuda.device(d.device):
            dt = torch.empty((Bsz, Ln, H, K), dtype=d.dtype, device=d.device)
            outs = [torch.empty((Bsz, Ln, G, K), dtype=d.dtype, device=d.device) for _ in range(4 if has_back else 2)]
            a = _args(d, w, H, G, has_back)
            a.bias = b.data_ptr()
            a.dt, a.Bm, a.Cm = dt.data_ptr(), outs[0].data_ptr(), outs[1].data_ptr()
            if has_back:
                a.Bm_back, a.Cm_back = outs[2].data_ptr(), outs[3].data_ptr()
            raw = None
            if wt is not None:
                raw = torch.empty_like(dt)
                a.weights, a.dt_raw = wt.data_ptr(), raw.data_ptr()
            L.check(lib.issm_param_gen_fwd(C.byref(a)), "issm_param_gen_fwd")
        ctx.save_for_backward(d, w, wt, raw)
        ctx.meta = (H, G, has_back, W.dtype, bias.dtype, R, None if weights is None else weights.dtype)
        return (dt, *outs)

    @staticmethod
    def backward(ctx, *grads):
        lib = L.load()
        d, w, wt, raw = ctx.saved_tensors
        H, G, has_back, wdt, bdt, R, wtdt = ctx.meta
        Bsz, Ln, K, M = d.shape
        g = [None if t is None else t.to(d.dtype).contiguous() for t in grads]
        need_dist, need_w, need_bias, need_wt = ctx.needs_input_grad[:4]
        with torch.cuda.device(d.device):
            a = _args(d, w, H, G, has_back)
            names = ("ddt", "dBm", "dCm", "dBm_back", "dCm_back")
            for n, t in zip(names, g):
                if t is not None:
                    setattr(a, n, t.data_ptr())
            ddist = torch.empty_like(d) if need_dist else None
            dbias = torch.empty((Bsz, Ln, R), dtype=torch.float32, device=d.device) if need_bias else None
            nb = lib.issm_param_gen_bwd_blocks(Bsz * Ln)
            dwp = torch.empty((max(nb, 1), H + 2 * G, M), dtype=torch.float32, device=d.device)
            dW = torch.zeros((H + 2 * G, M), dtype=torch.float32, device=d.device)
            if ddist is not None:
                a.ddist = ddist.data_ptr()
            if dbias is not None:
                a.dbias = dbias.data_ptr()
            a.dw_partial, a.dW = dwp.data_ptr(), dW.data_ptr()
            dwt = None
            if wt is not None:
                a.weights, a.dt_raw = wt.data_ptr(), raw.data_ptr()
                if need_wt:
                    dwt = torch.zeros((Bsz, Ln, K), dtype=torch.float32, device=d.device)
                    a.dweights = dwt.data_ptr()
            L.check(lib.issm_param_gen_bwd(C.byref(a)), "issm_param_gen_bwd")
        return (ddist, dW.to(wdt) if need_w else None, None if dbias is None else dbias.to(bdt),
                None if dwt is None else dwt.to(wtdt), None, None, None)


def scan_params(dist, W, bias, nheads: int, ngroups: int, has_back: bool = False, weights=None):
    """dist (B, L, K, M=16); W (H+2G, M): rows dt heads, B groups, C groups; bias (B, L, R) with columns
    [dt heads | B | C | B_back | C_back] (the last two when ``has_back``).  Returns dt (B,L,H,K), B, C
    (B,L,G,K) and, with ``has_back``, B_back, C_back.  Without ``weights`` dt is the raw sum (before
    softplus); with ``weights`` (B, L, K) -- the locality weight, or a 0/1 keep mask --
    dt = softplus(raw) * weights (dest_module.py:553-559)."""
    return ScanParamsFn.apply(dist, W, bias, weights, nheads, ngroups, has_back)
