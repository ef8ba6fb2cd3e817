"""The core of MultiHeadISSMScan as one autograd node.

Between the input projections and the output projections, MultiHeadISSMScan.forward (models/dest_module.py:528-581)
is a fixed chain: depthwise conv + SiLU of both branches (the reversed-order branch convolves the forward-order
branch's output, dest_module.py:530,534), generation of dt / B / C from the distance encoding, the
bidirectional scan, the average of the two directions, the gated RMSNorm.  Run as separate autograd Functions and
PyTorch ops that is some forty small operations forward and as many autograd nodes backward, and at the detector's
layer shape the host cannot issue them as fast as the GPU finishes them.  ``fused_scan_core`` makes the same calls
into libissm_hip.so back to back inside one Function and chains their backward passes by hand; the arithmetic is the
kernels' either way.  Used by ``scan_module.MultiHeadISSMScan`` for the bidirectional configuration with a distance
encoding the generation kernel is built for; every other configuration takes the step-by-step path."""
from __future__ import annotations

import ctypes as C

import torch

from . import _lib as L
from . import dwconv as _dw
from . import layernorm_gated as _ln
from . import param_gen as _pg
from .issm_combined import _Problem, _scan_bwd, _scan_fwd


def _kdt(t):
    return t.dtype if t.dtype in (torch.float32, torch.bfloat16) else torch.float32


def _transpose_states(lib, in0, in1, alpha, out_dtype):
    """(B, R, C) -> (B, C, R): alpha * (in0 + in1) in `out_dtype`; in1 may be None (issm_transpose_states)."""
    if in0.dtype not in (torch.float32, torch.bfloat16):
        in0 = in0.float()
        in1 = None if in1 is None else in1.float()
    in0 = in0.contiguous()
    in1 = None if in1 is None else in1.to(in0.dtype).contiguous()
    Bsz, R, Cn = in0.shape
    out = torch.empty((Bsz, Cn, R), dtype=out_dtype, device=in0.device)
    a = L.TransposeArgs()
    a.batch, a.rows, a.cols = Bsz, R, Cn
    a.in_dtype, a.out_dtype = L.dtype_code(in0.dtype), L.dtype_code(out_dtype)
    a.in0, a.in1, a.out = in0.data_ptr(), None if in1 is None else in1.data_ptr(), out.data_ptr()
    a.alpha = alpha
    a.stream = L.current_stream_ptr(in0.device)
    L.check(lib.issm_transpose_states(C.byref(a)), "issm_transpose_states")
    return out


class FusedScanCoreFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, zxbcdt, h0_lin, dist, weights, conv_w_f, conv_b_f, conv_w_b, conv_b_b, dt_w, bc_w, dt_bias, A_log, D,
                norm_w, d_inner, nheads, ngroups, chunk_size, dt_limit, eps):
        lib = L.load()
        dev = zxbcdt.device
        Bsz, Ln, _ = zxbcdt.shape
        H, G, di = nheads, ngroups, d_inner
        P, Cc = di // H, di + 2 * G
        K = dist.shape[2]
        kdt = _kdt(zxbcdt)
        zx = zxbcdt.detach().to(kdt)
        if zx.stride(-1) != 1:
            zx = zx.contiguous()
        z, xbc, dt_tok = zx[..., :di], zx[..., di:di + Cc], zx[..., di + Cc:]
        with torch.cuda.device(dev):
            st = L.current_stream_ptr(dev)
            # 1. both depthwise convolutions + SiLU
            # all small parameters in one fp32 buffer (one concatenation + one conversion instead of one per tensor);
            # adjacent pieces form the stacked operands the kernels take
            params = (conv_w_f, conv_w_b, conv_b_f, conv_b_b, dt_w, bc_w, dt_bias, A_log)
            sizes = [t.numel() for t in params]
            flat = torch.cat([t.detach().reshape(-1) for t in params]).float()
            pieces = torch.split(flat, sizes)
            cw = flat[:2 * Cc * _dw.TAPS].view(2, Cc, _dw.TAPS)
            cb = flat[2 * Cc * _dw.TAPS:2 * Cc * _dw.TAPS + 2 * Cc].view(2, Cc)
            W = flat[sum(sizes[:4]):sum(sizes[:6])].view(H + 2 * G, 16)      # rows: dt heads, B groups, C groups
            dt_bias32, A_log32 = pieces[6], pieces[7]
            x = torch.empty((2, Bsz, Ln, H, P), dtype=kdt, device=dev)       # the conv writes x and the B / C biases apart
            tail = torch.empty((2, Bsz, Ln, 2 * G), dtype=kdt, device=dev)
            pre = torch.empty((2, Bsz, Ln, Cc), dtype=kdt, device=dev)
            a = _dw._args(xbc, 2)
            a.w, a.bias, a.y, a.pre = cw.data_ptr(), cb.data_ptr(), x.data_ptr(), pre.data_ptr()
            a.split, a.y_tail = di, tail.data_ptr()
            a.chain = 1                                                      # key_conv_back reads key_conv's output
            L.check(lib.issm_dwconv_silu_fwd(C.byref(a)), "issm_dwconv_silu_fwd")
            x_f, x_b = x[0], x[1]
            # 2. dt / B / C (and the reversed-order B / C) from the distance encoding
            bias = torch.empty((Bsz, Ln, H + 4 * G), dtype=torch.float32, device=dev)
            torch.add(dt_tok, dt_bias32, out=bias[..., :H])
            bias[..., H:].unflatten(-1, (2, 2 * G)).copy_(tail.permute(1, 2, 0, 3))
            d = dist.detach().to(kdt).contiguous()
            wt = None if weights is None else weights.detach().float().contiguous()
            dt = torch.empty((Bsz, Ln, H, K), dtype=kdt, device=dev)
            bc = [torch.empty((Bsz, Ln, G, K), dtype=kdt, device=dev) for _ in range(4)]
            raw = torch.empty_like(dt) if wt is not None else None
            g = _pg._args(d, W, H, G, True)
            g.bias = bias.data_ptr()
            g.dt, g.Bm, g.Cm, g.Bm_back, g.Cm_back = (t.data_ptr() for t in (dt, *bc))
            if wt is not None:
                g.weights, g.dt_raw = wt.data_ptr(), raw.data_ptr()
            L.check(lib.issm_param_gen_fwd(C.byref(g)), "issm_param_gen_fwd")
            # 3. the bidirectional scan, queries as initial state
            A1 = torch.exp(A_log32).neg_()
            A = A1[:, None].expand(H, K)
            h0 = _transpose_states(lib, h0_lin.detach().reshape(Bsz, K, di), None, 1.0, _kdt(h0_lin)).view(Bsz, H, P, K)
            prob = _Problem([x_f, x_b], dt, A, [bc[0], bc[2]], [bc[1], bc[3]], chunk_size, D.detach(), [None, None], None,
                            h0, None, wt is None, dt_limit)
            outs, finals, ws = _scan_fwd(prob, True)
            # 4. gated RMSNorm (norm(x * silu(z))) of the two directions' average: the norm of s / 2 with eps is the norm
            # of s with 4 eps, so the sum goes in as it is and the halving never runs (nor its backward)
            key = torch.add(outs[0], outs[1]).view(Bsz * Ln, di)
            eps = 4.0 * eps
            z2 = z.reshape(Bsz * Ln, di) if z.is_contiguous() else z.as_strided((Bsz * Ln, di), (zx.stride(1), 1),
                                                                                 z.storage_offset())
            nw = norm_w.detach()
            nw = (nw if nw.dtype in (torch.float32, torch.bfloat16) else nw.float()).contiguous()
            key_n = torch.empty_like(key)
            rstd = torch.empty(Bsz * Ln, dtype=torch.float32, device=dev)
            n = _ln._norm_args(key, z2, nw, eps, None, False)
            n.y, n.y_row_stride, n.rstd = key_n.data_ptr(), key_n.stride(0), rstd.data_ptr()
            L.check(lib.issm_gated_rmsnorm_fwd(C.byref(n)), "issm_gated_rmsnorm_fwd")
            last = _transpose_states(lib, finals[0].view(Bsz, di, K), finals[1].view(Bsz, di, K), 0.5, _kdt(h0_lin))
        ctx.save_for_backward(xbc, pre, cw, d, W, wt, raw, key, z2, nw, rstd, A1)
        ctx.prob, ctx.ws = prob, ws
        ctx.meta = (Bsz, Ln, K, H, G, di, P, Cc, kdt, eps, st)
        ctx.dtypes = tuple(t.dtype for t in (zxbcdt, h0_lin, dist, conv_w_f, conv_b_f, conv_w_b, conv_b_b, dt_w, bc_w,
                                              dt_bias, A_log, D, norm_w))
        ctx.shapes = (conv_w_f.shape, conv_w_b.shape)
        return key_n.view(Bsz, Ln, di).to(zxbcdt.dtype), last.to(h0_lin.dtype)

    @staticmethod
    def backward(ctx, dkey_n, dlast):
        lib = L.load()
        xbc, pre, cw, d, W, wt, raw, key, z2, nw, rstd, A1 = ctx.saved_tensors
        Bsz, Ln, K, H, G, di, P, Cc, kdt, eps, _ = ctx.meta
        prob = ctx.prob
        dev = key.device
        (zdt, hdt, ddt_, wfdt, bfdt, wbdt, bbdt, dtwdt, bcwdt, dtbdt, aldt, Ddt, nwdt) = ctx.dtypes
        with torch.cuda.device(dev):
            # 4'. gated RMSNorm
            dy = dkey_n.to(kdt).reshape(Bsz * Ln, di).contiguous()
            dkey = torch.empty_like(key)
            Wd = di + Cc + H                      # row of d zxbcdt: [dz | d xbc | d dt]; each producer writes its part
            dzx = torch.empty((Bsz, Ln, Wd), dtype=kdt, device=dev)
            nb = lib.issm_rmsnorm_bwd_blocks(Bsz * Ln)
            dwp = torch.empty((nb, di), dtype=torch.float32, device=dev)
            dnw = torch.empty(di, dtype=torch.float32, device=dev)
            n = _ln._norm_args(key, z2, nw, eps, None, False)
            n.rstd = rstd.data_ptr()
            n.dy, n.dy_row_stride = dy.data_ptr(), dy.stride(0)
            n.dx, n.dx_row_stride = dkey.data_ptr(), dkey.stride(0)
            n.dz, n.dz_row_stride = dzx.data_ptr(), Wd
            n.dw_partial, n.dw = dwp.data_ptr(), dnw.data_ptr()
            L.check(lib.issm_gated_rmsnorm_bwd(C.byref(n)), "issm_gated_rmsnorm_bwd")
            # 3'. the scan: both directions receive the gradient of their sum, and half of the averaged final states'
            dyh = dkey.view(Bsz, Ln, H, P)
            dfin = _transpose_states(lib, dlast.reshape(Bsz, K, di), None, 0.5, torch.float32).view(Bsz, H, P, K)
            dxs, ddt, dA, dBs, dCs, dD, _, _, dh0 = _scan_bwd(prob, ctx.ws, [dyh, dyh], [dfin, dfin], want_dz=False)
            # 2'. parameter generation
            R0, R = H + 2 * G, H + 4 * G
            g = _pg._args(d, W, H, G, True)
            g.ddt, g.dBm, g.dCm, g.dBm_back, g.dCm_back = (t.data_ptr() for t in (ddt, dBs[0], dCs[0], dBs[1], dCs[1]))
            ddist = torch.empty_like(d) if ctx.needs_input_grad[2] else None
            dbias = torch.empty((Bsz, Ln, R), dtype=torch.float32, device=dev)
            nbp = lib.issm_param_gen_bwd_blocks(Bsz * Ln)
            dwpart = torch.empty((max(nbp, 1), R0, 16), dtype=torch.float32, device=dev)
            dW = torch.empty((R0, 16), dtype=torch.float32, device=dev)
            g.ddist = None if ddist is None else ddist.data_ptr()
            g.dbias, g.dw_partial, g.dW = dbias.data_ptr(), dwpart.data_ptr(), dW.data_ptr()
            dbias_sum = torch.empty(R, dtype=torch.float32, device=dev)
            g.dbias_sum = dbias_sum.data_ptr()
            if wt is not None:
                g.weights, g.dt_raw = wt.data_ptr(), raw.data_ptr()
            L.check(lib.issm_param_gen_bwd(C.byref(g)), "issm_param_gen_bwd")
            d_dt_tok = dbias[..., :H]
            # 1'. the convolutions: gradients of (x, b-bias, c-bias) per branch
            dtail = torch.empty((2, Bsz, Ln, 2 * G), dtype=kdt, device=dev)
            dtail.copy_(dbias[..., H:].unflatten(-1, (2, 2 * G)).permute(2, 0, 1, 3))
            rows = lib.issm_dwconv_partial_rows(Bsz, Ln)
            part = torch.empty((max(rows, 1), 2, 8, Cc), dtype=torch.float32, device=dev)
            dcw = torch.empty((2, Cc, _dw.TAPS), dtype=torch.float32, device=dev)
            dcb = torch.empty((2, Cc), dtype=torch.float32, device=dev)
            a = _dw._args(xbc, 2)
            a.w, a.pre = cw.data_ptr(), pre.data_ptr()
            a.split, a.chain = di, 1
            a.dy[0], a.dy[1] = dxs[0].data_ptr(), dxs[1].data_ptr()
            a.dy_tail[0], a.dy_tail[1] = dtail[0].data_ptr(), dtail[1].data_ptr()
            a.du = dzx.data_ptr() + di * dzx.element_size()
            a.du_batch_stride, a.du_token_stride = Ln * Wd, Wd
            a.partial, a.dw, a.dbias = part.data_ptr(), dcw.data_ptr(), dcb.data_ptr()
            L.check(lib.issm_dwconv_silu_bwd(C.byref(a)), "issm_dwconv_silu_bwd")
            dzx[..., di + Cc:].copy_(d_dt_tok)
            dA_log = dA.sum(-1).mul_(A1)
            dh0_lin = _transpose_states(lib, dh0.reshape(Bsz, di, K), None, 1.0, hdt if hdt in (torch.float32, torch.bfloat16) else torch.float32)
            ddt_bias = dbias_sum[:H]
            # parameter gradients: one buffer, one conversion to the parameters' dtype when they share one
            grads = [dcw[0], dcb[0], dcw[1], dcb[1], dW[:H], dW[H:], ddt_bias, dA_log, dD, dnw]
            pdts = (wfdt, bfdt, wbdt, bbdt, dtwdt, bcwdt, dtbdt, aldt, Ddt, nwdt)
            if len(set(pdts)) == 1 and pdts[0] != torch.float32:
                sizes = [t.numel() for t in grads]
                grads = list(torch.split(torch.cat([t.reshape(-1) for t in grads]).to(pdts[0]), sizes))
            else:
                grads = [t.to(dt_) for t, dt_ in zip(grads, pdts)]
        wf_shape, wb_shape = ctx.shapes
        grads[0], grads[2] = grads[0].reshape(wf_shape), grads[2].reshape(wb_shape)
        grads[4], grads[5] = grads[4].reshape(H, 16), grads[5].reshape(2 * G, 16)
        grads[8] = grads[8].reshape(prob.D.shape)
        return (dzx.to(zdt), dh0_lin.to(hdt), None if ddist is None else ddist.to(ddt_), None, *grads,
                None, None, None, None, None, None)


def fused_scan_core(zxbcdt, h0_lin, dist, weights, conv_f, conv_b, dt_proj_w, bc_proj_w, dt_bias, A_log, D, norm_w, d_inner,
                    nheads, ngroups, chunk_size, dt_limit, eps):
    """zxbcdt (B, L, 2 d_inner + 2G + H): output of key_proj; h0_lin (B, K, d_inner): output of query_proj;
    dist (B, L, K, 16); weights (B, L, K) fp32 or None; conv_f / conv_b: the two depthwise Conv1d modules.
    Returns the normalised key (B, L, d_inner) and the averaged final state (B, K, d_inner)."""
    return FusedScanCoreFn.apply(zxbcdt, h0_lin, dist, weights, conv_f.weight, conv_f.bias, conv_b.weight, conv_b.bias,
                                 dt_proj_w, bc_proj_w, dt_bias, A_log, D, norm_w, d_inner, nheads, ngroups, chunk_size,
                                 tuple(dt_limit), eps)
