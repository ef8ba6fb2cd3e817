"""Host-side mirror of the module that calls the scan: DEST's `MultiHeadISSMScan`
(models/dest_module.py:425-612) and its `PointLiteConv` (models/dest_module.py:400-422).

Parameter names, shapes and initialisation ranges follow the reference, so a reference
state_dict loads unchanged.  What differs is how the scan is fed:

* dt and B/C are produced directly in the layouts the kernels read, (B, L, H, K) and
  (B, L, G, K) with K contiguous (the reference builds them as transposed views and lets the
  operator copy them, dest_module.py:543-553 and issm_combined.py:64-76);
* without a mask the softplus of dt runs inside the scan kernels (`dt_softplus=True`), which
  also removes the separate softplus backward pass;
* both scan directions go through one fused call with reversed addressing instead of
  five `torch.flip` copies and a second operator call (dest_module.py:565-575).

The dense projections, the depthwise conv and LayerNorm stay ordinary PyTorch modules.
"""
from __future__ import annotations

import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import param_gen
from .dwconv import dwconv_silu
from .fused_layer import fused_scan_core
from .issm_combined import ISSM_biscan_combined, ISSM_chunk_scan_combined
from .layernorm_gated import RMSNorm as RMSNormGated


class _LinearTokens(torch.autograd.Function):
    """y = x W^T for a (tokens, features) activation with thousands of tokens and a few hundred features (the four
    projections of the layer).  Forward and input gradient are the library GEMMs nn.Linear uses; the weight gradient
    dW = dy^T x contracts over the tokens, and as one GEMM its (out x in) result makes only a few dozen tiles -- a
    fraction of the GPU, 54 us for 8192 x 288 -> 586 in bf16.  Here the tokens are cut into slices that run as one
    batched GEMM and the slices' results are summed (24 us)."""

    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx, x, w):
        # under autocast F.linear runs in the autocast dtype; what is saved must be in that dtype too, or the
        # backward's `dy @ w` would mix dtypes
        if torch.is_autocast_enabled("cuda"):
            adt = torch.get_autocast_dtype("cuda")
            x, w = x.to(adt), w.to(adt)
        ctx.save_for_backward(x, w)
        return F.linear(x, w)

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, dy):
        x, w = ctx.saved_tensors
        dy = dy.to(x.dtype)
        dx = dw = None
        if ctx.needs_input_grad[0]:
            dx = dy @ w
        if ctx.needs_input_grad[1]:
            x2, dy2 = x.reshape(-1, x.shape[-1]), dy.reshape(-1, dy.shape[-1])
            tokens = x2.shape[0]
            slices = 4 if x2.dtype == torch.bfloat16 else 2   # fastest of 2 .. 32 on MI355X at 2048 and 8192 tokens
            if tokens < 1024 or tokens % slices:
                slices = 1
            if slices > 1:
                dw = torch.bmm(dy2.view(slices, tokens // slices, -1).transpose(1, 2),
                               x2.view(slices, tokens // slices, -1)).sum(0)
            else:
                dw = dy2.t() @ x2
        return dx, dw


def _linear(module: nn.Linear, x):
    if module.bias is not None or not x.is_cuda:
        return module(x)
    return _LinearTokens.apply(x, module.weight)


class PointLiteConv(nn.Module):
    """Depthwise 7-tap conv along the (serialised) point order + SiLU; `xyz` is unused, as in the
    reference (dest_module.py:413-422)."""

    def __init__(self, in_channels: int, out_channels: int):
        super().__init__()
        self.dwconv = nn.Conv1d(in_channels, out_channels, kernel_size=7, stride=1, padding=3, bias=True,
                                groups=out_channels)
        self.act = nn.SiLU()

    def forward(self, xyz, feature):
        return dwconv_silu(feature, [self.dwconv.weight], [self.dwconv.bias])[0]


class MultiHeadISSMScan(nn.Module):
    def __init__(self, d_model: int = 512, d_state: int = 64, d_dist: int = 4, chunk_size: int = 256,
                 nheads: int = 4, ngroups: int = 1, expand: int = 2, use_biscan: bool = True,
                 A_init_range=(1, 16), dt_min: float = 0.0001, dt_max: float = 0.1, dt_init_floor: float = 1e-4,
                 dt_limit=(0.0, float("inf")), layer_idx=None):
        super().__init__()
        self.d_model, self.d_state, self.d_dist, self.chunk_size = d_model, d_state, d_dist, chunk_size
        self.nheads, self.ngroups, self.expand, self.use_biscan = nheads, ngroups, expand, use_biscan
        self.d_inner = expand * d_model
        self.headdim = self.d_inner // nheads
        self.dt_limit = dt_limit
        self.layer_idx = layer_idx
        self.fused = True   # run the chain between the projections as one autograd node when the configuration allows

        # [z, x, b_bias, c_bias, dt_bias] from the key tokens (dest_module.py:471-474)
        self.key_proj = nn.Linear(d_model, 2 * self.d_inner + 2 * ngroups + nheads, bias=False)
        d_key_conv = self.d_inner + 2 * ngroups
        self.key_conv = PointLiteConv(d_key_conv, d_key_conv)
        if use_biscan:
            self.key_conv_back = PointLiteConv(d_key_conv, d_key_conv)
        self.query_proj = nn.Linear(d_model, self.d_inner, bias=False)
        self.bc_proj = nn.Linear(d_dist, 2 * ngroups, bias=False)
        self.dt_proj = nn.Linear(d_dist, nheads, bias=False)

        # dt bias = softplus^-1 of a log-uniform dt (dest_module.py:485-495)
        dt = torch.exp(torch.rand(nheads) * (math.log(dt_max) - math.log(dt_min)) + math.log(dt_min))
        dt = torch.clamp(dt, min=dt_init_floor)
        self.dt_bias = nn.Parameter(dt + torch.log(-torch.expm1(-dt)))
        self.dt_bias._no_weight_decay = True

        assert A_init_range[0] > 0 and A_init_range[1] >= A_init_range[0]
        self.A_log = nn.Parameter(torch.log(torch.empty(nheads, dtype=torch.float32).uniform_(*A_init_range)))
        self.A_log._no_weight_decay = True
        self.D = nn.Parameter(torch.ones(nheads))
        self.D._no_weight_decay = True

        self.out_key_proj = nn.Linear(self.d_inner, d_model, bias=False)
        self.out_query_proj = nn.Linear(self.d_inner, d_model, bias=False)
        self.key_norm = RMSNormGated(self.d_inner, eps=1e-5, norm_before_gate=False)
        self.query_norm = nn.LayerNorm(self.d_inner)

    def scan_inputs(self, in_key, in_query, dist, key_xyz, mask=None):
        """Everything the scan consumes (dest_module.py:528-559), in kernel layouts.

        Returns a dict with z (B,L,d_inner), x / x_back (B,L,H,P), dt (B,L,H,K) -- raw (pre-softplus)
        when `softplus_in_kernel` -- A (H,K), B/C and their *_back (B,L,G,K), initial_states (B,H,P,K).
        """
        H, G, P = self.nheads, self.ngroups, self.headdim
        zxbcdt = _linear(self.key_proj, in_key)
        z, xbc, dt_tok = torch.split(zxbcdt, [self.d_inner, self.d_inner + 2 * G, H], dim=-1)
        if self.use_biscan:
            # key_conv_back runs on key_conv's OUTPUT (dest_module.py:530 reassigns xbc before :534 uses it):
            # one chained pass, xbc_b = silu(conv_back(silu(conv(xbc))))
            convs = (self.key_conv.dwconv, self.key_conv_back.dwconv)
            xbc_f, xbc_b = dwconv_silu(xbc, [c.weight for c in convs], [c.bias for c in convs], chain=True)
        else:
            xbc_f = self.key_conv(key_xyz, xbc)
        x, b_bias, c_bias = torch.split(xbc_f, [self.d_inner, G, G], dim=-1)
        out = dict(z=z, x=x.contiguous().unflatten(-1, (H, P)))
        # queries become the initial state: one state column per query (dest_module.py:537-538)
        h0 = _linear(self.query_proj, in_query)                                   # (B, K, H*P)
        out["initial_states"] = h0.unflatten(-1, (H, P)).permute(0, 2, 3, 1)   # (B, H, P, K) view
        out["A"] = (-torch.exp(self.A_log.float()))[:, None].expand(H, self.d_state)
        dt_tok_bias = dt_tok + self.dt_bias.to(dt_tok.dtype)
        if self.use_biscan:
            x_b, b_bias_b, c_bias_b = torch.split(xbc_b, [self.d_inner, G, G], dim=-1)
            out["x_back"] = x_b.contiguous().unflatten(-1, (H, P))
        if param_gen.supported(dist, H, G):
            # one pass over dist writes every (B,L,H|G,K) operand (dest_module.py:541-553)
            W = torch.cat([self.dt_proj.weight, self.bc_proj.weight], dim=0)
            cols = [dt_tok_bias, b_bias, c_bias] + ([b_bias_b, c_bias_b] if self.use_biscan else [])
            # a float mask weighs dt, a bool mask drops entries (dest_module.py:555-559): both are a factor on softplus(raw)
            wts = None
            if mask is not None:
                wts = mask.float() if mask.is_floating_point() else (~mask).float()
            res = param_gen.scan_params(dist, W, torch.cat(cols, dim=-1).float(), H, G, self.use_biscan, wts)
            dt_raw, out["B"], out["C"] = res[:3]
            if self.use_biscan:
                out["B_back"], out["C_back"] = res[3:]
            if mask is not None:
                out["dt"], out["softplus_in_kernel"] = dt_raw, False
                return out
        else:
            # W (G|H, M) @ dist^T (B,L,M,K): the product is written straight into (B,L,G|H,K), K contiguous
            dist_t = dist.transpose(-1, -2)
            b_base = torch.matmul(self.bc_proj.weight[:G], dist_t)
            c_base = torch.matmul(self.bc_proj.weight[G:], dist_t)
            out["B"] = b_base + b_bias.unsqueeze(-1)
            out["C"] = c_base + c_bias.unsqueeze(-1)
            if self.use_biscan:
                out["B_back"] = b_base + b_bias_b.unsqueeze(-1)
                out["C_back"] = c_base + c_bias_b.unsqueeze(-1)
            dt_raw = torch.matmul(self.dt_proj.weight, dist_t) + dt_tok_bias.unsqueeze(-1)
        if mask is None:
            out["dt"], out["softplus_in_kernel"] = dt_raw, True
        else:
            dt = F.softplus(dt_raw)
            if mask.dtype == torch.float32:
                dt = dt * mask.unsqueeze(2).to(dt.dtype)
            else:
                dt = dt.masked_fill(mask.unsqueeze(2), 0.0)
            out["dt"], out["softplus_in_kernel"] = dt, False
        return out

    def forward(self, in_key, in_query, dist, key_xyz, mask=None):
        """in_key (B,L,D), in_query (B,K,D), dist (B,L,K,M), mask (B,L,K) float weights or bool
        "drop" flags -> out_key (B,L,D), out_query (B,K,D)   (dest_module.py:515-585)."""
        if self.fused and self.use_biscan and param_gen.supported(dist, self.nheads, self.ngroups) and \
                not (mask is not None and mask.requires_grad):
            # the whole chain between the projections as one autograd node (same kernels, far fewer host operations)
            wts = None if mask is None else (mask.float() if mask.is_floating_point() else (~mask).float())
            key, last = fused_scan_core(_linear(self.key_proj, in_key), _linear(self.query_proj, in_query), dist, wts,
                                        self.key_conv.dwconv, self.key_conv_back.dwconv, self.dt_proj.weight,
                                        self.bc_proj.weight, self.dt_bias, self.A_log, self.D, self.key_norm.weight,
                                        self.d_inner, self.nheads, self.ngroups, self.chunk_size, self.dt_limit,
                                        self.key_norm.eps)
            return _linear(self.out_key_proj, key), _linear(self.out_query_proj, self.query_norm(last))
        s = self.scan_inputs(in_key, in_query, dist, key_xyz, mask)
        kw = dict(D=self.D, initial_states=s["initial_states"], dt_softplus=s["softplus_in_kernel"],
                  dt_limit=self.dt_limit)
        if self.use_biscan:
            key, key_back, last, last_back = ISSM_biscan_combined(
                s["x"], s["x_back"], s["dt"], s["A"], s["B"], s["B_back"], s["C"], s["C_back"], self.chunk_size, **kw)
            key = (key + key_back) / 2
            last = (last + last_back) / 2
        else:
            key, last = ISSM_chunk_scan_combined(s["x"], s["dt"], s["A"], s["B"], s["C"], self.chunk_size,
                                                 return_final_states=True, **kw)
        key = self.key_norm(key.flatten(-2), s["z"])
        out_key = _linear(self.out_key_proj, key)
        last = last.permute(0, 3, 1, 2).flatten(-2).to(in_query.dtype)      # (B, K, H*P)
        out_query = _linear(self.out_query_proj, self.query_norm(last))
        return out_key, out_query
