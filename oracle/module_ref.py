"""CPU restatement (test infrastructure, never imported by the product path) of DEST's
``MultiHeadISSMScan.forward`` (models/dest_module.py:515-585) in the reference's own order of operations --
transposed views, flipped copies, two scan calls -- in whatever dtype the given tensors have (the tests use
fp64), with the scan taken from ``oracle.issm_ref.issm_scan_sequential`` and the gated norm from
``oracle.issm_ref.gated_rmsnorm_ref``.

One detail of the reference that is easy to misread: dest_module.py:530 REASSIGNS ``xbc = key_conv(xbc)``, so the
reversed-order branch at :534, ``key_conv_back(key_xyz, xbc)``, convolves the forward-order branch's OUTPUT
(SiLU included), not the ``key_proj`` output.  ``tests/test_module_cpu.py`` pins that order on a case where the two
readings differ visibly.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

from . import issm_ref as R


def point_lite_conv(sd, prefix, t):
    """PointLiteConv.forward (dest_module.py:413-422): depthwise Conv1d(7, padding 3) over the token order, then SiLU."""
    w, b = sd[prefix + ".dwconv.weight"], sd[prefix + ".dwconv.bias"]
    return F.silu(F.conv1d(t.transpose(1, 2), w, b, padding=3, groups=w.shape[0])).transpose(1, 2)


def multi_head_issm_scan_ref(sd, cfg, in_key, in_query, dist, mask, intermediates=None):
    """sd: state_dict of the module (reference parameter names); cfg: nheads, ngroups, d_inner, d_state, use_biscan.
    Returns (out_key, out_query).  If `intermediates` is a dict it receives x, x_back, B, C, B_back, C_back, dt."""
    H, G, d_inner = cfg["nheads"], cfg["ngroups"], cfg["d_inner"]
    P, K = d_inner // H, cfg["d_state"]
    zxbcdt = in_key @ sd["key_proj.weight"].T                                          # :528
    z, xbc, dt_tok = torch.split(zxbcdt, [d_inner, d_inner + 2 * G, H], dim=-1)        # :529
    xbc = point_lite_conv(sd, "key_conv", xbc)                                         # :530 (xbc reassigned)
    x, b_bias, c_bias = torch.split(xbc, [d_inner, G, G], dim=-1)                      # :531
    if cfg["use_biscan"]:
        xbc_back = point_lite_conv(sd, "key_conv_back", xbc)                           # :534 (the convolved xbc)
        x_b, bb, cb = torch.split(xbc_back, [d_inner, G, G], dim=-1)
    h0 = (in_query @ sd["query_proj.weight"].T).reshape(in_query.shape[0], K, H, P).permute(0, 2, 3, 1)   # :537-538
    A = (-torch.exp(sd["A_log"]))[:, None].expand(H, K)                                # :541-542
    bc = dist @ sd["bc_proj.weight"].T                                                 # :543
    b_base, c_base = torch.split(bc, [G, G], dim=-1)
    Bm = b_base.transpose(-1, -2) + b_bias.unsqueeze(-1)                               # :545-546
    Cm = c_base.transpose(-1, -2) + c_bias.unsqueeze(-1)
    dt = F.softplus((dist @ sd["dt_proj.weight"].T).transpose(-1, -2) + dt_tok.unsqueeze(-1)
                    + sd["dt_bias"].reshape(1, 1, -1, 1))                              # :552-553
    if mask is not None:                                                               # :555-559
        if mask.dtype == torch.bool:
            dt = dt.masked_fill(mask.unsqueeze(2), 0.0)
        else:
            dt = dt * mask.unsqueeze(2).to(dt.dtype)
    hp = lambda t: t.reshape(*t.shape[:2], H, P)
    scan = lambda x_, dt_, B_, C_: R.issm_scan_sequential(hp(x_), dt_, A, B_, C_, D=sd["D"], initial_states=h0)
    key, last = scan(x, dt, Bm, Cm)                                                    # :565
    if intermediates is not None:
        intermediates.update(x=x, B=Bm, C=Cm, dt=dt)
    if cfg["use_biscan"]:
        fl = lambda t: torch.flip(t, dims=[1])
        B_back = b_base.transpose(-1, -2) + bb.unsqueeze(-1)                           # :549-550
        C_back = c_base.transpose(-1, -2) + cb.unsqueeze(-1)
        if intermediates is not None:
            intermediates.update(x_back=x_b, B_back=B_back, C_back=C_back)
        key_b, last_b = scan(fl(x_b), fl(dt), fl(B_back), fl(C_back))                  # :568-572
        key = (key + fl(key_b)) / 2                                                    # :573-575
        last = (last + last_b) / 2
    key = R.gated_rmsnorm_ref(key.flatten(-2), sd["key_norm.weight"], z=z, eps=1e-5, norm_before_gate=False)  # :578-579
    out_key = key @ sd["out_key_proj.weight"].T
    last = last.permute(0, 3, 1, 2).flatten(-2)                                        # :582
    last = F.layer_norm(last, (d_inner,), sd["query_norm.weight"], sd["query_norm.bias"], 1e-5)
    return out_key, last @ sd["out_query_proj.weight"].T
