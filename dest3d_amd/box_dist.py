"""Box-to-point distance encoding (``BoxDistFun``) and locality weight of DEST's decoder layer, on MI355X.

Mirrors models/dest_module.py:147-195 (``BoxDistFun``: same constructor arguments, buffer and parameter names, so
a reference ``state_dict`` loads unchanged) and :240-249 (``local_weight``).  The per-(point, box) work -- corner
deltas, rotation, signed-log compression, trilinear sampling of the learned table, the sum over 8 corners, and the
exponential weight -- runs in one kernel of libissm_hip.so with the table in LDS; ``dist`` comes out contiguous as
(B, nP, nQ, C), the layout the scan's parameter generation reads.  Only the table (hence the small MLP that
produces it) receives a gradient: the reference detaches the corners, and point positions and angles are inputs.
There is no fallback path."""
from __future__ import annotations

import ctypes as C
import math
from typing import Optional

import torch
import torch.nn as nn

from . import _lib as L

CHANNELS = 16      # table channels the kernels are built for (DEST's decoder: BoxDistFun(out_dim=16))
MAX_NODES = 1024   # table nodes that fit the LDS copy


def box_parametrization_to_corners(center, size, angle):
    """The 8 corners (..., 8, 3) of boxes given centre (..., 3), size (..., 3) = (l, w, h) and heading (...),
    in the frame of the inputs; corner order of dest_module.py:62-70 after the camera/lidar axis changes of
    :26-38 are composed: x = cx + sx l/2 cos + sz w/2 sin, y = cy - sx l/2 sin + sz w/2 cos, z = cz - sy h/2."""
    sx = center.new_tensor([1, 1, -1, -1, 1, 1, -1, -1])
    sy = center.new_tensor([1, 1, 1, 1, -1, -1, -1, -1])
    sz = center.new_tensor([1, -1, -1, 1, 1, -1, -1, 1])
    lx = size[..., 0:1] / 2 * sx
    hy = size[..., 2:3] / 2 * sy
    wz = size[..., 1:2] / 2 * sz
    c, s = torch.cos(angle).unsqueeze(-1), torch.sin(angle).unsqueeze(-1)
    x = center[..., 0:1] + lx * c + wz * s
    y = center[..., 1:2] - lx * s + wz * c
    z = center[..., 2:3] - hy
    return torch.stack([x, y, z], dim=-1)


def _f32c(t: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    return None if t is None else t.detach().float().contiguous()


class BoxDistFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, table, key_xyz, corners, angle, qcenter, radius, weight_dist, log_scale, max_value, out_dtype,
                want_dist, want_weights):
        L.require_gpu(key_xyz, "key_xyz")
        lib = L.load()
        Bsz, nP = key_xyz.shape[:2]
        nQ = corners.shape[1]
        key, cor, ang = _f32c(key_xyz), _f32c(corners), _f32c(angle)
        as_boxes = cor.dim() == 3          # (B, nQ, 7) boxes instead of (B, nQ, 8, 3) corners
        assert cor.shape[2:] == ((7,) if as_boxes else (8, 3))
        a = L.BoxDistArgs()
        a.batch, a.seqlen, a.nquery = Bsz, nP, nQ
        a.dtype = L.dtype_code(out_dtype)
        a.key = key.data_ptr()
        if as_boxes:
            a.boxes, a.min_radius = cor.data_ptr(), 0.64
        else:
            a.corners = cor.data_ptr()
        a.angle = None if ang is None else ang.data_ptr()
        a.log_scale, a.max_value = float(log_scale), float(max_value)
        a.stream = L.current_stream_ptr(key.device)
        a.D = a.H = a.W = 1
        dist = weights = tab = qc = rad = None
        with torch.cuda.device(key.device):
            if want_dist:
                assert table.dim() == 4 and table.shape[0] == CHANNELS, "table must be (16, D, H, W)"
                tab = _f32c(table)
                a.D, a.H, a.W = tab.shape[1:]
                a.table = tab.data_ptr()
                dist = torch.empty((Bsz, nP, nQ, CHANNELS), dtype=out_dtype, device=key.device)
                a.dist = dist.data_ptr()
            if want_weights:
                weights = torch.empty((Bsz, nP, nQ), dtype=torch.float32, device=key.device)
                a.weight_dist = float(weight_dist)
                if qcenter is not None:
                    qc, rad = _f32c(qcenter), _f32c(radius)
                    a.qcenter, a.radius = qc.data_ptr(), rad.data_ptr()
                else:
                    assert as_boxes, "weights need (qcenter, radius) or boxes"
                a.weights = weights.data_ptr()
            L.check(lib.issm_box_dist_fwd(C.byref(a)), "issm_box_dist_fwd")
        ctx.save_for_backward(key, cor, ang)
        ctx.meta = (None if table is None else (tuple(table.shape), table.dtype), log_scale, max_value, out_dtype)
        ctx.mark_non_differentiable(*[t for t in (weights,) if t is not None])
        return dist, weights

    @staticmethod
    def backward(ctx, ddist, _dweights):
        key, cor, ang = ctx.saved_tensors
        tmeta, log_scale, max_value, out_dtype = ctx.meta
        dtable = None
        if ddist is not None and tmeta is not None and ctx.needs_input_grad[0]:
            lib = L.load()
            (Cn, D, H, W), tdt = tmeta
            Bsz, nP = key.shape[:2]
            nQ = cor.shape[1]
            g = ddist.to(out_dtype).contiguous()
            with torch.cuda.device(key.device):
                a = L.BoxDistArgs()
                a.batch, a.seqlen, a.nquery, a.D, a.H, a.W = Bsz, nP, nQ, D, H, W
                a.dtype = L.dtype_code(out_dtype)
                a.key = key.data_ptr()
                if cor.dim() == 3:
                    a.boxes, a.min_radius = cor.data_ptr(), 0.64
                else:
                    a.corners = cor.data_ptr()
                a.angle = None if ang is None else ang.data_ptr()
                a.log_scale, a.max_value = float(log_scale), float(max_value)
                nbytes = lib.issm_box_dist_bwd_scratch_bytes(Bsz, nP, nQ, D, H, W)
                partial = torch.empty(nbytes // 8, dtype=torch.int64, device=key.device)
                out = torch.zeros((Cn, D, H, W), dtype=torch.float32, device=key.device)
                a.ddist, a.partial, a.dtable = g.data_ptr(), partial.data_ptr(), out.data_ptr()
                a.stream = L.current_stream_ptr(key.device)
                L.check(lib.issm_box_dist_bwd(C.byref(a)), "issm_box_dist_bwd")
            dtable = out.to(tdt)
        return (dtable,) + (None,) * 11


def box_dist(table, key_xyz, corners, angle=None, log_scale=512.0, max_value=4.0, out_dtype=None):
    """table (16, D, H, W), key_xyz (B, nP, 3), corners (B, nQ, 8, 3), angle (B, nQ) or None -> (B, nP, nQ, 16)."""
    out_dtype = out_dtype or (table.dtype if table.dtype in (torch.float32, torch.bfloat16) else torch.float32)
    return BoxDistFn.apply(table, key_xyz, corners, angle, None, None, 0.0, log_scale, max_value, out_dtype,
                           True, False)[0]


def local_weight(key_xyz, query_pos, weight_dist=15.0, min_radius=0.64):
    """exp(weight_dist * min(radius - |key - centre|, 0)), radius = max(|size|, min_radius); query_pos (B, nQ, 6)
    = centre + size -> (B, nP, nQ) fp32   (dest_module.py:240-249)."""
    radius = query_pos[..., 3:].float().square().sum(-1).sqrt().clamp_min(min_radius)
    corners = query_pos.new_zeros((*query_pos.shape[:2], 8, 3))
    return BoxDistFn.apply(None, key_xyz, corners, None, query_pos[..., :3], radius, float(weight_dist), 512.0, 4.0,
                           torch.float32, False, True)[1]


class BoxDistFun(nn.Module):
    """Learned relative-position encoding between key points and query boxes (dest_module.py:147-195)."""

    def __init__(self, log_scale: int = 512, rpe_quant: str = "bilinear_4_10", out_dim: int = 4, rpe_dim: int = 128):
        super().__init__()
        self.log_scale = log_scale
        self.interp_method, max_value, num_points = rpe_quant.split("_")
        max_value, num_points = float(max_value), int(num_points)
        if self.interp_method != "bilinear":
            raise NotImplementedError("the HIP kernel samples the table trilinearly ('bilinear' grid_sample mode)")
        if out_dim != CHANNELS or num_points ** 3 > MAX_NODES:
            raise NotImplementedError(f"built for out_dim == {CHANNELS} and at most {MAX_NODES} table nodes")
        lin = torch.linspace(-max_value, max_value, num_points, dtype=torch.float32)
        table = torch.stack(torch.meshgrid(lin, lin, lin, indexing="ij"), dim=-1).unsqueeze(0)
        self.register_buffer("relative_coords_table", table)
        self.max_value = max_value
        self.cpb_mlps = nn.Sequential(nn.Linear(3, rpe_dim, bias=True), nn.ReLU(inplace=False),
                                      nn.Linear(rpe_dim, out_dim, bias=False))

    def rpe_table(self) -> torch.Tensor:
        """(out_dim, n, n, n): the MLP evaluated on the coordinate lattice (dest_module.py:191)."""
        return self.cpb_mlps(self.relative_coords_table.to(self.cpb_mlps[0].weight.dtype))[0].permute(3, 0, 1, 2)

    def forward(self, key_xyz, query_xyz, query_size, query_angle, weight_query_pos=None, weight_dist=15.0):
        """-> dist (B, nP, nQ, out_dim).  With ``weight_query_pos`` (B, nQ, 6) the locality weights (B, nP, nQ)
        of ``local_weight`` are computed in the same pass and returned as a second value."""
        # the kernel derives the corners (and, for the weights, centre and radius) from the boxes themselves
        boxes = torch.cat([query_xyz, query_size, query_angle.unsqueeze(-1)], dim=-1).detach()
        table = self.rpe_table()
        out_dtype = table.dtype if table.dtype in (torch.float32, torch.bfloat16) else torch.float32
        if weight_query_pos is None:
            return BoxDistFn.apply(table, key_xyz, boxes, query_angle, None, None, 0.0, self.log_scale, self.max_value,
                                   out_dtype, True, False)[0]
        same_boxes = (weight_query_pos.shape[-1] == 6 and query_xyz.data_ptr() == weight_query_pos.data_ptr()
                      and query_size.data_ptr() == weight_query_pos[..., 3:].data_ptr()
                      and query_xyz.stride() == weight_query_pos[..., :3].stride())
        if same_boxes:        # query_pos[..., :3] / query_pos[..., 3:], as the decoder layer calls it
            qc = rad = None   # the weight's boxes are the encoding's: centre and radius come from `boxes`
        else:
            qc = weight_query_pos[..., :3]
            rad = weight_query_pos[..., 3:].float().square().sum(-1).sqrt().clamp_min(0.64)
        return BoxDistFn.apply(table, key_xyz, boxes, query_angle, qc, rad, float(weight_dist), self.log_scale,
                               self.max_value, out_dtype, True, True)
