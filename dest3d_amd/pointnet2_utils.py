"""Point-set operators of the PointNet++ backbone on MI355X, with the Python surface of the reference's
pointnet2/pointnet2_utils.py: ``furthest_point_sample``, ``gather_operation``, ``three_nn``, ``three_interpolate``,
``grouping_operation``, ``ball_query`` (autograd Functions, :51-291), ``QueryAndGroup`` (:294-376) and ``GroupAll``
(:379-425).  Arithmetic runs in libissm_hip.so (``issm_pn2_*``); there is no fallback path."""
from __future__ import annotations

import ctypes as C

import torch
import torch.nn as nn
from torch.autograd import Function

from . import _lib as L


def _f(t):
    return t.detach().float().contiguous()


def _i(t):
    return t.detach().to(torch.int32).contiguous()


def _st(t):
    return L.current_stream_ptr(t.device)


class FurthestPointSampling(Function):
    @staticmethod
    def forward(ctx, xyz, npoint):
        """xyz (B, N, 3) -> int32 indices (B, npoint) of a furthest-point subset, starting from point 0."""
        L.require_gpu(xyz, "xyz")
        lib = L.load()
        x = _f(xyz)
        Bsz, N, _ = x.shape
        with torch.cuda.device(x.device):
            out = torch.zeros((Bsz, npoint), dtype=torch.int32, device=x.device)
            temp = torch.empty((Bsz, N), dtype=torch.float32, device=x.device) if N > 24576 else None
            L.check(lib.issm_pn2_furthest_point_sampling(Bsz, N, npoint, x.data_ptr(), None if temp is None else temp.data_ptr(),
                                                         out.data_ptr(), _st(x)), "issm_pn2_furthest_point_sampling")
        ctx.mark_non_differentiable(out)
        return out

    @staticmethod
    def backward(ctx, a=None):
        return None, None


furthest_point_sample = FurthestPointSampling.apply


class GatherOperation(Function):
    @staticmethod
    def forward(ctx, features, idx):
        """features (B, C, N), idx (B, npoint) -> (B, C, npoint)."""
        L.require_gpu(features, "features")
        lib = L.load()
        f, ix = _f(features), _i(idx)
        Bsz, Cn, N = f.shape
        M = ix.shape[1]
        with torch.cuda.device(f.device):
            out = torch.empty((Bsz, Cn, M), dtype=torch.float32, device=f.device)
            L.check(lib.issm_pn2_gather_points(Bsz, Cn, N, M, f.data_ptr(), ix.data_ptr(), out.data_ptr(), _st(f)),
                    "issm_pn2_gather_points")
        ctx.for_backwards = (ix, Cn, N, features.dtype)
        return out.to(features.dtype)

    @staticmethod
    def backward(ctx, grad_out):
        lib = L.load()
        ix, Cn, N, dt = ctx.for_backwards
        g = _f(grad_out)
        Bsz, _, M = g.shape
        with torch.cuda.device(g.device):
            out = torch.zeros((Bsz, Cn, N), dtype=torch.float32, device=g.device)
            L.check(lib.issm_pn2_gather_points_grad(Bsz, Cn, N, M, g.data_ptr(), ix.data_ptr(), out.data_ptr(), _st(g)),
                    "issm_pn2_gather_points_grad")
        return out.to(dt), None


gather_operation = GatherOperation.apply


class ThreeNN(Function):
    @staticmethod
    def forward(ctx, unknown, known):
        """unknown (B, n, 3), known (B, m, 3) -> distances (B, n, 3) to, and int32 indices of, the 3 nearest known."""
        L.require_gpu(unknown, "unknown")
        lib = L.load()
        u, k = _f(unknown), _f(known)
        Bsz, n, _ = u.shape
        m = k.shape[1]
        with torch.cuda.device(u.device):
            dist2 = torch.empty((Bsz, n, 3), dtype=torch.float32, device=u.device)
            idx = torch.empty((Bsz, n, 3), dtype=torch.int32, device=u.device)
            L.check(lib.issm_pn2_three_nn(Bsz, n, m, u.data_ptr(), k.data_ptr(), dist2.data_ptr(), idx.data_ptr(), _st(u)),
                    "issm_pn2_three_nn")
        ctx.mark_non_differentiable(idx)
        return torch.sqrt(dist2), idx

    @staticmethod
    def backward(ctx, a=None, b=None):
        return None, None


three_nn = ThreeNN.apply


class ThreeInterpolate(Function):
    @staticmethod
    def forward(ctx, features, idx, weight):
        """features (B, c, m), idx / weight (B, n, 3) -> (B, c, n): weighted sum of three features per target."""
        L.require_gpu(features, "features")
        lib = L.load()
        f, ix, w = _f(features), _i(idx), _f(weight)
        Bsz, c, m = f.shape
        n = ix.shape[1]
        with torch.cuda.device(f.device):
            out = torch.empty((Bsz, c, n), dtype=torch.float32, device=f.device)
            L.check(lib.issm_pn2_three_interpolate(Bsz, c, m, n, f.data_ptr(), ix.data_ptr(), w.data_ptr(), out.data_ptr(),
                                                   _st(f)), "issm_pn2_three_interpolate")
        ctx.three_interpolate_for_backward = (ix, w, m, features.dtype)
        return out.to(features.dtype)

    @staticmethod
    def backward(ctx, grad_out):
        lib = L.load()
        ix, w, m, dt = ctx.three_interpolate_for_backward
        g = _f(grad_out)
        Bsz, c, n = g.shape
        with torch.cuda.device(g.device):
            # accumulated channel-last (coalesced atomics); the transpose is the gradient in the features' layout
            out = torch.zeros((Bsz, m, c), dtype=torch.float32, device=g.device)
            L.check(lib.issm_pn2_three_interpolate_grad_cl(Bsz, c, n, m, g.data_ptr(), ix.data_ptr(), w.data_ptr(),
                                                           out.data_ptr(), _st(g)), "issm_pn2_three_interpolate_grad_cl")
        return out.transpose(1, 2).to(dt), None, None


three_interpolate = ThreeInterpolate.apply


class GroupingOperation(Function):
    @staticmethod
    def forward(ctx, features, idx):
        """features (B, C, N), idx (B, npoint, nsample) -> (B, C, npoint, nsample)."""
        L.require_gpu(features, "features")
        lib = L.load()
        f, ix = _f(features), _i(idx)
        Bsz, Cn, N = f.shape
        _, M, S = ix.shape
        with torch.cuda.device(f.device):
            out = torch.empty((Bsz, Cn, M, S), dtype=torch.float32, device=f.device)
            L.check(lib.issm_pn2_group_points(Bsz, Cn, N, M, S, f.data_ptr(), ix.data_ptr(), out.data_ptr(), _st(f)),
                    "issm_pn2_group_points")
        ctx.for_backwards = (ix, N, features.dtype)
        return out.to(features.dtype)

    @staticmethod
    def backward(ctx, grad_out):
        lib = L.load()
        ix, N, dt = ctx.for_backwards
        g = _f(grad_out)
        Bsz, Cn, M, S = g.shape
        with torch.cuda.device(g.device):
            # accumulated channel-last (coalesced atomics); the transpose is the gradient in the features' layout
            out = torch.zeros((Bsz, N, Cn), dtype=torch.float32, device=g.device)
            L.check(lib.issm_pn2_group_points_grad_cl(Bsz, Cn, N, M, S, g.data_ptr(), ix.data_ptr(), out.data_ptr(), _st(g)),
                    "issm_pn2_group_points_grad_cl")
        return out.transpose(1, 2).to(dt), None


grouping_operation = GroupingOperation.apply


class BallQuery(Function):
    @staticmethod
    def forward(ctx, radius, nsample, xyz, new_xyz):
        """xyz (B, N, 3), new_xyz (B, npoint, 3) -> int32 (B, npoint, nsample): the first nsample points (in index
        order) within radius of each centre; missing slots repeat the first hit, no hit leaves zeros."""
        L.require_gpu(xyz, "xyz")
        lib = L.load()
        x, q = _f(xyz), _f(new_xyz)
        Bsz, N, _ = x.shape
        M = q.shape[1]
        with torch.cuda.device(x.device):
            idx = torch.zeros((Bsz, M, nsample), dtype=torch.int32, device=x.device)
            L.check(lib.issm_pn2_ball_query(Bsz, N, M, float(radius), nsample, q.data_ptr(), x.data_ptr(), idx.data_ptr(),
                                            _st(x)), "issm_pn2_ball_query")
        ctx.mark_non_differentiable(idx)
        return idx

    @staticmethod
    def backward(ctx, a=None):
        return None, None, None, None


ball_query = BallQuery.apply


class QueryAndGroup(nn.Module):
    """Ball query, then grouping of coordinates (relative to the centre) and features (pointnet2_utils.py:294-376)."""

    def __init__(self, radius, nsample, use_xyz=True, ret_grouped_xyz=False, normalize_xyz=False, sample_uniformly=False,
                 ret_unique_cnt=False):
        super().__init__()
        self.radius, self.nsample, self.use_xyz = radius, nsample, use_xyz
        self.ret_grouped_xyz = ret_grouped_xyz
        self.normalize_xyz = normalize_xyz
        self.sample_uniformly = sample_uniformly
        self.ret_unique_cnt = ret_unique_cnt
        if self.ret_unique_cnt:
            assert self.sample_uniformly

    def forward(self, xyz, new_xyz, features=None):
        idx = ball_query(self.radius, self.nsample, xyz, new_xyz)
        unique_cnt = None
        if self.sample_uniformly:
            # repeat the distinct hits at random instead of the first one (host loop, as in the reference)
            idx = idx.clone()
            unique_cnt = torch.zeros((idx.shape[0], idx.shape[1]))
            for b in range(idx.shape[0]):
                for r in range(idx.shape[1]):
                    uniq = torch.unique(idx[b, r, :])
                    unique_cnt[b, r] = uniq.shape[0]
                    pick = torch.randint(0, uniq.shape[0], (self.nsample - uniq.shape[0],), dtype=torch.long,
                                         device=uniq.device)
                    idx[b, r, :] = torch.cat((uniq, uniq[pick]))
        grouped_xyz = grouping_operation(xyz.transpose(1, 2).contiguous(), idx)   # (B, 3, npoint, nsample)
        grouped_xyz = grouped_xyz - new_xyz.transpose(1, 2).unsqueeze(-1)
        if self.normalize_xyz:
            grouped_xyz = grouped_xyz / self.radius
        if features is not None:
            grouped = grouping_operation(features, idx)
            new_features = torch.cat([grouped_xyz, grouped], dim=1) if self.use_xyz else grouped
        else:
            assert self.use_xyz, "Cannot have not features and not use xyz as a feature!"
            new_features = grouped_xyz
        ret = [new_features]
        if self.ret_grouped_xyz:
            ret.append(grouped_xyz)
        if self.ret_unique_cnt:
            ret.append(unique_cnt)
        return ret[0] if len(ret) == 1 else tuple(ret)


class GroupAll(nn.Module):
    """All points as one group (pointnet2_utils.py:379-425)."""

    def __init__(self, use_xyz=True, ret_grouped_xyz=False):
        super().__init__()
        self.use_xyz = use_xyz
        self.ret_grouped_xyz = ret_grouped_xyz

    def forward(self, xyz, new_xyz, features=None):
        grouped_xyz = xyz.transpose(1, 2).unsqueeze(2)
        if features is not None:
            grouped = features.unsqueeze(2)
            new_features = torch.cat([grouped_xyz, grouped], dim=1) if self.use_xyz else grouped
        else:
            new_features = grouped_xyz
        return (new_features, grouped_xyz) if self.ret_grouped_xyz else new_features
