"""Serialization of the key points along a 3-D Hilbert curve, on MI355X.

Mirrors models/dest_module.py:307-397 (``Serialization``: same constructor arguments, ``forward(points)`` filling
``index_list`` / ``reversed_index_list``, ``reorder_points``, ``reversed_reorder_points``).  The reference maps grid
coordinates to curve positions through a 2**27-entry table loaded from ``utils/hilbert/curve_template_3d_rank_9.pth``,
a file that is not part of its repository; here the position is computed by a kernel of libissm_hip.so (Skilling's
algorithm), so no file is needed -- and the curve's orientation may differ from that table's.  Ties (points in the
same 2 cm cell) keep their input order (stable sort), where the reference leaves them to the sort's whim.

With the fused scan only the small tensors need the permutation: the key positions (B, L, 3) and key features
(B, L, C).  Everything of size (B, L, K, .) is produced from the permuted positions directly in scan order."""
from __future__ import annotations

import ctypes as C
from typing import List, Sequence

import torch
import torch.nn as nn

from . import _lib as L

ORDERS = {"xyz": (0, 1, 2), "xzy": (0, 2, 1), "yxz": (1, 0, 2), "yzx": (1, 2, 0), "zxy": (2, 0, 1), "zyx": (2, 1, 0)}


def hilbert_codes(points: torch.Tensor, order: str = "xyz", bit: int = 9, cell: float = 1.0 / 50.0) -> torch.Tensor:
    """points (B, N, 3) -> int64 codes (B, N): position of every point's grid cell on the 3-D Hilbert curve."""
    if order not in ORDERS:
        raise NotImplementedError(order)
    L.require_gpu(points, "points")
    lib = L.load()
    p = points.detach().float().contiguous()
    with torch.cuda.device(p.device):
        mins = p.amin(dim=1).contiguous()
        codes = torch.empty(p.shape[:2], dtype=torch.int64, device=p.device)
        a = L.HilbertArgs()
        a.batch, a.npoint, a.bits = p.shape[0], p.shape[1], bit
        for i, v in enumerate(ORDERS[order]):
            a.order[i] = v
        a.cell = cell
        a.points, a.mins, a.codes = p.data_ptr(), mins.data_ptr(), codes.data_ptr()
        a.stream = L.current_stream_ptr(p.device)
        L.check(lib.issm_hilbert_codes(C.byref(a)), "issm_hilbert_codes")
    return codes


def hilbert_order(points: torch.Tensor, orders: Sequence[str] = ("xyz",), bit: int = 9, cell: float = 1.0 / 50.0):
    """points (B, N, 3), N <= 4096 -> (index, inverse), both (len(orders), B, N) int64: index[o, b] lists the points
    of sample b along the curve of order o (equal to a stable argsort of ``hilbert_codes``), inverse[o, b] is its
    inverse permutation.  One kernel launch (libissm_hip.so: issm_hilbert_order)."""
    for o in orders:
        if o not in ORDERS:
            raise NotImplementedError(o)
    L.require_gpu(points, "points")
    lib = L.load()
    p = points.detach().float().contiguous()
    with torch.cuda.device(p.device):
        out = torch.empty(2, len(orders), p.shape[0], p.shape[1], dtype=torch.int64, device=p.device)
        a = L.HilbertOrderArgs()
        a.batch, a.npoint, a.bits, a.norder = p.shape[0], p.shape[1], bit, len(orders)
        for j, o in enumerate(orders):
            for i, v in enumerate(ORDERS[o]):
                a.order[j][i] = v
        a.cell = cell
        a.points, a.index, a.inverse = p.data_ptr(), out[0].data_ptr(), out[1].data_ptr()
        a.stream = L.current_stream_ptr(p.device)
        L.check(lib.issm_hilbert_order(C.byref(a)), "issm_hilbert_order")
    return out[0], out[1]


class Serialization(nn.Module):
    def __init__(self, order: Sequence[str] = ("xyz", "yxz"), bit: int = 9):
        super().__init__()
        self.order = list(order)
        self.bit = bit
        self.hilbert_spatial_size = 2 ** bit
        self.index_list: List[torch.Tensor] = []
        self.reversed_index_list: List[torch.Tensor] = []
        self.index = 0

    def forward(self, points, depth=None):
        """points (B, N, 3): fills ``index_list`` (per order, the indices that sort the points along the curve) and
        ``reversed_index_list`` (their inverses)   (dest_module.py:319-345)."""
        self.index_list, self.reversed_index_list = [], []
        if (points.is_cuda and 0 < points.shape[1] <= L.HILBERT_ORDER_MAX_POINTS and self.bit <= 17
                and len(self.order) <= 6):
            # minimum corner, curve positions, stable sort and inverse permutation of every order in one launch
            idx, inv = hilbert_order(points, self.order, self.bit)
            self.index_list, self.reversed_index_list = list(idx.unbind(0)), list(inv.unbind(0))
            return
        for o in self.order:
            code = hilbert_codes(points, o, self.bit)
            idx = torch.argsort(code, dim=-1, stable=True)
            self.index_list.append(idx)
            self.reversed_index_list.append(torch.argsort(idx, dim=-1))

    def encode(self, grid_coord, order="xyz"):
        """grid_coord (N, 3) integer cells -> curve positions (dest_module.py:347-362)."""
        pts = grid_coord.float().unsqueeze(0)
        zero = torch.zeros(1, 1, 3, device=pts.device)
        return hilbert_codes(torch.cat([zero, pts], dim=1), order, self.bit, cell=1.0)[0, 1:]

    @staticmethod
    def _gather(points, idx):
        return points.gather(dim=1, index=idx.unsqueeze(-1).expand(-1, -1, points.shape[-1]))

    def reorder_points(self, points, id=0):
        index = 0 if len(self.index_list) == 1 else id
        self.index = index
        return self._gather(points, self.index_list[index])

    def reversed_reorder_points(self, points):
        index = 0 if len(self.reversed_index_list) == 1 else self.index
        return self._gather(points, self.reversed_index_list[index])
