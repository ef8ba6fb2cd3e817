"""ctypes binding of libissm_hip.so (the C ABI declared in include/issm.h).

The library is the only compute path of this package: if it is missing, loading fails
loudly -- there is no PyTorch fallback.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional, Sequence

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libissm_hip.so")

ISSM_CHUNK = 64
ISSM_F32, ISSM_BF16 = 0, 1
FLAG_DT_SOFTPLUS, FLAG_D_HAS_HDIM, FLAG_SEQ_IDX = 1, 2, 4

EXPORTS = [
    "issm_abi_version", "issm_last_error", "issm_fwd_workspace_bytes", "issm_bwd_workspace_bytes",
    "issm_scan_fwd", "issm_scan_bwd", "issm_stage_chunk_local", "issm_stage_state_passing_fwd",
    "issm_stage_chunk_scan", "issm_stage_bwd_gate", "issm_stage_bwd_dstates",
    "issm_stage_state_passing_bwd", "issm_stage_bwd_chunk", "issm_bwd_chunk_redo_ints", "issm_stage_bwd_dx",
    "issm_stage_bwd_reduce",
    "issm_rmsnorm_bwd_blocks", "issm_gated_rmsnorm_fwd", "issm_gated_rmsnorm_bwd",
    "issm_gated_rmsnorm_bwd_noalloc",
    "issm_param_gen_bwd_blocks", "issm_param_gen_fwd", "issm_param_gen_bwd",
    "issm_dwconv_partial_rows", "issm_dwconv_silu_fwd", "issm_dwconv_silu_bwd",
    "issm_box_dist_bwd_scratch_bytes", "issm_box_dist_fwd", "issm_box_dist_bwd",
    "issm_hilbert_codes", "issm_hilbert_order", "issm_transpose_states",
    "issm_pn2_furthest_point_sampling", "issm_pn2_ball_query", "issm_pn2_group_points", "issm_pn2_group_points_grad",
    "issm_pn2_gather_points", "issm_pn2_gather_points_grad", "issm_pn2_three_nn", "issm_pn2_three_interpolate",
    "issm_pn2_three_interpolate_grad", "issm_pn2_group_points_grad_cl", "issm_pn2_three_interpolate_grad_cl",
]


class Dims(C.Structure):
    _fields_ = [(n, C.c_int32) for n in
                ("batch", "seqlen", "nheads", "headdim", "dstate", "ngroups", "chunk_size", "ndir")]


class Tensor(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("stride", C.c_int64 * 3)]


class ScanArgs(C.Structure):
    _fields_ = [
        ("dims", Dims),
        ("io_dtype", C.c_int32), ("dt_dtype", C.c_int32), ("h0_dtype", C.c_int32),
        ("flags", C.c_uint32),
        ("dt_min", C.c_float), ("dt_max", C.c_float),
        ("x", Tensor * 2), ("dt", Tensor), ("Bm", Tensor * 2), ("Cm", Tensor * 2), ("z", Tensor * 2),
        ("A", C.c_void_p), ("D", C.c_void_p), ("dt_bias", C.c_void_p),
        ("h0", Tensor),
        ("out", Tensor * 2),
        ("final_states", C.c_void_p * 2),
        ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t),
        ("saved", C.c_void_p),
        ("dout", Tensor * 2),
        ("dfinal", C.c_void_p * 2),
        ("dx", Tensor * 2), ("dB", Tensor * 2), ("dC", Tensor * 2), ("dz", Tensor * 2),
        ("ddt", Tensor),
        ("dA", C.c_void_p), ("dD", C.c_void_p), ("ddt_bias", C.c_void_p), ("dh0", C.c_void_p),
        ("bwd_workspace", C.c_void_p), ("bwd_workspace_bytes", C.c_size_t),
        ("stream", C.c_void_p),
        ("seq_idx", C.c_void_p), ("seq_idx_stride", C.c_int64 * 2),
    ]


class NormArgs(C.Structure):
    _fields_ = [
        ("rows", C.c_int64), ("ncols", C.c_int32), ("group_size", C.c_int32),
        ("dtype", C.c_int32), ("weight_dtype", C.c_int32), ("norm_before_gate", C.c_int32),
        ("eps", C.c_float),
        ("x", C.c_void_p), ("z", C.c_void_p), ("w", C.c_void_p),
        ("x_row_stride", C.c_int64), ("z_row_stride", C.c_int64),
        ("y", C.c_void_p), ("y_row_stride", C.c_int64),
        ("rstd", C.c_void_p),
        ("dy", C.c_void_p), ("dy_row_stride", C.c_int64),
        ("dx", C.c_void_p), ("dz", C.c_void_p),
        ("dx_row_stride", C.c_int64), ("dz_row_stride", C.c_int64),
        ("dw_partial", C.c_void_p), ("dw", C.c_void_p),
        ("stream", C.c_void_p),
        ("layer_norm", C.c_int32), ("bias", C.c_void_p), ("mean", C.c_void_p),
        ("db_partial", C.c_void_p), ("db", C.c_void_p),
    ]


class PGenArgs(C.Structure):
    _fields_ = [
        ("tokens", C.c_int64), ("K", C.c_int32), ("M", C.c_int32), ("H", C.c_int32), ("G", C.c_int32),
        ("dtype", C.c_int32), ("has_back", C.c_int32),
        ("dist", C.c_void_p), ("W", C.c_void_p), ("bias", C.c_void_p),
        ("dt", C.c_void_p), ("Bm", C.c_void_p), ("Cm", C.c_void_p), ("Bm_back", C.c_void_p), ("Cm_back", C.c_void_p),
        ("weights", C.c_void_p), ("dt_raw", C.c_void_p),
        ("ddt", C.c_void_p), ("dBm", C.c_void_p), ("dCm", C.c_void_p), ("dBm_back", C.c_void_p),
        ("dCm_back", C.c_void_p),
        ("ddist", C.c_void_p), ("dbias", C.c_void_p), ("dweights", C.c_void_p),
        ("dw_partial", C.c_void_p), ("dW", C.c_void_p),
        ("stream", C.c_void_p), ("dbias_sum", C.c_void_p),
    ]


class DwConvArgs(C.Structure):
    _fields_ = [
        ("batch", C.c_int32), ("seqlen", C.c_int32), ("channels", C.c_int32), ("nsets", C.c_int32),
        ("taps", C.c_int32), ("dtype", C.c_int32),
        ("u", C.c_void_p), ("u_batch_stride", C.c_int64), ("u_token_stride", C.c_int64),
        ("w", C.c_void_p), ("bias", C.c_void_p), ("y", C.c_void_p), ("pre", C.c_void_p),
        ("dy", C.c_void_p * 2), ("du", C.c_void_p), ("partial", C.c_void_p), ("dw", C.c_void_p),
        ("dbias", C.c_void_p), ("stream", C.c_void_p),
        ("split", C.c_int32), ("y_tail", C.c_void_p), ("dy_tail", C.c_void_p * 2),
        ("du_batch_stride", C.c_int64), ("du_token_stride", C.c_int64),
        ("chain", C.c_int32),
    ]


class BoxDistArgs(C.Structure):
    _fields_ = [
        ("batch", C.c_int32), ("seqlen", C.c_int32), ("nquery", C.c_int32),
        ("D", C.c_int32), ("H", C.c_int32), ("W", C.c_int32), ("dtype", C.c_int32),
        ("key", C.c_void_p), ("corners", C.c_void_p), ("boxes", C.c_void_p), ("min_radius", C.c_float),
        ("angle", C.c_void_p), ("table", C.c_void_p),
        ("log_scale", C.c_float), ("max_value", C.c_float),
        ("dist", C.c_void_p), ("qcenter", C.c_void_p), ("radius", C.c_void_p),
        ("weight_dist", C.c_float), ("weights", C.c_void_p),
        ("ddist", C.c_void_p), ("partial", C.c_void_p), ("dtable", C.c_void_p), ("stream", C.c_void_p),
    ]


class TransposeArgs(C.Structure):
    _fields_ = [
        ("batch", C.c_int32), ("rows", C.c_int32), ("cols", C.c_int32),
        ("in_dtype", C.c_int32), ("out_dtype", C.c_int32),
        ("in0", C.c_void_p), ("in1", C.c_void_p), ("out", C.c_void_p),
        ("alpha", C.c_float), ("stream", C.c_void_p),
    ]


class HilbertArgs(C.Structure):
    _fields_ = [
        ("batch", C.c_int32), ("npoint", C.c_int32), ("bits", C.c_int32), ("order", C.c_int32 * 3),
        ("cell", C.c_float), ("points", C.c_void_p), ("mins", C.c_void_p), ("codes", C.c_void_p),
        ("stream", C.c_void_p),
    ]


class HilbertOrderArgs(C.Structure):
    _fields_ = [
        ("batch", C.c_int32), ("npoint", C.c_int32), ("bits", C.c_int32), ("norder", C.c_int32),
        ("order", (C.c_int32 * 3) * 6), ("cell", C.c_float), ("points", C.c_void_p), ("index", C.c_void_p),
        ("inverse", C.c_void_p), ("stream", C.c_void_p),
    ]


HILBERT_ORDER_MAX_POINTS = 4096

_lib: Optional[C.CDLL] = None


def load() -> C.CDLL:
    """Load the shared library (once).  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m dest3d_amd.build` "
            "(hipcc, --offload-arch=gfx950).  This package has no fallback path.")
    lib = C.CDLL(LIB_PATH)
    lib.issm_last_error.restype = C.c_char_p
    P = C.POINTER
    lib.issm_fwd_workspace_bytes.argtypes = [P(ScanArgs), P(C.c_size_t)]
    lib.issm_bwd_workspace_bytes.argtypes = [P(ScanArgs), P(C.c_size_t)]
    lib.issm_scan_fwd.argtypes = [P(ScanArgs)]
    lib.issm_scan_bwd.argtypes = [P(ScanArgs)]
    vp = C.c_void_p
    lib.issm_stage_chunk_local.argtypes = [P(ScanArgs), vp, vp, vp]
    lib.issm_stage_state_passing_fwd.argtypes = [P(ScanArgs), vp, vp]
    lib.issm_stage_chunk_scan.argtypes = [P(ScanArgs), vp, vp, vp]
    lib.issm_stage_bwd_gate.argtypes = [P(ScanArgs), vp, vp]
    lib.issm_stage_bwd_dstates.argtypes = [P(ScanArgs), vp, vp, vp]
    lib.issm_stage_state_passing_bwd.argtypes = [P(ScanArgs), vp, vp, vp, vp, vp]
    lib.issm_stage_bwd_chunk.argtypes = [P(ScanArgs), C.c_int, vp, vp, vp, vp, vp, vp, vp, vp]
    lib.issm_bwd_chunk_redo_ints.argtypes = [P(ScanArgs)]
    lib.issm_bwd_chunk_redo_ints.restype = C.c_size_t
    lib.issm_stage_bwd_dx.argtypes = [P(ScanArgs), vp, vp, vp, vp]
    lib.issm_stage_bwd_reduce.argtypes = [P(ScanArgs), vp, vp, vp, vp]
    lib.issm_rmsnorm_bwd_blocks.argtypes = [C.c_int64]
    lib.issm_gated_rmsnorm_fwd.argtypes = [P(NormArgs)]
    lib.issm_gated_rmsnorm_bwd.argtypes = [P(NormArgs)]
    lib.issm_gated_rmsnorm_bwd_noalloc.argtypes = [P(NormArgs)]
    lib.issm_box_dist_bwd_scratch_bytes.argtypes = [C.c_int32] * 6
    lib.issm_hilbert_codes.argtypes = [P(HilbertArgs)]
    lib.issm_transpose_states.argtypes = [P(TransposeArgs)]
    lib.issm_hilbert_order.argtypes = [P(HilbertOrderArgs)]
    i32, f32 = C.c_int32, C.c_float
    lib.issm_pn2_furthest_point_sampling.argtypes = [i32, i32, i32, vp, vp, vp, vp]
    lib.issm_pn2_ball_query.argtypes = [i32, i32, i32, f32, i32, vp, vp, vp, vp]
    lib.issm_pn2_group_points.argtypes = [i32, i32, i32, i32, i32, vp, vp, vp, vp]
    lib.issm_pn2_group_points_grad.argtypes = [i32, i32, i32, i32, i32, vp, vp, vp, vp]
    lib.issm_pn2_gather_points.argtypes = [i32, i32, i32, i32, vp, vp, vp, vp]
    lib.issm_pn2_gather_points_grad.argtypes = [i32, i32, i32, i32, vp, vp, vp, vp]
    lib.issm_pn2_three_nn.argtypes = [i32, i32, i32, vp, vp, vp, vp, vp]
    lib.issm_pn2_three_interpolate.argtypes = [i32, i32, i32, i32, vp, vp, vp, vp, vp]
    lib.issm_pn2_three_interpolate_grad.argtypes = [i32, i32, i32, i32, vp, vp, vp, vp, vp]
    lib.issm_pn2_group_points_grad_cl.argtypes = [i32, i32, i32, i32, i32, vp, vp, vp, vp]
    lib.issm_pn2_three_interpolate_grad_cl.argtypes = [i32, i32, i32, i32, vp, vp, vp, vp, vp]
    lib.issm_box_dist_fwd.argtypes = [P(BoxDistArgs)]
    lib.issm_box_dist_bwd.argtypes = [P(BoxDistArgs)]
    lib.issm_dwconv_partial_rows.argtypes = [C.c_int32, C.c_int32]
    lib.issm_dwconv_silu_fwd.argtypes = [P(DwConvArgs)]
    lib.issm_dwconv_silu_bwd.argtypes = [P(DwConvArgs)]
    lib.issm_param_gen_bwd_blocks.argtypes = [C.c_int64]
    lib.issm_param_gen_fwd.argtypes = [P(PGenArgs)]
    lib.issm_param_gen_bwd.argtypes = [P(PGenArgs)]
    for name in EXPORTS:
        if name != "issm_last_error" and not name.endswith("_redo_ints"):
            getattr(lib, name).restype = C.c_int
    lib.issm_box_dist_bwd_scratch_bytes.restype = C.c_int64
    _lib = lib
    return lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        raise RuntimeError(f"{what} failed (status {rc}): {load().issm_last_error().decode()}")


def dtype_code(dt: torch.dtype) -> int:
    if dt == torch.float32:
        return ISSM_F32
    if dt == torch.bfloat16:
        return ISSM_BF16
    raise TypeError(f"unsupported dtype {dt}: the ISSM kernels take float32 or bfloat16")


def tensor_desc(t: Optional[torch.Tensor]) -> Tensor:
    """Descriptor of a 4-D tensor whose last dim is contiguous (or an absent tensor)."""
    d = Tensor()
    if t is None:
        d.ptr = None
        return d
    assert t.dim() == 4 and t.stride(-1) == 1, "innermost dimension must be contiguous"
    d.ptr = t.data_ptr()
    for i in range(3):
        d.stride[i] = t.stride(i)
    return d


def ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def current_stream_ptr(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def require_gpu(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on a HIP device: the ISSM operator has no CPU path")
