"""Builds libissm_hip.so (gfx950) in-tree with hipcc.  `python -m dest3d_amd.build`."""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libissm_hip.so")
SOURCES = ["issm_abi.hip", "issm_fwd.hip", "issm_fwd_tile.hip", "issm_bwd.hip", "issm_bwd_tile.hip", "rmsnorm_gated.hip", "param_gen.hip", "dwconv_silu.hip", "box_dist.hip", "box_dist_sorted.hip", "hilbert.hip", "pointnet2_ops.hip", "transpose_states.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffast-math", "-fno-finite-math-only",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-attributes",
]


# Sources whose results are integers decided by floating-point comparisons, compiled without -ffast-math:
#  - hilbert.hip: a floating-point quotient picks the cell; IEEE division (no reciprocal-multiply rewriting) puts a
#    point exactly on a cell boundary into the same cell as on the host;
#  - pointnet2_ops.hip: squared distances pick indices (furthest point, ball membership, three nearest).  Under
#    -ffast-math the backend fuses multiply and add whatever `#pragma clang fp contract(off)` says, and a distance one
#    unit in the last place off decides a near-tie differently from a plain fp32 evaluation.
EXACT_ARITHMETIC = {"hilbert.hip", "pointnet2_ops.hip"}


def _compile(src: str) -> str:
    obj = os.path.join(CSRC, src.replace(".hip", ".o"))
    flags = [f for f in FLAGS if f not in ("-ffast-math", "-fno-finite-math-only")] if src in EXACT_ARITHMETIC else FLAGS
    cmd = [HIPCC, *flags, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose: bool = True) -> str:
    """Compile every HIP source for gfx950 and link the shared library; returns its path."""
    with ThreadPoolExecutor(max_workers=min(4, len(SOURCES))) as ex:
        objs = list(ex.map(_compile, SOURCES))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    if verbose:
        print(f"built {LIB}")
    return LIB


if __name__ == "__main__":
    build()
