// Gated RMSNorm forward / backward for gfx950: one 64-lane wavefront per row group,
// HBM-bound streaming kernels with wave-level shuffles for the row reductions.
//   norm_before_gate = 0:  y = (x*silu(z)) * rstd * w,   rstd = 1/sqrt(mean((x*silu z)^2) + eps)
//   norm_before_gate = 1:  y = x * rstd * w * silu(z)
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "issm_dev.h"

namespace issm {


__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

__global__ __launch_bounds__(NTHREADS) void k_rmsnorm_fwd(NormP p) {
  const int lane = threadIdx.x & 63;
  const long item = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= p.rows * p.ngroups) return;
  const long row = item / p.ngroups;
  const int grp = item % p.ngroups;
  const int c0 = grp * p.gs;
  float ss = 0.0f;
  for (int c = lane; c < p.gs; c += 64) {
    float v = ldv(p.x, row * p.xs + c0 + c, p.dt);
    if (p.z && !p.nbg) {
      const float z = ldv(p.z, row * p.zs + c0 + c, p.dt);
      v *= z * sigmoidf_(z);
    }
    ss += v * v;
  }
  ss = wave_sum(ss);
  const float rstd = 1.0f / sqrtf(ss / (float)p.gs + p.eps);
  if (lane == 0 && p.rstd) p.rstd[(long)grp * p.rows + row] = rstd;
  for (int c = lane; c < p.gs; c += 64) {
    float v = ldv(p.x, row * p.xs + c0 + c, p.dt);
    float gate = 1.0f;
    if (p.z) {
      const float z = ldv(p.z, row * p.zs + c0 + c, p.dt);
      gate = z * sigmoidf_(z);
    }
    if (p.z && !p.nbg) v *= gate;
    float y = v * rstd * ldv(p.w, c0 + c, p.wdt);
    if (p.z && p.nbg) y *= gate;
    stv(p.y, row * p.ys + c0 + c, p.dt, y);
  }
}

// One wavefront per block; block b walks rows b, b+nblocks, ... and keeps its dw partial in LDS.
__global__ __launch_bounds__(64) void k_rmsnorm_bwd(NormP p) {
  extern __shared__ float dws[];
  const int lane = threadIdx.x;
  for (int c = lane; c < p.ncols; c += 64) dws[c] = 0.0f;
  for (long row = blockIdx.x; row < p.rows; row += p.nblocks) {
    for (int grp = 0; grp < p.ngroups; ++grp) {
      const int c0 = grp * p.gs;
      const float rstd = p.rstd[(long)grp * p.rows + row];
      float c1 = 0.0f;
      for (int c = lane; c < p.gs; c += 64) {
        float v = ldv(p.x, row * p.xs + c0 + c, p.dt);
        float d = ldv(p.dy, row * p.dys + c0 + c, p.dt);
        if (p.z) {
          const float z = ldv(p.z, row * p.zs + c0 + c, p.dt);
          const float gate = z * sigmoidf_(z);
          if (p.nbg) d *= gate; else v *= gate;
        }
        c1 += v * rstd * d * ldv(p.w, c0 + c, p.wdt);
      }
      c1 = wave_sum(c1) / (float)p.gs;
      for (int c = lane; c < p.gs; c += 64) {
        const float xo = ldv(p.x, row * p.xs + c0 + c, p.dt);
        const float dyo = ldv(p.dy, row * p.dys + c0 + c, p.dt);
        const float w = ldv(p.w, c0 + c, p.wdt);
        float z = 0.0f, sg = 0.0f, gate = 1.0f;
        if (p.z) {
          z = ldv(p.z, row * p.zs + c0 + c, p.dt);
          sg = sigmoidf_(z);
          gate = z * sg;
        }
        const float v = (p.z && !p.nbg) ? xo * gate : xo;
        const float d = (p.z && p.nbg) ? dyo * gate : dyo;
        const float xhat = v * rstd;
        float dxv = (w * d - xhat * c1) * rstd;
        dws[c0 + c] += d * xhat;
        if (p.z) {
          float dzv;
          if (p.nbg) dzv = dyo * (xhat * w) * sg * (1.0f + z * (1.0f - sg));
          else {
            dzv = dxv * xo * sg * (1.0f + z * (1.0f - sg));
            dxv *= gate;
          }
          if (p.dz) stv(p.dz, row * p.dzs + c0 + c, p.dt, dzv);
        }
        stv(p.dx, row * p.dxs + c0 + c, p.dt, dxv);
      }
    }
  }
  for (int c = lane; c < p.ncols; c += 64) p.dw_partial[(long)blockIdx.x * p.ncols + c] = dws[c];
}

// dw[c] = sum over the per-block partials, in a fixed order: block = 32 columns x 8 row groups, row group g
// adds partials g, g+8, ... with four independent accumulators, then the 8 group sums are combined in order.
__global__ __launch_bounds__(NTHREADS) void k_rmsnorm_dw(NormP p) {
  __shared__ float red[NTHREADS];
  const int c = blockIdx.x * 32 + (threadIdx.x & 31), g = threadIdx.x >> 5;
  float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
  if (c < p.ncols) {
    int b = g;
    for (; b + 24 < p.nblocks; b += 32) {
      a0 += p.dw_partial[(long)b * p.ncols + c];
      a1 += p.dw_partial[(long)(b + 8) * p.ncols + c];
      a2 += p.dw_partial[(long)(b + 16) * p.ncols + c];
      a3 += p.dw_partial[(long)(b + 24) * p.ncols + c];
    }
    for (; b < p.nblocks; b += 8) a0 += p.dw_partial[(long)b * p.ncols + c];
  }
  red[threadIdx.x] = (a0 + a1) + (a2 + a3);
  __syncthreads();
  if (g == 0 && c < p.ncols) {
    float t = 0.0f;
#pragma unroll
    for (int k = 0; k < 8; ++k) t += red[k * 32 + (threadIdx.x & 31)];
    p.dw[c] = t;
  }
}

int launch_rmsnorm_fwd(const NormP& p, hipStream_t st) {
  const long items = p.rows * p.ngroups;
  hipLaunchKernelGGL(k_rmsnorm_fwd, dim3((unsigned)((items + 3) / 4)), dim3(NTHREADS), 0, st, p);
  return (int)hipGetLastError();
}

int launch_rmsnorm_bwd(const NormP& p, hipStream_t st) {
  hipLaunchKernelGGL(k_rmsnorm_bwd, dim3(p.nblocks), dim3(64), (size_t)p.ncols * sizeof(float), st, p);
  int e = (int)hipGetLastError();
  if (e) return e;
  hipLaunchKernelGGL(k_rmsnorm_dw, dim3((p.ncols + 31) / 32), dim3(NTHREADS), 0, st, p);
  return (int)hipGetLastError();
}

}  // namespace issm
