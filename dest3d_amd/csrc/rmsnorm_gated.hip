// Gated RMSNorm / LayerNorm forward and backward for gfx950: one 64-lane wavefront per row group,
// HBM-bound streaming kernels with wave-level shuffles for the row reductions.
//   norm_before_gate = 0:  y = xhat(x*silu(z)) * w + b
//   norm_before_gate = 1:  y = (xhat(x) * w + b) * silu(z)
//   xhat(v) = v * rstd,            rstd = 1/sqrt(mean(v^2) + eps)              (RMS statistics, p.ln = 0)
//   xhat(v) = (v - mean) * rstd,   rstd = 1/sqrt(mean((v - mean)^2) + eps)     (LayerNorm, p.ln = 1)
// b is optional (issm_triton/layernorm_gated.py:35-97 forward, :145-260 backward).
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
  auto gated_x = [&](int c) {
    float v = ldv(p.x, row * p.xs + c0 + c, p.dt);
    if (p.z && !p.nbg) {
      const float z = ldv(p.z, row * p.zs + c0 + c, p.dt);
      v *= z * sigmoidf_(z);
    }
    return v;
  };
  float mean = 0.0f;
  if (p.ln) {
    float sm = 0.0f;
    for (int c = lane; c < p.gs; c += 64) sm += gated_x(c);
    mean = wave_sum(sm) / (float)p.gs;
    if (lane == 0) p.mean[(long)grp * p.rows + row] = mean;
  }
  float ss = 0.0f;
  for (int c = lane; c < p.gs; c += 64) {
    const float v = gated_x(c) - mean;
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
    float y = (v - mean) * rstd * ldv(p.w, c0 + c, p.wdt);
    if (p.b) y += ldv(p.b, c0 + c, p.wdt);
    if (p.z && p.nbg) y *= gate;
    stv(p.y, row * p.ys + c0 + c, p.dt, y);
  }
}

// ---- fast paths: one group per row, ncols a multiple of 4 and at most 1024 ---------------------------------
// A lane owns vectors lane, lane + 64, ... of 4 consecutive columns; the row stays in registers between the
// reduction and the second use, loads and stores are 8 bytes (bf16) or 16 bytes (fp32) wide, and the backward keeps
// its dw partial in registers instead of read-modify-writing LDS.
// Rows may start at any element (a column slice of a wider row): the 4 elements are read through a type that only
// promises element alignment, which the compiler turns into one wide access on this target (unaligned global
// accesses are legal on gfx9 under HSA) -- one code path, no case distinction around the loads.  `al` is unused.
struct __attribute__((packed, aligned(2))) RowBf4 {
  unsigned lo, hi;
};
struct __attribute__((packed, aligned(4))) RowF4 {
  float x, y, z, w;
};
template <bool BF>
__device__ __forceinline__ f4 ld4(const void* p, long off, bool ok, int /*al*/) {
  // an absent lane reads offset 0 and the value is replaced by zero: no branch around the load, so that a thread's
  // loads stay in flight together
  f4 r;
  off = ok ? off : 0;
  if (BF) {
    const RowBf4 w = *(const RowBf4*)((const uint16_t*)p + off);
    r.x = __uint_as_float(w.lo << 16); r.y = __uint_as_float(w.lo & 0xffff0000u);
    r.z = __uint_as_float(w.hi << 16); r.w = __uint_as_float(w.hi & 0xffff0000u);
  } else {
    const RowF4 w = *(const RowF4*)((const float*)p + off);
    r = (f4){w.x, w.y, w.z, w.w};
  }
  if (!ok) r = (f4){0.0f, 0.0f, 0.0f, 0.0f};
  return r;
}
template <bool BF>
__device__ __forceinline__ void st4(void* p, long off, f4 v, int /*al*/) {
  if (BF) {
    RowBf4 w;
    w.lo = pack_bf16(v.x, v.y); w.hi = pack_bf16(v.z, v.w);
    *(RowBf4*)((uint16_t*)p + off) = w;
  } else {
    RowF4 w;
    w.x = v.x; w.y = v.y; w.z = v.z; w.w = v.w;
    *(RowF4*)((float*)p + off) = w;
  }
}
// alignment class of rows starting at q with `stride` elements between them
__device__ __forceinline__ int al_of(const void* q, long stride, bool bf) {
  const uintptr_t a = (uintptr_t)q | ((uintptr_t)(stride < 0 ? -stride : stride) * (bf ? 2 : 4));
  const uintptr_t full = bf ? 7 : 15;
  return (a & full) == 0 ? 0 : ((a & (full >> 1)) == 0 ? 1 : 2);
}
// The lane's norm weights (fp32 or bf16 by `wdt`), zero for absent vectors: one wide load each, and one branch on
// the dtype around all of them (a branch per load would make each wait for the previous one)
template <int NV>
__device__ __forceinline__ void ldw(const void* w, int lane, int nvec, int wdt, f4 (&out)[NV]) {
  if (wdt) {
#pragma unroll
    for (int v = 0; v < NV; ++v) out[v] = ld4<true>(w, 4 * (lane + 64 * v), lane + 64 * v < nvec, 0);
  } else {
#pragma unroll
    for (int v = 0; v < NV; ++v) out[v] = ld4<false>(w, 4 * (lane + 64 * v), lane + 64 * v < nvec, 0);
  }
}
__device__ __forceinline__ f4 silu4(f4 z, f4& sg) {
  f4 g;
#pragma unroll
  for (int i = 0; i < 4; ++i) { sg[i] = sigmoidf_(z[i]); g[i] = z[i] * sg[i]; }
  return g;
}

// EXT: LayerNorm statistics and / or a bias (p.ln, p.b); the plain RMS form compiles without either.
template <bool BF, int NV, bool EXT>
__global__ __launch_bounds__(NTHREADS) void k_rmsnorm_fwd_fast(NormP p) {
  const int lane = threadIdx.x & 63;
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= p.rows) return;
  const int nvec = p.ncols >> 2;
  const int ax = al_of(p.x, p.xs, BF), az = al_of(p.z, p.zs, BF), ay = al_of(p.y, p.ys, BF);
  // all loads of the row first (x, z, the weights), nothing between them: one memory round trip per row
  const void* zp = p.z ? p.z : p.x;  // without a gate the second load repeats the first and is not used
  const long zs = p.z ? p.zs : p.xs;
  f4 x[NV], gate[NV], wv[NV];
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    const int vi = lane + 64 * v;
    const bool ok = vi < nvec;
    x[v] = ld4<BF>(p.x, row * p.xs + 4 * vi, ok, ax);
    gate[v] = ld4<BF>(zp, row * zs + 4 * vi, ok, az);
  }
  ldw<NV>(p.w, lane, nvec, p.wdt, wv);
  f4 bv[EXT ? NV : 1];
  if constexpr (EXT) ldw<NV>(p.b ? p.b : p.w, lane, nvec, p.wdt, bv);  // without a bias: loaded, not used
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    if (p.z) {
      f4 sg;
      gate[v] = silu4(gate[v], sg);
      if (!p.nbg) x[v] *= gate[v];
    }
  }
  if (EXT && p.ln) {
    float sm = 0.0f;  // absent vectors were loaded as zeros
#pragma unroll
    for (int v = 0; v < NV; ++v) sm += (x[v].x + x[v].y) + (x[v].z + x[v].w);
    const float mean = wave_sum(sm) / (float)p.ncols;
    if (lane == 0) p.mean[row] = mean;
#pragma unroll
    for (int v = 0; v < NV; ++v)
      if (lane + 64 * v < nvec) x[v] -= mean;
  }
  float ss = 0.0f;
#pragma unroll
  for (int v = 0; v < NV; ++v) ss += (x[v].x * x[v].x + x[v].y * x[v].y) + (x[v].z * x[v].z + x[v].w * x[v].w);
  ss = wave_sum(ss);
  const float rstd = 1.0f / sqrtf(ss / (float)p.ncols + p.eps);
  if (lane == 0 && p.rstd) p.rstd[row] = rstd;
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    const int vi = lane + 64 * v;
    if (vi < nvec) {
      f4 y = x[v] * rstd * wv[v];
      if constexpr (EXT) { if (p.b) y += bv[v]; }
      if (p.z && p.nbg) y *= gate[v];
      st4<BF>(p.y, row * p.ys + 4 * vi, y, ay);
    }
  }
}

template <bool BF, int NV, bool EXT>
__global__ __launch_bounds__(64) void k_rmsnorm_bwd_fast(NormP p) {
  const int lane = threadIdx.x;
  const int nvec = p.ncols >> 2;
  const int ax = al_of(p.x, p.xs, BF), az = al_of(p.z, p.zs, BF), ady = al_of(p.dy, p.dys, BF);
  const int adx = al_of(p.dx, p.dxs, BF), adz = al_of(p.dz, p.dzs, BF);
  f4 w[NV], dwacc[NV], bv[EXT ? NV : 1], dbacc[EXT ? NV : 1];
#pragma unroll
  for (int v = 0; v < NV; ++v) dwacc[v] = (f4){0.0f, 0.0f, 0.0f, 0.0f};
  ldw<NV>(p.w, lane, nvec, p.wdt, w);
  if constexpr (EXT) {
    ldw<NV>(p.b ? p.b : p.w, lane, nvec, p.wdt, bv);  // without a bias: loaded, not used
#pragma unroll
    for (int v = 0; v < NV; ++v) dbacc[v] = (f4){0.0f, 0.0f, 0.0f, 0.0f};
  }
  // The loads of the next row are requested before the current row is worked on (x, dy, z and rstd back to back,
  // nothing between them), so that a row costs no memory round trip of its own.
  const void* zp = p.z ? p.z : p.x;  // without a gate the third load repeats the first and is not used
  const long zs = p.z ? p.zs : p.xs;
  f4 xn[NV], dyn[NV], zn[NV];
  float rstd_n = 0.0f, mean_n = 0.0f;
  auto fetch = [&](long row) {
    rstd_n = p.rstd[row];
    if (EXT && p.ln) mean_n = p.mean[row];
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      const int vi = lane + 64 * v;
      const bool ok = vi < nvec;
      xn[v] = ld4<BF>(p.x, row * p.xs + 4 * vi, ok, ax);
      dyn[v] = ld4<BF>(p.dy, row * p.dys + 4 * vi, ok, ady);
      zn[v] = ld4<BF>(zp, row * zs + 4 * vi, ok, az);
    }
  };
  if ((long)blockIdx.x < p.rows) fetch(blockIdx.x);
  for (long row = blockIdx.x; row < p.rows; row += p.nblocks) {
    const float rstd = rstd_n, mean = mean_n;  // mean stays 0 for RMS statistics
    f4 xo[NV], dyo[NV], z[NV], sg[NV], gate[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) { xo[v] = xn[v]; dyo[v] = dyn[v]; z[v] = zn[v]; }
    if (row + p.nblocks < p.rows) fetch(row + p.nblocks);
    // absent vectors carry dy = 0, so they add nothing to either sum although their x - mean is not zero
    float c1 = 0.0f, c2 = 0.0f;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      gate[v] = (f4){1.0f, 1.0f, 1.0f, 1.0f};
      if (p.z) gate[v] = silu4(z[v], sg[v]);
      f4 vv = (p.z && !p.nbg) ? xo[v] * gate[v] : xo[v];
      if (EXT) vv -= mean;
      const f4 d = (p.z && p.nbg) ? dyo[v] * gate[v] : dyo[v];
      const f4 wd = d * w[v];
      const f4 t = vv * rstd * wd;
      c1 += (t.x + t.y) + (t.z + t.w);
      if (EXT) c2 += (wd.x + wd.y) + (wd.z + wd.w);
    }
    c1 = wave_sum(c1) / (float)p.ncols;
    c2 = (EXT && p.ln) ? wave_sum(c2) / (float)p.ncols : 0.0f;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      const int vi = lane + 64 * v;
      if (vi < nvec) {
        f4 vv = (p.z && !p.nbg) ? xo[v] * gate[v] : xo[v];
        if (EXT) vv -= mean;
        const f4 d = (p.z && p.nbg) ? dyo[v] * gate[v] : dyo[v];
        const f4 xhat = vv * rstd;
        f4 dxv = (w[v] * d - (xhat * c1 + c2)) * rstd;
        dwacc[v] += d * xhat;
        if constexpr (EXT) dbacc[v] += d;
        if (p.z) {
          f4 dzv;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float ds = sg[v][i] * (1.0f + z[v][i] * (1.0f - sg[v][i]));  // d silu / dz
            float pre = xhat[i] * w[v][i];
            if constexpr (EXT) { if (p.b) pre += bv[v][i]; }
            dzv[i] = p.nbg ? dyo[v][i] * pre * ds : dxv[i] * xo[v][i] * ds;
          }
          if (!p.nbg) dxv *= gate[v];
          if (p.dz) st4<BF>(p.dz, row * p.dzs + 4 * vi, dzv, adz);
        }
        st4<BF>(p.dx, row * p.dxs + 4 * vi, dxv, adx);
      }
    }
  }
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    const int vi = lane + 64 * v;
    if (vi < nvec) {
      *(f4*)(p.dw_partial + (long)blockIdx.x * p.ncols + 4 * vi) = dwacc[v];
      if constexpr (EXT) { if (p.b) *(f4*)(p.db_partial + (long)blockIdx.x * p.ncols + 4 * vi) = dbacc[v]; }
    }
  }
}

static bool norm_fast_ok(const NormP& p) { return p.ngroups == 1 && (p.ncols & 3) == 0 && p.ncols <= 1024; }

// One wavefront per block; block b walks rows b, b+nblocks, ... and keeps its dw partial in LDS.
__global__ __launch_bounds__(64) void k_rmsnorm_bwd(NormP p) {
  extern __shared__ float dws[];  // dw partial (ncols), then the db partial (ncols) when there is a bias
  float* dbs = dws + p.ncols;
  const int lane = threadIdx.x;
  for (int c = lane; c < (p.b ? 2 : 1) * p.ncols; c += 64) dws[c] = 0.0f;
  for (long row = blockIdx.x; row < p.rows; row += p.nblocks) {
    for (int grp = 0; grp < p.ngroups; ++grp) {
      const int c0 = grp * p.gs;
      const float rstd = p.rstd[(long)grp * p.rows + row];
      const float mean = p.ln ? p.mean[(long)grp * p.rows + row] : 0.0f;
      float c1 = 0.0f, c2 = 0.0f;
      for (int c = lane; c < p.gs; c += 64) {
        float v = ldv(p.x, row * p.xs + c0 + c, p.dt);
        float d = ldv(p.dy, row * p.dys + c0 + c, p.dt);
        if (p.z) {
          const float z = ldv(p.z, row * p.zs + c0 + c, p.dt);
          const float gate = z * sigmoidf_(z);
          if (p.nbg) d *= gate; else v *= gate;
        }
        const float wd = d * ldv(p.w, c0 + c, p.wdt);
        c1 += (v - mean) * rstd * wd;
        c2 += wd;
      }
      c1 = wave_sum(c1) / (float)p.gs;
      c2 = p.ln ? wave_sum(c2) / (float)p.gs : 0.0f;
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
        const float v = ((p.z && !p.nbg) ? xo * gate : xo) - mean;
        const float d = (p.z && p.nbg) ? dyo * gate : dyo;
        const float xhat = v * rstd;
        float dxv = (w * d - (xhat * c1 + c2)) * rstd;
        dws[c0 + c] += d * xhat;
        if (p.b) dbs[c0 + c] += d;
        if (p.z) {
          float dzv;
          const float pre = p.b ? xhat * w + ldv(p.b, c0 + c, p.wdt) : xhat * w;
          if (p.nbg) dzv = dyo * pre * sg * (1.0f + z * (1.0f - sg));
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
  for (int c = lane; c < p.ncols; c += 64) {
    p.dw_partial[(long)blockIdx.x * p.ncols + c] = dws[c];
    if (p.b) p.db_partial[(long)blockIdx.x * p.ncols + c] = dbs[c];
  }
}

// dw[c] = sum over the per-block partials, in a fixed order: block = 8 columns x 32 row groups, row group g adds
// partials g, g+32, ... with two independent accumulators, then the 32 group sums are combined in order.
__global__ __launch_bounds__(NTHREADS) void k_rmsnorm_dw(NormP p, const float* __restrict__ partial,
                                                         float* __restrict__ out) {
  __shared__ float red[NTHREADS];
  const int c = blockIdx.x * 8 + (threadIdx.x & 7), g = threadIdx.x >> 3;
  float a0 = 0.0f, a1 = 0.0f;
  if (c < p.ncols) {
    int b = g;
    for (; b + 32 < p.nblocks; b += 64) {
      a0 += partial[(long)b * p.ncols + c];
      a1 += partial[(long)(b + 32) * p.ncols + c];
    }
    if (b < p.nblocks) a0 += partial[(long)b * p.ncols + c];
  }
  red[threadIdx.x] = a0 + a1;
  __syncthreads();
  if (g == 0 && c < p.ncols) {
    float t = 0.0f;
#pragma unroll
    for (int k = 0; k < 32; ++k) t += red[k * 8 + (threadIdx.x & 7)];
    out[c] = t;
  }
}

#define NORM_FAST_NV(KERNEL, GRID, BLOCK, BF_, EXT_)                                              \
  do {                                                                                           \
    const int nv = (p.ncols / 4 + 63) / 64;                                                      \
    if (nv <= 1) hipLaunchKernelGGL((KERNEL<BF_, 1, EXT_>), GRID, BLOCK, 0, st, p);              \
    else if (nv == 2) hipLaunchKernelGGL((KERNEL<BF_, 2, EXT_>), GRID, BLOCK, 0, st, p);         \
    else hipLaunchKernelGGL((KERNEL<BF_, 4, EXT_>), GRID, BLOCK, 0, st, p);                      \
  } while (0)
#define NORM_FAST(KERNEL, GRID, BLOCK)                                                            \
  do {                                                                                           \
    const bool ext = p.ln || p.b;                                                                \
    if (p.dt) {                                                                                  \
      if (ext) NORM_FAST_NV(KERNEL, GRID, BLOCK, true, true);                                    \
      else NORM_FAST_NV(KERNEL, GRID, BLOCK, true, false);                                       \
    } else {                                                                                     \
      if (ext) NORM_FAST_NV(KERNEL, GRID, BLOCK, false, true);                                   \
      else NORM_FAST_NV(KERNEL, GRID, BLOCK, false, false);                                      \
    }                                                                                            \
  } while (0)

int launch_rmsnorm_fwd(const NormP& p, hipStream_t st) {
  if (norm_fast_ok(p)) {
    NORM_FAST(k_rmsnorm_fwd_fast, dim3((unsigned)((p.rows + 3) / 4)), dim3(NTHREADS));
    return (int)hipGetLastError();
  }
  const long items = p.rows * p.ngroups;
  hipLaunchKernelGGL(k_rmsnorm_fwd, dim3((unsigned)((items + 3) / 4)), dim3(NTHREADS), 0, st, p);
  return (int)hipGetLastError();
}

int launch_rmsnorm_bwd(const NormP& p, hipStream_t st) {
  if (norm_fast_ok(p)) NORM_FAST(k_rmsnorm_bwd_fast, dim3(p.nblocks), dim3(64));
  else hipLaunchKernelGGL(k_rmsnorm_bwd, dim3(p.nblocks), dim3(64), (size_t)(p.b ? 2 : 1) * p.ncols * sizeof(float), st, p);
  int e = (int)hipGetLastError();
  if (e) return e;
  hipLaunchKernelGGL(k_rmsnorm_dw, dim3((p.ncols + 7) / 8), dim3(NTHREADS), 0, st, p, p.dw_partial, p.dw);
  if (p.b) hipLaunchKernelGGL(k_rmsnorm_dw, dim3((p.ncols + 7) / 8), dim3(NTHREADS), 0, st, p, p.db_partial, p.db);
  return (int)hipGetLastError();
}

}  // namespace issm
