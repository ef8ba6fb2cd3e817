// Point-set operators of the PointNet++ backbone for gfx950: furthest point sampling, ball query, grouping,
// gathering, 3-nearest-neighbour search and interpolation (the functions of the reference's `pointnet2._ext`,
// pointnet2/_ext_src/src/*.cpp).  Index arithmetic is exact; all tensors fp32 / int32, contiguous.
//
//  * furthest point sampling: one 512-thread workgroup per sample; a thread owns points tid, tid + 512, ... and keeps
//    their coordinates and running minimum distance in registers (up to 24576 points; beyond that coordinates are
//    re-read and distances kept in the caller's `temp`); per sample drawn: one pass over the thread's points, an
//    argmax over the wave with shuffles, over the 8 waves through LDS.  Ties go to the smaller index.
//  * ball query: one wave per query centre; 64 points are tested per step and compacted in index order with a
//    ballot, so the first `nsample` hits are found without a serial scan; the wave stops as soon as it has them.
//  * 3-NN: one thread per unknown point, known points staged through LDS 256 at a time.
//  * group / gather / interpolate: one thread per output element, innermost index fastest; the gradients scatter
//    with hardware float atomics (duplicates in idx are the rule), as the reference does -- either straight into
//    the (b, c, n) layout, one scattered cache line per lane, or (the *_cl entry points) into a channel-last
//    (b, n, c) buffer through an LDS transpose, 64 consecutive floats per instruction.
#include "issm_dev.h"

namespace issm {

constexpr int FPS_T = 512;    // threads of the sampling workgroup (two waves per SIMD: 256 registers each)

// Squared distance in plain fp32 steps (three subtractions, three products, two additions, each rounded): no fused
// multiply-add and no reordering, so the comparisons that pick indices agree with a straightforward fp32 evaluation.
__device__ __forceinline__ float sqdist(float ax, float ay, float az, float bx, float by, float bz) {
#pragma clang fp contract(off) reassociate(off)
  const float dx = ax - bx, dy = ay - by, dz = az - bz;
  const float xx = dx * dx, yy = dy * dy, zz = dz * dz;
  return (xx + yy) + zz;
}

struct ArgMax {
  float v;
  int i;
};
__device__ __forceinline__ ArgMax better(ArgMax a, ArgMax b) {  // larger value, then smaller index
  return (b.v > a.v || (b.v == a.v && b.i < a.i)) ? b : a;
}

// idxs[b][0] = 0; then repeatedly the point farthest from the chosen set.  Points with |p|^2 <= 1e-3 (padding at the
// origin) are never chosen and keep their distance, as in the reference (sampling_gpu.cu:105-106).
// PPT > 0: the thread's PPT points -- coordinates and running distance -- live in registers for the whole kernel
// (n <= 512 * PPT); PPT == 0: any n, coordinates re-read from memory (L2) and distances kept in `temp`.
template <int PPT>
__global__ __launch_bounds__(FPS_T) void k_fps(int n, int npoint, const float* __restrict__ xyz, float* __restrict__ temp,
                                                int* __restrict__ idxs) {
  __shared__ float sv[FPS_T / 64];
  __shared__ int si[FPS_T / 64];
  __shared__ int chosen;
  const int b = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const float* p = xyz + (long)b * n * 3;
  int* out = idxs + (long)b * npoint;
  constexpr int R = PPT > 0 ? PPT : 1;
  float px[R], py[R], pz[R], dreg[R];
  float* tmp = nullptr;
  if (PPT > 0) {
#pragma unroll
    for (int j = 0; j < R; ++j) {
      const int k = tid + j * FPS_T;
      px[j] = py[j] = pz[j] = 0.0f;  // a slot past n looks like a padding point: skipped
      if (k < n) { px[j] = p[k * 3]; py[j] = p[k * 3 + 1]; pz[j] = p[k * 3 + 2]; }
      // padding points get a distance that never wins; the others start at 1e10
      dreg[j] = sqdist(px[j], py[j], pz[j], 0.0f, 0.0f, 0.0f) > 1e-3f ? 1e10f : -2.0f;
    }
  } else {
    tmp = temp + (long)b * n;
    for (int k = tid; k < n; k += FPS_T) tmp[k] = 1e10f;
  }
  if (tid == 0) out[0] = 0;
  int old = 0;
  for (int s = 1; s < npoint; ++s) {
    const float ox = p[old * 3], oy = p[old * 3 + 1], oz = p[old * 3 + 2];
    float bv = -1.0f;
    int bi = 0;
    if (PPT > 0) {
#pragma unroll
      for (int j = 0; j < R; ++j) {
        const float d = fminf(dreg[j], sqdist(px[j], py[j], pz[j], ox, oy, oz));
        dreg[j] = d;
        if (d > bv) { bv = d; bi = tid + j * FPS_T; }  // indices ascend with j: the first maximum stays
      }
    } else {
      for (int k = tid; k < n; k += FPS_T) {
        const float x = p[k * 3], y = p[k * 3 + 1], z = p[k * 3 + 2];
        if (sqdist(x, y, z, 0.0f, 0.0f, 0.0f) > 1e-3f) {
          const float d = fminf(tmp[k], sqdist(x, y, z, ox, oy, oz));
          tmp[k] = d;
          if (d > bv) { bv = d; bi = k; }
        }
      }
    }
    ArgMax best = {bv, bi};
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      ArgMax other = {__shfl_xor(best.v, o, 64), __shfl_xor(best.i, o, 64)};
      best = better(best, other);
    }
    if (lane == 0) { sv[wave] = best.v; si[wave] = best.i; }
    __syncthreads();
    if (tid == 0) {
      ArgMax a = {sv[0], si[0]};
      for (int w = 1; w < FPS_T / 64; ++w) a = better(a, ArgMax{sv[w], si[w]});
      chosen = a.v > -1.0f ? a.i : 0;  // nothing but padding points: index 0, as the reference
      out[s] = chosen;
    }
    __syncthreads();
    old = chosen;
  }
}

// idx[b][j][0..nsample): the first nsample points (in index order) closer than radius to new_xyz[b][j]; missing
// slots repeat the first hit; no hit at all leaves zeros (ball_query_gpu.cu:20-44).
__global__ __launch_bounds__(NTHREADS) void k_ball_query(int n, int m, float radius2, int nsample,
                                                         const float* __restrict__ new_xyz, const float* __restrict__ xyz,
                                                         int* __restrict__ idx) {
  const int b = blockIdx.y, lane = threadIdx.x & 63;
  const int j = blockIdx.x * (NTHREADS / 64) + (threadIdx.x >> 6);
  if (j >= m) return;  // whole wave
  const float* q = new_xyz + ((long)b * m + j) * 3;
  const float qx = q[0], qy = q[1], qz = q[2];
  const float* p = xyz + (long)b * n * 3;
  int* out = idx + ((long)b * m + j) * nsample;
  int cnt = 0, first = 0;
  for (int k0 = 0; k0 < n && cnt < nsample; k0 += 64) {
    const int k = k0 + lane;
    bool hit = false;
    if (k < n) {
      hit = sqdist(qx, qy, qz, p[k * 3], p[k * 3 + 1], p[k * 3 + 2]) < radius2;
    }
    const unsigned long long mask = __ballot(hit);
    if (mask == 0) continue;
    if (cnt == 0) first = k0 + __builtin_ctzll(mask);
    const int slot = cnt + __popcll(mask & ((1ull << lane) - 1ull));
    if (hit && slot < nsample) out[slot] = k;
    cnt += __popcll(mask);
  }
  if (cnt > nsample) cnt = nsample;
  for (int s = cnt + lane; s < nsample; s += 64) out[s] = first;  // first == 0 when nothing was found
}

// out[b][c][j][s] = points[b][c][idx[b][j][s]]   (one thread per output element)
__global__ __launch_bounds__(NTHREADS) void k_group_points(long total, int c, int n, int ms, const float* __restrict__ points,
                                                           const int* __restrict__ idx, float* __restrict__ out) {
  const long e = (long)blockIdx.x * NTHREADS + threadIdx.x;
  if (e >= total) return;
  const int r = (int)(e % ms);
  const long bc = e / ms;
  const int b = (int)(bc / c);
  const int k = min(max(idx[(long)b * ms + r], 0), n - 1);  // a stray index must not leave the tensor
  out[e] = points[bc * n + k];
}
__global__ __launch_bounds__(NTHREADS) void k_group_points_grad(long total, int c, int n, int ms,
                                                                const float* __restrict__ grad_out,
                                                                const int* __restrict__ idx, float* __restrict__ grad_points) {
  const long e = (long)blockIdx.x * NTHREADS + threadIdx.x;
  if (e >= total) return;
  const int r = (int)(e % ms);
  const long bc = e / ms;
  const int b = (int)(bc / c);
  const int k = min(max(idx[(long)b * ms + r], 0), n - 1);
  unsafeAtomicAdd(grad_points + bc * n + k, grad_out[e]);
}

// 3 nearest known points of every unknown point: squared distances ascending, ties to the smaller index
__global__ __launch_bounds__(NTHREADS) void k_three_nn(int n, int m, const float* __restrict__ unknown,
                                                       const float* __restrict__ known, float* __restrict__ dist2,
                                                       int* __restrict__ idx) {
  __shared__ float kx[NTHREADS], ky[NTHREADS], kz[NTHREADS];
  const int b = blockIdx.y;
  const int j = blockIdx.x * NTHREADS + threadIdx.x;
  const bool live = j < n;
  float ux = 0.0f, uy = 0.0f, uz = 0.0f;
  if (live) {
    const float* u = unknown + ((long)b * n + j) * 3;
    ux = u[0]; uy = u[1]; uz = u[2];
  }
  float b1 = __builtin_huge_valf(), b2 = b1, b3 = b1;  // fewer than 3 known points leave +inf (the reference's 1e40)
  int i1 = 0, i2 = 0, i3 = 0;
  const float* kp = known + (long)b * m * 3;
  for (int k0 = 0; k0 < m; k0 += NTHREADS) {
    const int kk = k0 + threadIdx.x;
    if (kk < m) { kx[threadIdx.x] = kp[kk * 3]; ky[threadIdx.x] = kp[kk * 3 + 1]; kz[threadIdx.x] = kp[kk * 3 + 2]; }
    __syncthreads();
    const int lim = min(NTHREADS, m - k0);
    for (int t = 0; t < lim; ++t) {
      const float d = sqdist(ux, uy, uz, kx[t], ky[t], kz[t]);
      const int k = k0 + t;
      if (d < b1) { b3 = b2; i3 = i2; b2 = b1; i2 = i1; b1 = d; i1 = k; }
      else if (d < b2) { b3 = b2; i3 = i2; b2 = d; i2 = k; }
      else if (d < b3) { b3 = d; i3 = k; }
    }
    __syncthreads();
  }
  if (live) {
    float* dd = dist2 + ((long)b * n + j) * 3;
    int* ii = idx + ((long)b * n + j) * 3;
    dd[0] = b1; dd[1] = b2; dd[2] = b3;
    ii[0] = i1; ii[1] = i2; ii[2] = i3;
  }
}

// out[b][c][j] = sum_k weight[b][j][k] * points[b][c][idx[b][j][k]]
__global__ __launch_bounds__(NTHREADS) void k_three_interpolate(long total, int c, int m, int n, const float* __restrict__ points,
                                                                const int* __restrict__ idx, const float* __restrict__ weight,
                                                                float* __restrict__ out) {
  const long e = (long)blockIdx.x * NTHREADS + threadIdx.x;
  if (e >= total) return;
  const int j = (int)(e % n);
  const long bc = e / n;
  const int b = (int)(bc / c);
  const long o = ((long)b * n + j) * 3;
  const float* src = points + bc * m;
  float acc = 0.0f;
#pragma unroll
  for (int k = 0; k < 3; ++k) acc += weight[o + k] * src[min(max(idx[o + k], 0), m - 1)];
  out[e] = acc;
}
__global__ __launch_bounds__(NTHREADS) void k_three_interpolate_grad(long total, int c, int n, int m,
                                                                     const float* __restrict__ grad_out,
                                                                     const int* __restrict__ idx,
                                                                     const float* __restrict__ weight,
                                                                     float* __restrict__ grad_points) {
  const long e = (long)blockIdx.x * NTHREADS + threadIdx.x;
  if (e >= total) return;
  const int j = (int)(e % n);
  const long bc = e / n;
  const int b = (int)(bc / c);
  const long o = ((long)b * n + j) * 3;
  float* dst = grad_points + bc * m;
  const float g = grad_out[e];
#pragma unroll
  for (int k = 0; k < 3; ++k) unsafeAtomicAdd(dst + min(max(idx[o + k], 0), m - 1), g * weight[o + k]);
}

// Gradients into a channel-last buffer, out_cl (b, n, c) += ...: a 64 x 64 tile of grad_out (channels x entries) is
// read along the entries (coalesced), turned in LDS, and added with lanes running over channels, so one atomic
// instruction covers 64 consecutive floats of one point instead of 64 scattered cache lines.
// K3 == false: grouping, entries e = (j, s) with index idx[b][e], value grad_out[b][ch][e];
// K3 == true: interpolation, entries j with three indices and weights each, value grad_out[b][ch][j] * weight[b][j][k].
template <bool K3>
__global__ __launch_bounds__(NTHREADS) void k_scatter_channel_last(int c, int n, int ne, const float* __restrict__ grad_out,
                                                                   const int* __restrict__ idx, const float* __restrict__ weight,
                                                                   float* __restrict__ out_cl) {
  __shared__ float tile[64][65];
  const int b = blockIdx.z, c0 = blockIdx.y * 64, e0 = blockIdx.x * 64;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int r = wave; r < 64; r += NTHREADS / 64) {
    const int ch = c0 + r, e = e0 + lane;
    tile[r][lane] = (ch < c && e < ne) ? grad_out[((long)b * c + ch) * ne + e] : 0.0f;
  }
  __syncthreads();
  const int ch = c0 + lane;
  for (int r = wave; r < 64; r += NTHREADS / 64) {
    const int e = e0 + r;
    if (e >= ne) break;  // wave-uniform
    const float g = tile[lane][r];
    if (K3) {
#pragma unroll
      for (int k = 0; k < 3; ++k) {
        const long o = ((long)b * ne + e) * 3 + k;
        const int p = min(max(idx[o], 0), n - 1);
        if (ch < c) unsafeAtomicAdd(out_cl + ((long)b * n + p) * c + ch, g * weight[o]);
      }
    } else {
      const int p = min(max(idx[(long)b * ne + e], 0), n - 1);
      if (ch < c) unsafeAtomicAdd(out_cl + ((long)b * n + p) * c + ch, g);
    }
  }
}

int launch_scatter_channel_last(bool k3, int b, int c, int n, int ne, const float* grad_out, const int* idx,
                                const float* weight, float* out_cl, hipStream_t st) {
  const dim3 g((ne + 63) / 64, (c + 63) / 64, b), t(NTHREADS);
  if (k3) hipLaunchKernelGGL(k_scatter_channel_last<true>, g, t, 0, st, c, n, ne, grad_out, idx, weight, out_cl);
  else hipLaunchKernelGGL(k_scatter_channel_last<false>, g, t, 0, st, c, n, ne, grad_out, idx, weight, out_cl);
  return (int)hipGetLastError();
}

static unsigned blocks_for(long total) { return (unsigned)((total + NTHREADS - 1) / NTHREADS); }

int launch_fps(int b, int n, int npoint, const float* xyz, float* temp, int* idxs, hipStream_t st) {
  const dim3 g(b), t(FPS_T);
  if (n <= FPS_T * 4) hipLaunchKernelGGL(k_fps<4>, g, t, 0, st, n, npoint, xyz, temp, idxs);
  else if (n <= FPS_T * 8) hipLaunchKernelGGL(k_fps<8>, g, t, 0, st, n, npoint, xyz, temp, idxs);
  else if (n <= FPS_T * 16) hipLaunchKernelGGL(k_fps<16>, g, t, 0, st, n, npoint, xyz, temp, idxs);
  else if (n <= FPS_T * 24) hipLaunchKernelGGL(k_fps<24>, g, t, 0, st, n, npoint, xyz, temp, idxs);
  else if (n <= FPS_T * 32) hipLaunchKernelGGL(k_fps<32>, g, t, 0, st, n, npoint, xyz, temp, idxs);
  else if (n <= FPS_T * 40) hipLaunchKernelGGL(k_fps<40>, g, t, 0, st, n, npoint, xyz, temp, idxs);
  else if (n <= FPS_T * 48) hipLaunchKernelGGL(k_fps<48>, g, t, 0, st, n, npoint, xyz, temp, idxs);
  else hipLaunchKernelGGL(k_fps<0>, g, t, 0, st, n, npoint, xyz, temp, idxs);
  return (int)hipGetLastError();
}
int launch_ball_query(int b, int n, int m, float radius, int nsample, const float* new_xyz, const float* xyz, int* idx,
                      hipStream_t st) {
  hipLaunchKernelGGL(k_ball_query, dim3((m + 3) / 4, b), dim3(NTHREADS), 0, st, n, m, radius * radius, nsample, new_xyz, xyz,
                     idx);
  return (int)hipGetLastError();
}
int launch_group_points(int b, int c, int n, int ms, const float* points, const int* idx, float* out, hipStream_t st) {
  const long total = (long)b * c * ms;
  hipLaunchKernelGGL(k_group_points, dim3(blocks_for(total)), dim3(NTHREADS), 0, st, total, c, n, ms, points, idx, out);
  return (int)hipGetLastError();
}
int launch_group_points_grad(int b, int c, int n, int ms, const float* grad_out, const int* idx, float* grad_points,
                             hipStream_t st) {
  const long total = (long)b * c * ms;
  hipLaunchKernelGGL(k_group_points_grad, dim3(blocks_for(total)), dim3(NTHREADS), 0, st, total, c, n, ms, grad_out, idx,
                     grad_points);
  return (int)hipGetLastError();
}
int launch_three_nn(int b, int n, int m, const float* unknown, const float* known, float* dist2, int* idx, hipStream_t st) {
  hipLaunchKernelGGL(k_three_nn, dim3((n + NTHREADS - 1) / NTHREADS, b), dim3(NTHREADS), 0, st, n, m, unknown, known, dist2,
                     idx);
  return (int)hipGetLastError();
}
int launch_three_interpolate(int b, int c, int m, int n, const float* points, const int* idx, const float* weight, float* out,
                             hipStream_t st) {
  const long total = (long)b * c * n;
  hipLaunchKernelGGL(k_three_interpolate, dim3(blocks_for(total)), dim3(NTHREADS), 0, st, total, c, m, n, points, idx, weight,
                     out);
  return (int)hipGetLastError();
}
int launch_three_interpolate_grad(int b, int c, int n, int m, const float* grad_out, const int* idx, const float* weight,
                                  float* grad_points, hipStream_t st) {
  const long total = (long)b * c * n;
  hipLaunchKernelGGL(k_three_interpolate_grad, dim3(blocks_for(total)), dim3(NTHREADS), 0, st, total, c, n, m, grad_out, idx,
                     weight, grad_points);
  return (int)hipGetLastError();
}

}  // namespace issm
