// Box-to-point distance encoding and locality weight: the two (B, L, K) fields DEST computes right before the scan
// (gfx950).
//
// BoxDistFun.forward (models/dest_module.py:174-195): for every (key point l, query box k) and each of the box's 8
// corners, delta = corner - key, rotated in the x-y plane by the query angle, compressed by a signed log
// (sign(v) log2(|v| s + 1) / log2 8 / max_value), and used as the sampling position of a trilinear grid_sample
// (padding zeros, align_corners False) into a small learned table (C = 16 channels over D x H x W = 10^3 nodes); the
// 8 samples are summed into dist[b][l][k][0..15].  local_weight (dest_module.py:240-249):
// w[b][l][k] = exp(weight_dist * min(radius_k - |key_l - centre_k|, 0)).
// As tensor ops this materialises (B, 8K, L, 3) deltas several times and gathers 8 * 8 * 16 table entries per (l, k)
// from global memory.  Here the table (node-major: 16 channels of a node contiguous) lives in LDS, a wave owns one
// box (corners in scalar registers) and walks the key points with one (l, k) pair per lane, and the output row (16
// values) leaves as one contiguous store; no intermediate exists.  The backward is the table gradient only (corners are detached in the
// reference, key positions and angles are inputs): the same walk, scattering weight * ddist into an LDS copy of the
// table, then a sum of the per-workgroup copies.  The LDS copy is 64-bit fixed point (terms scaled by
// 2^34 / max|ddist|, found by a first pass): LDS integer atomics run about twice as fast as ds_add_f32 here, and
// integer sums do not depend on the order of the adds, so the gradient is reproducible bit for bit.
#include "box_dist_dev.h"

namespace issm {

// Locality weights: thread = (l, k) pair, k along the lanes (coalesced stores).
__global__ __launch_bounds__(NTHREADS) void k_box_dist_weights(BoxDistP p) {
  const Items it = my_items(p);
  float qx = 0.0f, qy = 0.0f, qz = 0.0f, radius = 0.0f;
  long cur = -1;
  for (long item = it.i0; item < it.i1; ++item) {
    const int l = (int)(item % p.L);
    const long bk = item / p.L;
    const int b = (int)(bk / it.kchunks), k = (int)(bk % it.kchunks) * NTHREADS + threadIdx.x;
    if (k >= p.K) continue;
    if (bk != cur) {
      if (p.qcenter) {
        const float* q = p.qcenter + ((long)b * p.K + k) * 3;
        qx = q[0]; qy = q[1]; qz = q[2];
        radius = p.radius[(long)b * p.K + k];
      } else {  // from the box: centre, radius = max(|size|, min_radius)
        const float* q = p.boxes + ((long)b * p.K + k) * 7;
        qx = q[0]; qy = q[1]; qz = q[2];
        radius = fmaxf(sqrtf(q[3] * q[3] + q[4] * q[4] + q[5] * q[5]), p.min_radius);
      }
      cur = bk;
    }
    const float* key = p.key + ((long)b * p.L + l) * 3;  // uniform
    const float ex = key[0] - qx, ey = key[1] - qy, ez = key[2] - qz;
    const float d = sqrtf(ex * ex + ey * ey + ez * ez);
    p.weights[((long)b * p.L + l) * p.K + k] = __expf(p.weight_dist * fminf(radius - d, 0.0f));
  }
}

template <bool BF>
__device__ __forceinline__ void store_dist(const BoxDistP& p, long o, const f4 (&acc)[4]) {
  if (BF) {
    uint4* dst = (uint4*)((uint16_t*)p.dist + o * BD_C);
    dst[0] = make_uint4(pack_bf16(acc[0].x, acc[0].y), pack_bf16(acc[0].z, acc[0].w), pack_bf16(acc[1].x, acc[1].y),
                        pack_bf16(acc[1].z, acc[1].w));
    dst[1] = make_uint4(pack_bf16(acc[2].x, acc[2].y), pack_bf16(acc[2].z, acc[2].w), pack_bf16(acc[3].x, acc[3].y),
                        pack_bf16(acc[3].z, acc[3].w));
  } else {
    f4* dst = (f4*)((float*)p.dist + o * BD_C);
#pragma unroll
    for (int j = 0; j < 4; ++j) dst[j] = acc[j];
  }
}

__device__ __forceinline__ float wave_uniform(float v) {
  return __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(v)));
}

// dist: a wave owns one box (its corners and rotations in scalar registers) and BD_SEG key points, a lane one point
// at a time.  Pairs whose corners share a 3 x 3 x 3 window take the short path at once; the others (a box next to
// or around the point: about four in ten at detector scales) are queued in LDS and then walked corner by corner in
// full waves -- done in place, the long path would run for every wave with most lanes idle, and cost more than the
// rest together.  The eight waves of a workgroup own adjacent boxes, so a point's eight rows are neighbours in memory.
// The table lies node-major in LDS with 20 floats from node to node: a lane reads its node's 16 channels as four
// 16-byte pieces, and with 16 floats per node the lanes of one read would meet in the 16 banks that (node mod 4)
// selects; 20 n mod 64 runs through all sixteen 4-bank groups as n does.
constexpr int BD_SEG = 1024;   // points per wave
constexpr int BD_FWD_T = 512;  // 8 waves = 8 adjacent boxes per workgroup, one workgroup (96 KB of LDS) per CU
constexpr int BD_NS = 20;      // floats from node to node
template <bool BF>
__global__ __launch_bounds__(BD_FWD_T) void k_box_dist_fwd(BoxDistP p) {
  __shared__ __attribute__((aligned(16))) float tab[BD_MAXCELLS * BD_NS];
  __shared__ unsigned short queue[BD_FWD_T / 64][BD_SEG];
  const int cells = p.D * p.H * p.W;
  for (int e = threadIdx.x; e < cells * BD_C; e += BD_FWD_T) {
    const int ch = e / cells, cell = e - ch * cells;
    tab[cell * BD_NS + ch] = p.table[e];
  }
  __syncthreads();
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int kgroups = (p.K + 7) / 8, nseg = (p.L + BD_SEG - 1) / BD_SEG;
  const int kgroup = blockIdx.x % kgroups, bs = blockIdx.x / kgroups;
  const int seg = bs % nseg, b = bs / nseg, k = kgroup * 8 + wave;
  const bool live = k < p.K;  // uniform per wave
  const int l0 = seg * BD_SEG, n = min(BD_SEG, p.L - l0);
  const float scale = 1.0f / (3.0f * p.max_value);
  BoxLane bx;
  int queued = 0;
  if (live) {
    load_box(p, b, k, bx);
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      bx.cx[c] = wave_uniform(bx.cx[c]); bx.cy[c] = wave_uniform(bx.cy[c]); bx.cz[c] = wave_uniform(bx.cz[c]);
      bx.cs[c] = wave_uniform(bx.cs[c]); bx.sn[c] = wave_uniform(bx.sn[c]);
    }
    for (int base = 0; base < n; base += 64) {
      const int li = base + lane;
      const bool valid = li < n;
      const float* key = p.key + ((long)b * p.L + l0 + (valid ? li : n - 1)) * 3;
      const float kx = key[0], ky = key[1], kz = key[2];
      Window win;
      const bool one_window = corner_window(p, bx, kx, ky, kz, scale, win);
      if (valid && one_window) {
        f4 acc[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j] = (f4){0.0f, 0.0f, 0.0f, 0.0f};
        for_window(p, win, [&](int off, float w) {
          const f4* src = (const f4*)(tab + off);
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[j] += w * src[j];
        }, BD_NS);
        store_dist<BF>(p, ((long)b * p.L + l0 + li) * p.K + k, acc);
      }
      const unsigned long long rest = __ballot(valid && !one_window);
      if (valid && !one_window) queue[wave][queued + __popcll(rest & ((1ull << lane) - 1ull))] = (unsigned short)li;
      queued += __popcll(rest);
    }
  }
  __syncthreads();
  if (!live) return;
  for (int i = lane; i < queued; i += 64) {
    const int li = queue[wave][i];
    const float* key = p.key + ((long)b * p.L + l0 + li) * 3;
    const float kx = key[0], ky = key[1], kz = key[2];
    f4 acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[j] = (f4){0.0f, 0.0f, 0.0f, 0.0f};
    // A rolled loop that always works on slot 0 and then rotates the box's registers by one corner: fully unrolled,
    // the compiler issues the LDS reads of all 8 corners first and spills them.
#pragma unroll 1
    for (int c = 0; c < 8; ++c) {
      const float dx = bx.cx[0] - kx, dy = bx.cy[0] - ky, dz = bx.cz[0] - kz;
      const float rx = dx * bx.cs[0] - dy * bx.sn[0], ry = dx * bx.sn[0] + dy * bx.cs[0];
      Tri t;
      trilinear(p, node_pos(rx, p.log_scale, scale, p.W), node_pos(ry, p.log_scale, scale, p.H),
                node_pos(dz, p.log_scale, scale, p.D), t, BD_NS);
#pragma unroll
      for (int n8 = 0; n8 < 8; ++n8) {
        const f4* src = (const f4*)(tab + t.off[n8]);
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j] += t.w[n8] * src[j];
      }
      rotate_box(bx);
    }
    store_dist<BF>(p, ((long)b * p.L + l0 + li) * p.K + k, acc);
  }
}

__global__ void k_box_dist_clear(unsigned* scal) { scal[0] = 0u; }

// max |ddist| (bit pattern of a non-negative float orders like the unsigned integer)
template <bool BF>
__global__ __launch_bounds__(NTHREADS) void k_box_dist_gmax(BoxDistP p, unsigned* scal) {
  const long n = (long)p.B * p.L * p.K * BD_C;
  float m = 0.0f;
  for (long e = ((long)blockIdx.x * NTHREADS + threadIdx.x) * 8; e < n; e += (long)gridDim.x * NTHREADS * 8) {
    if (BF) {
      const uint4 v = *(const uint4*)((const uint16_t*)p.ddist + e);
      const unsigned w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int j = 0; j < 4; ++j)
        m = fmaxf(m, fmaxf(fabsf(__uint_as_float(w[j] << 16)), fabsf(__uint_as_float(w[j] & 0xffff0000u))));
    } else {
      const f4 a = *(const f4*)((const float*)p.ddist + e), c = *(const f4*)((const float*)p.ddist + e + 4);
      m = fmaxf(m, fmaxf(fmaxf(fabsf(a.x), fabsf(a.y)), fmaxf(fabsf(a.z), fabsf(a.w))));
      m = fmaxf(m, fmaxf(fmaxf(fabsf(c.x), fabsf(c.y)), fmaxf(fabsf(c.z), fabsf(c.w))));
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
  if ((threadIdx.x & 63) == 0 && m > 0.0f && m == m) atomicMax(scal, __float_as_uint(m));
}

// Table gradient: partial[wg][cell][ch] = sum over the workgroup's (l, k) pairs and corners of weight * ddist.
template <bool BF>
__global__ __launch_bounds__(NTHREADS) void k_box_dist_bwd(BoxDistP p) {
  __shared__ __attribute__((aligned(16))) unsigned long long tab[BD_MAXCELLS * BD_C];  // 128 KB: one workgroup per CU
  const int cells = p.D * p.H * p.W;
  for (int e = threadIdx.x; e < cells * BD_C; e += NTHREADS) tab[e] = 0ull;
  __syncthreads();
  const float fx_scale = bd_scale((const unsigned*)p.partial);
  const Items it = my_items(p);
  const float scale = 1.0f / (3.0f * p.max_value);
  int rot[BD_C];
#pragma unroll
  for (int j = 0; j < BD_C; ++j) rot[j] = (j + threadIdx.x) & 15;
  BoxLane bx;
  long cur = -1;
  for (long item = it.i0; item < it.i1; ++item) {
    const int l = (int)(item % p.L);
    const long bk = item / p.L;
    const int b = (int)(bk / it.kchunks), k = (int)(bk % it.kchunks) * NTHREADS + threadIdx.x;
    if (k >= p.K) continue;
    if (bk != cur) {
      load_box(p, b, k, bx);
      cur = bk;
    }
    const float* key = p.key + ((long)b * p.L + l) * 3;
    const float kx = key[0], ky = key[1], kz = key[2];
    const long o = ((long)b * p.L + l) * p.K + k;
    float g[BD_C];
    if (BF) {
      const uint4* src = (const uint4*)((const uint16_t*)p.ddist + o * BD_C);
      const uint4 a = src[0], c = src[1];
      const unsigned w[8] = {a.x, a.y, a.z, a.w, c.x, c.y, c.z, c.w};
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        g[2 * j] = __uint_as_float(w[j] << 16);
        g[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
      }
    } else {
      const f4* src = (const f4*)((const float*)p.ddist + o * BD_C);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const f4 v = src[j];
        g[4 * j] = v.x; g[4 * j + 1] = v.y; g[4 * j + 2] = v.z; g[4 * j + 3] = v.w;
      }
    }
#pragma unroll
    for (int j = 0; j < BD_C; ++j) g[j] *= fx_scale;
    // Lane r adds channel (j + r) mod 16 at step j.  Samples crowd into few nodes (the signed log maps most
    // distances near +-1), so many lanes of a wave hit the same node at once: with every lane on channel j that is
    // one LDS address and the adds serialise; rotated, the lanes of a node spread over its 16 channels.
#pragma unroll
    for (int bit = 8; bit >= 1; bit >>= 1) {
      const bool on = (threadIdx.x & bit) != 0;
      float t[BD_C];
#pragma unroll
      for (int j = 0; j < BD_C; ++j) t[j] = on ? g[(j + bit) & 15] : g[j];
#pragma unroll
      for (int j = 0; j < BD_C; ++j) g[j] = t[j];
    }
    Window win;
    if (corner_window(p, bx, kx, ky, kz, scale, win)) {
      for_window(p, win, [&](int off, float w) {
        unsigned long long* dst = tab + off;
#pragma unroll
        for (int j = 0; j < BD_C; ++j) atomicAdd(dst + rot[j], (unsigned long long)__float2ll_rn(w * g[j]));
      });
    } else {
#pragma unroll 1
      for (int c = 0; c < 8; ++c) {
        const float dx = bx.cx[0] - kx, dy = bx.cy[0] - ky, dz = bx.cz[0] - kz;
        const float rx = dx * bx.cs[0] - dy * bx.sn[0], ry = dx * bx.sn[0] + dy * bx.cs[0];
        Tri t;
        trilinear(p, node_pos(rx, p.log_scale, scale, p.W), node_pos(ry, p.log_scale, scale, p.H),
                  node_pos(dz, p.log_scale, scale, p.D), t);
#pragma unroll
        for (int n = 0; n < 8; ++n) {
          if (t.w[n] != 0.0f) {
            unsigned long long* dst = tab + t.off[n];
#pragma unroll
            for (int j = 0; j < BD_C; ++j) atomicAdd(dst + rot[j], (unsigned long long)__float2ll_rn(t.w[n] * g[j]));
          }
        }
        rotate_box(bx);
      }
    }
  }
  __syncthreads();
  unsigned long long* out = (unsigned long long*)p.partial + 2 + (long)blockIdx.x * cells * BD_C;
  for (int e = threadIdx.x; e < cells * BD_C; e += NTHREADS) out[e] = tab[e];
}

// dtable[ch][cell] = (sum over workgroups of partial[wg][cell][ch], exact in 64 bits) / scale
__global__ __launch_bounds__(NTHREADS) void k_box_dist_dtable(BoxDistP p) {
  const int cells = p.D * p.H * p.W;
  const int e = blockIdx.x * NTHREADS + threadIdx.x;  // e = cell * 16 + ch
  if (e >= cells * BD_C) return;
  const long long* part = (const long long*)p.partial + 2;
  long long a = 0;
  for (int w = 0; w < p.nwg_bwd; ++w) a += part[(long)w * cells * BD_C + e];
  const int cell = e / BD_C, ch = e % BD_C;
  p.dtable[(long)ch * cells + cell] = (float)((double)a / (double)bd_scale((const unsigned*)p.partial));
}

int box_dist_workgroups(int B, int L, int K) {
  const long items = (long)B * ((K + NTHREADS - 1) / NTHREADS) * L;
  return (int)(items < 512 ? items : 512);  // forward: two 64 KB workgroups per CU
}
int box_dist_bwd_workgroups(int B, int L, int K) {
  const long items = (long)B * ((K + NTHREADS - 1) / NTHREADS) * L;
  return (int)(items < 256 ? items : 256);  // backward: one 128 KB workgroup per CU
}

int launch_box_dist_fwd(const BoxDistP& p, hipStream_t st) {
  const dim3 b(NTHREADS);
  if (p.dist) {
    const dim3 g((unsigned)((long)p.B * ((p.L + BD_SEG - 1) / BD_SEG) * ((p.K + 7) / 8)));
    if (p.dtype) hipLaunchKernelGGL(k_box_dist_fwd<true>, g, dim3(BD_FWD_T), 0, st, p);
    else hipLaunchKernelGGL(k_box_dist_fwd<false>, g, dim3(BD_FWD_T), 0, st, p);
  }
  if (p.weights) hipLaunchKernelGGL(k_box_dist_weights, dim3(p.nwg), b, 0, st, p);
  return (int)hipGetLastError();
}

int launch_box_dist_bwd_sorted(const BoxDistP& p, hipStream_t st);
long box_dist_sorted_scratch_bytes(int B, int L, int K, int D, int H, int W);

// few pairs: scatter with LDS atomics (one launch of work); many pairs: sort by window, then dense sums
constexpr long BD_SORT_MIN_PAIRS = 1 << 16;

long box_dist_bwd_scratch_bytes(int B, int L, int K, int D, int H, int W) {
  const long atomic_path = 16 + (long)box_dist_bwd_workgroups(B, L, K) * D * H * W * BD_C * 8;
  if ((long)B * L * K < BD_SORT_MIN_PAIRS) return atomic_path;
  const long sorted_path = box_dist_sorted_scratch_bytes(B, L, K, D, H, W);
  return sorted_path > atomic_path ? sorted_path : atomic_path;
}

int launch_box_dist_bwd(const BoxDistP& p, hipStream_t st) {
  if ((long)p.B * p.L * p.K >= BD_SORT_MIN_PAIRS) return launch_box_dist_bwd_sorted(p, st);
  const dim3 g(p.nwg_bwd), b(NTHREADS);
  unsigned* scal = (unsigned*)p.partial;
  hipLaunchKernelGGL(k_box_dist_clear, dim3(1), dim3(1), 0, st, scal);
  if (p.dtype) hipLaunchKernelGGL(k_box_dist_gmax<true>, dim3(512), b, 0, st, p, scal);
  else hipLaunchKernelGGL(k_box_dist_gmax<false>, dim3(512), b, 0, st, p, scal);
  if (p.dtype) hipLaunchKernelGGL(k_box_dist_bwd<true>, g, b, 0, st, p);
  else hipLaunchKernelGGL(k_box_dist_bwd<false>, g, b, 0, st, p);
  int e = (int)hipGetLastError();
  if (e) return e;
  const int n = p.D * p.H * p.W * BD_C;
  hipLaunchKernelGGL(k_box_dist_dtable, dim3((n + NTHREADS - 1) / NTHREADS), b, 0, st, p);
  return (int)hipGetLastError();
}

}  // namespace issm
