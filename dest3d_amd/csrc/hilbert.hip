// Space-filling-curve codes of the key points (gfx950): the serialization order of the scan.
//
// Serialization.forward / encode (models/dest_module.py:307-356): every point is quantised to a grid of `cell`
// metres relative to its sample's minimum corner, clamped to 2^bits - 1 per axis, the three grid coordinates are
// permuted by the order string, and mapped to a position on the 3-D Hilbert curve; the caller argsorts the codes.
// The reference reads the curve from a 2^27-entry lookup table that is not shipped with it; here the position is
// computed (Skilling's transpose algorithm, first coordinate most significant, about 25 integer operations per bit).
// One thread per point, one launch per order; memory bound and tiny (24 bytes in, 8 out per point).
#include "issm_dev.h"

namespace issm {

__device__ __forceinline__ long hilbert3(unsigned x0, unsigned x1, unsigned x2, int bits) {
  unsigned X[3] = {x0, x1, x2};
  const unsigned M = 1u << (bits - 1);
  for (unsigned Q = M; Q > 1; Q >>= 1) {
    const unsigned P = Q - 1;
#pragma unroll
    for (int i = 0; i < 3; ++i) {
      if (X[i] & Q) {
        X[0] ^= P;
      } else {
        const unsigned t = (X[0] ^ X[i]) & P;
        X[0] ^= t;
        X[i] ^= t;
      }
    }
  }
  X[1] ^= X[0];
  X[2] ^= X[1];
  unsigned t = 0;
  for (unsigned Q = M; Q > 1; Q >>= 1)
    if (X[2] & Q) t ^= Q - 1;
  X[0] ^= t; X[1] ^= t; X[2] ^= t;
  long h = 0;
  for (int b = bits - 1; b >= 0; --b) {
#pragma unroll
    for (int i = 0; i < 3; ++i) h = (h << 1) | ((X[i] >> b) & 1u);
  }
  return h;
}

// Cell index of a truncated quotient: [0, cap], with NaN (a NaN coordinate, or Inf - Inf) sent to cell 0 by an explicit
// test instead of reaching the float-to-int conversion, whose result for NaN is not defined.
__device__ __forceinline__ unsigned cell_index(float v, int cap) {
  return v >= (float)cap ? (unsigned)cap : (v > 0.0f ? (unsigned)(int)v : 0u);
}
// Minimum that keeps a NaN once seen, as torch.amin does (fminf would drop it): a sample with a NaN coordinate then
// gets the same corner, and so the same cells, from the one-workgroup kernel and from the host-side reduction.
__device__ __forceinline__ float min_keep_nan(float a, float b) { return a != a ? a : (b != b ? b : fminf(a, b)); }

__global__ __launch_bounds__(NTHREADS) void k_hilbert_codes(HilbertP p) {
  const long id = (long)blockIdx.x * NTHREADS + threadIdx.x;
  if (id >= (long)p.B * p.N) return;
  const int b = (int)(id / p.N);
  const float* q = p.points + id * 3;
  const float* mn = p.mins + (long)b * 3;
  unsigned g[3];
  const int cap = (1 << p.bits) - 1;
#pragma unroll
  for (int i = 0; i < 3; ++i) {
    // a correctly rounded division, as torch.div(..., rounding_mode="trunc") performs on the host: this file is built
    // without fast-math, which would turn it into a multiplication by an approximate reciprocal and move points that
    // sit exactly on a cell boundary into the neighbouring cell
    g[i] = cell_index(truncf((q[i] - mn[i]) / p.cell), cap);
  }
  p.codes[id] = hilbert3(g[p.perm[0]], g[p.perm[1]], g[p.perm[2]], p.bits);
}

// The whole serialization of a sample in one workgroup: minimum corner, curve positions, a stable sort of the
// positions and the inverse permutation (Serialization.forward, models/dest_module.py:319-345, for all its orders in
// one launch).  Workgroup = (order, sample).  Keys are (position << 12 | point index): unique, so a bitonic network in
// LDS sorts them stably; up to 4096 points (32 KB of keys).  The separate steps (a reduction, a launch per order, two
// library sorts per order) took 75 us per order at 1024 points, nearly all of it launches.
constexpr int HO_MAXN = 4096, HO_IDXBITS = 12;
__global__ __launch_bounds__(NTHREADS) void k_hilbert_order(HilbertOrderP p) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  unsigned long long* keys = reinterpret_cast<unsigned long long*>(smem_raw);
  __shared__ float red[3][NTHREADS / 64];
  const int tid = threadIdx.x;
  const int b = blockIdx.x % p.B, o = blockIdx.x / p.B;
  const float* pts = p.points + (long)b * p.N * 3;
  // minimum corner of the sample (exact: a minimum does not depend on the order it is taken in)
  float mn[3] = {INFINITY, INFINITY, INFINITY};
  for (int j = tid; j < p.N; j += NTHREADS) {
#pragma unroll
    for (int i = 0; i < 3; ++i) mn[i] = min_keep_nan(mn[i], pts[3 * j + i]);
  }
#pragma unroll
  for (int i = 0; i < 3; ++i) {
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) mn[i] = min_keep_nan(mn[i], __shfl_xor(mn[i], d, 64));
    if ((tid & 63) == 0) red[i][tid >> 6] = mn[i];
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 3; ++i) {
    mn[i] = red[i][0];
#pragma unroll
    for (int w = 1; w < NTHREADS / 64; ++w) mn[i] = min_keep_nan(mn[i], red[i][w]);
  }
  const int cap = (1 << p.bits) - 1;
  const int p0 = p.perm[o][0], p1 = p.perm[o][1], p2 = p.perm[o][2];
  for (int j = tid; j < p.NP; j += NTHREADS) {
    unsigned long long key = ~0ull;  // padding sorts last
    if (j < p.N) {
      unsigned g[3];
#pragma unroll
      for (int i = 0; i < 3; ++i) {
        g[i] = cell_index(truncf((pts[3 * j + i] - mn[i]) / p.cell), cap);  // the same correctly rounded division as above
      }
      key = ((unsigned long long)hilbert3(g[p0], g[p1], g[p2], p.bits) << HO_IDXBITS) | (unsigned)j;
    }
    keys[j] = key;
  }
  __syncthreads();
  // bitonic network: NP / 2 compare-exchanges per step, every step behind a barrier
  for (int k = 2; k <= p.NP; k <<= 1) {
    for (int d = k >> 1; d > 0; d >>= 1) {
      for (int t = tid; t < (p.NP >> 1); t += NTHREADS) {
        const int lo = ((t & ~(d - 1)) << 1) | (t & (d - 1)), hi = lo | d;
        const bool up = (lo & k) == 0;
        const unsigned long long a = keys[lo], c = keys[hi];
        if ((a > c) == up) {
          keys[lo] = c;
          keys[hi] = a;
        }
      }
      __syncthreads();
    }
  }
  long* index = p.index + ((long)o * p.B + b) * p.N;
  long* inverse = p.inverse ? p.inverse + ((long)o * p.B + b) * p.N : nullptr;
  for (int j = tid; j < p.N; j += NTHREADS) {
    const int src = (int)(keys[j] & ((1u << HO_IDXBITS) - 1u));
    index[j] = src;
    if (inverse) inverse[src] = j;
  }
}

int launch_hilbert_order(const HilbertOrderP& p, hipStream_t st) {
  hipLaunchKernelGGL(k_hilbert_order, dim3((unsigned)(p.B * p.norder)), dim3(NTHREADS), (size_t)p.NP * 8, st, p);
  return (int)hipGetLastError();
}

int launch_hilbert_codes(const HilbertP& p, hipStream_t st) {
  const long n = (long)p.B * p.N;
  hipLaunchKernelGGL(k_hilbert_codes, dim3((unsigned)((n + NTHREADS - 1) / NTHREADS)), dim3(NTHREADS), 0, st, p);
  return (int)hipGetLastError();
}

}  // namespace issm
