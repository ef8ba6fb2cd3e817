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
    const float v = truncf((q[i] - mn[i]) / p.cell);
    int c = v >= (float)cap ? cap : (int)v;
    g[i] = (unsigned)(c < 0 ? 0 : c);
  }
  p.codes[id] = hilbert3(g[p.perm[0]], g[p.perm[1]], g[p.perm[2]], p.bits);
}

int launch_hilbert_codes(const HilbertP& p, hipStream_t st) {
  const long n = (long)p.B * p.N;
  hipLaunchKernelGGL(k_hilbert_codes, dim3((unsigned)((n + NTHREADS - 1) / NTHREADS)), dim3(NTHREADS), 0, st, p);
  return (int)hipGetLastError();
}

}  // namespace issm
