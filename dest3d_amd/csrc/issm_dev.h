// Device-side building blocks shared by the ISSM kernels (gfx950 / CDNA4 only).
//
// Tiling conventions used by every kernel in this directory
//  * one workgroup = 256 threads = 4 wavefronts of 64 lanes;
//  * time is cut into chunks of CS = 64 tokens, the state dimension into slices of
//    NS = 64 columns; a "unit" is one (batch*direction, chunk, head);
//  * every LDS tile is a row-major float array whose leading dimension is
//    (width + 4): with ld = 4 (mod 8) both fragment access patterns below are free
//    of bank conflicts;
//  * matrix products run on v_mfma_f32_16x16x4_f32.  Lane (m = lane & 15,
//    g = lane >> 4) feeds the j-th of four back-to-back MFMAs with k = kb + 4g + j,
//    so that an operand stored with k contiguous ("M-major", tile[m][k]) is fetched
//    with one 128-bit LDS read and an operand stored with m contiguous ("K-major",
//    tile[k][m]) with four 32-bit reads.  The accumulator register r of that lane
//    holds element (row = 4g + r, col = m) of the 16x16 result.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace issm {

constexpr int CS = 64;         // tokens per chunk
constexpr int NS = 64;         // state columns per slice (forward kernels)
constexpr int LDN = NS + 4;    // leading dimension of [*][NS] tiles
constexpr int NSB = 32;        // state columns per slice (backward chunk kernel)
constexpr int LDNB = NSB + 4;
constexpr int LDC = CS + 4;    // leading dimension of [*][CS] tiles
constexpr int MAXP = 64;       // largest head dimension built
constexpr int LDP = MAXP + 4;  // leading dimension of [*][P] tiles
constexpr int NTHREADS = 256;
constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;

typedef float f4 __attribute__((ext_vector_type(4)));

struct TensorD {
  const void* ptr;
  long s0, s1, s2;  // element strides of dims 0,1,2 (innermost contiguous)
};

// Kernel parameter block (passed by value).
struct KP {
  int B, L, H, P, N, G, ndir, nc, hpg;
  int dir0;  // first direction handled by this launch (kernels launched per direction)
  int io_dt, dt_dt, h0_dt;  // 0 = f32, 1 = bf16
  unsigned flags;
  float dt_min, dt_max;
  TensorD x[2], Bm[2], Cm[2], z[2], out[2], dout[2], dx[2], dB[2], dC[2], dz[2];
  TensorD dt, ddt, h0;
  const float* A;
  const float* D;
  const float* dt_bias;
  float* final_states[2];
  const float* dfinal[2];
};

enum : unsigned { F_SOFTPLUS = 1u, F_D_HDIM = 2u };

// Parameter block of the gated RMSNorm kernels.
struct NormP {
  long rows;
  int ncols, gs, ngroups;
  int dt, wdt, nbg;
  float eps;
  const void *x, *z, *w;
  long xs, zs;
  void* y;
  long ys;
  float* rstd;
  const void* dy;
  long dys;
  void *dx, *dz;
  long dxs, dzs;
  float* dw_partial;
  float* dw;
  int nblocks;
};


__device__ __forceinline__ float bf16_to_f(uint16_t v) { return __uint_as_float(((uint32_t)v) << 16); }
__device__ __forceinline__ uint16_t f_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);  // NaN
  u += 0x7fffu + ((u >> 16) & 1u);  // round to nearest even
  return (uint16_t)(u >> 16);
}
__device__ __forceinline__ float ldv(const void* p, long i, int dt) {
  return dt ? bf16_to_f(((const uint16_t*)p)[i]) : ((const float*)p)[i];
}
__device__ __forceinline__ void stv(void* p, long i, int dt, float v) {
  if (dt) ((uint16_t*)p)[i] = f_to_bf16(v); else ((float*)p)[i] = v;
}
__device__ __forceinline__ float ex2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float sigmoidf_(float x) { return 1.0f / (1.0f + __expf(-x)); }

// Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous range
// of logical ids so that units sharing B/C tiles (the heads of one chunk) share an L2.
__device__ __forceinline__ int xcd_remap(int bid, int nblocks) {
  if (nblocks & 7) return bid;
  return (bid & 7) * (nblocks >> 3) + (bid >> 3);
}

__device__ __forceinline__ f4 mfma4(float a, float b, f4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

// acc += A(16 x 16k) * B(16k x 16) for k in [kb, kb+16); both operands M-major:
// A[m][k] at a[(m0+m)*lda + k], B[n][k] at b[(n0+n)*ldb + k].
__device__ __forceinline__ void mma16_mm(f4& acc, const float* a, int lda, int m0, const float* b, int ldb,
                                         int n0, int kb, int lane) {
  const int m = lane & 15, g = lane >> 4;
  f4 av = *(const f4*)(a + (m0 + m) * lda + kb + 4 * g);
  f4 bv = *(const f4*)(b + (n0 + m) * ldb + kb + 4 * g);
  acc = mfma4(av.x, bv.x, acc);
  acc = mfma4(av.y, bv.y, acc);
  acc = mfma4(av.z, bv.z, acc);
  acc = mfma4(av.w, bv.w, acc);
}
// both operands K-major: A[k][m] at a[k*lda + m0+m], B[k][n] at b[k*ldb + n0+n]
__device__ __forceinline__ void mma16_kk(f4& acc, const float* a, int lda, int m0, const float* b, int ldb,
                                         int n0, int kb, int lane) {
  const int m = lane & 15, g = lane >> 4;
  const float* ap = a + (kb + 4 * g) * lda + m0 + m;
  const float* bp = b + (kb + 4 * g) * ldb + n0 + m;
#pragma unroll
  for (int j = 0; j < 4; ++j) acc = mfma4(ap[j * lda], bp[j * ldb], acc);
}
// A M-major, B K-major
__device__ __forceinline__ void mma16_mk(f4& acc, const float* a, int lda, int m0, const float* b, int ldb,
                                         int n0, int kb, int lane) {
  const int m = lane & 15, g = lane >> 4;
  f4 av = *(const f4*)(a + (m0 + m) * lda + kb + 4 * g);
  const float* bp = b + (kb + 4 * g) * ldb + n0 + m;
  acc = mfma4(av.x, bp[0], acc);
  acc = mfma4(av.y, bp[ldb], acc);
  acc = mfma4(av.z, bp[2 * ldb], acc);
  acc = mfma4(av.w, bp[3 * ldb], acc);
}
// A K-major, B M-major
__device__ __forceinline__ void mma16_km(f4& acc, const float* a, int lda, int m0, const float* b, int ldb,
                                         int n0, int kb, int lane) {
  const int m = lane & 15, g = lane >> 4;
  const float* ap = a + (kb + 4 * g) * lda + m0 + m;
  f4 bv = *(const f4*)(b + (n0 + m) * ldb + kb + 4 * g);
  acc = mfma4(ap[0], bv.x, acc);
  acc = mfma4(ap[lda], bv.y, acc);
  acc = mfma4(ap[2 * lda], bv.z, acc);
  acc = mfma4(ap[3 * lda], bv.w, acc);
}

// Decode a unit id -> (b, dir, c, h); h is fastest so that the heads of one chunk run
// back to back and share the B/C tiles in cache.
struct Unit {
  int b, dir, bt, c, h, g;
};
__device__ __forceinline__ Unit decode_unit(const KP& p, int u) {
  Unit r;
  r.h = u % p.H;
  u /= p.H;
  r.c = u % p.nc;
  r.bt = u / p.nc;
  r.dir = r.bt % p.ndir;
  r.b = r.bt / p.ndir;
  r.g = r.h / p.hpg;
  return r;
}
// physical row of logical time t for a direction
__device__ __forceinline__ int phys_row(const KP& p, int dir, int t) { return dir ? p.L - 1 - t : t; }

// dt transform of one element (bias -> softplus -> clamp), also returns the
// pre-activation for the backward masks.
__device__ __forceinline__ float dt_act(const KP& p, float pre) {
  float v = pre;
  if (p.flags & F_SOFTPLUS) v = (pre <= 20.0f) ? log1pf(__expf(pre)) : pre;
  return fminf(fmaxf(v, p.dt_min), p.dt_max);
}

// Slice prologue for a slice of NSL (64 or 32) state columns.  Thread (rg = tid / NSL,
// col = tid % NSL) owns RPT = 64*NSL/256 consecutive rows of column n0+col of one unit.
// Loads dt, applies the transform, forms the inclusive running sum of dt' * A * log2(e)
// down the chunk (so decays are exp2 of differences) and leaves
//   csS[l][col] = running sum (log2 domain),  dtS[l][col] = dt'
// in LDS (leading dimension NSL+4).  `tot` is a [256/NSL][NSL] scratch.  pre[i] receives
// dt + bias of the owned rows.  Rows past the end of the sequence and columns past N read
// as dt' = 0.  Ends with a barrier.
template <int NSL>
__device__ __forceinline__ void prep_slice(const KP& p, const Unit& u, int n0, float* csS, float* dtS,
                                           float* tot, float* pre) {
  constexpr int RPT = CS * NSL / NTHREADS, LD = NSL + 4;
  const int tid = threadIdx.x, rg = tid / NSL, col = tid % NSL;
  const int n = n0 + col;
  const bool vn = n < p.N;
  const float A2 = vn ? p.A[u.h * p.N + n] * LOG2E : 0.0f;
  const float bias = (vn && p.dt_bias) ? p.dt_bias[u.h * p.N + n] : 0.0f;
  const long base = (long)u.b * p.dt.s0 + (long)u.h * p.dt.s2 + n;
  float dtp[RPT], cs[RPT], raw[RPT];
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const int t = u.c * CS + rg * RPT + i;
    const bool v = vn && t < p.L;
    raw[i] = v ? ldv(p.dt.ptr, base + (long)phys_row(p, u.dir, t) * p.dt.s1, p.dt_dt) : 0.0f;
  }
  float run = 0.0f;
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const int t = u.c * CS + rg * RPT + i;
    const bool v = vn && t < p.L;
    pre[i] = raw[i] + bias;
    dtp[i] = v ? dt_act(p, pre[i]) : 0.0f;
    run += dtp[i] * A2;
    cs[i] = run;
  }
  tot[rg * NSL + col] = run;
  __syncthreads();
  float off = 0.0f;
  for (int g = 0; g < rg; ++g) off += tot[g * NSL + col];
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    csS[(rg * RPT + i) * LD + col] = cs[i] + off;
    dtS[(rg * RPT + i) * LD + col] = dtp[i];
  }
  __syncthreads();
}

// Rows of a (B,L,G|H,N)-shaped operand into LDS: dst[l][col] for the 64 rows of the unit's
// chunk, columns n0..n0+NSL-1 (zero outside the sequence / past N).
template <int NSL>
__device__ __forceinline__ void load_ln_tile(const KP& p, const Unit& u, const TensorD& t, int dtype, int third,
                                             int n0, float* dst) {
  constexpr int RPT = CS * NSL / NTHREADS, LD = NSL + 4;
  const int tid = threadIdx.x, rg = tid / NSL, col = tid % NSL;
  const int n = n0 + col;
  const long base = (long)u.b * t.s0 + (long)third * t.s2 + n;
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const int l = rg * RPT + i, tt = u.c * CS + l;
    const bool v = (n < p.N) && (tt < p.L);
    dst[l * LD + col] = v ? ldv(t.ptr, base + (long)phys_row(p, u.dir, tt) * t.s1, dtype) : 0.0f;
  }
}

// The unit's (64 x P) tile of a (B,L,H,P) tensor into LDS dst[l][p] (leading dimension ld),
// zero padded to ppad columns.
__device__ __forceinline__ void load_lp_tile(const KP& p, const Unit& u, const TensorD& t, int dtype, float* dst,
                                             int ppad, int ld) {
  const long base = (long)u.b * t.s0 + (long)u.h * t.s2;
  for (int e = threadIdx.x; e < CS * ppad; e += NTHREADS) {
    const int l = e / ppad, pp = e - l * ppad, tt = u.c * CS + l;
    const bool v = (pp < p.P) && (tt < p.L);
    dst[l * ld + pp] = v ? ldv(t.ptr, base + (long)phys_row(p, u.dir, tt) * t.s1 + pp, dtype) : 0.0f;
  }
}
// Same for an fp32 contiguous (Bt,L,H,P) workspace tensor stored in physical time order.
__device__ __forceinline__ void load_lp_tile_ws(const KP& p, const Unit& u, const float* src, float* dst, int ppad,
                                                int ld) {
  const long base = ((long)u.bt * p.L) * p.H * p.P + (long)u.h * p.P;
  for (int e = threadIdx.x; e < CS * ppad; e += NTHREADS) {
    const int l = e / ppad, pp = e - l * ppad, tt = u.c * CS + l;
    const bool v = (pp < p.P) && (tt < p.L);
    dst[l * ld + pp] = v ? src[base + (long)phys_row(p, u.dir, tt) * p.H * p.P + pp] : 0.0f;
  }
}

// Index helpers for the fp32 intermediates.
//   states  (Bt, nc+1, H, P, N): slot c = state entering chunk c, slot nc = final state
//   dstates (Bt, nc,   H, P, N)
//   per-chunk vectors (Bt, nc, H, N); square blocks (Bt, nc, H, 64, 64)
__device__ __forceinline__ long st_off(const KP& p, int bt, int c, int h) {
  return (((long)bt * (p.nc + 1) + c) * p.H + h) * p.P * p.N;
}
__device__ __forceinline__ long dst_off(const KP& p, int bt, int c, int h) {
  return (((long)bt * p.nc + c) * p.H + h) * p.P * p.N;
}
__device__ __forceinline__ long vec_off(const KP& p, int bt, int c, int h) {
  return (((long)bt * p.nc + c) * p.H + h) * p.N;
}
__device__ __forceinline__ long sq_off(const KP& p, int bt, int c, int h) {
  return (((long)bt * p.nc + c) * p.H + h) * CS * CS;
}

}  // namespace issm
