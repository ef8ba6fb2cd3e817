// Forward kernels of the ISSM chunked scan for gfx950.
//
//   k_chunk_local   dt transform + cumsum, chunk-local end states S_c and the intra-chunk
//                   matrix M_c = "C.A.B^T" in one pass over dt
//   k_state_fwd     inter-chunk recurrence (HBM streaming)
//   k_chunk_scan    y = (C*exp(cs)) H^T + tril(M) x + D x, optional gate
//
// The decay exp(cs[l]-cs[s]) sits inside the contraction over the state index n, so
// M = sum_n C[l,n] B[s,n] dt'[s,n] exp(cs[l,n]-cs[s,n]) is not a plain GEMM.  It is
// evaluated exactly on the matrix cores by a binary hierarchy over the rows of a chunk:
// a pair (l > s) belongs to level w = highest set bit of (l xor s); at that level both
// rows sit in the same aligned block of 2w rows, s in its lower half, l in its upper half,
// and with r = last row of the lower half
//        exp(cs[l]-cs[s]) = exp(cs[l]-cs[r]) * exp(cs[r]-cs[s]).
// dt' >= 0 makes cs monotone in l for every n, so both factors lie between 1 and the
// product: nothing overflows that the exact value would not.  Level w therefore is an
// ordinary product Cw . Bw^T of rescaled operands, restricted to its blocks; the diagonal
// l == s is the plain product C . (B dt')^T.
#include "issm_dev.h"

namespace issm {

struct FwdLocalSmem {
  float xs[CS * LDP];    // x tile [l][p]
  float cs[CS * LDN];    // running sum of dt'*A*log2e [l][n]
  float bd[CS * LDN];    // B*dt' [l][n]
  float cc[CS * LDN];    // C [l][n]
  float opa[CS * LDN];   // level operand Cw / decayed B
  float opb[CS * LDN];   // level operand Bw
  float tot[4 * NS];
};

template <int PT>
__global__ __launch_bounds__(NTHREADS) void k_chunk_local(KP p, float* __restrict__ states,
                                                          float* __restrict__ cs_last, float* __restrict__ cabt) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  FwdLocalSmem& s = *reinterpret_cast<FwdLocalSmem*>(smem_raw);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rg = tid >> 6, col = tid & 63;
  const Unit u = decode_unit(p, xcd_remap(blockIdx.x, gridDim.x));
  const int ppad = PT * 16;

  load_lp_tile(p, u, p.x[u.dir], p.io_dt, s.xs, ppad, LDP);

  // accumulators of M: level 32, 16 and the four sub-16 levels + diagonal of the wave's diagonal tile
  f4 a32 = {0, 0, 0, 0}, a16 = {0, 0, 0, 0}, a8 = {0, 0, 0, 0}, a4 = {0, 0, 0, 0}, a2 = {0, 0, 0, 0},
     a1 = {0, 0, 0, 0}, a0 = {0, 0, 0, 0};
  const bool want_m = cabt != nullptr;
  const bool want_s = states != nullptr;

  for (int n0 = 0; n0 < p.N; n0 += NS) {
    float pre[16];
    prep_slice<NS>(p, u, n0, s.cs, s.opa /* dt' parked here */, s.tot, pre);
    // bd = B*dt', cc = C
    {
      const int n = n0 + col;
      const TensorD& tb = p.Bm[u.dir];
      const TensorD& tc = p.Cm[u.dir];
      const long bb = (long)u.b * tb.s0 + (long)u.g * tb.s2 + n;
      const long cb = (long)u.b * tc.s0 + (long)u.g * tc.s2 + n;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int l = rg * 16 + i, tt = u.c * CS + l;
        const bool v = (n < p.N) && (tt < p.L);
        const int pr = phys_row(p, u.dir, tt);
        const float bv = v ? ldv(tb.ptr, bb + (long)pr * tb.s1, p.io_dt) : 0.0f;
        const float cv = v ? ldv(tc.ptr, cb + (long)pr * tc.s1, p.io_dt) : 0.0f;
        s.bd[l * LDN + col] = bv * s.opa[l * LDN + col];
        s.cc[l * LDN + col] = cv;
      }
    }
    if (rg == 3 && n0 + col < p.N)
      cs_last[vec_off(p, u.bt, u.c, u.h) + n0 + col] = s.cs[63 * LDN + col] * LN2;
    __syncthreads();

    if (want_s) {
      // decayed B: B*dt'*exp(cs_last - cs[l])
      const float last = s.cs[63 * LDN + col];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int l = rg * 16 + i;
        s.opa[l * LDN + col] = s.bd[l * LDN + col] * ex2(last - s.cs[l * LDN + col]);
      }
      __syncthreads();
      // S[p][n] = sum_l x[l][p] * Bdec[l][n]; wave owns 16 columns
      f4 acc[PT];
#pragma unroll
      for (int pt = 0; pt < PT; ++pt) acc[pt] = (f4){0, 0, 0, 0};
#pragma unroll
      for (int kb = 0; kb < CS; kb += 16)
#pragma unroll
        for (int pt = 0; pt < PT; ++pt) mma16_kk(acc[pt], s.xs, LDP, pt * 16, s.opa, LDN, wave * 16, kb, lane);
      const int n = n0 + wave * 16 + (lane & 15);
      float* dst = states + st_off(p, u.bt, u.c, u.h);
#pragma unroll
      for (int pt = 0; pt < PT; ++pt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int pp = pt * 16 + 4 * (lane >> 4) + r;
          if (pp < p.P && n < p.N) dst[(long)pp * p.N + n] = acc[pt][r];
        }
    }

    if (want_m) {
      // diagonal level: C . (B dt')^T on the wave's diagonal tile
#pragma unroll
      for (int kb = 0; kb < NS; kb += 16) mma16_mm(a0, s.cc, LDN, wave * 16, s.bd, LDN, wave * 16, kb, lane);
#pragma unroll
      for (int lv = 5; lv >= 0; --lv) {
        const int w = 1 << lv;
        __syncthreads();  // previous users of opa/opb are done
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int l = rg * 16 + i;
          const int ref = (l & ~(2 * w - 1)) + w - 1;
          const float cr = s.cs[ref * LDN + col], cl = s.cs[l * LDN + col];
          const bool upper = (l & w) != 0;
          // upper rows act as l (left factor), lower rows as s (right factor)
          const float e = ex2(upper ? cl - cr : cr - cl);
          s.opa[l * LDN + col] = upper ? s.cc[l * LDN + col] * e : 0.0f;
          s.opb[l * LDN + col] = upper ? 0.0f : s.bd[l * LDN + col] * e;
        }
        __syncthreads();
        if (lv == 5) {
          const int ti = 2 + (wave >> 1), tj = wave & 1;
#pragma unroll
          for (int kb = 0; kb < NS; kb += 16) mma16_mm(a32, s.opa, LDN, ti * 16, s.opb, LDN, tj * 16, kb, lane);
        } else if (lv == 4) {
          if (wave < 2) {
            const int ti = wave ? 3 : 1, tj = wave ? 2 : 0;
#pragma unroll
            for (int kb = 0; kb < NS; kb += 16) mma16_mm(a16, s.opa, LDN, ti * 16, s.opb, LDN, tj * 16, kb, lane);
          }
        } else {
          f4& acc = lv == 3 ? a8 : lv == 2 ? a4 : lv == 1 ? a2 : a1;
#pragma unroll
          for (int kb = 0; kb < NS; kb += 16) mma16_mm(acc, s.opa, LDN, wave * 16, s.opb, LDN, wave * 16, kb, lane);
        }
      }
    }
    __syncthreads();
  }

  if (want_m) {
    float* m = cabt + sq_off(p, u.bt, u.c, u.h);
    const int cm = lane & 15, g = lane >> 4;
    // level 32 tile
    {
      const int ti = 2 + (wave >> 1), tj = wave & 1;
#pragma unroll
      for (int r = 0; r < 4; ++r) m[(ti * 16 + 4 * g + r) * CS + tj * 16 + cm] = a32[r];
    }
    if (wave < 2) {
      const int ti = wave ? 3 : 1, tj = wave ? 2 : 0;
#pragma unroll
      for (int r = 0; r < 4; ++r) m[(ti * 16 + 4 * g + r) * CS + tj * 16 + cm] = a16[r];
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int l = 4 * g + r, sc = cm;  // within the diagonal tile
      const int d = l ^ sc;
      float v = d == 0 ? a0[r] : d >= 8 ? a8[r] : d >= 4 ? a4[r] : d >= 2 ? a2[r] : a1[r];
      if (sc > l) v = 0.0f;
      m[(wave * 16 + l) * CS + wave * 16 + sc] = v;
    }
  }
}

// ---------------------------------------------------------------- state passing
// One thread carries 4 adjacent state columns of one (bt, h, p) through all chunks.
// Slot c of `states` holds S_c on entry and H_c (state at the start of chunk c) on exit;
// slot nc receives the final state.
__global__ __launch_bounds__(NTHREADS) void k_state_fwd(KP p, float* __restrict__ states,
                                                        const float* __restrict__ cs_last) {
  const int nq = (p.N + 3) >> 2;
  const long total = (long)p.B * p.ndir * p.H * p.P * nq;
  const long id = (long)blockIdx.x * NTHREADS + threadIdx.x;
  if (id >= total) return;
  const int q = id % nq;
  long r = id / nq;
  const int pp = r % p.P;
  r /= p.P;
  const int h = r % p.H;
  const int bt = r / p.H;
  const int b = bt / p.ndir, dir = bt % p.ndir;
  const int n = q * 4;
  const bool full = (n + 3 < p.N) && ((p.N & 3) == 0);
  float st[4] = {0, 0, 0, 0};
  if (p.h0.ptr) {
    const long o = (long)b * p.h0.s0 + (long)h * p.h0.s1 + (long)pp * p.h0.s2 + n;
    for (int j = 0; j < 4; ++j)
      if (n + j < p.N) st[j] = ldv(p.h0.ptr, o + j, p.h0_dt);
  }
  const long cstride = (long)p.H * p.P * p.N;
  float* sp = states + st_off(p, bt, 0, h) + (long)pp * p.N + n;
  const float* cl = cs_last + vec_off(p, bt, 0, h) + n;
  for (int c = 0; c < p.nc; ++c) {
    float sv[4], dv[4];
    if (full) {
      const f4 t = *(const f4*)sp;
      const f4 d = *(const f4*)cl;
      sv[0] = t.x; sv[1] = t.y; sv[2] = t.z; sv[3] = t.w;
      dv[0] = d.x; dv[1] = d.y; dv[2] = d.z; dv[3] = d.w;
      *(f4*)sp = (f4){st[0], st[1], st[2], st[3]};
    } else {
      for (int j = 0; j < 4; ++j) {
        const bool v = n + j < p.N;
        sv[j] = v ? sp[j] : 0.0f;
        dv[j] = v ? cl[j] : 0.0f;
        if (v) sp[j] = st[j];
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) st[j] = __expf(dv[j]) * st[j] + sv[j];
    sp += cstride;
    cl += (long)p.H * p.N;
  }
  // slot nc keeps the final state for the backward pass
  for (int j = 0; j < 4; ++j)
    if (n + j < p.N) sp[j] = st[j];
  if (p.final_states[dir]) {
    float* f = p.final_states[dir] + (((long)b * p.H + h) * p.P + pp) * p.N + n;
    for (int j = 0; j < 4; ++j)
      if (n + j < p.N) f[j] = st[j];
  }
}

// ------------------------------------------------------------------ chunk scan
struct FwdScanSmem {
  float xs[CS * LDP];   // x [s][p]
  float ms[CS * LDC];   // tril(M) [l][s]
  float cs[CS * LDN];
  float ct[CS * LDN];   // C * exp2(cs) [l][n]
  float hs[MAXP * LDN]; // H [p][n]
  float tot[4 * NS];
};

template <int PT>
__global__ __launch_bounds__(NTHREADS) void k_chunk_scan(KP p, const float* __restrict__ states,
                                                         const float* __restrict__ cabt, float* __restrict__ out_x) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  FwdScanSmem& s = *reinterpret_cast<FwdScanSmem*>(smem_raw);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rg = tid >> 6, col = tid & 63;
  const Unit u = decode_unit(p, xcd_remap(blockIdx.x, gridDim.x));
  const int ppad = PT * 16;

  load_lp_tile(p, u, p.x[u.dir], p.io_dt, s.xs, ppad, LDP);
  {
    const float* m = cabt + sq_off(p, u.bt, u.c, u.h);
    for (int e = tid; e < CS * CS; e += NTHREADS) {
      const int l = e >> 6, sc = e & 63;
      s.ms[l * LDC + sc] = sc <= l ? m[e] : 0.0f;
    }
  }
  f4 acc[PT];
#pragma unroll
  for (int pt = 0; pt < PT; ++pt) acc[pt] = (f4){0, 0, 0, 0};

  const float* hsrc = states + st_off(p, u.bt, u.c, u.h);
  for (int n0 = 0; n0 < p.N; n0 += NS) {
    float pre[16];
    prep_slice<NS>(p, u, n0, s.cs, s.ct /* dt' unused */, s.tot, pre);
    {
      const int n = n0 + col;
      const TensorD& tc = p.Cm[u.dir];
      const long cb = (long)u.b * tc.s0 + (long)u.g * tc.s2 + n;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int l = rg * 16 + i, tt = u.c * CS + l;
        const bool v = (n < p.N) && (tt < p.L);
        const float cv = v ? ldv(tc.ptr, cb + (long)phys_row(p, u.dir, tt) * tc.s1, p.io_dt) : 0.0f;
        s.ct[l * LDN + col] = cv * ex2(s.cs[l * LDN + col]);
      }
      for (int e = tid; e < ppad * NS; e += NTHREADS) {
        const int pp = e >> 6, c2 = e & 63;
        const bool v = pp < p.P && n0 + c2 < p.N;
        s.hs[pp * LDN + c2] = v ? hsrc[(long)pp * p.N + n0 + c2] : 0.0f;
      }
    }
    __syncthreads();
    // y[l][p] += sum_n Ct[l][n] H[p][n]; wave owns 16 rows
#pragma unroll
    for (int kb = 0; kb < NS; kb += 16)
#pragma unroll
      for (int pt = 0; pt < PT; ++pt) mma16_mm(acc[pt], s.ct, LDN, wave * 16, s.hs, LDN, pt * 16, kb, lane);
    __syncthreads();
  }
  // y[l][p] += sum_{s<=l} M[l][s] x[s][p]; rows of this wave only need s < 16(wave+1)
  for (int kb = 0; kb < (wave + 1) * 16; kb += 16)
#pragma unroll
    for (int pt = 0; pt < PT; ++pt) mma16_mk(acc[pt], s.ms, LDC, wave * 16, s.xs, LDP, pt * 16, kb, lane);

  const TensorD& to = p.out[u.dir];
  const TensorD& tz = p.z[u.dir];
#pragma unroll
  for (int pt = 0; pt < PT; ++pt)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int l = wave * 16 + 4 * (lane >> 4) + r, pp = pt * 16 + (lane & 15);
      const int tt = u.c * CS + l;
      if (tt >= p.L || pp >= p.P) continue;
      const int pr = phys_row(p, u.dir, tt);
      float v = acc[pt][r];
      if (p.D) v += ((p.flags & F_D_HDIM) ? p.D[u.h * p.P + pp] : p.D[u.h]) * s.xs[l * LDP + pp];
      if (tz.ptr) {
        if (out_x) out_x[(((long)u.bt * p.L + pr) * p.H + u.h) * p.P + pp] = v;
        const float zz = ldv(tz.ptr, (long)u.b * tz.s0 + (long)pr * tz.s1 + (long)u.h * tz.s2 + pp, p.io_dt);
        v *= zz * sigmoidf_(zz);
      }
      stv(const_cast<void*>(to.ptr), (long)u.b * to.s0 + (long)pr * to.s1 + (long)u.h * to.s2 + pp, p.io_dt, v);
    }
}

// ------------------------------------------------------------------- launchers
int launch_chunk_local(const KP& p, float* states, float* cs_last, float* cabt, hipStream_t st) {
  const int units = p.B * p.ndir * p.nc * p.H;
  const int pt = (p.P + 15) / 16;
  const size_t sm = sizeof(FwdLocalSmem);
#define LAUNCH(PT_)                                                                                        \
  { hipError_t e_ = hipFuncSetAttribute((const void*)k_chunk_local<PT_>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)sm); if (e_ != hipSuccess) return (int)e_; } \
  hipLaunchKernelGGL(k_chunk_local<PT_>, dim3(units), dim3(NTHREADS), sm, st, p, states, cs_last, cabt)
  switch (pt) {
    case 1: LAUNCH(1); break;
    case 2: LAUNCH(2); break;
    case 3: LAUNCH(3); break;
    default: LAUNCH(4); break;
  }
#undef LAUNCH
  return (int)hipGetLastError();
}

int launch_state_fwd(const KP& p, float* states, const float* cs_last, hipStream_t st) {
  const long total = (long)p.B * p.ndir * p.H * p.P * ((p.N + 3) / 4);
  const int blocks = (int)((total + NTHREADS - 1) / NTHREADS);
  hipLaunchKernelGGL(k_state_fwd, dim3(blocks), dim3(NTHREADS), 0, st, p, states, cs_last);
  return (int)hipGetLastError();
}

int launch_chunk_scan(const KP& p, const float* states, const float* cabt, float* out_x, hipStream_t st) {
  const int units = p.B * p.ndir * p.nc * p.H;
  const int pt = (p.P + 15) / 16;
  const size_t sm = sizeof(FwdScanSmem);
#define LAUNCH(PT_)                                                                                       \
  { hipError_t e_ = hipFuncSetAttribute((const void*)k_chunk_scan<PT_>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)sm); if (e_ != hipSuccess) return (int)e_; } \
  hipLaunchKernelGGL(k_chunk_scan<PT_>, dim3(units), dim3(NTHREADS), sm, st, p, states, cabt, out_x)
  switch (pt) {
    case 1: LAUNCH(1); break;
    case 2: LAUNCH(2); break;
    case 3: LAUNCH(3); break;
    default: LAUNCH(4); break;
  }
#undef LAUNCH
  return (int)hipGetLastError();
}

}  // namespace issm
