// Backward kernels of the ISSM chunked scan for gfx950.
//
//   k_bwd_gate      z-gate backward (elementwise)
//   k_bwd_dstates   dH_c = dy^T (C*exp(cs))  and  dM = tril(dy x^T)
//   k_state_bwd     reverse inter-chunk recurrence (HBM streaming)
//   k_bwd_chunk     per (chunk, group, 32-column slice), looping over the heads of the
//                   group: ddt, dB, dC and the per-unit partial sums of dA / ddt_bias
//   k_bwd_dx        dx and the per-unit partial sums of dD
//   k_bwd_reduce    fixed-order sums of the partials (bit-reproducible, no atomics)
//
// With Bd = B dt', E(l,s) = exp(cs[l]-cs[s]) and per state column n
//   Q[m] = sum_p x[m,p] dS[p],  R[l] = sum_p dy[l,p] H[p],
//   G[m] = sum_{l>=m} dM[l,m] C[l] E(l,m),  F[l] = sum_{s<=l} dM[l,s] Bd[s] E(l,s),
//   E1 = exp(cs_last-cs) Q + G,   X2 = exp(cs) R + F
// the gradients are dB = sum_heads dt' E1, dC = sum_heads X2, ddt' = B E1 + A da,
// da[k] = sum_{l>=k} (C X2 - Bd E1)[l] + (sum_p dS[p] H_next[p]), the last term entering at
// the chunk's last row.  G and F carry the decay inside the contraction; they use the same
// binary row hierarchy as the forward intra-chunk matrix (see issm_fwd.hip).
#include "issm_dev.h"

namespace issm {

// ------------------------------------------------------------------- z gate
// out_x, dy_ws: fp32 (Bt,L,H,P) contiguous in physical time order.
__global__ __launch_bounds__(NTHREADS) void k_bwd_gate(KP p, const float* __restrict__ out_x,
                                                       float* __restrict__ dy_ws) {
  const long total = (long)p.B * p.ndir * p.L * p.H * p.P;
  const long id = (long)blockIdx.x * NTHREADS + threadIdx.x;
  if (id >= total) return;
  const int pp = id % p.P;
  long r = id / p.P;
  const int h = r % p.H;
  r /= p.H;
  const int l = r % p.L;
  const int bt = r / p.L;
  const int b = bt / p.ndir, dir = bt % p.ndir;
  const TensorD& tz = p.z[dir];
  const TensorD& td = p.dout[dir];
  const TensorD& tdz = p.dz[dir];
  const float z = ldv(tz.ptr, (long)b * tz.s0 + (long)l * tz.s1 + (long)h * tz.s2 + pp, p.io_dt);
  const float d = ldv(td.ptr, (long)b * td.s0 + (long)l * td.s1 + (long)h * td.s2 + pp, p.io_dt);
  const float sg = sigmoidf_(z);
  dy_ws[id] = d * z * sg;
  if (tdz.ptr)
    stv(const_cast<void*>(tdz.ptr), (long)b * tdz.s0 + (long)l * tdz.s1 + (long)h * tdz.s2 + pp, p.io_dt,
        d * out_x[id] * sg * (1.0f + z * (1.0f - sg)));
}

// ------------------------------------------------------------ dstates and dM
template <int PT>
struct BwdStSmem {
  static constexpr int LDPT = PT * 16 + 4;
  float dys[CS * LDPT];
  float xs[CS * LDPT];
  float cs[CS * LDN];
  float ct[CS * LDN];
  float tot[4 * NS];
};

template <int PT>
__global__ __launch_bounds__(NTHREADS) void k_bwd_dstates(KP p, const float* __restrict__ dy_ws,
                                                          float* __restrict__ dstates, float* __restrict__ dm) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  typedef BwdStSmem<PT> SM;
  SM& s = *reinterpret_cast<SM*>(smem_raw);
  constexpr int LDPT = SM::LDPT;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rg = tid >> 6, col = tid & 63;
  const Unit u = decode_unit(p, xcd_remap(blockIdx.x, gridDim.x));
  const int ppad = PT * 16;

  if (dy_ws) load_lp_tile_ws(p, u, dy_ws, s.dys, ppad, LDPT);
  else load_lp_tile(p, u, p.dout[u.dir], p.io_dt, s.dys, ppad, LDPT);
  load_lp_tile(p, u, p.x[u.dir], p.io_dt, s.xs, ppad, LDPT);
  __syncthreads();

  if (dm) {
    float* m = dm + sq_off(p, u.bt, u.c, u.h);
    const int cm = lane & 15, g = lane >> 4;
    for (int j = 0; j <= wave; ++j) {
      f4 acc = {0, 0, 0, 0};
#pragma unroll
      for (int kb = 0; kb < ppad; kb += 16) mma16_mm(acc, s.dys, LDPT, wave * 16, s.xs, LDPT, j * 16, kb, lane);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int l = wave * 16 + 4 * g + r, sc = j * 16 + cm;
        m[l * CS + sc] = sc <= l ? acc[r] : 0.0f;
      }
    }
  }
  if (!dstates) return;

  for (int n0 = 0; n0 < p.N; n0 += NS) {
    float pre[16];
    prep_slice<NS>(p, u, n0, s.cs, s.ct, s.tot, pre);
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
    }
    __syncthreads();
    f4 acc[PT];
#pragma unroll
    for (int pt = 0; pt < PT; ++pt) acc[pt] = (f4){0, 0, 0, 0};
#pragma unroll
    for (int kb = 0; kb < CS; kb += 16)
#pragma unroll
      for (int pt = 0; pt < PT; ++pt) mma16_kk(acc[pt], s.dys, LDPT, pt * 16, s.ct, LDN, wave * 16, kb, lane);
    const int n = n0 + wave * 16 + (lane & 15);
    float* dst = dstates + dst_off(p, u.bt, u.c, u.h);
#pragma unroll
    for (int pt = 0; pt < PT; ++pt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int pp = pt * 16 + 4 * (lane >> 4) + r;
        if (pp < p.P && n < p.N) dst[(long)pp * p.N + n] = acc[pt][r];
      }
    __syncthreads();
  }
}

// ------------------------------------------------------- reverse state passing
// Block = (bt, h, 64 state columns); thread (pg = tid >> 4, nq = tid & 15) carries rows
// p = pg, pg+16, ... of 4 adjacent columns.  dstates[c] holds dH_c on entry and dS_c (gradient
// of the chunk-local end state) on exit.  g_last[c][n] = sum_p dS_c[p,n] * H_{c+1}[p,n].
__global__ __launch_bounds__(NTHREADS) void k_state_bwd(KP p, const float* __restrict__ states,
                                                        const float* __restrict__ cs_last,
                                                        float* __restrict__ dstates, float* __restrict__ g_last,
                                                        float* __restrict__ dh0_dir) {
  __shared__ float red[16 * 64];
  const int nsl = (p.N + 63) / 64;
  int bid = blockIdx.x;
  const int ns = bid % nsl;
  bid /= nsl;
  const int h = bid % p.H;
  const int bt = bid / p.H;
  const int b = bt / p.ndir, dir = bt % p.ndir;
  const int tid = threadIdx.x, pg = tid >> 4, nq = tid & 15;
  const int n = ns * 64 + nq * 4;
  float carry[4][4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int pp = pg + 16 * k;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const bool v = pp < p.P && n + j < p.N && p.dfinal[dir];
      carry[k][j] = v ? p.dfinal[dir][(((long)b * p.H + h) * p.P + pp) * p.N + n + j] : 0.0f;
    }
  }
  for (int c = p.nc - 1; c >= 0; --c) {
    float gp[4] = {0, 0, 0, 0};
    float dec[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) dec[j] = n + j < p.N ? __expf(cs_last[vec_off(p, bt, c, h) + n + j]) : 0.0f;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int pp = pg + 16 * k;
      if (pp >= p.P) continue;
      const float* hn = states + st_off(p, bt, c + 1, h) + (long)pp * p.N + n;
      float* dd = dstates + dst_off(p, bt, c, h) + (long)pp * p.N + n;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (n + j >= p.N) continue;
        const float dh = dd[j];
        dd[j] = carry[k][j];
        gp[j] += hn[j] * carry[k][j];
        carry[k][j] = dec[j] * carry[k][j] + dh;
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) red[pg * 64 + nq * 4 + j] = gp[j];
    __syncthreads();
    if (tid < 64) {
      float sum = 0.0f;
#pragma unroll
      for (int k = 0; k < 16; ++k) sum += red[k * 64 + tid];
      if (ns * 64 + tid < p.N) g_last[vec_off(p, bt, c, h) + ns * 64 + tid] = sum;
    }
    __syncthreads();
  }
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int pp = pg + 16 * k;
    if (pp >= p.P) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (n + j < p.N) dh0_dir[((((long)dir * p.B + b) * p.H + h) * p.P + pp) * p.N + n + j] = carry[k][j];
  }
}

// -------------------------------------------------------------- chunk backward
template <int PT>
struct BwdChunkSmem {
  static constexpr int LDPT = PT * 16 + 4;
  float cs[CS * LDNB];
  float dts[CS * LDNB];
  float bs[CS * LDNB];
  float ccs[CS * LDNB];
  float opa[CS * LDNB];  // level operand Bw, later E1
  float opb[CS * LDNB];  // level operand Cw, later X2
  float xs[CS * LDPT];
  float dys[CS * LDPT];
  float dms[CS * LDC];
  float dss[PT * 16 * LDNB];
  float hs[PT * 16 * LDNB];
  float tot[8 * NSB];
  float red[2 * 8 * NSB];
};

// partials: partA (Bt*nc, H, N) then partBias (Bt*nc, H, N)
template <int PT>
__global__ __launch_bounds__(NTHREADS) void k_bwd_chunk(KP p, const float* __restrict__ dy_ws,
                                                        const float* __restrict__ states,
                                                        const float* __restrict__ dstates,
                                                        const float* __restrict__ dm,
                                                        const float* __restrict__ g_last, float* __restrict__ partA,
                                                        float* __restrict__ partBias) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  typedef BwdChunkSmem<PT> SM;
  SM& s = *reinterpret_cast<SM*>(smem_raw);
  constexpr int LDPT = SM::LDPT;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rg = tid >> 5, col = tid & 31;  // column-thread layout: rows 8rg..8rg+7
  const int cm = lane & 15, g4 = lane >> 4;
  const int ppad = PT * 16;
  const int nsl = (p.N + NSB - 1) / NSB;
  Unit u;
  {
    int id = xcd_remap(blockIdx.x, gridDim.x);
    const int ns = id % nsl;
    id /= nsl;
    u.g = id % p.G;
    id /= p.G;
    u.c = id % p.nc;
    u.b = id / p.nc;
    u.dir = p.dir0;
    u.bt = u.b * p.ndir + u.dir;
    u.h = 0;
    const int n0 = ns * NSB;
    const int n = n0 + col;
    const bool vn = n < p.N;

    load_ln_tile<NSB>(p, u, p.Bm[u.dir], p.io_dt, u.g, n0, s.bs);
    load_ln_tile<NSB>(p, u, p.Cm[u.dir], p.io_dt, u.g, n0, s.ccs);
    float dBacc[8], dCacc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) dBacc[i] = dCacc[i] = 0.0f;

    for (int hh = 0; hh < p.hpg; ++hh) {
      u.h = u.g * p.hpg + hh;
      float pre[8];
      prep_slice<NSB>(p, u, n0, s.cs, s.dts, s.tot, pre);
      if (dy_ws) load_lp_tile_ws(p, u, dy_ws, s.dys, ppad, LDPT);
      else load_lp_tile(p, u, p.dout[u.dir], p.io_dt, s.dys, ppad, LDPT);
      load_lp_tile(p, u, p.x[u.dir], p.io_dt, s.xs, ppad, LDPT);
      {
        const float* m = dm + sq_off(p, u.bt, u.c, u.h);
        for (int e = tid; e < CS * CS; e += NTHREADS) {
          const int l = e >> 6, sc = e & 63;
          s.dms[l * LDC + sc] = sc <= l ? m[e] : 0.0f;
        }
        const float* ds = dstates + dst_off(p, u.bt, u.c, u.h);
        const float* hp = states + st_off(p, u.bt, u.c, u.h);
        for (int e = tid; e < ppad * NSB; e += NTHREADS) {
          const int pp = e >> 5, c2 = e & 31;
          const bool v = pp < p.P && n0 + c2 < p.N;
          s.dss[pp * LDNB + c2] = v ? ds[(long)pp * p.N + n0 + c2] : 0.0f;
          s.hs[pp * LDNB + c2] = v ? hp[(long)pp * p.N + n0 + c2] : 0.0f;
        }
      }
      __syncthreads();

      // Q, R and the diagonal (l == s) terms, in accumulator layout: wave owns rows 16*wave..+15
      f4 e1[2], x2[2];
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        f4 q = {0, 0, 0, 0}, r = {0, 0, 0, 0};
#pragma unroll
        for (int kb = 0; kb < ppad; kb += 16) {
          mma16_mk(q, s.xs, LDPT, wave * 16, s.dss, LDNB, nt * 16, kb, lane);
          mma16_mk(r, s.dys, LDPT, wave * 16, s.hs, LDNB, nt * 16, kb, lane);
        }
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
          const int row = wave * 16 + 4 * g4 + rr, cx = nt * 16 + cm;
          const float cl = s.cs[row * LDNB + cx], last = s.cs[63 * LDNB + cx];
          const float dd = s.dms[row * LDC + row];
          e1[nt][rr] = ex2(last - cl) * q[rr] + dd * s.ccs[row * LDNB + cx];
          x2[nt][rr] = ex2(cl) * r[rr] + dd * s.bs[row * LDNB + cx] * s.dts[row * LDNB + cx];
        }
      }

      // hierarchy levels of F and G
#pragma unroll
      for (int lv = 5; lv >= 0; --lv) {
        const int w = 1 << lv;
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int l = rg * 8 + i;
          const int ref = (l & ~(2 * w - 1)) + w - 1;
          const float cr = s.cs[ref * LDNB + col], cl = s.cs[l * LDNB + col];
          const bool upper = (l & w) != 0;
          const float e = ex2(upper ? cl - cr : cr - cl);
          s.opa[l * LDNB + col] = upper ? 0.0f : s.bs[l * LDNB + col] * s.dts[l * LDNB + col] * e;
          s.opb[l * LDNB + col] = upper ? s.ccs[l * LDNB + col] * e : 0.0f;
        }
        __syncthreads();
        const int I = wave;
        // F: rows of this tile that are "upper" at this level; K runs over s
        int fk0 = 0, fk1 = 0, gk0 = 0, gk1 = 0;
        if (lv == 5) {
          if (I >= 2) { fk0 = 0; fk1 = 32; } else { gk0 = 32; gk1 = 64; }
        } else if (lv == 4) {
          if (I & 1) { fk0 = 16 * (I - 1); fk1 = 16 * I; } else { gk0 = 16 * (I + 1); gk1 = 16 * (I + 2); }
        } else {
          fk0 = gk0 = 16 * I;
          fk1 = gk1 = 16 * I + 16;
        }
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) {
          f4 fw = {0, 0, 0, 0}, gw = {0, 0, 0, 0};
          for (int kb = fk0; kb < fk1; kb += 16) {
            // A = dM[l][s] (M-major), B = Bw[s][n] (K-major)
            f4 av = *(const f4*)(s.dms + (I * 16 + cm) * LDC + kb + 4 * g4);
            if (lv < 3) {
#pragma unroll
              for (int j = 0; j < 4; ++j)
                if (((cm ^ (4 * g4 + j)) >= 2 * w)) av[j] = 0.0f;
            }
            const float* bp = s.opa + (kb + 4 * g4) * LDNB + nt * 16 + cm;
            fw = mfma4(av.x, bp[0], fw);
            fw = mfma4(av.y, bp[LDNB], fw);
            fw = mfma4(av.z, bp[2 * LDNB], fw);
            fw = mfma4(av.w, bp[3 * LDNB], fw);
          }
          for (int kb = gk0; kb < gk1; kb += 16) {
            // A[m][k=l] = dM[l][m] (K-major), B = Cw[l][n] (K-major)
            const float* ap = s.dms + (kb + 4 * g4) * LDC + I * 16 + cm;
            const float* bp = s.opb + (kb + 4 * g4) * LDNB + nt * 16 + cm;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              float a = ap[j * LDC];
              if (lv < 3 && ((cm ^ (4 * g4 + j)) >= 2 * w)) a = 0.0f;
              gw = mfma4(a, bp[j * LDNB], gw);
            }
          }
#pragma unroll
          for (int rr = 0; rr < 4; ++rr) {
            const int row = wave * 16 + 4 * g4 + rr, cx = nt * 16 + cm;
            const int ref = (row & ~(2 * w - 1)) + w - 1;
            const float cr = s.cs[ref * LDNB + cx], cl = s.cs[row * LDNB + cx];
            if (row & w) x2[nt][rr] += ex2(cl - cr) * fw[rr];
            else e1[nt][rr] += ex2(cr - cl) * gw[rr];
          }
        }
      }
      __syncthreads();
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
          const int row = wave * 16 + 4 * g4 + rr, cx = nt * 16 + cm;
          s.opa[row * LDNB + cx] = e1[nt][rr];
          s.opb[row * LDNB + cx] = x2[nt][rr];
        }
      __syncthreads();

      // column phase: thread owns rows 8rg..8rg+7 of column col
      float ddtp[8], dcs[8], dv[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int l = rg * 8 + i;
        const float E1 = s.opa[l * LDNB + col], X2 = s.opb[l * LDNB + col];
        const float b = s.bs[l * LDNB + col], c = s.ccs[l * LDNB + col], d = s.dts[l * LDNB + col];
        dv[i] = d;
        dBacc[i] += d * E1;
        dCacc[i] += X2;
        ddtp[i] = b * E1;
        dcs[i] = c * X2 - b * d * E1;
      }
      if (rg == 7 && vn) dcs[7] += g_last[vec_off(p, u.bt, u.c, u.h) + n];
      float run = 0.0f;
#pragma unroll
      for (int i = 7; i >= 0; --i) {
        run += dcs[i];
        dcs[i] = run;
      }
      s.tot[rg * NSB + col] = run;
      __syncthreads();
      float off = 0.0f;
      for (int g = rg + 1; g < 8; ++g) off += s.tot[g * NSB + col];
      const float An = vn ? p.A[u.h * p.N + n] : 0.0f;
      float sumA = 0.0f, sumB = 0.0f;
      const TensorD& tdd = p.ddt;
      const long dbase = (long)u.b * tdd.s0 + (long)u.h * tdd.s2 + n;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int l = rg * 8 + i, tt = u.c * CS + l;
        const float da = dcs[i] + off;
        sumA += da * dv[i];
        float val = ddtp[i] + da * An;
        float sp = pre[i];
        if (p.flags & F_SOFTPLUS) sp = (pre[i] <= 20.0f) ? log1pf(__expf(pre[i])) : pre[i];
        if (sp < p.dt_min || sp > p.dt_max) val = 0.0f;
        if ((p.flags & F_SOFTPLUS) && pre[i] <= 20.0f) val *= sigmoidf_(pre[i]);
        if (vn && tt < p.L) {
          sumB += val;
          if (tdd.ptr) {
            const long o = dbase + (long)phys_row(p, u.dir, tt) * tdd.s1;
            if (p.dir0 > 0) val += ldv(tdd.ptr, o, p.dt_dt);
            stv(const_cast<void*>(tdd.ptr), o, p.dt_dt, val);
          }
        }
      }
      s.red[rg * NSB + col] = sumA;
      s.red[8 * NSB + rg * NSB + col] = sumB;
      __syncthreads();
      if (rg == 0 && vn) {
        float a = 0.0f, bsum = 0.0f;
#pragma unroll
        for (int g = 0; g < 8; ++g) {
          a += s.red[g * NSB + col];
          bsum += s.red[8 * NSB + g * NSB + col];
        }
        partA[vec_off(p, u.bt, u.c, u.h) + n] = a;
        partBias[vec_off(p, u.bt, u.c, u.h) + n] = bsum;
      }
      __syncthreads();
    }

    const TensorD& tB = p.dB[u.dir];
    const TensorD& tC = p.dC[u.dir];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int tt = u.c * CS + rg * 8 + i;
      if (!vn || tt >= p.L) continue;
      const int pr = phys_row(p, u.dir, tt);
      if (tB.ptr) stv(const_cast<void*>(tB.ptr), (long)u.b * tB.s0 + (long)pr * tB.s1 + (long)u.g * tB.s2 + n, p.io_dt, dBacc[i]);
      if (tC.ptr) stv(const_cast<void*>(tC.ptr), (long)u.b * tC.s0 + (long)pr * tC.s1 + (long)u.g * tC.s2 + n, p.io_dt, dCacc[i]);
    }
  }
}

// ------------------------------------------------------------------------- dx
template <int PT>
struct BwdDxSmem {
  static constexpr int LDPT = PT * 16 + 4;
  float dys[CS * LDPT];
  float ms[CS * LDC];
  float cs[CS * LDN];
  float bt[CS * LDN];
  float dss[PT * 16 * LDN];
  float tot[4 * NS];
};

// partD: (Bt*nc*H, P) per-unit sums over rows of dy*x
template <int PT>
__global__ __launch_bounds__(NTHREADS) void k_bwd_dx(KP p, const float* __restrict__ dy_ws,
                                                     const float* __restrict__ dstates,
                                                     const float* __restrict__ cabt, float* __restrict__ partD) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  typedef BwdDxSmem<PT> SM;
  SM& s = *reinterpret_cast<SM*>(smem_raw);
  constexpr int LDPT = SM::LDPT;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rg = tid >> 6, col = tid & 63;
  const Unit u = decode_unit(p, xcd_remap(blockIdx.x, gridDim.x));
  const int ppad = PT * 16;

  if (dy_ws) load_lp_tile_ws(p, u, dy_ws, s.dys, ppad, LDPT);
  else load_lp_tile(p, u, p.dout[u.dir], p.io_dt, s.dys, ppad, LDPT);
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
  const float* ds = dstates + dst_off(p, u.bt, u.c, u.h);

  for (int n0 = 0; n0 < p.N; n0 += NS) {
    float pre[16];
    prep_slice<NS>(p, u, n0, s.cs, s.bt, s.tot, pre);
    {
      const int n = n0 + col;
      const TensorD& tb = p.Bm[u.dir];
      const long bb = (long)u.b * tb.s0 + (long)u.g * tb.s2 + n;
      const float last = s.cs[63 * LDN + col];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int l = rg * 16 + i, tt = u.c * CS + l;
        const bool v = (n < p.N) && (tt < p.L);
        const float bv = v ? ldv(tb.ptr, bb + (long)phys_row(p, u.dir, tt) * tb.s1, p.io_dt) : 0.0f;
        s.bt[l * LDN + col] = bv * s.bt[l * LDN + col] * ex2(last - s.cs[l * LDN + col]);
      }
      for (int e = tid; e < ppad * NS; e += NTHREADS) {
        const int pp = e >> 6, c2 = e & 63;
        const bool v = pp < p.P && n0 + c2 < p.N;
        s.dss[pp * LDN + c2] = v ? ds[(long)pp * p.N + n0 + c2] : 0.0f;
      }
    }
    __syncthreads();
#pragma unroll
    for (int kb = 0; kb < NS; kb += 16)
#pragma unroll
      for (int pt = 0; pt < PT; ++pt) mma16_mm(acc[pt], s.bt, LDN, wave * 16, s.dss, LDN, pt * 16, kb, lane);
    __syncthreads();
  }
  // dx[m][p] += sum_{l>=m} M[l][m] dy[l][p]
  for (int kb = wave * 16; kb < CS; kb += 16)
#pragma unroll
    for (int pt = 0; pt < PT; ++pt) mma16_kk(acc[pt], s.ms, LDC, wave * 16, s.dys, LDPT, pt * 16, kb, lane);

  const TensorD& tx = p.x[u.dir];
  const TensorD& tdx = p.dx[u.dir];
  float* prod = s.cs;  // reuse: [64][LDN] is at least [64][ppad]
#pragma unroll
  for (int pt = 0; pt < PT; ++pt)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int l = wave * 16 + 4 * (lane >> 4) + r, pp = pt * 16 + (lane & 15);
      const int tt = u.c * CS + l;
      float pv = 0.0f;
      if (tt < p.L && pp < p.P) {
        const int pr = phys_row(p, u.dir, tt);
        const float dyv = s.dys[l * LDPT + pp];
        float v = acc[pt][r];
        if (p.D) {
          v += ((p.flags & F_D_HDIM) ? p.D[u.h * p.P + pp] : p.D[u.h]) * dyv;
          pv = dyv * ldv(tx.ptr, (long)u.b * tx.s0 + (long)pr * tx.s1 + (long)u.h * tx.s2 + pp, p.io_dt);
        }
        if (tdx.ptr)
          stv(const_cast<void*>(tdx.ptr), (long)u.b * tdx.s0 + (long)pr * tdx.s1 + (long)u.h * tdx.s2 + pp, p.io_dt, v);
      }
      prod[l * LDN + pp] = pv;
    }
  if (p.D && partD) {
    __syncthreads();
    if (tid < ppad) {
      float sum = 0.0f;
      for (int l = 0; l < CS; ++l) sum += prod[l * LDN + tid];
      if (tid < p.P) partD[(((long)u.bt * p.nc + u.c) * p.H + u.h) * p.P + tid] = sum;
    }
  }
}

// ------------------------------------------------------------------- reductions
// dA[h,n] = sum_j partA[j,h,n];  ddt_bias likewise;  dD[h(,p)] = sum_j partD[j,h,p];
// dh0 = sum over directions.  One thread per output element, fixed summation order.
__global__ __launch_bounds__(NTHREADS) void k_bwd_reduce(KP p, const float* __restrict__ partA,
                                                         const float* __restrict__ partBias,
                                                         const float* __restrict__ partD,
                                                         const float* __restrict__ dh0_dir, float* __restrict__ dA,
                                                         float* __restrict__ dbias, float* __restrict__ dD,
                                                         float* __restrict__ dh0) {
  const long id = (long)blockIdx.x * NTHREADS + threadIdx.x;
  const long nHN = (long)p.H * p.N;
  const int J = p.B * p.ndir * p.nc;
  const long nD = (p.flags & F_D_HDIM) ? (long)p.H * p.P : p.H;
  const long nS = (long)p.B * p.H * p.P * p.N;
  if (id < nHN) {
    if (dA) {
      float a = 0.0f;
      for (int j = 0; j < J; ++j) a += partA[(long)j * nHN + id];
      dA[id] = a;
    }
    if (dbias) {
      float a = 0.0f;
      for (int j = 0; j < J; ++j) a += partBias[(long)j * nHN + id];
      dbias[id] = a;
    }
  }
  if (id < nD && dD) {
    float a = 0.0f;
    if (p.flags & F_D_HDIM) {
      for (int j = 0; j < J; ++j) a += partD[(long)j * p.H * p.P + id];
    } else {
      for (int j = 0; j < J; ++j)
        for (int pp = 0; pp < p.P; ++pp) a += partD[((long)j * p.H + id) * p.P + pp];
    }
    dD[id] = a;
  }
  if (id < nS && dh0) {
    float a = dh0_dir[id];
    if (p.ndir > 1) a += dh0_dir[nS + id];
    dh0[id] = a;
  }
}

// -------------------------------------------------------------------- launchers
#define ISSM_PT_SWITCH(pt, STMT) \
  switch (pt) {                  \
    case 1: { constexpr int PT_ = 1; STMT; } break; \
    case 2: { constexpr int PT_ = 2; STMT; } break; \
    case 3: { constexpr int PT_ = 3; STMT; } break; \
    default: { constexpr int PT_ = 4; STMT; } break; \
  }

int launch_bwd_gate(const KP& p, const float* out_x, float* dy_ws, hipStream_t st) {
  const long total = (long)p.B * p.ndir * p.L * p.H * p.P;
  hipLaunchKernelGGL(k_bwd_gate, dim3((unsigned)((total + NTHREADS - 1) / NTHREADS)), dim3(NTHREADS), 0, st, p, out_x,
                     dy_ws);
  return (int)hipGetLastError();
}

int launch_bwd_dstates(const KP& p, const float* dy_ws, float* dstates, float* dm, hipStream_t st) {
  const int units = p.B * p.ndir * p.nc * p.H;
  const int pt = (p.P + 15) / 16;
  ISSM_PT_SWITCH(pt, {
    const size_t sm = sizeof(BwdStSmem<PT_>);
    { hipError_t e_ = hipFuncSetAttribute((const void*)k_bwd_dstates<PT_>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)sm); if (e_ != hipSuccess) return (int)e_; }
    hipLaunchKernelGGL(k_bwd_dstates<PT_>, dim3(units), dim3(NTHREADS), sm, st, p, dy_ws, dstates, dm);
  });
  return (int)hipGetLastError();
}

int launch_state_bwd(const KP& p, const float* states, const float* cs_last, float* dstates, float* g_last,
                     float* dh0_dir, hipStream_t st) {
  const int blocks = p.B * p.ndir * p.H * ((p.N + 63) / 64);
  hipLaunchKernelGGL(k_state_bwd, dim3(blocks), dim3(NTHREADS), 0, st, p, states, cs_last, dstates, g_last, dh0_dir);
  return (int)hipGetLastError();
}

int launch_bwd_chunk(const KP& p, const float* dy_ws, const float* states, const float* dstates, const float* dm,
                     const float* g_last, float* partA, float* partBias, hipStream_t st) {
  const int blocks = p.B * p.nc * p.G * ((p.N + NSB - 1) / NSB);
  const int pt = (p.P + 15) / 16;
  ISSM_PT_SWITCH(pt, {
    const size_t sm = sizeof(BwdChunkSmem<PT_>);
    { hipError_t e_ = hipFuncSetAttribute((const void*)k_bwd_chunk<PT_>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)sm); if (e_ != hipSuccess) return (int)e_; }
    hipLaunchKernelGGL(k_bwd_chunk<PT_>, dim3(blocks), dim3(NTHREADS), sm, st, p, dy_ws, states, dstates, dm, g_last,
                       partA, partBias);
  });
  return (int)hipGetLastError();
}

int launch_bwd_dx(const KP& p, const float* dy_ws, const float* dstates, const float* cabt, float* partD,
                  hipStream_t st) {
  const int units = p.B * p.ndir * p.nc * p.H;
  const int pt = (p.P + 15) / 16;
  ISSM_PT_SWITCH(pt, {
    const size_t sm = sizeof(BwdDxSmem<PT_>);
    { hipError_t e_ = hipFuncSetAttribute((const void*)k_bwd_dx<PT_>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)sm); if (e_ != hipSuccess) return (int)e_; }
    hipLaunchKernelGGL(k_bwd_dx<PT_>, dim3(units), dim3(NTHREADS), sm, st, p, dy_ws, dstates, cabt, partD);
  });
  return (int)hipGetLastError();
}

int launch_bwd_reduce(const KP& p, const float* partA, const float* partBias, const float* partD,
                      const float* dh0_dir, float* dA, float* dbias, float* dD, float* dh0, hipStream_t st) {
  long n = (long)p.H * p.N;
  const long nS = (long)p.B * p.H * p.P * p.N;
  if (dh0 && nS > n) n = nS;
  const long nD = (long)p.H * p.P;
  if (nD > n) n = nD;
  hipLaunchKernelGGL(k_bwd_reduce, dim3((unsigned)((n + NTHREADS - 1) / NTHREADS)), dim3(NTHREADS), 0, st, p, partA,
                     partBias, partD, dh0_dir, dA, dbias, dD, dh0);
  return (int)hipGetLastError();
}

}  // namespace issm
