// Chunk backward of the ISSM scan in tile-base form (gfx950): ddt, dB, dC and the partial sums of dA / ddt_bias.
//
// Same job and same workgroup shape as k_bwd_chunk (issm_bwd.hip): workgroup = (batch, chunk, group, 64 state columns)
// of one direction, looping over the heads of the group; lane (cm, g4) of a wave owns state column cm and the 16 chunk
// rows {16J + 4 g4 + j}.  What differs is how the decay exp2(cs[l] - cs[s]) inside the sums
//   F[l] = sum_{s<=l} dM[l,s] Bd[s] exp2(cs[l]-cs[s]),   G[s] = sum_{l>=s} dM[l,s] C[l] exp2(cs[l]-cs[s])
// is taken apart.  With pc = running sum of a = dt' A log2(e) restarted at every 16-row tile and base(J) = sum of the
// tiles before J,
//   exp2(cs[l] - cs[s]) = up[l] . E(I,J) . iup[s],   up = exp2(pc), iup = exp2(-pc), E(I,J) = exp2(base(I) - base(J))
// for l in tile I >= tile J of s.  up and iup are two exponentials per element, E ten per column, and then every block
// (I, J) of F and G is a plain 16x16x16 product of the dM block with the tile's operand rows (Bd iup for F, C up for G)
// whose result is scaled by E(I,J): no per-level operands, no pairs evaluated in the vector ALU.  The state terms fit the
// same form: exp2(cs[l]) = up[l] E(I,0) and exp2(cs_last - cs[s]) = E(4,J) iup[s].
//
// iup grows like 2^(decay across one tile), so the form is only used where every tile's sum stays within SPAN_LIMIT
// (|tt| <= 96: operands below 2^96, no overflow before the factors meet).  A head of a workgroup where some column
// exceeds it -- very large dt' |A| -- is left out here, marked in `redo`, and evaluated by the level-hierarchy kernel
// (k_bwd_chunk / k_bwd_chunk_bf with `redo`), which has no such limit.  Operands: bf16 inputs -> one bf16 instruction
// per block, operands rounded once; fp32 inputs -> operands cut to 16 significand bits and split exactly into (hi, lo)
// bf16 pairs, a.b = (ah.bl + al.bh) + (ah.bh + al.bl), each bracket one K = 32 instruction.  d/d(cs) is formed as
// (operand as the matrix instruction took it) x (product) on both rows of a pair, so the two entries of a pair cancel
// to fp32 rounding in the suffix sums.
//
// Built for complete tiles only (sequence length and state dimension multiples of 64, no packed sequences, x / dout
// rows that allow 8- / 16-byte accesses, no z gate, x / B / C and dt of one type); every other call takes the
// level-hierarchy kernel alone.  That is what lets the kernel issue every global load of a head without a branch, one
// head ahead: the wave then knows how many requests are outstanding at every point and waits for exactly the ones it
// needs (a load inside a branch, even a uniform one, makes the compiler wait for all outstanding loads at the join).
#include "issm_dev.h"

namespace issm {

constexpr float SPAN_LIMIT = 96.0f;

template <int PT, bool SPLIT>
struct BwdTileSmem {
  static constexpr int KW = 16 * PT, LDP = KW + 8;  // x / dy tiles [l][p]
  static constexpr int LDM = CS + 8;                // T[i][j] = dM[max(i,j)][min(i,j)]
  static constexpr int NH = SPLIT ? 2 : 1;          // hi (and lo) copies
  uint16_t xs[NH * CS * LDP];
  uint16_t dys[NH * CS * LDP];
  uint16_t tm[NH * CS * LDM];
  float dbc[32 * NTHREADS];  // per-lane dB / dC accumulators [k][tid]
  // bf16 inputs, two head tiles: the group's B and C values of every lane, packed in pairs, [i][tid] (i < 8: B, then C).
  // They are the same for every head of the group; read from global memory again per head they miss the L2 (the heads'
  // streams have been through it in between) and were a third of the kernel's reads.  fp32 inputs have no room for them
  // at two workgroups per CU, wider heads no registers to spare for the change (they spill and lose what it gains).
  static constexpr bool BCL = !SPLIT && PT == 2;
  unsigned bc[BCL ? 16 * NTHREADS : 1];
  int bad[4];                // per wave: some column of the head exceeds SPAN_LIMIT
};

__device__ __forceinline__ bf8 cat_bf4(bf4 a, bf4 b) { return __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7); }

// PNF: the head dimension fills its 16-row tiles (P == 16 PT); ACC: ddt holds the other direction's share already and
// this launch adds to it; P32 (bf16 only): that share travels in fp32 through p.ddt_part -- the first direction's launch
// writes it there, the second reads it from there and writes the once-rounded sum to ddt.
template <int PT, bool IOB, bool PNF, bool ACC, bool P32>
__global__ __launch_bounds__(NTHREADS, 2) void k_bwd_tile(KP p, const float* __restrict__ states,
                                                          const float* __restrict__ dstates,
                                                          const float* __restrict__ dm,
                                                          const float* __restrict__ g_last, float* __restrict__ partA,
                                                          float* __restrict__ partBias, int* __restrict__ redo) {
  constexpr bool SPLIT = !IOB;
  extern __shared__ __align__(16) unsigned char smem_raw[];
  typedef BwdTileSmem<PT, SPLIT> SM;
  SM& s = *reinterpret_cast<SM*>(smem_raw);
  constexpr int LDP = SM::LDP, LDM = SM::LDM, KT = (PT + 1) / 2;
  constexpr bool BCL = SM::BCL;
  constexpr int KP_ = PT * 4;  // dS / H values per lane
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int cm = lane & 15, g4 = lane >> 4;
  const int nsl = p.N / NS;
  Unit u;
  const int wg = xcd_remap(blockIdx.x, gridDim.x);
  int id = wg;
  const int ns = id % nsl;
  id /= nsl;
  u.g = id % p.G;
  id /= p.G;
  u.c = p.c_lo + id % p.ncl;
  u.b = id / p.ncl;
  u.dir = p.dir0;
  u.bt = u.b * p.ndir + u.dir;
  u.h = u.g * p.hpg;
  const int n = ns * NS + wave * 16 + cm;
  const RowMap rm = make_rowmap<true>(p, u, g4, ns * NS);

#pragma unroll
  for (int k = 0; k < 16; ++k) s.dbc[k * NTHREADS + tid] = s.dbc[(16 + k) * NTHREADS + tid] = 0.0f;

  if constexpr (BCL) {
    float tb[16], tc[16];
    lane_load_ln<true>(p.Bm[u.dir], u.b, u.g, n, true, g4, rm, tb);
    lane_load_ln<true>(p.Cm[u.dir], u.b, u.g, n, true, g4, rm, tc);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      s.bc[i * NTHREADS + tid] = pack_bf16(tb[2 * i], tb[2 * i + 1]);  // exact: the values are bf16 numbers
      s.bc[(8 + i) * NTHREADS + tid] = pack_bf16(tc[2 * i], tc[2 * i + 1]);
    }
  }

  // the reversed direction's launch follows the forward one's and shares dt, x, B, C and ddt with it: it walks the
  // heads backwards, so what the first launch touched last (and the last-level cache still holds) is read first
  auto head_of = [&](int hh) { return u.g * p.hpg + (p.dir0 ? p.hpg - 1 - hh : hh); };

  // Everything a head reads from global memory is requested one head ahead, at the point of the previous head where
  // few registers are live (after its matrix products), so that the requests are in flight while that head's suffix
  // sums and stores run.  (B and C of the lane's rows are the same for every head of the group; they are fetched again
  // per head -- from the cache -- rather than held in 32 registers across the loop.)
  // What one head reads: the thread's share of the tiles the four waves stage in LDS (T: rows tid >> 3 and
  // 32 + (tid >> 3), columns 8 (tid & 7) .. + 7 of the hi -- and lo -- matrix; x, dy: group i of the thread is row
  // e4 / 4PT, columns 4 (e4 % 4PT) .. + 3 with e4 = tid + 256 i) and the lane's column operands.  Requested in the order
  // of first use, without a branch; rows of x / dy past the head dimension are read from the tensor's first elements and
  // count as zero.
  uint4 l_th0, l_th1, l_tl0, l_tl1;
  f4 l_xv[SPLIT ? PT : 1], l_dv[SPLIT ? PT : 1];
  uint2 l_nx[SPLIT ? 1 : PT], l_ny[SPLIT ? 1 : PT];
  float l_raw[16], l_A, l_bias, l_gl, l_dsv[KP_], l_hv[KP_], l_Bv[BCL ? 1 : 16], l_Cv[BCL ? 1 : 16];
  auto request = [&](int hnext) {
    constexpr int G4 = 4 * PT;
    int tq = tid;
    asm volatile("" : "+v"(tq));
    const int mrow = tq >> 3, mcol = (tq & 7) * 8;
    const uint16_t* dmb = reinterpret_cast<const uint16_t*>(dm + sq_off(p, u.bt, u.c, hnext));
    l_th0 = *(const uint4*)(dmb + mrow * CS + mcol);
    l_th1 = *(const uint4*)(dmb + (32 + mrow) * CS + mcol);
    if constexpr (SPLIT) {
      l_tl0 = *(const uint4*)(dmb + CS * CS + mrow * CS + mcol);
      l_tl1 = *(const uint4*)(dmb + CS * CS + (32 + mrow) * CS + mcol);
    }
    {
      typedef typename std::conditional<IOB, uint16_t, float>::type T;
      const TensorD& tx = p.x[u.dir];
      const TensorD& ty = p.dout[u.dir];
      const T* qx = (const T*)tx.ptr + ((long)u.b * tx.s0 + (long)hnext * tx.s2);
      const T* qy = (const T*)ty.ptr + ((long)u.b * ty.s0 + (long)hnext * ty.s2);
      const long t0 = u.dir ? p.L - 1 - u.c * CS : u.c * CS, sgn = u.dir ? -1 : 1;
#pragma unroll
      for (int i = 0; i < PT; ++i) {
        const int e4 = tq + i * NTHREADS, l = e4 / G4, p4 = (e4 % G4) * 4;
        const bool ok = p4 < p.P;
        const long ox = ok ? (t0 + sgn * l) * tx.s1 + p4 : 0, oy = ok ? (t0 + sgn * l) * ty.s1 + p4 : 0;
        if constexpr (SPLIT) {
          const f4 a = *(const f4*)(qy + oy), b = *(const f4*)(qx + ox);
          l_dv[i] = ok ? a : (f4){0, 0, 0, 0};
          l_xv[i] = ok ? b : (f4){0, 0, 0, 0};
        } else {
          const uint2 a = *(const uint2*)(qy + oy), b = *(const uint2*)(qx + ox);
          l_ny[i] = ok ? a : make_uint2(0u, 0u);
          l_nx[i] = ok ? b : make_uint2(0u, 0u);
        }
      }
    }
    lane_load_ln<IOB>(p.dt, u.b, hnext, n, true, g4, rm, l_raw);
    l_A = p.A[hnext * p.N + n];
    {
      const float* bp = p.dt_bias ? p.dt_bias : p.A;  // no bias: any readable address, the value is dropped
      const float b = bp[hnext * p.N + n];
      l_bias = p.dt_bias ? b : 0.0f;
    }
    l_gl = g_last[vec_off(p, u.bt, u.c, hnext) + n];  // (every lane of the column; the last lane group uses it)
    lane_load_pn<KP_>(dstates + dst_off(p, u.bt, u.c, hnext), p.P, p.N, n, true, g4, PNF, l_dsv);
    lane_load_pn<KP_>(states + st_off(p, u.bt, u.c, hnext), p.P, p.N, n, true, g4, PNF, l_hv);
    if constexpr (!BCL) {
      lane_load_ln<IOB>(p.Bm[u.dir], u.b, u.g, n, true, g4, rm, l_Bv);
      lane_load_ln<IOB>(p.Cm[u.dir], u.b, u.g, n, true, g4, rm, l_Cv);
    }
  };
  request(head_of(0));

  for (int hh = 0; hh < p.hpg; ++hh) {
    u.h = head_of(hh);
    __syncthreads();  // the previous head no longer reads the tiles
    {
      int tq = tid;
      asm volatile("" : "+v"(tq));
      const int mrow = tq >> 3, mcol = (tq & 7) * 8;
      constexpr int G4 = 4 * PT;
      *(uint4*)(s.tm + mrow * LDM + mcol) = l_th0;
      *(uint4*)(s.tm + (32 + mrow) * LDM + mcol) = l_th1;
      if constexpr (SPLIT) {
        *(uint4*)(s.tm + CS * LDM + mrow * LDM + mcol) = l_tl0;
        *(uint4*)(s.tm + CS * LDM + (32 + mrow) * LDM + mcol) = l_tl1;
#pragma unroll
        for (int i = 0; i < PT; ++i) {
          const int e4 = tq + i * NTHREADS, o = (e4 / G4) * LDP + (e4 % G4) * 4;
          const float wy[4] = {l_dv[i][0], l_dv[i][1], l_dv[i][2], l_dv[i][3]};
          const float wx[4] = {l_xv[i][0], l_xv[i][1], l_xv[i][2], l_xv[i][3]};
          bf4 h, l;
          split4(wy, h, l);
          *(bf4*)(s.dys + o) = h;
          *(bf4*)(s.dys + CS * LDP + o) = l;
          split4(wx, h, l);
          *(bf4*)(s.xs + o) = h;
          *(bf4*)(s.xs + CS * LDP + o) = l;
        }
      } else {
        lp_store_raw<PT, LDP>(l_ny, s.dys, tq);
        lp_store_raw<PT, LDP>(l_nx, s.xs, tq);
      }
    }

    // ---- dt transform and the per-tile running sums, before the barrier that publishes the tiles: the same barrier
    // then also publishes whether any column of the workgroup is out of the form's range
    Coef cf;
    cf.A = l_A;
    cf.bias = l_bias;
    const float An = cf.A;
    float dtp[16], dfac[16], pc[16], tt[4];
    lane_dt<true>(p, cf, true, g4, rm, l_raw, dtp, dfac);
    lane_tile_sums(An * LOG2E, cm, g4, rm, dtp, pc, tt);
    {
      const float worst = fmaxf(fmaxf(fabsf(tt[0]), fabsf(tt[1])), fmaxf(fabsf(tt[2]), fabsf(tt[3])));
      const bool bad = !(worst <= SPAN_LIMIT);  // also true for NaN
      const int wbad = __any(bad) ? 1 : 0;
      if (lane == 0) s.bad[wave] = wbad;
    }
    __syncthreads();
    const int4 bd = *(const int4*)s.bad;
    const bool skip = (bd.x | bd.y | bd.z | bd.w) != 0;  // uniform: the whole head is left to the level-hierarchy kernel
    if (tid == 0) redo[(p.dir0 * (int)gridDim.x + wg) * p.hpg + hh] = skip ? 1 : 0;
    const uint16_t* xs_ = s.xs;
    const uint16_t* dys_ = s.dys;
    const uint16_t* tm_ = s.tm;

    float dcs[16], val[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) dcs[k] = val[k] = 0.0f;
    if (!skip) {
      // ---- decay factors and the operand rows
      __builtin_amdgcn_sched_barrier(0);
      float up[16], iup[16];
#pragma unroll
      for (int k = 0; k < 16; ++k) {
        up[k] = ex2(pc[k]);
        iup[k] = ex2(-pc[k]);
      }
      // E(I,J) = exp2(base(I) - base(J)), 0 <= J < I <= 4 (base(0) = 0, base(4) = the chunk's total)
      float bs[5];
      bs[0] = 0.0f;
#pragma unroll
      for (int J = 0; J < 4; ++J) bs[J + 1] = bs[J] + tt[J];
      float E[5][4];
#pragma unroll
      for (int I = 1; I < 5; ++I)
#pragma unroll
        for (int J = 0; J < I; ++J) E[I][J] = ex2(bs[I] - bs[J]);
      auto unpk = [](const unsigned (&a)[8], int k) {
        return __uint_as_float((k & 1) ? (a[k >> 1] & 0xffff0000u) : (a[k >> 1] << 16));
      };
      auto half_of = [](unsigned w, int k) { return __uint_as_float((k & 1) ? (w & 0xffff0000u) : (w << 16)); };
      // Cu = C up (operand of the G blocks), Bi = B dt' iup (operand of the F blocks)
      bf4 Ch[4], Bh[4], Cl[4], Bl[4];
#pragma unroll
      for (int J = 0; J < 4; ++J)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int k = 4 * J + j;
          float cu, bi;
          if constexpr (!BCL) {
            cu = l_Cv[k] * up[k];
            bi = l_Bv[k] * dtp[k] * iup[k];
          } else {  // out of the workgroup's LDS copy of the group's B and C
            cu = half_of(s.bc[(8 + (k >> 1)) * NTHREADS + tid], k) * up[k];
            bi = half_of(s.bc[(k >> 1) * NTHREADS + tid], k) * dtp[k] * iup[k];
          }
          if (SPLIT) {
            cu = trunc16(cu);
            bi = trunc16(bi);
          }
          Ch[J][j] = (__bf16)cu;
          Bh[J][j] = (__bf16)bi;
          if (SPLIT) {
            Cl[J][j] = (__bf16)(cu - (float)Ch[J][j]);  // exact: 16 bits = 8 + 8
            Bl[J][j] = (__bf16)(bi - (float)Bh[J][j]);
          }
        }
      // B (and, for bf16 inputs, C) as the column phase needs them: bf16 inputs are bf16 numbers and stay packed, two
      // to a register
      unsigned bvp[8], cvp[8];
      float bvf[SPLIT ? 16 : 1];
      if constexpr (BCL) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          bvp[i] = s.bc[i * NTHREADS + tid];
          cvp[i] = s.bc[(8 + i) * NTHREADS + tid];
        }
      } else if constexpr (!SPLIT) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          bvp[i] = pack_bf16(l_Bv[2 * i], l_Bv[2 * i + 1]);
          cvp[i] = pack_bf16(l_Cv[2 * i], l_Cv[2 * i + 1]);
        }
      } else {
#pragma unroll
        for (int k = 0; k < 16; ++k) bvf[k] = l_Bv[k];
      }
      __builtin_amdgcn_sched_barrier(0);

      int cq = cm, gq = g4;
      asm volatile("" : "+v"(cq), "+v"(gq));
      // dS and H of the lane's column as (hi, lo) bf16 pairs: the B operands of Q = x . dS and R = dy . H (products over
      // the head dimension, K = 32 per step; k-slot s of step t <-> lane value 8 t + s).  They are fp32 states: the last
      // row's Bd . E1 cancels against the state term g = sum_p dS H_next in d/d(cs), and a dS rounded to 8 bits would
      // leave that difference far above the input rounding.
      bf8 dsh[KT], dsl[KT], hh_[KT], hl_[KT];
#pragma unroll
      for (int t = 0; t < KT; ++t) {
        float a[8], b[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          a[j] = 8 * t + j < KP_ ? l_dsv[(8 * t + j) % KP_] : 0.0f;
          b[j] = 8 * t + j < KP_ ? l_hv[(8 * t + j) % KP_] : 0.0f;
        }
        split8(a, dsh[t], dsl[t]);
        split8(b, hh_[t], hl_[t]);
      }
      unsigned mf[2], mg[2];  // bf16-pair masks of the diagonal block for this lane's four columns 4 g4 + j
#pragma unroll
      for (int w = 0; w < 2; ++w) {
        const int c0 = 4 * gq + 2 * w;
        mf[w] = (c0 <= cq ? 0xffffu : 0u) | (c0 + 1 <= cq ? 0xffff0000u : 0u);
        mg[w] = (c0 >= cq ? 0xffffu : 0u) | (c0 + 1 >= cq ? 0xffff0000u : 0u);
      }
      auto block = [&](uint2 ah, uint2 al, bf4 bh, bf4 bl) -> f4 {
        f4 acc = {0, 0, 0, 0};
        const bf4 a_h = __builtin_bit_cast(bf4, ah);
        if constexpr (SPLIT) {
          // (ah + al) . (bh + bl) in full: the same A fragment against (bl | bh) and (bh | bl).  All four terms, so
          // that F and G see one and the same product dM16 . B16 . C16 for a pair of rows
          const bf8 a2 = cat_bf4(a_h, __builtin_bit_cast(bf4, al));
          acc = mfma_bf(a2, cat_bf4(bl, bh), acc);
          return mfma_bf(a2, cat_bf4(bh, bl), acc);
        } else {
          return mfma_bf16k(a_h, bh, acc);
        }
      };

      // ---- tile by tile: the state terms of the lane's four rows of tile R, the blocks of F and G that end in them,
      // and their share of the column phase.  Row block R of T (rows 16 R + cm) serves the F blocks (R, c <= R) and, T
      // being symmetric, the G blocks (c >= R, R); on the diagonal block F keeps the columns <= the row and G those >= it.
#pragma unroll
      for (int R = 0; R < 4; ++R) {
        f4 xf = {0, 0, 0, 0}, xg = {0, 0, 0, 0};  // the blocks' sums
        f4 sf, sg;                                // the state terms
        {
          f4 q = {0, 0, 0, 0}, r = {0, 0, 0, 0};
#pragma unroll
          for (int t = 0; t < KT; ++t) {
            const bool half = (PT & 1) && t == KT - 1;
            const bf8 xfr = half ? split_frag<LDP, true>(xs_, R * 16 + cq, gq, t) : split_frag<LDP>(xs_, R * 16 + cq, gq, t);
            const bf8 yfr = half ? split_frag<LDP, true>(dys_, R * 16 + cq, gq, t) : split_frag<LDP>(dys_, R * 16 + cq, gq, t);
            q = mfma_bf(xfr, dsl[t], q);
            r = mfma_bf(yfr, hl_[t], r);
            if constexpr (SPLIT) {
              const uint16_t* xl_ = xs_ + CS * LDP;
              const uint16_t* yl_ = dys_ + CS * LDP;
              const bf8 xg_ = half ? split_frag<LDP, true>(xl_, R * 16 + cq, gq, t) : split_frag<LDP>(xl_, R * 16 + cq, gq, t);
              const bf8 yg_ = half ? split_frag<LDP, true>(yl_, R * 16 + cq, gq, t) : split_frag<LDP>(yl_, R * 16 + cq, gq, t);
              q = mfma_bf(xg_, dsh[t], q);
              r = mfma_bf(yg_, hh_[t], r);
            }
            q = mfma_bf(xfr, dsh[t], q);
            r = mfma_bf(yfr, hh_[t], r);
          }
#pragma unroll
          for (int rr = 0; rr < 4; ++rr) {
            sg[rr] = E[4][R] * q[rr];
            sf[rr] = R == 0 ? r[rr] : E[R][0] * r[rr];
          }
        }
        uint2 th[4], tl[4];
        const uint16_t* row = tm_ + (16 * R + cq) * LDM + 4 * gq;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          th[c] = *(const uint2*)(row + 16 * c);
          if (SPLIT) tl[c] = *(const uint2*)(row + CS * LDM + 16 * c);
          else tl[c] = make_uint2(0u, 0u);
        }
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          if (c <= R) {  // F block (R, c)
            uint2 ah = th[c], al = tl[c];
            if (c == R) {
              ah.x &= mf[0]; ah.y &= mf[1];
              al.x &= mf[0]; al.y &= mf[1];
            }
            const f4 acc = block(ah, al, Bh[c], Bl[c]);
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) xf[rr] = c == R ? xf[rr] + acc[rr] : fmaf(E[R][c < R ? c : 0], acc[rr], xf[rr]);
          }
          if (c >= R) {  // G block (c, R)
            uint2 ah = th[c], al = tl[c];
            if (c == R) {
              ah.x &= mg[0]; ah.y &= mg[1];
              al.x &= mg[0]; al.y &= mg[1];
            }
            const f4 acc = block(ah, al, Ch[c], Cl[c]);
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) xg[rr] = c == R ? xg[rr] + acc[rr] : fmaf(E[c > R ? c : 4][R], acc[rr], xg[rr]);
          }
        }
        // The rows' share of the column phase.  d/d(cs) = C X2 - Bd E1 takes the blocks' sums times the operands as the
        // matrix instructions took them: a pair of rows then enters both of its rows as one and the same product and
        // cancels in the suffix sums to fp32 rounding.  The state terms cancel against the state pass's column sums,
        // which were formed from unrounded states: with bf16 inputs they take the unrounded operands (B and C are
        // exact, the decays fp32); with fp32 inputs the 16-bit operands are as accurate as the split products Q and R.
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
          const int k = 4 * R + rr;
          const float bv = SPLIT ? bvf[k] : unpk(bvp, k);
          const float E1 = iup[k] * (sg[rr] + xg[rr]), X2 = up[k] * (sf[rr] + xf[rr]);
          s.dbc[k * NTHREADS + tid] += dtp[k] * E1;
          s.dbc[(16 + k) * NTHREADS + tid] += X2;
          val[k] = bv * E1;
          if constexpr (SPLIT) {
            const float c16 = (float)Ch[R][rr] + (float)Cl[R][rr], b16 = (float)Bh[R][rr] + (float)Bl[R][rr];
            dcs[k] = c16 * (xf[rr] + sf[rr]) - b16 * (xg[rr] + sg[rr]);
          } else {
            const float c16 = (float)Ch[R][rr], b16 = (float)Bh[R][rr];
            dcs[k] = (c16 * xf[rr] - b16 * xg[rr]) + (unpk(cvp, k) * up[k] * sf[rr] - bv * dtp[k] * iup[k] * sg[rr]);
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    pin16(dcs); pin16(val);

    // ---- this direction's predecessor in ddt, then the next head's requests: all of them stay in flight through the
    // rest of this head, which only waits for the predecessor's values (requested before them)
    const float gl_keep = l_gl;
    float old[16];
    if constexpr (ACC) {
      if constexpr (P32) lane_load_ln<false>(p.ddt_part, u.b, u.h, n, true, g4, rm, old);
      else lane_load_ln<IOB>(p.ddt, u.b, u.h, n, true, g4, rm, old);
    }
    request(head_of(min(hh + 1, p.hpg - 1)));  // (unconditional: the last head is requested again and not used)
    __builtin_amdgcn_sched_barrier(0);
    if (skip) {
      // the level-hierarchy kernel adds this head's share to ddt later: it must find the other direction's, or zero
      if constexpr (!ACC) {  // (val is all zero here)
        if constexpr (P32) lane_store_ln<false>(p.ddt_part, u.b, u.h, n, true, g4, rm, val);
        else lane_store_ln<IOB>(p.ddt, u.b, u.h, n, true, g4, rm, val);
      } else if constexpr (P32) {
        lane_store_ln<IOB>(p.ddt, u.b, u.h, n, true, g4, rm, old);  // the other direction's share moves into ddt
      }
      continue;
    }

    // ---- the rest of the column phase: suffix sums over the rows, ddt, the partial sums
    // (fresh opaque lane coordinates: the cross-lane fetch addresses are formed here rather than kept across the loop and
    // reloaded from scratch behind the requests in flight)
    int cm2 = cm, g42 = g4;
    asm volatile("" : "+v"(cm2), "+v"(g42));
    dcs[15] += g42 == 3 ? gl_keep : 0.0f;
    {
      // suffix sums up the 64 rows; the cross-lane steps of the four tiles are issued together
      float c[4], v[4], t[4];
#pragma unroll
      for (int J = 3; J >= 0; --J) {
        float a = 0.0f;
#pragma unroll
        for (int j = 3; j >= 0; --j) {
          a += dcs[4 * J + j];
          dcs[4 * J + j] = a;
        }
        c[J] = a;
      }
#pragma unroll
      for (int J = 0; J < 4; ++J) t[J] = __shfl_down(c[J], 16, 64);
#pragma unroll
      for (int J = 0; J < 4; ++J) v[J] = g42 <= 2 ? c[J] + t[J] : c[J];
#pragma unroll
      for (int J = 0; J < 4; ++J) t[J] = __shfl_down(v[J], 32, 64);
#pragma unroll
      for (int J = 0; J < 4; ++J) v[J] = g42 <= 1 ? v[J] + t[J] : v[J];  // inclusive from the last lane group down
#pragma unroll
      for (int J = 0; J < 4; ++J) t[J] = __shfl(v[J], cm2, 64);           // tile totals
      float carry = 0.0f;  // sum over all rows after the current tile
#pragma unroll
      for (int J = 3; J >= 0; --J) {
        const float add = carry + (v[J] - c[J]);
#pragma unroll
        for (int j = 0; j < 4; ++j) dcs[4 * J + j] += add;
        carry += t[J];
      }
    }
    float sumA = 0.0f, sumB = 0.0f;
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const float da = dcs[k];
      sumA += da * dtp[k];
      val[k] = (val[k] + da * An) * dfac[k];
      sumB += val[k];
    }
    if constexpr (ACC) {
#pragma unroll
      for (int k = 0; k < 16; ++k) val[k] += old[k];
    }
    if constexpr (!ACC && P32) lane_store_ln<false>(p.ddt_part, u.b, u.h, n, true, g4, rm, val);
    else lane_store_ln<IOB>(p.ddt, u.b, u.h, n, true, g4, rm, val);
    sumA = scan_g_incl(sumA, g4);
    sumB = scan_g_incl(sumB, g4);
    if (g4 == 3) {
      // (an opaque copy of the column: the two per-lane addresses are then formed here instead of being kept, as 64-bit
      // values, across the head loop -- a reload from scratch at this point would wait for every request in flight)
      int nq = n;
      asm volatile("" : "+v"(nq));
      partA[vec_off(p, u.bt, u.c, u.h) + nq] = sumA;
      partBias[vec_off(p, u.bt, u.c, u.h) + nq] = sumB;
    }
  }

  {
    float vb[16], vc[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      vb[k] = s.dbc[k * NTHREADS + tid];
      vc[k] = s.dbc[(16 + k) * NTHREADS + tid];
    }
    if (p.dB[u.dir].ptr) lane_store_ln<IOB>(p.dB[u.dir], u.b, u.g, n, true, g4, rm, vb);
    if (p.dC[u.dir].ptr) lane_store_ln<IOB>(p.dC[u.dir], u.b, u.g, n, true, g4, rm, vc);
  }
}

// Whether the tile-base kernel is built for this call (otherwise the level-hierarchy kernel does all the work): complete
// tiles, x / B / C and dt of one type, x and dout rows that allow vector accesses, no gate, ddt wanted, and -- fp32
// inputs with four head tiles would need split x / dy tiles and T that leave one workgroup per CU -- P <= 48 for fp32.
bool bwd_tile_available(const KP& p, const float* dy_ws) {
  if (p.full_tiles != 1 || dy_ws || p.io_dt != p.dt_dt || !p.ddt.ptr) return false;
  if (p.io_dt == 0 && p.P > 48) return false;
  const int es = p.io_dt ? 2 : 4;
  for (int d = 0; d < p.ndir; ++d) {
    const TensorD* ts[2] = {&p.x[d], &p.dout[d]};
    for (const TensorD* t : ts)
      if ((p.P & 3) || ((t->s0 | t->s1 | t->s2) & 3) || (((uintptr_t)t->ptr) & (4 * es - 1))) return false;
  }
  return true;
}

template <int PT, bool IOB>
static int launch_bwd_tile_t(const KP& p, int blocks, const float* states, const float* dstates, const float* dm,
                             const float* g_last, float* partA, float* partBias, int* redo, hipStream_t st) {
  const size_t sm = sizeof(BwdTileSmem<PT, !IOB>);
  const bool pnf = p.P == 16 * PT, acc = p.dir0 > 0;
  auto go = [&](auto kern) -> int {
    if (sm > 64 * 1024)
      if (int e = (int)hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)sm))
        return e;
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(NTHREADS), sm, st, p, states, dstates, dm, g_last, partA, partBias, redo);
    return 0;
  };
  if constexpr (IOB) {
    if (p.ddt_part.ptr) {
      if (pnf) return acc ? go(&k_bwd_tile<PT, IOB, true, true, true>) : go(&k_bwd_tile<PT, IOB, true, false, true>);
      return acc ? go(&k_bwd_tile<PT, IOB, false, true, true>) : go(&k_bwd_tile<PT, IOB, false, false, true>);
    }
  }
  if (pnf) return acc ? go(&k_bwd_tile<PT, IOB, true, true, false>) : go(&k_bwd_tile<PT, IOB, true, false, false>);
  return acc ? go(&k_bwd_tile<PT, IOB, false, true, false>) : go(&k_bwd_tile<PT, IOB, false, false, false>);
}

int launch_bwd_tile(const KP& p, const float* states, const float* dstates, const float* dm, const float* g_last,
                    float* partA, float* partBias, int* redo, hipStream_t st) {
  const int blocks = p.B * p.nc * p.G * (p.N / NS);
  const int pt = (p.P + 15) / 16;
  int e = 0;
  if (p.io_dt) {
    if (pt <= 2) e = launch_bwd_tile_t<2, true>(p, blocks, states, dstates, dm, g_last, partA, partBias, redo, st);
    else if (pt == 3) e = launch_bwd_tile_t<3, true>(p, blocks, states, dstates, dm, g_last, partA, partBias, redo, st);
    else e = launch_bwd_tile_t<4, true>(p, blocks, states, dstates, dm, g_last, partA, partBias, redo, st);
  } else {
    if (pt <= 2) e = launch_bwd_tile_t<2, false>(p, blocks, states, dstates, dm, g_last, partA, partBias, redo, st);
    else e = launch_bwd_tile_t<3, false>(p, blocks, states, dstates, dm, g_last, partA, partBias, redo, st);
  }
  if (e) return e;
  return (int)hipGetLastError();
}

}  // namespace issm
