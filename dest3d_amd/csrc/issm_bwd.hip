// Backward kernels of the ISSM chunked scan for gfx950.
//
//   k_bwd_gate      z-gate backward (elementwise)
//   k_bwd_dstates   dH_c = dy^T (C*exp(cs))  and  dM = tril(dy x^T)
//   k_state_bwd_full / k_state_bwd   reverse inter-chunk recurrence (HBM streaming)
//   k_bwd_chunk     per (chunk, group, 64-column slice), looping over the heads of the
//                   group: ddt, dB, dC and the per-unit partial sums of dA / ddt_bias
//   k_bwd_dx        dx and the per-unit partial sums of dD
//   k_bwd_reduce    fixed-order sums of the partials (bit-reproducible, no atomics), one launch
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
// BF (bf16 inputs): the dy and x tiles are kept as bf16 (exact) and every product runs on the bf16 matrix instruction.
// fp32 inputs: (hi, lo) bf16 pairs of the tiles (hi first), three bf16 instructions per product -- an fp32 matrix
// instruction would keep the vector ALU from issuing while it runs.
template <int PT, bool BF>
struct BwdStSmem {
  static constexpr int NH = BF ? 1 : 2;
  // bf16 tiles [l][p]; four columns of padding instead of eight where the (hi, lo) tiles of four head tiles would
  // otherwise take 55 KB and leave two workgroups per CU instead of three
  static constexpr int LDP = PT * 16 + ((NH == 2 && PT >= 4) ? 4 : 8);
  static constexpr int LDT = CS + 8;        // transposed dy tile [p][l]
  uint16_t dys[NH * CS * LDP];
  uint16_t xs[NH * CS * LDP];
  uint16_t dyt_hi[PT * 16 * LDT];             // dy tile transposed, [p][l]: operand of dH
  uint16_t dyt_lo[BF ? 8 : PT * 16 * LDT];
};

// dH[p][n] = sum_l dy[l][p] * C[l][n] exp2(cs[l][n]): contraction over rows, so the B operand
// comes straight from the registers of the column-lane layout; each wave walks its own 16
// columns of every 64-column slice without any barrier after the dy / x tiles are staged.
template <int PT, bool IOB, bool DTB, bool FULL>
__device__ __forceinline__ void k_bwd_dstates_body(const KP& p, const float* __restrict__ dy_ws, float* __restrict__ dstates, float* __restrict__ dm) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  typedef BwdStSmem<PT, IOB> SM;
  SM& s = *reinterpret_cast<SM*>(smem_raw);
  constexpr int LDP = SM::LDP, LDT = SM::LDT;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int cm = lane & 15, g4 = lane >> 4;
  const Unit u = decode_unit(p, xcd_remap(blockIdx.x, gridDim.x));

  int n = wave * 16 + cm;
  bool vn = FULL || n < p.N;
  RowMap rm;
  Coef cf;
  float raw[16], cv[16];
  if (dstates) {
    rm = make_rowmap<FULL>(p, u, g4, 0);
    lane_load_ln<DTB>(p.dt, u.b, u.h, n, vn, g4, rm, raw);
    cf = lane_coef(p, u.h, n, vn);
    lane_load_ln<IOB>(p.Cm[u.dir], u.b, u.g, n, vn, g4, rm, cv);
  }
  {
    float dv[CS * PT * 16 / NTHREADS], xv[CS * PT * 16 / NTHREADS];
    dy_load<IOB, PT, FULL>(p, u, dy_ws, dv);
    lp_load<IOB, PT, FULL>(p, u, p.x[u.dir], xv);
    if constexpr (IOB) {
      lp_store_bf<PT, LDP>(dv, s.dys, tid);
      lp_store_bf<PT, LDP>(xv, s.xs, tid);
    } else {
      lp_store_split<PT, LDP>(dv, s.dys, s.dys + CS * LDP, tid);
      lp_store_split<PT, LDP>(xv, s.xs, s.xs + CS * LDP, tid);
    }
    if (dstates) lp_store_split_t<PT, LDT, !IOB>(dv, s.dyt_hi, s.dyt_lo);
  }
  __syncthreads();

  if (dm) {
    float* m = dm + sq_off(p, u.bt, u.c, u.h);
    for (int j = 0; j <= wave; ++j) {
      f4 acc = {0, 0, 0, 0};
      constexpr int KT = (PT + 1) / 2;
#pragma unroll
      for (int t = 0; t < KT; ++t) {
        const bool half = (PT & 1) && t == KT - 1;  // an odd number of 16-column tiles: the last step is half full
        auto frag = [&](const uint16_t* tile, int row) {
          return half ? split_frag<LDP, true>(tile, row, g4, t) : split_frag<LDP>(tile, row, g4, t);
        };
        const bf8 a = frag(s.dys, wave * 16 + cm), b = frag(s.xs, j * 16 + cm);
        if constexpr (IOB) acc = mfma_bf(a, b, acc);
        else acc = mfma_split(a, frag(s.dys + CS * LDP, wave * 16 + cm), b, frag(s.xs + CS * LDP, j * 16 + cm), acc);
      }
      {
        // The block goes out as the symmetric bf16 matrix T[i][j] = dM[max(i,j)][min(i,j)] (8 KB at the start of the
        // unit's 16 KB): the F sums of the chunk backward contract over the columns of dM and the G sums over its rows,
        // and with T both are rows of one tile, contiguous for a lane's k-slots.  bf16 inputs: T is dM rounded to
        // bf16.  fp32 inputs: a second matrix of the same shape follows in the next 8 KB with the bf16 rounding of what
        // the first one left, dM = hi + lo to 16 significand bits.
        uint16_t* mb = reinterpret_cast<uint16_t*>(m);
        const int sc = j * 16 + cm, l0 = wave * 16 + 4 * g4;
#pragma unroll
        for (int half = 0; half < (IOB ? 1 : 2); ++half) {
          const unsigned w0 = pack_bf16(acc[0], acc[1]), w1 = pack_bf16(acc[2], acc[3]);
          const uint16_t h[4] = {(uint16_t)w0, (uint16_t)(w0 >> 16), (uint16_t)w1, (uint16_t)(w1 >> 16)};
          if (j < wave) {  // a block below the diagonal blocks: whole, and whole again mirrored
#pragma unroll
            for (int r = 0; r < 4; ++r) mb[(l0 + r) * CS + sc] = h[r];
            *(uint2*)(mb + sc * CS + l0) = make_uint2(w0, w1);
          } else {  // a diagonal block: the lane's entries on or below the diagonal, each mirrored
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              if (sc <= l0 + r) mb[(l0 + r) * CS + sc] = h[r];
              if (sc < l0 + r) mb[sc * CS + l0 + r] = h[r];
            }
          }
#pragma unroll
          for (int r = 0; r < 4; ++r) acc[r] -= bf16_to_f(h[r]);
          mb += CS * CS;
        }
      }
    }
  }
  if (!dstates) return;

  for (int n0 = 0; n0 < p.N; n0 += NS) {
    float ct[16];
    {
      float dtp[16], cs[16], dummy[16];
      lane_prep<false>(p, cf, vn, cm, g4, rm, raw, dtp, cs, dummy);
#pragma unroll
      for (int k = 0; k < 16; ++k) ct[k] = cv[k] * ex2(cs[k]);
    }
    const int n_cur = n;
    const bool vn_cur = vn;
    if (n0 + NS < p.N) {
      n = n0 + NS + wave * 16 + cm;
      vn = FULL || n < p.N;
      rm = make_rowmap<FULL>(p, u, g4, n0 + NS);
      lane_load_ln<DTB>(p.dt, u.b, u.h, n, vn, g4, rm, raw);
      cf = lane_coef(p, u.h, n, vn);
      lane_load_ln<IOB>(p.Cm[u.dir], u.b, u.g, n, vn, g4, rm, cv);
    }
    f4 acc[PT];
#pragma unroll
    for (int pt = 0; pt < PT; ++pt) acc[pt] = (f4){0, 0, 0, 0};
    rows_product_split<PT, LDT, IOB ? 0 : 1>(acc, s.dyt_hi, s.dyt_lo, [&](int k) { return ct[k]; }, cm, g4);
    float* dst = dstates + dst_off(p, u.bt, u.c, u.h);
#pragma unroll
    for (int pt = 0; pt < PT; ++pt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int pp = pt * 16 + 4 * g4 + r;
        if (pp < p.P && vn_cur) dst[(long)pp * p.N + n_cur] = acc[pt][r];
      }
  }
}
template <int PT, bool IOB, bool DTB, bool FULL>
__global__ __launch_bounds__(NTHREADS) void k_bwd_dstates(KP p, const float* __restrict__ dy_ws, float* __restrict__ dstates, float* __restrict__ dm) {
  k_bwd_dstates_body<PT, IOB, DTB, FULL>(p, dy_ws, dstates, dm);
}
// One launch for a sequence whose last chunk is ragged: complete-tile code for the complete chunks, the general code
// for the last one (uniform per workgroup).
template <int PT, bool IOB, bool DTB>
__global__ __launch_bounds__(NTHREADS) void k_bwd_dstates_mixed(KP p, const float* __restrict__ dy_ws, float* __restrict__ dstates, float* __restrict__ dm) {
  if (decode_unit(p, xcd_remap(blockIdx.x, gridDim.x)).c == p.nc - 1) k_bwd_dstates_body<PT, IOB, DTB, false>(p, dy_ws, dstates, dm);
  else k_bwd_dstates_body<PT, IOB, DTB, true>(p, dy_ws, dstates, dm);
}


// ------------------------------------------------------- reverse state passing
// Block = (bt, h, 64 state columns); thread (pg = tid >> 4, nq = tid & 15) carries rows
// p = pg, pg+16, ... of 4 adjacent columns.  dstates[c] holds dH_c on entry and dS_c (gradient
// of the chunk-local end state) on exit.  g_last[c][n] = sum_p dS_c[p,n] * H_{c+1}[p,n].
template <int NQ>
__global__ __launch_bounds__(NTHREADS) void k_state_bwd(KP p, const float* __restrict__ states,
                                                        const float* __restrict__ cs_last,
                                                        float* __restrict__ dstates, float* __restrict__ g_last,
                                                        float* __restrict__ dh0_dir) {
  // NQ column quads per workgroup: NCOL columns, PGN row groups, a thread carries rows pg, pg + PGN, ...
  constexpr int NCOL = NQ * 4, PGN = NTHREADS / NQ, KR = (MAXP + PGN - 1) / PGN;
  __shared__ float red[PGN * NCOL];
  const int nsl = (p.N + NCOL - 1) / NCOL;
  int bid = blockIdx.x;
  const int ns = bid % nsl;
  bid /= nsl;
  const int h = bid % p.H;
  const int bt = bid / p.H;
  const int b = bt / p.ndir, dir = bt % p.ndir;
  const int tid = threadIdx.x, pg = tid / NQ, nq = tid % NQ;
  const int n = ns * NCOL + nq * 4;
  const bool vec = ((p.N & 3) == 0) && (n + 3 < p.N);
  float carry[KR][4];
#pragma unroll
  for (int k = 0; k < KR; ++k) {
    const int pp = pg + PGN * k;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const bool v = pp < p.P && n + j < p.N && p.dfinal[dir];
      carry[k][j] = v ? p.dfinal[dir][(((long)b * p.H + h) * p.P + pp) * p.N + n + j] : 0.0f;
    }
  }
  // operands of one chunk: decay exponent, H_{c+1} and dH_c of the thread's rows
  auto load_chunk = [&](int c, float (&dec)[4], float (&hn)[KR][4], float (&dh)[KR][4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) dec[j] = n + j < p.N ? cs_last[vec_off(p, bt, c, h) + n + j] : 0.0f;
#pragma unroll
    for (int k = 0; k < KR; ++k) {
      const int pp = pg + PGN * k;
      const float* hp = states + st_off(p, bt, c + 1, h) + (long)pp * p.N + n;
      const float* dd = dstates + dst_off(p, bt, c, h) + (long)pp * p.N + n;
      if (vec && pp < p.P) {
        const f4 a = *(const f4*)hp, d = *(const f4*)dd;
#pragma unroll
        for (int j = 0; j < 4; ++j) { hn[k][j] = a[j]; dh[k][j] = d[j]; }
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const bool v = pp < p.P && n + j < p.N;
          hn[k][j] = v ? hp[j] : 0.0f;
          dh[k][j] = v ? dd[j] : 0.0f;
        }
      }
    }
  };
  // The operands of the next two chunks are always in flight (the loads do not depend on the carry), so the
  // recurrence never waits for memory and enough bytes are outstanding to keep HBM busy.
  float dec[4], hn[KR][4], dh[KR][4], dec_1[4], hn_1[KR][4], dh_1[KR][4];
  load_chunk(p.nc - 1, dec, hn, dh);
  if (p.nc > 1) load_chunk(p.nc - 2, dec_1, hn_1, dh_1);
  for (int c = p.nc - 1; c >= 0; --c) {
    float gp[4] = {0, 0, 0, 0};
    float dec_n[4], hn_n[KR][4], dh_n[KR][4];
    if (c > 1) load_chunk(c - 2, dec_n, hn_n, dh_n);
#pragma unroll
    for (int j = 0; j < 4; ++j) dec[j] = __expf(dec[j]);
#pragma unroll
    for (int k = 0; k < KR; ++k) {
      const int pp = pg + PGN * k;
      float* dd = dstates + dst_off(p, bt, c, h) + (long)pp * p.N + n;
      if (vec && pp < p.P) {
        *(f4*)dd = (f4){carry[k][0], carry[k][1], carry[k][2], carry[k][3]};
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (pp < p.P && n + j < p.N) dd[j] = carry[k][j];
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        gp[j] += hn[k][j] * carry[k][j];
        carry[k][j] = dec[j] * carry[k][j] + dh[k][j];
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) red[pg * NCOL + nq * 4 + j] = gp[j];
    __syncthreads();
    if (tid < 64) {
      // 64 lanes over NCOL columns: a lane sums every (64 / NCOL)-th row group of its column, then the lanes of a
      // column (NCOL apart) are added
      constexpr int PARTS = 64 / NCOL;
      const int col = tid % NCOL, part = tid / NCOL;
      float sum = 0.0f;
#pragma unroll
      for (int k = 0; k < PGN / PARTS; ++k) sum += red[(k * PARTS + part) * NCOL + col];
#pragma unroll
      for (int d = NCOL; d < 64; d <<= 1) sum += __shfl_xor(sum, d, 64);
      if (part == 0 && ns * NCOL + col < p.N) g_last[vec_off(p, bt, c, h) + ns * NCOL + col] = sum;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 4; ++j) { dec[j] = dec_1[j]; dec_1[j] = dec_n[j]; }
#pragma unroll
    for (int k = 0; k < KR; ++k)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        hn[k][j] = hn_1[k][j]; dh[k][j] = dh_1[k][j];
        hn_1[k][j] = hn_n[k][j]; dh_1[k][j] = dh_n[k][j];
      }
  }
#pragma unroll
  for (int k = 0; k < KR; ++k) {
    const int pp = pg + PGN * k;
    if (pp >= p.P) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (n + j < p.N) dh0_dir[((((long)dir * p.B + b) * p.H + h) * p.P + pp) * p.N + n + j] = carry[k][j];
  }
}

// The same recurrence for N a multiple of the slice width, with no conditional access anywhere: every load of the
// loop is issued on every path, so the compiler can count the loads still in flight and the prefetched operands of
// the next chunks stay in flight across the barrier (with loads inside branches it waits for all of them before each
// store, which exposes the full memory latency once per chunk; few workgroups walking many chunks -- batch 2, 256
// chunks -- then run at that pace).  A thread owns KM rows, pg + PGN k; for rows past the head dimension it stands in
// for the head's last row: it issues the same loads (so that every load of the loop is unconditional) but stores
// nothing and adds nothing to the column sums -- what a stand-in computes is never used, so it does not matter that
// the row's owner overwrites dH with dS while the stand-in's prefetches of that row are in flight.
template <int NQ, int KM, int R, bool BATCH>
__global__ __launch_bounds__(NTHREADS) void k_state_bwd_full(KP p, const float* __restrict__ states,
                                                             const float* __restrict__ cs_last,
                                                             float* __restrict__ dstates, float* __restrict__ g_last,
                                                             float* __restrict__ dh0_dir) {
  constexpr int NCOL = NQ * 4, PGN = NTHREADS / NQ;
  // The column sums g = sum_p H dS need the rows of all four waves.  Two ways to add them up:
  //  - per step (BATCH = false): every thread leaves its partial sums in local memory and, behind the step's barrier,
  //    the first wave adds each column's PGN of them.  That exchange (local-memory round trips one after the other)
  //    lies on the path from one chunk to the next, which a chip full of workgroups hides: from 256 workgroups on
  //    this form is as fast as the other or up to 10 % faster;
  //  - K steps at once (BATCH = true): the steps only deposit partial sums -- 16 per column: a wave's lanes of one
  //    16-lane row share a column quad, after one in-row rotation for NQ = 8 -- and one thread per (step, column)
  //    adds them behind one barrier per K steps.  With few workgroups walking hundreds of chunks the pace of the
  //    exchange is the run time: 1.3-1.6x faster up to 128 workgroups (batch 2, 256 chunks: 145 -> 110 us).
  // Two buffers, used in turn, either way.
  constexpr int K = !BATCH ? 1 : R * NCOL <= NTHREADS ? R : R / 2;
  static_assert(R % K == 0 && K * NCOL <= NTHREADS && (NQ == 8 || NQ == 16), "batches of K steps tile the ring");
  __shared__ __align__(16) float red2[2][BATCH ? K * NCOL * 16 : PGN * NCOL];
  int par = 0;
  const int nsl = p.N / NCOL;
  int bid = blockIdx.x;
  const int ns = bid % nsl;
  bid /= nsl;
  const int h = bid % p.H;
  const int bt = bid / p.H;
  const int b = bt / p.ndir, dir = bt % p.ndir;
  const int tid = threadIdx.x, pg = tid / NQ, nq = tid % NQ;
  const int n = ns * NCOL + nq * 4;
  const int part = (tid >> 6) * 4 + ((tid & 63) >> 4);  // (wave, 16-lane row): which of a column's 16 partial sums
  const bool deposits = NQ == 16 || !(tid & 8);
  long rowk[KM];   // offsets of the thread's rows
  bool own[KM];    // a row of its own (stores, takes part in the column sums) or a stand-in (loads only)
#pragma unroll
  for (int k = 0; k < KM; ++k) {
    rowk[k] = (long)min(pg + PGN * k, p.P - 1) * p.N + n;
    own[k] = pg + PGN * k < p.P;
  }
  const long cstep = (long)p.H * p.P * p.N, vstep = (long)p.H * p.N;  // from chunk to chunk
  f4 carry[KM];
#pragma unroll
  for (int k = 0; k < KM; ++k) {
    carry[k] = (f4){0, 0, 0, 0};
    if (p.dfinal[dir]) carry[k] = *(const f4*)(p.dfinal[dir] + ((long)b * p.H + h) * p.P * p.N + rowk[k]);
  }
  const float* hp = states + st_off(p, bt, p.nc, h);      // H_{c+1}, c = nc - 1
  float* dd = dstates + dst_off(p, bt, p.nc - 1, h);      // dH_c in, dS_c out
  const float* cl = cs_last + vec_off(p, bt, p.nc - 1, h) + n;
  float* gl = g_last + vec_off(p, bt, p.nc - 1, h) + ns * NCOL;  // of the first step of the current batch
  // Operands of R chunks in R register slots: the one being used and the next R - 1, the last of which is requested
  // at the top of a step (the final steps request chunk 0 again: in range, unused).  Step j = nc-1-c uses slot
  // j % R; the loop is unrolled over the slots so that none is ever copied (a copy would wait for its load).
  f4 dec[R], hn[R][KM], dh[R][KM];
  auto request = [&](int slot, int back_chunks) {
    const long back = (long)back_chunks * cstep;
    dec[slot] = *(const f4*)(cl - (long)back_chunks * vstep);
#pragma unroll
    for (int k = 0; k < KM; ++k) {
      hn[slot][k] = *(const f4*)(hp - back + rowk[k]);
      dh[slot][k] = *(const f4*)(dd - back + rowk[k]);
    }
  };
#pragma unroll
  for (int i = 0; i < R - 1; ++i) request(i, min(i, p.nc - 1));
  auto step = [&](int cur, int pre, int c) {
    request(pre, min(c, R - 1));
    f4 gp = {0, 0, 0, 0}, e;
#pragma unroll
    for (int j = 0; j < 4; ++j) e[j] = __expf(dec[cur][j]);
#pragma unroll
    for (int k = 0; k < KM; ++k) {
      if (own[k]) *(f4*)(dd + rowk[k]) = carry[k];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        gp[j] += own[k] ? hn[cur][k][j] * carry[k][j] : 0.0f;
        carry[k][j] = e[j] * carry[k][j] + dh[cur][k][j];
      }
    }
    if (!BATCH) {
      *(f4*)(red2[par] + pg * NCOL + nq * 4) = gp;
    } else {
      if (NQ == 8) {
        // lanes l and l ^ 8 of a 16-lane row hold the same column quad: rotate the row by 8 and add
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float own_sum = gp[j];  // a scalar copy: the bit cast below must not be applied to a vector element
          gp[j] = own_sum + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
                                                          0, __builtin_bit_cast(int, own_sum), 0x128, 0xf, 0xf, false));
        }
      }
      if (deposits) {
        // the 16 partial sums of a column are added in the order of their places, whatever lane filled them: the
        // place is rotated by the column so that a wave's stores spread over the banks
        float* red = red2[par] + ((cur % K) * NCOL + nq * 4) * 16;
#pragma unroll
        for (int j = 0; j < 4; ++j) red[j * 16 + ((part + nq * 4 + j) & 15)] = gp[j];
      }
    }
    hp -= cstep; dd -= cstep; cl -= vstep;
  };
  // The column sums of the batch's first cnt steps: thread = (step, column).
  auto add_up = [&](int cnt) {
    __syncthreads();  // the other buffer is filled next; this one again after the next barrier
    if (!BATCH) {
      if (tid < 64) {
        // 64 lanes over NCOL columns: a lane sums every (64 / NCOL)-th row group of its column, then the lanes of a
        // column (NCOL apart) are added
        constexpr int PARTS = 64 / NCOL;
        const int col = tid % NCOL, prt = tid / NCOL;
        const float* red = red2[par];
        float sum = 0.0f;
#pragma unroll
        for (int k = 0; k < PGN / PARTS; ++k) sum += red[(k * PARTS + prt) * NCOL + col];
#pragma unroll
        for (int d = NCOL; d < 64; d <<= 1) sum += __shfl_xor(sum, d, 64);
        if (prt == 0) gl[col] = sum;
      }
    } else if (tid < cnt * NCOL) {
      const f4* r = (const f4*)(red2[par] + tid * 16);
      const f4 a = r[0], b4 = r[1], c4 = r[2], d4 = r[3];
      const f4 s4 = (a + b4) + (c4 + d4);
      gl[-(long)(tid / NCOL) * vstep + tid % NCOL] = (s4[0] + s4[1]) + (s4[2] + s4[3]);
    }
    gl -= (long)cnt * vstep;
    par ^= 1;
  };
  int c = p.nc - 1;
  for (; c >= R - 1; c -= R) {
#pragma unroll
    for (int i = 0; i < R; ++i) {
      step(i, (i + R - 1) % R, c - i);
      if ((i + 1) % K == 0) add_up(K);
    }
  }
#pragma unroll
  for (int i = 0; i < R - 1; ++i) {  // uniform: the last nc % R chunks
    if (c - i >= 0) {
      step(i, (i + R - 1) % R, c - i);
      if ((i + 1) % K == 0) add_up(K);
      else if (c - i == 0) add_up(i % K + 1);
    }
  }
#pragma unroll
  for (int k = 0; k < KM; ++k)
    if (own[k]) *(f4*)(dh0_dir + (((long)dir * p.B + b) * p.H + h) * p.P * p.N + rowk[k]) = carry[k];
}

// -------------------------------------------------------------- chunk backward
// Workgroup = (batch, chunk, group, 64 state columns) of one direction, looping over the heads of
// the group.  Column-lane layout: cumulative sums, decays, level operands, E1, X2 and the suffix
// sums live in registers of one lane; only x, dy and dM (shared by the four waves) go through LDS.
template <int PT>
struct BwdChunkSmem {
  static constexpr int KW = 16 * PT;  // stored width; the K = 32 steps read missing columns as zero
  // Four head tiles (P > 48): the dM tile takes the place of the x tile once the products over the head dimension
  // are done, which keeps the workgroup under half of the CU's LDS (two workgroups per CU instead of one).
  static constexpr bool DM_OVER_X = PT > 3;
  SplitTile<KW> xs;   // x tile [l][p] as bf16 (hi, lo)
  SplitTile<KW> dys;  // dy tile
  float dms_own[DM_OVER_X ? 4 : CS * LDC];
  float dbc[32 * NTHREADS];  // per-lane dB / dC accumulators [k][tid]
  __device__ __forceinline__ float* dms() { return DM_OVER_X ? reinterpret_cast<float*>(&xs) : dms_own; }
};
static_assert(sizeof(SplitTile<64>) >= CS * LDC * sizeof(float), "the dM tile must fit in the x tile's place");

// F[l] = sum_{s<=l} dM[l,s] Bd[s] exp2(cs[l]-cs[s]) and G[s] = sum_{l>=s} dM[l,s] C[l] exp2(cs[l]-cs[s]) per state
// column, accumulated into x2 (F) and e1 (G).  A pair (l > s) is handled at the level w = highest set
// bit of (l xor s); the lane's rows are 16J + 4 g4 + j, so
//   w = 32, 16  ->  the pair lies in different 16-row tiles: role (upper / lower half of the 2w-block)
//                   is a compile-time function of J;
//   w = 8, 4    ->  same tile, different lane groups g4: role depends on g4;
//   w = 2, 1, 0 ->  both rows belong to the same lane: evaluated directly, one exp2 per pair.
// At the levels >= 4 a row contributes  op = Bd * exp2(ref - cs)  if it is in the lower half of its
// block and  op = C * exp2(cs - ref)  if it is in the upper half (ref = cs of the last row of the lower
// half): both factors are <= 1.

// Levels 32 (LV = 5) and 16 (LV = 4): products of 16x16 blocks of dM with the operand rows.
template <int LV>
__device__ __forceinline__ void bwd_big_level(const float (&cs)[16], const float (&Bd)[16], const float (&Cv)[16],
                                              const float* __restrict__ dms, float (&e1)[16], float (&x2)[16], int cm,
                                              int g4) {
  float op[16], ee[16];
  // reference rows: one cross-lane fetch (level 32) or two (level 16), before anything waits for them
  const float ref_a = __shfl(LV == 4 ? cs[3] : cs[7], cm + 48, 64);
  const float ref_b = LV == 4 ? __shfl(cs[11], cm + 48, 64) : ref_a;
#pragma unroll
  for (int J = 0; J < 4; ++J) {
    const float ref = (J & 2) ? ref_b : ref_a;
    const bool upper = LV == 4 ? (J & 1) : (J & 2);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = 4 * J + j;
      const float e = ex2(upper ? cs[k] - ref : ref - cs[k]);
      ee[k] = e;
      op[k] = (upper ? Cv[k] : Bd[k]) * e;
    }
  }
#pragma unroll
  for (int I = 0; I < 4; ++I) {
    f4 acc = {0, 0, 0, 0};
    if (LV == 5) {
      if (I >= 2) {  // F: rows of tiles 2,3 gather from the lower rows s in tiles 0,1
        const f4 av0 = *(const f4*)(dms + (I * 16 + cm) * LDC + 4 * g4);
        const f4 av1 = *(const f4*)(dms + (I * 16 + cm) * LDC + 16 + 4 * g4);
#pragma unroll
        for (int j = 0; j < 4; ++j) acc = mfma4(av0[j], op[j], acc);
#pragma unroll
        for (int j = 0; j < 4; ++j) acc = mfma4(av1[j], op[4 + j], acc);
      } else {  // G: rows of tiles 0,1 gather from the upper rows l in tiles 2,3 (all eight reads first)
        float a8[8];
#pragma unroll
        for (int J = 2; J < 4; ++J)
#pragma unroll
          for (int j = 0; j < 4; ++j) a8[4 * (J - 2) + j] = dms[(J * 16 + 4 * g4 + j) * LDC + I * 16 + cm];
#pragma unroll
        for (int J = 2; J < 4; ++J)
#pragma unroll
          for (int j = 0; j < 4; ++j) acc = mfma4(a8[4 * (J - 2) + j], op[4 * J + j], acc);
      }
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) {
        if (I >= 2) x2[4 * I + rr] += ee[4 * I + rr] * acc[rr];
        else e1[4 * I + rr] += ee[4 * I + rr] * acc[rr];
      }
    } else {
      if (I & 1) {
        const f4 av = *(const f4*)(dms + (I * 16 + cm) * LDC + (I - 1) * 16 + 4 * g4);
#pragma unroll
        for (int j = 0; j < 4; ++j) acc = mfma4(av[j], op[4 * (I - 1) + j], acc);
      } else {
        const float* ap = dms + ((I + 1) * 16 + 4 * g4) * LDC + I * 16 + cm;
#pragma unroll
        for (int j = 0; j < 4; ++j) acc = mfma4(ap[j * LDC], op[4 * (I + 1) + j], acc);
      }
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) {
        if (I & 1) x2[4 * I + rr] += ee[4 * I + rr] * acc[rr];
        else e1[4 * I + rr] += ee[4 * I + rr] * acc[rr];
      }
    }
  }
}

// Levels 8 (LV = 3) and 4 (LV = 2), inside a diagonal 16x16 tile.  With T_w[i][j] = dM[max(i,j)][min(i,j)] if
// the pair (i, j) belongs to level w and 0 otherwise (a symmetric matrix), Z = T_w . op holds the F sum on
// the upper rows and the G sum on the lower rows: one product serves both, and no operand needs masking,
// because T_w pairs an upper row only with lower rows of its block and vice versa.
template <int LV>
__device__ __forceinline__ void bwd_mid_level(const float (&cs)[16], const float (&Bd)[16], const float (&Cv)[16],
                                              const float* __restrict__ dms, float (&e1)[16], float (&x2)[16], int cm,
                                              int g4) {
  const bool up = LV == 2 ? (g4 & 1) : (g4 & 2);  // role of the lane's rows 4 g4 + j
  const float upf = up ? 1.0f : 0.0f, lof = up ? 0.0f : 1.0f;
  // A operand: row i = cm of T_w, columns kk = 4 g4 + jj.  Non-zero only where (i, kk) is a level-w pair.
  const int cg = cm >> 2;
  const bool iup = LV == 2 ? (cg & 1) : (cg & 2);
  const bool nz = LV == 2 ? (g4 == (cg ^ 1)) : ((g4 >> 1) != (cg >> 1));
  const int a_base = iup ? cm * LDC + 4 * g4 : 4 * g4 * LDC + cm;  // dM[i][kk] (i upper) or dM[kk][i] (i lower)
  const int a_step = iup ? 1 : LDC;
  float op[16], ee[16], refs[4];
#pragma unroll
  for (int J = 0; J < 4; ++J)  // the four cross-lane fetches together
    refs[J] = LV == 2 ? __shfl(cs[4 * J + 3], cm + 16 * (g4 & 2), 64) : __shfl(cs[4 * J + 3], cm + 16, 64);
#pragma unroll
  for (int J = 0; J < 4; ++J) {
    const float ref = refs[J];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = 4 * J + j;
      const float d = cs[k] - ref;
      const float e = ex2(up ? d : -d);
      ee[k] = e;
      op[k] = (up ? Cv[k] : Bd[k]) * e;
    }
  }
  // all 16 dM values first, then the products: read one by one, each read's LDS latency would sit in front of its
  // matrix instruction (two waves per SIMD do not hide it)
  float av[16];
#pragma unroll
  for (int I = 0; I < 4; ++I)
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) av[4 * I + jj] = dms[I * (16 * LDC + 16) + a_base + jj * a_step];
#pragma unroll
  for (int I = 0; I < 4; ++I) {
    f4 acc = {0, 0, 0, 0};
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) acc = mfma4(nz ? av[4 * I + jj] : 0.0f, op[4 * I + jj], acc);
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
      const float v = ee[4 * I + rr] * acc[rr];
      x2[4 * I + rr] = fmaf(v, upf, x2[4 * I + rr]);
      e1[4 * I + rr] = fmaf(v, lof, e1[4 * I + rr]);
    }
  }
}

// Levels 2, 1 and the diagonal: the pairs inside each group of four consecutive rows owned by the lane.
__device__ __forceinline__ void bwd_small_levels(const float (&cs)[16], const float (&Bd)[16], const float (&Cv)[16],
                                                 const float* __restrict__ dms, float (&e1)[16], float (&x2)[16],
                                                 int g4) {
#pragma unroll
  for (int J = 0; J < 4; ++J) {
    const float* blk = dms + (16 * J + 4 * g4) * LDC + 16 * J + 4 * g4;  // dM[row jl][col js] of the group
    f4 m[4];
#pragma unroll
    for (int jl = 0; jl < 4; ++jl) m[jl] = *(const f4*)(blk + jl * LDC);
#pragma unroll
    for (int jl = 0; jl < 4; ++jl) {
      const int kl = 4 * J + jl;
      e1[kl] = fmaf(m[jl][jl], Cv[kl], e1[kl]);
      x2[kl] = fmaf(m[jl][jl], Bd[kl], x2[kl]);
#pragma unroll
      for (int js = 0; js < jl; ++js) {
        const int ks = 4 * J + js;
        const float wgt = m[jl][js] * ex2(cs[kl] - cs[ks]);
        e1[ks] = fmaf(wgt, Cv[kl], e1[ks]);
        x2[kl] = fmaf(wgt, Bd[ks], x2[kl]);
      }
    }
  }
}

// partA, partBias: (Bt*nc, H, N) per-unit partial sums of dA and ddt_bias
template <int PT, bool IOB, bool DTB, bool FULL>
__device__ __forceinline__ void k_bwd_chunk_body(const KP& p, const float* __restrict__ dy_ws, const float* __restrict__ states, const float* __restrict__ dstates, const float* __restrict__ dm, const float* __restrict__ g_last, float* __restrict__ partA, float* __restrict__ partBias, const int* __restrict__ redo, const int dir_here, const bool mirror) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  typedef BwdChunkSmem<PT> SM;
  SM& s = *reinterpret_cast<SM*>(smem_raw);
  constexpr int KW = SM::KW, LDS_ = SplitTile<KW>::LD, KT = (PT + 1) / 2;
  constexpr int KP_ = PT * 4;  // dS / H values per lane
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int cm = lane & 15, g4 = lane >> 4;
  const int nsl = (p.N + NS - 1) / NS;
  Unit u;
  // `redo` (one word per direction, workgroup and head, written by the tile-base kernel): only the marked heads are
  // evaluated here, and their ddt / dB / dC are added to what that kernel left (zero, or the other direction's share).
  // `mirror`: the workgroup's chunk index counts from the other end -- the chunk of this direction that covers the
  // same tokens as the un-mirrored chunk of the other direction (one workgroup then adds both directions' shares to
  // those tokens' ddt one after the other, and no two workgroups ever update one address).
  int id = xcd_remap(blockIdx.x, gridDim.x);
  const int ns = id % nsl;
  id /= nsl;
  u.g = id % p.G;
  id /= p.G;
  const int cj = id % p.ncl;
  u.c = p.c_lo + (mirror ? p.ncl - 1 - cj : cj);
  u.b = id / p.ncl;
  if (redo) {
    const int nblk = p.B * p.ncl * p.G * nsl;
    const int wg = ((u.b * p.ncl + (u.c - p.c_lo)) * p.G + u.g) * nsl + ns;  // as the tile-base kernel counts them
    redo += (dir_here * nblk + wg) * p.hpg;
    int any = 0;
    for (int hh = 0; hh < p.hpg; ++hh) any |= redo[hh];
    if (!any) return;
  }
  u.dir = dir_here;
  u.bt = u.b * p.ndir + u.dir;
  u.h = u.g * p.hpg;
  const int n = ns * NS + wave * 16 + cm;
  const bool vn = FULL || n < p.N;

  // rows past the end of the sequence and absent columns: lane_row(k) >= lim
  const RowMap rm = make_rowmap<FULL>(p, u, g4, ns * NS);
  const int lim = vn ? rm.nvalid - 4 * g4 : 0;
  auto rowk = [&](int k) { return 16 * (k >> 2) + (k & 3); };
  const bool pn_full = FULL && p.P == PT * 16;

  float Bv[16], Cv[16];
  lane_load_ln<IOB>(p.Bm[u.dir], u.b, u.g, n, vn, g4, rm, Bv);
  lane_load_ln<IOB>(p.Cm[u.dir], u.b, u.g, n, vn, g4, rm, Cv);
  // dB / dC accumulators over the heads of the group: private to the lane, kept in LDS
#pragma unroll
  for (int k = 0; k < 16; ++k) s.dbc[k * NTHREADS + tid] = s.dbc[(16 + k) * NTHREADS + tid] = 0.0f;

  for (int hh = 0; hh < p.hpg; ++hh) {
    if (redo && !redo[hh]) continue;
    // the reversed direction's launch follows the forward one's and shares dt, x, B, C and ddt with it: it walks the
    // heads backwards, so what the first launch touched last (and the last-level cache still holds) is read first
    u.h = u.g * p.hpg + (dir_here ? p.hpg - 1 - hh : hh);
    // ---- global loads of this head
    float raw[16], dsv[KP_], hv[KP_];
    lane_load_ln<DTB>(p.dt, u.b, u.h, n, vn, g4, rm, raw);
    const Coef cf = lane_coef(p, u.h, n, vn);
    const float gl = (g4 == 3 && vn) ? g_last[vec_off(p, u.bt, u.c, u.h) + n] : 0.0f;
    lane_load_pn<KP_>(dstates + dst_off(p, u.bt, u.c, u.h), p.P, p.N, n, vn, g4, pn_full, dsv);
    lane_load_pn<KP_>(states + st_off(p, u.bt, u.c, u.h), p.P, p.N, n, vn, g4, pn_full, hv);
    f4 mkeep[SM::DM_OVER_X ? 4 : 1];  // the thread's part of the dM tile until the x tile's place is free
    {
      float xv[CS * PT * 16 / NTHREADS], dv[CS * PT * 16 / NTHREADS];
      f4 mv[4];
      int tq = tid;
      asm volatile("" : "+v"(tq));
      dy_load<IOB, PT, FULL>(p, u, dy_ws, dv, tq);
      lp_load<IOB, PT, FULL>(p, u, p.x[u.dir], xv, tq);
      tril_load_hl(dm + sq_off(p, u.bt, u.c, u.h), mv, tq);
      __syncthreads();  // the previous head no longer reads the LDS tiles
      lp_store_split<PT, LDS_>(dv, s.dys.hi, s.dys.lo, tq);
      lp_store_split<PT, LDS_>(xv, s.xs.hi, s.xs.lo, tq);
      if constexpr (!SM::DM_OVER_X) tril_store(mv, s.dms(), tq);
      else {
#pragma unroll
        for (int v = 0; v < 4; ++v) mkeep[v] = mv[v];
      }
    }
    __syncthreads();

    // ---- dt transform and running sum down the chunk (log2 domain)
    const float An = cf.A;
    float dtp[16], cs[16], dfac[16];
    float last;
    {
      last = lane_prep<true>(p, cf, vn, cm, g4, rm, raw, dtp, cs, dfac);
    }
    float Bd[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) Bd[k] = Bv[k] * dtp[k];
    pin16(cs); pin16(Bd);

    // ---- Q, R, diagonal terms.  e1 / x2 [I][r] <-> row 16I + 4 g4 + r <-> index k = 4I + r
    // (LDS fragment addresses are derived from per-head opaque copies of the lane coordinates so that
    // they are recomputed instead of being kept live across the whole head loop)
    int cq = cm, gq = g4;
    asm volatile("" : "+v"(cq), "+v"(gq));
    float e1[16], x2[16];
    {
      // Q = x . dS and R = dy . H contract over the head dimension: split-bf16 products, K = 32 per step.
      // k-slot s of step t <-> lane value q = 8 t + s <-> p = 16 (q >> 2) + 4 g4 + (q & 3).
      // (Q first, then R: only one pair of split operands is live at a time)
      auto product = [&](const float (&v)[KP_], const uint16_t* thi, const uint16_t* tlo, f4 (&res)[4]) {
        bf8 bh[KT], bl[KT];
#pragma unroll
        for (int t = 0; t < KT; ++t) {
          float a[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) a[j] = 8 * t + j < KP_ ? v[(8 * t + j) % KP_] : 0.0f;
          split8(a, bh[t], bl[t]);
        }
#pragma unroll
        for (int I = 0; I < 4; ++I) {
          res[I] = (f4){0, 0, 0, 0};
#pragma unroll
          for (int t = 0; t < KT; ++t) {
            // the last step of an odd number of 16-column tiles has only its first half
            const bool half = (PT & 1) && t == KT - 1;
            const bf8 ah = half ? split_frag<LDS_, true>(thi, I * 16 + cq, gq, t) : split_frag<LDS_>(thi, I * 16 + cq, gq, t);
            const bf8 al = half ? split_frag<LDS_, true>(tlo, I * 16 + cq, gq, t) : split_frag<LDS_>(tlo, I * 16 + cq, gq, t);
            res[I] = mfma_split(ah, al, bh[t], bl[t], res[I]);
          }
        }
      };
      if constexpr (KT == 1) {
        // one K step: both products interleaved (two independent accumulation chains)
        float a[8], b[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) { a[j] = dsv[j]; b[j] = hv[j]; }
        bf8 dsh, dsl, hh_, hl_;
        split8(a, dsh, dsl);
        split8(b, hh_, hl_);
#pragma unroll
        for (int I = 0; I < 4; ++I) {
          const bf8 xh = split_frag<LDS_>(s.xs.hi, I * 16 + cq, gq, 0), xl = split_frag<LDS_>(s.xs.lo, I * 16 + cq, gq, 0);
          const bf8 yh = split_frag<LDS_>(s.dys.hi, I * 16 + cq, gq, 0), yl = split_frag<LDS_>(s.dys.lo, I * 16 + cq, gq, 0);
          const f4 q = mfma_split(xh, xl, dsh, dsl, (f4){0, 0, 0, 0});
          const f4 r = mfma_split(yh, yl, hh_, hl_, (f4){0, 0, 0, 0});
#pragma unroll
          for (int rr = 0; rr < 4; ++rr) {
            e1[4 * I + rr] = ex2(last - cs[4 * I + rr]) * q[rr];
            x2[4 * I + rr] = ex2(cs[4 * I + rr]) * r[rr];
          }
        }
      } else {
        f4 q[4];
        product(dsv, s.xs.hi, s.xs.lo, q);
#pragma unroll
        for (int I = 0; I < 4; ++I)
#pragma unroll
          for (int rr = 0; rr < 4; ++rr) e1[4 * I + rr] = ex2(last - cs[4 * I + rr]) * q[I][rr];
        product(hv, s.dys.hi, s.dys.lo, q);
#pragma unroll
        for (int I = 0; I < 4; ++I)
#pragma unroll
          for (int rr = 0; rr < 4; ++rr) x2[4 * I + rr] = ex2(cs[4 * I + rr]) * q[I][rr];
      }
    }

    if constexpr (SM::DM_OVER_X) {
      __syncthreads();  // every wave is done with the x tile
      int tq = tid;
      asm volatile("" : "+v"(tq));
      tril_store(mkeep, s.dms(), tq);
      __syncthreads();
    }
    // ---- hierarchy levels of F and G; scheduling barriers keep one level's operands live at a time
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" : "+v"(cq), "+v"(gq));
    pin16(cs); pin16(e1); pin16(x2);
    bwd_big_level<5>(cs, Bd, Cv, s.dms(), e1, x2, cq, gq);
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" : "+v"(cq), "+v"(gq));
    pin16(cs); pin16(e1); pin16(x2);
    bwd_big_level<4>(cs, Bd, Cv, s.dms(), e1, x2, cq, gq);
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" : "+v"(cq), "+v"(gq));
    pin16(cs); pin16(e1); pin16(x2);
    bwd_mid_level<3>(cs, Bd, Cv, s.dms(), e1, x2, cq, gq);
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" : "+v"(cq), "+v"(gq));
    pin16(cs); pin16(e1); pin16(x2);
    bwd_mid_level<2>(cs, Bd, Cv, s.dms(), e1, x2, cq, gq);
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" : "+v"(cq), "+v"(gq));
    pin16(cs); pin16(e1); pin16(x2);
    // the second direction adds to the first one's ddt: fetch it while the last levels run
    float old[16];
    if ((redo || dir_here > 0) && p.ddt.ptr) lane_load_ln<DTB>(p.ddt, u.b, u.h, n, vn, g4, rm, old);
    __builtin_amdgcn_sched_barrier(0);
    bwd_small_levels(cs, Bd, Cv, s.dms(), e1, x2, gq);
    __builtin_amdgcn_sched_barrier(0);

    // ---- column phase: everything below is local to the lane except the scans over rows
    pin16(e1); pin16(x2);
    float dcs[16], val[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const float E1 = e1[k], X2 = x2[k];
      s.dbc[k * NTHREADS + tid] += dtp[k] * E1;
      s.dbc[(16 + k) * NTHREADS + tid] += X2;
      val[k] = Bv[k] * E1;
      dcs[k] = Cv[k] * X2 - Bd[k] * E1;
    }
    dcs[15] += gl;
    {
      // suffix sums up the 64 rows; the cross-lane steps of the four tiles are issued together (see lane_prep)
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
      for (int J = 0; J < 4; ++J) v[J] = g4 <= 2 ? c[J] + t[J] : c[J];
#pragma unroll
      for (int J = 0; J < 4; ++J) t[J] = __shfl_down(v[J], 32, 64);
#pragma unroll
      for (int J = 0; J < 4; ++J) v[J] = g4 <= 1 ? v[J] + t[J] : v[J];  // inclusive from the last lane group down
#pragma unroll
      for (int J = 0; J < 4; ++J) t[J] = __shfl(v[J], cm, 64);           // tile totals
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
      if (rm.full || rowk(k) < lim) sumB += val[k];
      if (redo || dir_here > 0) val[k] += old[k];
    }
    if (p.ddt.ptr) lane_store_ln<DTB>(p.ddt, u.b, u.h, n, vn, g4, rm, val);
    sumA = scan_g_incl(sumA, g4);
    sumB = scan_g_incl(sumB, g4);
    if (g4 == 3 && vn) {
      partA[vec_off(p, u.bt, u.c, u.h) + n] = sumA;
      partBias[vec_off(p, u.bt, u.c, u.h) + n] = sumB;
    }
  }

  {
    float vb[16], vc[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      vb[k] = s.dbc[k * NTHREADS + tid];
      vc[k] = s.dbc[(16 + k) * NTHREADS + tid];
    }
    if (redo) {
      float ob[16], oc[16];
      if (p.dB[u.dir].ptr) lane_load_ln<IOB>(p.dB[u.dir], u.b, u.g, n, vn, g4, rm, ob);
      if (p.dC[u.dir].ptr) lane_load_ln<IOB>(p.dC[u.dir], u.b, u.g, n, vn, g4, rm, oc);
#pragma unroll
      for (int k = 0; k < 16; ++k) {
        vb[k] += ob[k];
        vc[k] += oc[k];
      }
    }
    if (p.dB[u.dir].ptr) lane_store_ln<IOB>(p.dB[u.dir], u.b, u.g, n, vn, g4, rm, vb);
    if (p.dC[u.dir].ptr) lane_store_ln<IOB>(p.dC[u.dir], u.b, u.g, n, vn, g4, rm, vc);
  }
}
template <int PT, bool IOB, bool DTB, bool FULL>
__global__ __launch_bounds__(NTHREADS, 2) void k_bwd_chunk(KP p, const float* __restrict__ dy_ws, const float* __restrict__ states, const float* __restrict__ dstates, const float* __restrict__ dm, const float* __restrict__ g_last, float* __restrict__ partA, float* __restrict__ partBias, const int* __restrict__ redo, int ndirs) {
  // (ndirs > 1 only with `redo`: the marked heads of directions p.dir0, p.dir0 + 1, .. one after the other)
  for (int d = 0; d < ndirs; ++d) {
    if (d) __syncthreads();
    k_bwd_chunk_body<PT, IOB, DTB, FULL>(p, dy_ws, states, dstates, dm, g_last, partA, partBias, redo, p.dir0 + d, d > 0);
  }
}
// One launch for a sequence whose last chunk is ragged: complete-tile code for the complete chunks, the general code
// for the last one (uniform per workgroup).
template <int PT, bool IOB, bool DTB>
__global__ __launch_bounds__(NTHREADS, 2) void k_bwd_chunk_mixed(KP p, const float* __restrict__ dy_ws, const float* __restrict__ states, const float* __restrict__ dstates, const float* __restrict__ dm, const float* __restrict__ g_last, float* __restrict__ partA, float* __restrict__ partBias) {
  if (p.c_lo + (xcd_remap(blockIdx.x, gridDim.x) / ((p.N + NS - 1) / NS) / p.G) % p.ncl == p.nc - 1) k_bwd_chunk_body<PT, IOB, DTB, false>(p, dy_ws, states, dstates, dm, g_last, partA, partBias, nullptr, p.dir0, false);
  else k_bwd_chunk_body<PT, IOB, DTB, true>(p, dy_ws, states, dstates, dm, g_last, partA, partBias, nullptr, p.dir0, false);
}


// ------------------------------------------------- chunk backward, bf16 inputs
// The same computation for bf16 x / B / C / dy: every matrix product runs on v_mfma_f32_16x16x32_bf16 with operands
// rounded once to bf16 (the reference casts its dot operands to the input dtype as well, issm_cabt_bmm.py:42-43;
// running sums, decays, states and all accumulation stay fp32).  x and dy are bf16 already, so their tiles are exact
// copies; dM arrives from k_bwd_dstates as the symmetric bf16 matrix T[i][j] = dM[max(i,j)][min(i,j)]: the F sums
// contract over the columns of dM and the G sums over its rows, and in T both are rows, contiguous for a lane's k-slots.
// The tiles of a head are requested at the top of its turn, behind its column operands, and copied to LDS as raw
// bf16.  (Holding the next head's tiles in registers while the levels run -- two sets of tiles in LDS, one barrier per
// head -- was 1 - 2 % faster as long as there were registers for it; the d/d(cs) accumulator below has taken them.)
template <int PT>
struct BwdChunkBfSmem {
  static constexpr int KW = 16 * PT, LDP = KW + 8;  // x / dy tiles [l][p]
  static constexpr int LDM = CS + 8;                // dM tile [row][col]
  uint16_t xs[CS * LDP], dys[CS * LDP];
  uint16_t dm[CS * LDM];  // T[i][j] = dM[max(i,j)][min(i,j)]
  float dbc[32 * NTHREADS];
};

__device__ __forceinline__ bf8 pack_bf8(const float (&v)[8]) {
  bf8 r;
#pragma unroll
  for (int j = 0; j < 8; ++j) r[j] = (__bf16)v[j];
  return r;
}
// four values in k-slots 0..3, zeros in 4..7
__device__ __forceinline__ bf8 pack_bf4_lo(float a, float b, float c, float d) {
  bf8 r = {0, 0, 0, 0, 0, 0, 0, 0};
  r[0] = (__bf16)a; r[1] = (__bf16)b; r[2] = (__bf16)c; r[3] = (__bf16)d;
  return r;
}
__device__ __forceinline__ bf8 frag4_lo(const uint16_t* q, bool keep = true) {
  uint2 w = *(const uint2*)q;
  if (!keep) w = make_uint2(0u, 0u);
  const bf4 a = __builtin_bit_cast(bf4, w);
  const bf4 z = {0, 0, 0, 0};
  return __builtin_shufflevector(a, z, 0, 1, 2, 3, 4, 5, 6, 7);
}

template <int LDM, int LV>
__device__ __forceinline__ void bwd_big_level_bf(const float (&cs)[16], const float (&Bv)[16], const float (&dtp)[16], const float (&Cv)[16],
                                                 const uint16_t* __restrict__ dmr, const uint16_t* __restrict__ dmt,
                                                 float (&e1)[16], float (&x2)[16], float (&dcs)[16], int cm, int g4) {
  float op[16], ee[16];
  const float ref_a = __shfl(LV == 4 ? cs[3] : cs[7], cm + 48, 64);
  const float ref_b = LV == 4 ? __shfl(cs[11], cm + 48, 64) : ref_a;
#pragma unroll
  for (int J = 0; J < 4; ++J) {
    const float ref = (J & 2) ? ref_b : ref_a;
    const bool upper = LV == 4 ? (J & 1) : (J & 2);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = 4 * J + j;
      const float e = ex2(upper ? cs[k] - ref : ref - cs[k]);
      ee[k] = e;
      op[k] = (upper ? Cv[k] : Bv[k] * dtp[k]) * e;
    }
  }
  if (LV == 5) {
    float lo8[8], hi8[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) { lo8[j] = op[j]; hi8[j] = op[8 + j]; }
    const bf8 blo = pack_bf8(lo8), bhi = pack_bf8(hi8);
    // two products at a time (F: rows of tiles 2, 3 gather from tiles 0, 1; then G: rows of tiles 0, 1 gather from
    // tiles 2, 3), so that only two operand fragments and two results are live at once
    const f4 z = {0, 0, 0, 0};
    {
      const bf8 a2 = split_frag<LDM>(dmr, 32 + cm, g4, 0), a3 = split_frag<LDM>(dmr, 48 + cm, g4, 0);
      const f4 f2 = mfma_bf(a2, blo, z), f3 = mfma_bf(a3, blo, z);
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) {
        x2[8 + rr] += ee[8 + rr] * f2[rr];
        x2[12 + rr] += ee[12 + rr] * f3[rr];
        dcs[8 + rr] += (float)bhi[rr] * f2[rr];
        dcs[12 + rr] += (float)bhi[4 + rr] * f3[rr];
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    {
      const bf8 a0 = split_frag<LDM>(dmt, cm, g4, 1), a1 = split_frag<LDM>(dmt, 16 + cm, g4, 1);
      const f4 g0 = mfma_bf(a0, bhi, z), g1 = mfma_bf(a1, bhi, z);
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) {
        e1[rr] += ee[rr] * g0[rr];
        e1[4 + rr] += ee[4 + rr] * g1[rr];
        dcs[rr] -= (float)blo[rr] * g0[rr];
        dcs[4 + rr] -= (float)blo[4 + rr] * g1[rr];
      }
    }
  } else {
    bf8 b[4];
#pragma unroll
    for (int I = 0; I < 4; ++I) {
      const int K = (I & 1) ? I - 1 : I + 1;  // the tile contracted over
      b[I] = pack_bf4_lo(op[4 * K], op[4 * K + 1], op[4 * K + 2], op[4 * K + 3]);
    }
    const f4 z = {0, 0, 0, 0};
#pragma unroll
    for (int I = 0; I < 4; ++I) {
      const int K = (I & 1) ? I - 1 : I + 1;
      if (I == 2) __builtin_amdgcn_sched_barrier(0);  // two products at a time
      const f4 acc = mfma_bf(frag4_lo(((I & 1) ? dmr : dmt) + (I * 16 + cm) * LDM + K * 16 + 4 * g4), b[I], z);
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) {
        const float fr = (float)b[(I & 1) ? I - 1 : I + 1][rr];  // this row's operand as the partner tile's product took it
        if (I & 1) {
          x2[4 * I + rr] += ee[4 * I + rr] * acc[rr];
          dcs[4 * I + rr] += fr * acc[rr];
        } else {
          e1[4 * I + rr] += ee[4 * I + rr] * acc[rr];
          dcs[4 * I + rr] -= fr * acc[rr];
        }
      }
    }
  }
}

template <int LDM, int LV>
__device__ __forceinline__ void bwd_mid_level_bf(const float (&cs)[16], const float (&Bv)[16], const float (&dtp)[16], const float (&Cv)[16],
                                                 const uint16_t* __restrict__ dmr, const uint16_t* __restrict__ dmt,
                                                 float (&e1)[16], float (&x2)[16], float (&dcs)[16], int cm, int g4) {
  const bool up = LV == 2 ? (g4 & 1) : (g4 & 2);  // role of the lane's rows 4 g4 + j
  const float upf = up ? 1.0f : 0.0f, lof = up ? 0.0f : 1.0f;
  // A operand: row i = cm of T_w (see bwd_mid_level), columns 4 g4 + jj; non-zero only where (i, kk) is a level-w pair
  const int cg = cm >> 2;
  const bool iup = LV == 2 ? (cg & 1) : (cg & 2);
  const bool nz = LV == 2 ? (g4 == (cg ^ 1)) : ((g4 >> 1) != (cg >> 1));
  const uint16_t* abase = (iup ? dmr : dmt) + cm * LDM + 4 * g4;
  float op[16], ee[16], refs[4];
#pragma unroll
  for (int J = 0; J < 4; ++J)
    refs[J] = LV == 2 ? __shfl(cs[4 * J + 3], cm + 16 * (g4 & 2), 64) : __shfl(cs[4 * J + 3], cm + 16, 64);
  bf8 a[4];
#pragma unroll
  for (int I = 0; I < 4; ++I) a[I] = frag4_lo(abase + I * (16 * LDM + 16), nz);
#pragma unroll
  for (int J = 0; J < 4; ++J) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = 4 * J + j;
      const float e = ex2(up ? cs[k] - refs[J] : refs[J] - cs[k]);
      ee[k] = e;
      op[k] = (up ? Cv[k] : Bv[k] * dtp[k]) * e;
    }
  }
  const f4 z = {0, 0, 0, 0};
#pragma unroll
  for (int I = 0; I < 4; ++I) {
    const bf8 bo = pack_bf4_lo(op[4 * I], op[4 * I + 1], op[4 * I + 2], op[4 * I + 3]);
    const f4 acc = mfma_bf(a[I], bo, z);
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
      const float v = ee[4 * I + rr] * acc[rr];
      x2[4 * I + rr] = fmaf(v, upf, x2[4 * I + rr]);
      e1[4 * I + rr] = fmaf(v, lof, e1[4 * I + rr]);
      dcs[4 * I + rr] = fmaf((float)bo[rr] * acc[rr], upf - lof, dcs[4 * I + rr]);
    }
  }
}

template <int LDM>
__device__ __forceinline__ void bwd_small_levels_bf(const float (&cs)[16], const float (&Bv)[16], const float (&dtp)[16], const float (&Cv)[16],
                                                    const uint16_t* __restrict__ dmr, float (&e1)[16], float (&x2)[16],
                                                    int g4) {
#pragma unroll
  for (int J = 0; J < 4; ++J) {
    const uint16_t* blk = dmr + (16 * J + 4 * g4) * LDM + 16 * J + 4 * g4;  // dM[row jl][col js] of the group
    uint2 m[4];
#pragma unroll
    for (int jl = 0; jl < 4; ++jl) m[jl] = *(const uint2*)(blk + jl * LDM);
    float Bd[4];
#pragma unroll
    for (int jl = 0; jl < 4; ++jl) Bd[jl] = Bv[4 * J + jl] * dtp[4 * J + jl];
    auto at = [&](int jl, int js) {
      const unsigned w = js < 2 ? m[jl].x : m[jl].y;
      return __uint_as_float((js & 1) ? (w & 0xffff0000u) : (w << 16));
    };
#pragma unroll
    for (int jl = 0; jl < 4; ++jl) {
      const int kl = 4 * J + jl;
      const float d = at(jl, jl);
      e1[kl] = fmaf(d, Cv[kl], e1[kl]);
      x2[kl] = fmaf(d, Bd[jl], x2[kl]);
#pragma unroll
      for (int js = 0; js < jl; ++js) {
        const int ks = 4 * J + js;
        const float wgt = at(jl, js) * ex2(cs[kl] - cs[ks]);
        e1[ks] = fmaf(wgt, Cv[kl], e1[ks]);
        x2[kl] = fmaf(wgt, Bd[js], x2[kl]);
      }
    }
  }
}

template <int PT, bool DTB, bool FULL>
__device__ __forceinline__ void k_bwd_chunk_bf_body(const KP& p, const float* __restrict__ dy_ws, const float* __restrict__ states, const float* __restrict__ dstates, const float* __restrict__ dm, const float* __restrict__ g_last, float* __restrict__ partA, float* __restrict__ partBias, const int* __restrict__ redo, const int dir_here, const bool mirror) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  typedef BwdChunkBfSmem<PT> SM;
  SM& s = *reinterpret_cast<SM*>(smem_raw);
  constexpr int LDP = SM::LDP, LDM = SM::LDM, KT = (PT + 1) / 2;
  constexpr int KP_ = PT * 4;  // dS / H values per lane
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int cm = lane & 15, g4 = lane >> 4;
  const int nsl = (p.N + NS - 1) / NS;
  Unit u;
  // `redo` (one word per direction, workgroup and head, written by the tile-base kernel): only the marked heads are
  // evaluated here, and their ddt / dB / dC are added to what that kernel left (zero, or the other direction's share).
  // `mirror`: the workgroup's chunk index counts from the other end -- the chunk of this direction that covers the
  // same tokens as the un-mirrored chunk of the other direction (one workgroup then adds both directions' shares to
  // those tokens' ddt one after the other, and no two workgroups ever update one address).
  int id = xcd_remap(blockIdx.x, gridDim.x);
  const int ns = id % nsl;
  id /= nsl;
  u.g = id % p.G;
  id /= p.G;
  const int cj = id % p.ncl;
  u.c = p.c_lo + (mirror ? p.ncl - 1 - cj : cj);
  u.b = id / p.ncl;
  if (redo) {
    const int nblk = p.B * p.ncl * p.G * nsl;
    const int wg = ((u.b * p.ncl + (u.c - p.c_lo)) * p.G + u.g) * nsl + ns;  // as the tile-base kernel counts them
    redo += (dir_here * nblk + wg) * p.hpg;
    int any = 0;
    for (int hh = 0; hh < p.hpg; ++hh) any |= redo[hh];
    if (!any) return;
  }
  u.dir = dir_here;
  u.bt = u.b * p.ndir + u.dir;
  u.h = u.g * p.hpg;
  const int n = ns * NS + wave * 16 + cm;
  const bool vn = FULL || n < p.N;
  const RowMap rm = make_rowmap<FULL>(p, u, g4, ns * NS);
  const int lim = vn ? rm.nvalid - 4 * g4 : 0;
  auto rowk = [&](int k) { return 16 * (k >> 2) + (k & 3); };
  const bool pn_full = FULL && p.P == PT * 16;

  float Bv[16], Cv[16];
  lane_load_ln<true>(p.Bm[u.dir], u.b, u.g, n, vn, g4, rm, Bv);
  lane_load_ln<true>(p.Cm[u.dir], u.b, u.g, n, vn, g4, rm, Cv);
#pragma unroll
  for (int k = 0; k < 16; ++k) s.dbc[k * NTHREADS + tid] = s.dbc[(16 + k) * NTHREADS + tid] = 0.0f;

  // The reversed direction's launch follows the forward one's and shares dt, x, B, C and ddt with it: it walks the
  // heads backwards, so what the first launch touched last (and the last-level cache still holds) is read first.
  auto head_of = [&](int hh) { return u.g * p.hpg + (dir_here ? p.hpg - 1 - hh : hh); };
  // a head's tiles on their way from global memory to LDS: raw bf16 pairs (x, dy) and the thread's two 16-byte pieces
  // of T (rows tq >> 3 and 32 + (tq >> 3), columns 8 (tq & 7) .. + 7)
  uint2 nx[PT], ny[PT];
  uint4 nm0, nm1;
  // (the thread index is made opaque at each use: the per-lane addresses derived from it are then formed next to the
  // accesses instead of being kept, as 64-bit values, across the whole head loop)
  auto request = [&](int h) {
    int tq = tid;
    asm volatile("" : "+v"(tq));
    const int mrow = tq >> 3, mcol = (tq & 7) * 8;
    Unit v = u;
    v.h = h;
    dy_load_bf<PT, FULL>(p, v, dy_ws, ny, tq);
    lp_load_bf<PT, FULL>(p, v, p.x[u.dir], nx, tq);
    const uint16_t* dmb = reinterpret_cast<const uint16_t*>(dm + sq_off(p, u.bt, u.c, h));
    nm0 = *(const uint4*)(dmb + mrow * CS + mcol);
    nm1 = *(const uint4*)(dmb + (32 + mrow) * CS + mcol);
  };
  auto deposit = [&]() {
    int tq = tid;
    asm volatile("" : "+v"(tq));
    const int mrow = tq >> 3, mcol = (tq & 7) * 8;
    lp_store_raw<PT, LDP>(ny, s.dys, tq);
    lp_store_raw<PT, LDP>(nx, s.xs, tq);
    *(uint4*)(s.dm + mrow * LDM + mcol) = nm0;
    *(uint4*)(s.dm + (32 + mrow) * LDM + mcol) = nm1;
  };

  for (int hh = 0; hh < p.hpg; ++hh) {
    if (redo && !redo[hh]) continue;
    u.h = head_of(hh);
    // ---- global loads of this head
    float raw[16], dsv[KP_], hv[KP_];
    lane_load_ln<DTB>(p.dt, u.b, u.h, n, vn, g4, rm, raw);
    const Coef cf = lane_coef(p, u.h, n, vn);
    const float gl = (g4 == 3 && vn) ? g_last[vec_off(p, u.bt, u.c, u.h) + n] : 0.0f;
    lane_load_pn<KP_>(dstates + dst_off(p, u.bt, u.c, u.h), p.P, p.N, n, vn, g4, pn_full, dsv);
    lane_load_pn<KP_>(states + st_off(p, u.bt, u.c, u.h), p.P, p.N, n, vn, g4, pn_full, hv);
    request(u.h);
    __syncthreads();  // the previous head no longer reads the tiles
    deposit();
    __syncthreads();
    const uint16_t* xs_ = s.xs;
    const uint16_t* dys_ = s.dys;
    const uint16_t* dm_ = s.dm;

    const float An = cf.A;
    float dtp[16], cs[16], dfac[16];
    const float last = lane_prep<true>(p, cf, vn, cm, g4, rm, raw, dtp, cs, dfac);
    pin16(cs);

    int cq = cm, gq = g4;
    asm volatile("" : "+v"(cq), "+v"(gq));
    float e1[16], x2[16];
    {
      // Q = x . dS and R = dy . H over the head dimension, K = 32 per step; k-slot s of step t <-> lane value 8 t + s.
      // x and dy are exact in bf16; dS and H are fp32 states and enter as (hi, lo) pairs -- two instructions per step:
      // the last row's Bd . E1 cancels against the state term g = sum_p dS H_next in d/d(cs), and a dS rounded to 8
      // bits would leave that difference with a relative error far above the bf16 level.
      bf8 dsh[KT], dsl[KT], hh_[KT], hl_[KT];
#pragma unroll
      for (int t = 0; t < KT; ++t) {
        float a[8], b[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          a[j] = 8 * t + j < KP_ ? dsv[(8 * t + j) % KP_] : 0.0f;
          b[j] = 8 * t + j < KP_ ? hv[(8 * t + j) % KP_] : 0.0f;
        }
        split8(a, dsh[t], dsl[t]);
        split8(b, hh_[t], hl_[t]);
      }
#pragma unroll
      for (int I = 0; I < 4; ++I) {
        f4 q = {0, 0, 0, 0}, r = {0, 0, 0, 0};
#pragma unroll
        for (int t = 0; t < KT; ++t) {
          const bool half = (PT & 1) && t == KT - 1;
          const bf8 xf = half ? split_frag<LDP, true>(xs_, I * 16 + cq, gq, t) : split_frag<LDP>(xs_, I * 16 + cq, gq, t);
          const bf8 yf = half ? split_frag<LDP, true>(dys_, I * 16 + cq, gq, t) : split_frag<LDP>(dys_, I * 16 + cq, gq, t);
          q = mfma_bf(xf, dsl[t], q);
          r = mfma_bf(yf, hl_[t], r);
          q = mfma_bf(xf, dsh[t], q);
          r = mfma_bf(yf, hh_[t], r);
        }
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
          e1[4 * I + rr] = ex2(last - cs[4 * I + rr]) * q[rr];
          x2[4 * I + rr] = ex2(cs[4 * I + rr]) * r[rr];
        }
      }
    }

    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" : "+v"(cq), "+v"(gq));
    pin16(cs); pin16(e1); pin16(x2);
    bwd_small_levels_bf<LDM>(cs, Bv, dtp, Cv, dm_, e1, x2, gq);
    __builtin_amdgcn_sched_barrier(0);
    // d/d(cs) so far (state terms and in-lane pairs, all fp32): C . X2 - Bd . E1.  The matrix levels add their share to
    // it directly, as (the operand as the matrix instruction took it, rounded to bf16) x (the product): a pair (i, j)
    // then enters row i and, negated, row j as the same product of the same three numbers, and the suffix sums below,
    // in which the two cancel for every row before j, are left with fp32 rounding instead of bf16 rounding.
    float dcs[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) dcs[k] = Cv[k] * x2[k] - Bv[k] * dtp[k] * e1[k];
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" : "+v"(cq), "+v"(gq));
    pin16(cs); pin16(e1); pin16(x2); pin16(dcs);
    bwd_big_level_bf<LDM, 5>(cs, Bv, dtp, Cv, dm_, dm_, e1, x2, dcs, cq, gq);
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" : "+v"(cq), "+v"(gq));
    pin16(cs); pin16(e1); pin16(x2); pin16(dcs);
    bwd_big_level_bf<LDM, 4>(cs, Bv, dtp, Cv, dm_, dm_, e1, x2, dcs, cq, gq);
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" : "+v"(cq), "+v"(gq));
    pin16(cs); pin16(e1); pin16(x2); pin16(dcs);
    bwd_mid_level_bf<LDM, 3>(cs, Bv, dtp, Cv, dm_, dm_, e1, x2, dcs, cq, gq);
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" : "+v"(cq), "+v"(gq));
    pin16(cs); pin16(e1); pin16(x2); pin16(dcs);
    // the second direction adds to the first one's ddt: fetch it while the last level runs
    float old[16];
    if ((redo || dir_here > 0) && p.ddt.ptr) lane_load_ln<DTB>(p.ddt, u.b, u.h, n, vn, g4, rm, old);
    __builtin_amdgcn_sched_barrier(0);
    bwd_mid_level_bf<LDM, 2>(cs, Bv, dtp, Cv, dm_, dm_, e1, x2, dcs, cq, gq);
    __builtin_amdgcn_sched_barrier(0);

    // ---- column phase (as in k_bwd_chunk)
    pin16(e1); pin16(x2); pin16(dcs);
    float val[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const float E1 = e1[k], X2 = x2[k];
      s.dbc[k * NTHREADS + tid] += dtp[k] * E1;
      s.dbc[(16 + k) * NTHREADS + tid] += X2;
      val[k] = Bv[k] * E1;
    }
    dcs[15] += gl;
    {
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
      for (int J = 0; J < 4; ++J) v[J] = g4 <= 2 ? c[J] + t[J] : c[J];
#pragma unroll
      for (int J = 0; J < 4; ++J) t[J] = __shfl_down(v[J], 32, 64);
#pragma unroll
      for (int J = 0; J < 4; ++J) v[J] = g4 <= 1 ? v[J] + t[J] : v[J];
#pragma unroll
      for (int J = 0; J < 4; ++J) t[J] = __shfl(v[J], cm, 64);
      float carry = 0.0f;
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
      if (rm.full || rowk(k) < lim) sumB += val[k];
    }
    if ((redo || dir_here > 0) && p.ddt.ptr) {
#pragma unroll
      for (int k = 0; k < 16; ++k) val[k] += old[k];
    }
    if (p.ddt.ptr) lane_store_ln<DTB>(p.ddt, u.b, u.h, n, vn, g4, rm, val);
    sumA = scan_g_incl(sumA, g4);
    sumB = scan_g_incl(sumB, g4);
    if (g4 == 3 && vn) {
      partA[vec_off(p, u.bt, u.c, u.h) + n] = sumA;
      partBias[vec_off(p, u.bt, u.c, u.h) + n] = sumB;
    }
  }

  {
    float vb[16], vc[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      vb[k] = s.dbc[k * NTHREADS + tid];
      vc[k] = s.dbc[(16 + k) * NTHREADS + tid];
    }
    if (redo) {
      float ob[16], oc[16];
      if (p.dB[u.dir].ptr) lane_load_ln<true>(p.dB[u.dir], u.b, u.g, n, vn, g4, rm, ob);
      if (p.dC[u.dir].ptr) lane_load_ln<true>(p.dC[u.dir], u.b, u.g, n, vn, g4, rm, oc);
#pragma unroll
      for (int k = 0; k < 16; ++k) {
        vb[k] += ob[k];
        vc[k] += oc[k];
      }
    }
    if (p.dB[u.dir].ptr) lane_store_ln<true>(p.dB[u.dir], u.b, u.g, n, vn, g4, rm, vb);
    if (p.dC[u.dir].ptr) lane_store_ln<true>(p.dC[u.dir], u.b, u.g, n, vn, g4, rm, vc);
  }
}
template <int PT, bool DTB, bool FULL>
__global__ __launch_bounds__(NTHREADS, 2) void k_bwd_chunk_bf(KP p, const float* __restrict__ dy_ws, const float* __restrict__ states, const float* __restrict__ dstates, const float* __restrict__ dm, const float* __restrict__ g_last, float* __restrict__ partA, float* __restrict__ partBias, const int* __restrict__ redo, int ndirs) {
  for (int d = 0; d < ndirs; ++d) {
    if (d) __syncthreads();
    k_bwd_chunk_bf_body<PT, DTB, FULL>(p, dy_ws, states, dstates, dm, g_last, partA, partBias, redo, p.dir0 + d, d > 0);
  }
}
// One launch for a sequence whose last chunk is ragged: complete-tile code for the complete chunks, the general code
// for the last one (uniform per workgroup).
template <int PT, bool DTB>
__global__ __launch_bounds__(NTHREADS, 2) void k_bwd_chunk_bf_mixed(KP p, const float* __restrict__ dy_ws, const float* __restrict__ states, const float* __restrict__ dstates, const float* __restrict__ dm, const float* __restrict__ g_last, float* __restrict__ partA, float* __restrict__ partBias) {
  if (p.c_lo + (xcd_remap(blockIdx.x, gridDim.x) / ((p.N + NS - 1) / NS) / p.G) % p.ncl == p.nc - 1) k_bwd_chunk_bf_body<PT, DTB, false>(p, dy_ws, states, dstates, dm, g_last, partA, partBias, nullptr, p.dir0, false);
  else k_bwd_chunk_bf_body<PT, DTB, true>(p, dy_ws, states, dstates, dm, g_last, partA, partBias, nullptr, p.dir0, false);
}


// ------------------------------------------------------------------------- dx
// BF (bf16 inputs): the operands of the product over the state index are bf16 tiles read as matrix fragments of 8
// adjacent columns; fp32 inputs: (hi, lo) pairs of such tiles from two head tiles on, fp32 tiles for one.  `prod` (the
// dy * x products of the skip gradient) is its own small tile for bf16 inputs.
#ifndef DX_SPLIT_FROM
#define DX_SPLIT_FROM 2
#endif
template <int PT, bool BF>
struct BwdDxSmem {
  static constexpr int LDPT = PT * 16 + 4;
  static constexpr int LDK = NS + 8;
  // fp32 inputs: the product over the state index on (hi, lo) bf16 tiles, hi.hi + hi.lo + lo.hi, instead of fp32
  // matrix instructions, which take the vector ALU's issue slots (28 - 45 % of this kernel's cycles, never beside its
  // vector work); the bf16 instructions run beside it.  (DX_SPLIT_FROM: head tiles from which this form is used.)
  static constexpr bool SPL = !BF && PT >= DX_SPLIT_FROM;
  static constexpr bool B16 = BF || SPL;
  static constexpr int NH = SPL ? 2 : 1;
  float dys[CS * LDPT];
  typename std::conditional<B16, uint16_t, float>::type bt[NH * CS * (B16 ? LDK : LDN)];        // B dt' exp2(last - cs) [m][n]
  typename std::conditional<B16, uint16_t, float>::type dss[NH * PT * 16 * (B16 ? LDK : LDN)];  // dS [p][n]
  float prod_own[BF ? CS * LDPT : 4];  // dy * x; with fp32 inputs it takes the place of `bt`
  __device__ __forceinline__ float* prod() { return BF ? prod_own : reinterpret_cast<float*>(bt); }
  static constexpr int LDPROD = B16 ? LDPT : LDN;
  static_assert(!SPL || sizeof(uint16_t) * NH * CS * LDK >= sizeof(float) * CS * LDPT, "dy * x fits in the place of bt");
};
// a (16 PT x 64) slab of fp32 values as (hi, lo) bf16 pairs into LDS hi / lo [p][col], row stride LD
template <int PT, int LD>
__device__ __forceinline__ void pn_store_hl(const PnRegs<PT>& r, uint16_t* hi, uint16_t* lo, int tid = threadIdx.x) {
  typedef PnRegs<PT> R;
#pragma unroll
  for (int i = 0; i < R::CNT; ++i) {
    const int e = tid + i * NTHREADS, pp = e / R::Q, c4 = (e % R::Q) * 4;
    const float w[4] = {r.v[i][0], r.v[i][1], r.v[i][2], r.v[i][3]};
    bf4 h, l;
    split4(w, h, l);
    if (e < R::TOT) {
      *(bf4*)(hi + pp * LD + c4) = h;
      *(bf4*)(lo + pp * LD + c4) = l;
    }
  }
}
template <int PT, int LD>
__device__ __forceinline__ void pn_store_bf16(const PnRegs<PT>& r, uint16_t* dst, int tid = threadIdx.x) {
  typedef PnRegs<PT> R;
#pragma unroll
  for (int i = 0; i < R::CNT; ++i) {
    const int e = tid + i * NTHREADS, pp = e / R::Q, c4 = (e % R::Q) * 4;
    if (e < R::TOT) *(uint2*)(dst + pp * LD + c4) = make_uint2(pack_bf16(r.v[i][0], r.v[i][1]), pack_bf16(r.v[i][2], r.v[i][3]));
  }
}
template <int LD>
__device__ __forceinline__ bf8 frag8(const uint16_t* tile, int row, int g4, int t) {
  return *(const bf8*)(tile + row * LD + 32 * t + 8 * g4);
}

// partD: (Bt*nc*H, P) per-unit sums over rows of dy*x
template <int PT, bool IOB, bool DTB, bool FULL>
__device__ __forceinline__ void k_bwd_dx_body(const KP& p, const float* __restrict__ dy_ws, const float* __restrict__ dstates, const float* __restrict__ cabt, float* __restrict__ partD) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  typedef BwdDxSmem<PT, IOB> SM;
  SM& s = *reinterpret_cast<SM*>(smem_raw);
  constexpr int LDPT = SM::LDPT, LDK = SM::LDK, LDPR = SM::LDPROD;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int cm = lane & 15, g4 = lane >> 4;
  const Unit u = decode_unit(p, xcd_remap(blockIdx.x, gridDim.x));
  const float* ds = dstates + dst_off(p, u.bt, u.c, u.h);

  int n = wave * 16 + cm;
  bool vn = FULL || n < p.N;
  RowMap rm;
  Coef cf;
  rm = make_rowmap<FULL>(p, u, g4, 0);
  float raw[16], bv[16];
  PnRegs<PT> sv;
  lane_load_ln<DTB>(p.dt, u.b, u.h, n, vn, g4, rm, raw);
  cf = lane_coef(p, u.h, n, vn);
  lane_load_ln<IOB>(p.Bm[u.dir], u.b, u.g, n, vn, g4, rm, bv);
  pn_load<PT>(p, ds, 0, sv);
  // M^T of this wave's 16 columns goes straight into matrix-operand registers (lane (column cm, group g4) holds
  // rows 16 kb + 4 g4 .. + 3 of the blocks kb >= wave, the upper triangle of the diagonal block zeroed): no LDS tile,
  // which lets a fourth workgroup live on the CU
  float mf[4][4];
  {
    const float* mcol = cabt + sq_off(p, u.bt, u.c, u.h) + (4 * g4) * CS + wave * 16 + cm;
#pragma unroll
    for (int kb = 0; kb < 4; ++kb)
#pragma unroll
      for (int j = 0; j < 4; ++j) mf[kb][j] = mcol[(16 * max(kb, wave) + j) * CS];  // no branch between the loads
#pragma unroll
    for (int kb = 0; kb < 4; ++kb)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (kb < wave || (kb == wave && cm > 4 * g4 + j)) mf[kb][j] = 0.0f;
  }
  {
    float dv[CS * PT * 16 / NTHREADS];
    dy_load<IOB, PT, FULL>(p, u, dy_ws, dv);
    lp_store<PT>(dv, s.dys, LDPT);
  }
  f4 acc[PT];
#pragma unroll
  for (int pt = 0; pt < PT; ++pt) acc[pt] = (f4){0, 0, 0, 0};

  for (int n0 = 0; n0 < p.N; n0 += NS) {
    {
      float dtp[16], cs[16], dummy[16];
      const float last = lane_prep<false>(p, cf, vn, cm, g4, rm, raw, dtp, cs, dummy);
      if constexpr (IOB) {
        float btv[16];
#pragma unroll
        for (int k = 0; k < 16; k += 2) {
          btv[k] = bv[k] * dtp[k] * ex2(last - cs[k]);
          btv[k + 1] = bv[k + 1] * dtp[k + 1] * ex2(last - cs[k + 1]);
          const unsigned h2 = pack_bf16(btv[k], btv[k + 1]);
          s.bt[lane_row(k, g4) * LDK + wave * 16 + cm] = (uint16_t)h2;
          s.bt[lane_row(k + 1, g4) * LDK + wave * 16 + cm] = (uint16_t)(h2 >> 16);
        }
      } else if constexpr (SM::SPL) {
#pragma unroll
        for (int k = 0; k < 16; k += 2) {
          const float b0 = bv[k] * dtp[k] * ex2(last - cs[k]), b1 = bv[k + 1] * dtp[k + 1] * ex2(last - cs[k + 1]);
          const unsigned h2 = pack_bf16(b0, b1);
          const unsigned l2 = pack_bf16(b0 - __uint_as_float(h2 << 16), b1 - __uint_as_float(h2 & 0xffff0000u));
          const int o0 = lane_row(k, g4) * LDK + wave * 16 + cm, o1 = lane_row(k + 1, g4) * LDK + wave * 16 + cm;
          s.bt[o0] = (uint16_t)h2;
          s.bt[o1] = (uint16_t)(h2 >> 16);
          s.bt[CS * LDK + o0] = (uint16_t)l2;
          s.bt[CS * LDK + o1] = (uint16_t)(l2 >> 16);
        }
      } else {
#pragma unroll
        for (int k = 0; k < 16; ++k)
          s.bt[lane_row(k, g4) * LDN + wave * 16 + cm] = bv[k] * dtp[k] * ex2(last - cs[k]);
      }
    }
    if constexpr (IOB) pn_store_bf16<PT, LDK>(sv, s.dss);
    else if constexpr (SM::SPL) pn_store_hl<PT, LDK>(sv, s.dss, s.dss + PT * 16 * LDK);
    else pn_store<PT>(sv, s.dss);
    if (n0 + NS < p.N) {
      n = n0 + NS + wave * 16 + cm;
      vn = FULL || n < p.N;
      rm = make_rowmap<FULL>(p, u, g4, n0 + NS);
      lane_load_ln<DTB>(p.dt, u.b, u.h, n, vn, g4, rm, raw);
      cf = lane_coef(p, u.h, n, vn);
      lane_load_ln<IOB>(p.Bm[u.dir], u.b, u.g, n, vn, g4, rm, bv);
      pn_load<PT>(p, ds, n0 + NS, sv);
    }
    __syncthreads();
    if constexpr (IOB) {
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const bf8 a = frag8<LDK>(s.bt, wave * 16 + cm, g4, t);
#pragma unroll
        for (int pt = 0; pt < PT; ++pt) acc[pt] = mfma_bf(a, frag8<LDK>(s.dss, pt * 16 + cm, g4, t), acc[pt]);
      }
    } else if constexpr (SM::SPL) {
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const bf8 ah = frag8<LDK>(s.bt, wave * 16 + cm, g4, t), al = frag8<LDK>(s.bt + CS * LDK, wave * 16 + cm, g4, t);
#pragma unroll
        for (int pt = 0; pt < PT; ++pt)
          acc[pt] = mfma_split(ah, al, frag8<LDK>(s.dss, pt * 16 + cm, g4, t),
                               frag8<LDK>(s.dss + PT * 16 * LDK, pt * 16 + cm, g4, t), acc[pt]);
      }
    } else {
#pragma unroll
      for (int kb = 0; kb < NS; kb += 16)
#pragma unroll
        for (int pt = 0; pt < PT; ++pt) mma16_mm(acc[pt], s.bt, LDN, wave * 16, s.dss, LDN, pt * 16, kb, lane);
    }
    __syncthreads();
  }
  // dx[m][p] += sum_{l>=m} M[l][m] dy[l][p]
#pragma unroll
  for (int kb = 0; kb < 4; ++kb)
    if (kb >= wave) {  // uniform
      // the lane's four M values and four dy values are the operands of one K = 16 bf16 instruction as they stand
      // (k-slot j of lane group g4 <-> row 16 kb + 4 g4 + j), both as (hi, lo) pairs
      bf4 ah, al;
      split4(mf[kb], ah, al);
#pragma unroll
      for (int pt = 0; pt < PT; ++pt) {
        const float* bp = s.dys + (16 * kb + 4 * g4) * LDPT + pt * 16 + cm;
        const float yw[4] = {bp[0], bp[LDPT], bp[2 * LDPT], bp[3 * LDPT]};
        bf4 bh, bl;
        split4(yw, bh, bl);
        acc[pt] = mfma_bf16k(al, bh, acc[pt]);
        acc[pt] = mfma_bf16k(ah, bl, acc[pt]);  // (also for bf16 inputs: a gated dy is an fp32 product)
        acc[pt] = mfma_bf16k(ah, bh, acc[pt]);
      }
    }

  const TensorD& tx = p.x[u.dir];
  const TensorD& tdx = p.dx[u.dir];
  float* prod = s.prod();  // [64][LDPR]
#pragma unroll
  for (int pt = 0; pt < PT; ++pt) {
    int ox[4], odx[4];
    float xv[4], v[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int l = wave * 16 + 4 * g4 + r, pp = pt * 16 + cm, tt = u.c * CS + l;
      const bool ok = tt < p.L && pp < p.P;
      const int pr = ok ? phys_row(p, u.dir, tt) : 0;
      ox[r] = (ok && p.D) ? pr * (int)tx.s1 + pp : -1;
      odx[r] = (ok && tdx.ptr) ? pr * (int)tdx.s1 + pp : -1;
    }
    gload<IOB, 4>(tx.ptr, (long)u.b * tx.s0 + (long)u.h * tx.s2, ox, xv);
    float dcoef = 0.0f;  // skip coefficient of the lane's column, read once
    if (p.D) dcoef = (p.flags & F_D_HDIM) ? p.D[u.h * p.P + min(pt * 16 + cm, p.P - 1)] : p.D[u.h];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int l = wave * 16 + 4 * g4 + r, pp = pt * 16 + cm;
      const float dyv = s.dys[l * LDPT + pp];
      v[r] = fmaf(dcoef, dyv, acc[pt][r]);
      prod[l * LDPR + pp] = dyv * xv[r];
    }
    gstore<IOB, 4>(const_cast<void*>(tdx.ptr), (long)u.b * tdx.s0 + (long)u.h * tdx.s2, odx, v);
  }
  if (p.D && partD) {
    __syncthreads();
    if (tid < PT * 16) {
      float sum = 0.0f;
      for (int l = 0; l < CS; ++l) sum += prod[l * LDPR + tid];
      if (tid < p.P) partD[(((long)u.bt * p.nc + u.c) * p.H + u.h) * p.P + tid] = sum;
    }
  }
}
template <int PT, bool IOB, bool DTB, bool FULL>
__global__ __launch_bounds__(NTHREADS, (PT <= 2 && FULL) ? 4 : 1) void k_bwd_dx(KP p, const float* __restrict__ dy_ws, const float* __restrict__ dstates, const float* __restrict__ cabt, float* __restrict__ partD) {
  k_bwd_dx_body<PT, IOB, DTB, FULL>(p, dy_ws, dstates, cabt, partD);
}
// One launch for a sequence whose last chunk is ragged: complete-tile code for the complete chunks, the general code
// for the last one (uniform per workgroup).
template <int PT, bool IOB, bool DTB>
__global__ __launch_bounds__(NTHREADS, (PT <= 2 && false) ? 4 : 1) void k_bwd_dx_mixed(KP p, const float* __restrict__ dy_ws, const float* __restrict__ dstates, const float* __restrict__ cabt, float* __restrict__ partD) {
  if (decode_unit(p, xcd_remap(blockIdx.x, gridDim.x)).c == p.nc - 1) k_bwd_dx_body<PT, IOB, DTB, false>(p, dy_ws, dstates, cabt, partD);
  else k_bwd_dx_body<PT, IOB, DTB, true>(p, dy_ws, dstates, cabt, partD);
}


// ------------------------------------------------------------------- reductions
// All final reductions run as ONE launch (they are independent of each other and tiny, so separate
// launches would cost more in dispatch latency than in work); blocks are dealt to the jobs in order.
struct ReduceJobs {
  const float *partA, *partBias, *partD, *dh0_dir;
  float *dA, *dbias, *dD, *dh0;
  int J, nHN, H, P, d_hdim, ndir;
  long n_h0;
  int b_A, b_bias, b_D, b_h0;  // first block of each job; b_h0 .. gridDim.x is the dh0 job
};

// Column sums of a (J, ncols) fp32 matrix in a fixed order (bit-reproducible, no atomics):
// block = 32 columns x 8 row groups; row group g adds rows g, g+8, ... and the 8 group sums are
// combined in order.
__device__ __forceinline__ void colsum_block(const float* __restrict__ src, int J, int ncols, float* __restrict__ dst,
                                             int blk, float* red) {
  const int c = blk * 32 + (threadIdx.x & 31), g = threadIdx.x >> 5;
  float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
  if (c < ncols) {
    int j = g;
#pragma unroll 2
    for (; j + 24 < J; j += 32) {
      a0 += src[(long)j * ncols + c];
      a1 += src[(long)(j + 8) * ncols + c];
      a2 += src[(long)(j + 16) * ncols + c];
      a3 += src[(long)(j + 24) * ncols + c];
    }
    for (; j < J; j += 8) a0 += src[(long)j * ncols + c];
  }
  red[threadIdx.x] = (a0 + a1) + (a2 + a3);
  __syncthreads();
  if (g == 0 && c < ncols) {
    float t = 0.0f;
#pragma unroll
    for (int k = 0; k < 8; ++k) t += red[k * 32 + (threadIdx.x & 31)];
    dst[c] = t;
  }
}

// dD[h] = sum over units and p of partD[(j*H + h)*P + p]: one block per head.
__device__ __forceinline__ void dd_scalar_block(const float* __restrict__ partD, int J, int H, int P,
                                                float* __restrict__ dD, int h, float* red) {
  // element e = j P + p of the head's (J, P) slab; a thread takes e = tid, tid + 256, ...: (j, p) advance without a
  // division, and four elements are requested before any is added (with 8 blocks in the launch the latency of a
  // load is the run time: one element per trip made this the longest block of the kernel)
  const int dj = NTHREADS / P, dp = NTHREADS % P;
  int jj = (int)threadIdx.x / P, pp = (int)threadIdx.x % P;
  const long row = (long)H * P;
  const float* src = partD + (long)h * P;
  float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
  auto next = [&](int& j_, int& p_) {
    p_ += dp;
    j_ += dj + (p_ >= P ? 1 : 0);
    p_ -= p_ >= P ? P : 0;
  };
  while (jj < J) {
    int j1 = jj, p1 = pp;
    next(j1, p1);
    int j2 = j1, p2 = p1;
    next(j2, p2);
    int j3 = j2, p3 = p2;
    next(j3, p3);
    const float v0 = src[jj * row + pp];   // (rows past the end read row 0 and add nothing: no branch around a load)
    const float v1 = src[(j1 < J ? j1 : 0) * row + p1];
    const float v2 = src[(j2 < J ? j2 : 0) * row + p2];
    const float v3 = src[(j3 < J ? j3 : 0) * row + p3];
    a0 += v0;
    a1 += j1 < J ? v1 : 0.0f;
    a2 += j2 < J ? v2 : 0.0f;
    a3 += j3 < J ? v3 : 0.0f;
    jj = j3; pp = p3;
    next(jj, pp);
  }
  red[threadIdx.x] = (a0 + a1) + (a2 + a3);
  __syncthreads();
  for (int o = NTHREADS / 2; o > 0; o >>= 1) {
    if (threadIdx.x < o) red[threadIdx.x] += red[threadIdx.x + o];
    __syncthreads();
  }
  if (threadIdx.x == 0) dD[h] = red[0];
}

__global__ __launch_bounds__(NTHREADS) void k_bwd_reduce(ReduceJobs j) {
  __shared__ float red[NTHREADS];
  const int b = blockIdx.x;
  if (b < j.b_bias) {
    colsum_block(j.partA, j.J, j.nHN, j.dA, b - j.b_A, red);
  } else if (b < j.b_D) {
    colsum_block(j.partBias, j.J, j.nHN, j.dbias, b - j.b_bias, red);
  } else if (b < j.b_h0) {
    if (j.d_hdim) colsum_block(j.partD, j.J, j.H * j.P, j.dD, b - j.b_D, red);
    else dd_scalar_block(j.partD, j.J, j.H, j.P, j.dD, b - j.b_D, red);
  } else {
    // dh0 = sum over directions of dh0_dir
    const long id = (long)(b - j.b_h0) * NTHREADS + threadIdx.x;
    if (id < j.n_h0) {
      float a = j.dh0_dir[id];
      if (j.ndir > 1) a += j.dh0_dir[j.n_h0 + id];
      j.dh0[id] = a;
    }
  }
}

// -------------------------------------------------------------------- launchers
template <typename K>
static int set_lds(K kernel, size_t bytes) {
  return (int)hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
}

int launch_bwd_gate(const KP& p, const float* out_x, float* dy_ws, hipStream_t st) {
  const long total = (long)p.B * p.ndir * p.L * p.H * p.P;
  hipLaunchKernelGGL(k_bwd_gate, dim3((unsigned)((total + NTHREADS - 1) / NTHREADS)), dim3(NTHREADS), 0, st, p, out_x,
                     dy_ws);
  return (int)hipGetLastError();
}

int launch_bwd_dstates(const KP& p, const float* dy_ws, float* dstates, float* dm, hipStream_t st) {
  const int units = p.B * p.ndir * p.nc * p.H;
  ISSM_DISPATCH(p, {
    const size_t sm = sizeof(BwdStSmem<PT_, IOB_>);
    constexpr auto kern = MIXED_ ? &k_bwd_dstates_mixed<PT_, IOB_, DTB_> : &k_bwd_dstates<PT_, IOB_, DTB_, FULL_>;
    if (int e = set_lds(kern, sm)) return e;
    hipLaunchKernelGGL(kern, dim3(units), dim3(NTHREADS), sm, st, p, dy_ws, dstates, dm);
  });
  return (int)hipGetLastError();
}

int launch_state_bwd(const KP& p, const float* states, const float* cs_last, float* dstates, float* g_last,
                     float* dh0_dir, hipStream_t st) {
  // One workgroup walks the chunks of its columns one after the other.  Complete shapes take the variant without
  // conditional accesses; with few (batch, head) pairs narrower column slices put more workgroups on the chip.
  const int wide = p.B * p.ndir * p.H * ((p.N + 63) / 64);
#define ISSM_STATE_BWD_FULL(NQ_, KM_, R_, BATCH_)                                                                          \
  hipLaunchKernelGGL((k_state_bwd_full<NQ_, KM_, R_, BATCH_>), dim3(p.B * p.ndir * p.H * (p.N / (4 * NQ_))), dim3(NTHREADS), \
                     0, st, p, states, cs_last, dstates, g_last, dh0_dir)
  if (p.N % 32 == 0 && (wide < 256 || p.N % 64 != 0)) {
    // few workgroups walking many chunks: the column sums of several steps behind one barrier
    const bool batch = p.B * p.ndir * p.H * (p.N / 32) <= 128 && p.nc >= 32;
    if (p.P <= 32) { if (batch) ISSM_STATE_BWD_FULL(8, 1, 6, true); else ISSM_STATE_BWD_FULL(8, 1, 6, false); }
    else { if (batch) ISSM_STATE_BWD_FULL(8, 2, 4, true); else ISSM_STATE_BWD_FULL(8, 2, 4, false); }
  } else if (p.N % 64 == 0) {
    switch ((p.P + 15) / 16) {
      case 1: ISSM_STATE_BWD_FULL(16, 1, 3, false); break;
      case 2: ISSM_STATE_BWD_FULL(16, 2, 3, false); break;
      case 3: ISSM_STATE_BWD_FULL(16, 3, 3, false); break;
      default: ISSM_STATE_BWD_FULL(16, 4, 3, false); break;
    }
  } else if (wide < 256) {
    const int blocks = p.B * p.ndir * p.H * ((p.N + 15) / 16);
    hipLaunchKernelGGL(k_state_bwd<4>, dim3(blocks), dim3(NTHREADS), 0, st, p, states, cs_last, dstates, g_last, dh0_dir);
  } else {
    hipLaunchKernelGGL(k_state_bwd<16>, dim3(wide), dim3(NTHREADS), 0, st, p, states, cs_last, dstates, g_last, dh0_dir);
  }
#undef ISSM_STATE_BWD_FULL
  return (int)hipGetLastError();
}

template <int PT, bool IOB, bool DTB, bool FULL, bool MIXED>
static int launch_bwd_chunk_t(const KP& p, int blocks, const float* dy_ws, const float* states, const float* dstates,
                              const float* dm, const float* g_last, float* partA, float* partBias, const int* redo,
                              int ndirs, hipStream_t st) {
  if constexpr (MIXED) {  // (never with `redo`: the tile-base kernel takes complete tiles only)
    if constexpr (IOB) {
      const size_t sm = sizeof(BwdChunkBfSmem<PT>);
      if (int e = set_lds(&k_bwd_chunk_bf_mixed<PT, DTB>, sm)) return e;
      hipLaunchKernelGGL((k_bwd_chunk_bf_mixed<PT, DTB>), dim3(blocks), dim3(NTHREADS), sm, st, p, dy_ws, states, dstates, dm, g_last, partA, partBias);
    } else {
      const size_t sm = sizeof(BwdChunkSmem<PT>);
      if (int e = set_lds(&k_bwd_chunk_mixed<PT, false, DTB>, sm)) return e;
      hipLaunchKernelGGL((k_bwd_chunk_mixed<PT, false, DTB>), dim3(blocks), dim3(NTHREADS), sm, st, p, dy_ws, states, dstates, dm, g_last, partA, partBias);
    }
  } else if constexpr (IOB) {  // bf16 inputs: every product on the bf16 matrix instructions
    const size_t sm = sizeof(BwdChunkBfSmem<PT>);
    if (int e = set_lds(&k_bwd_chunk_bf<PT, DTB, FULL>, sm)) return e;
    hipLaunchKernelGGL((k_bwd_chunk_bf<PT, DTB, FULL>), dim3(blocks), dim3(NTHREADS), sm, st, p, dy_ws, states, dstates, dm, g_last, partA, partBias, redo, ndirs);
  } else {
    const size_t sm = sizeof(BwdChunkSmem<PT>);
    if (int e = set_lds(&k_bwd_chunk<PT, false, DTB, FULL>, sm)) return e;
    hipLaunchKernelGGL((k_bwd_chunk<PT, false, DTB, FULL>), dim3(blocks), dim3(NTHREADS), sm, st, p, dy_ws, states, dstates, dm, g_last, partA, partBias, redo, ndirs);
  }
  return 0;
}

bool bwd_tile_available(const KP& p, const float* dy_ws);
int launch_bwd_tile(const KP& p, const float* states, const float* dstates, const float* dm, const float* g_last,
                    float* partA, float* partBias, int* redo, hipStream_t st);

// Chunk backward of direction p.dir0.  With a `redo` buffer (issm_bwd_chunk_redo_ints words) the tile-base kernel
// (issm_bwd_tile.hip) does the work and marks the heads outside its range; launch_bwd_chunk_redo then evaluates those
// with the level-hierarchy kernel.  Without one, or for calls the tile-base kernel is not built for (ragged tiles, packed
// sequences, a gate, mixed input types), the level-hierarchy kernel evaluates everything and *redo_pending stays 0.
int launch_bwd_chunk(const KP& p, const float* dy_ws, const float* states, const float* dstates, const float* dm,
                     const float* g_last, float* partA, float* partBias, int* redo, int* redo_pending, hipStream_t st) {
  const int blocks = p.B * p.nc * p.G * ((p.N + NS - 1) / NS);
  if (redo && bwd_tile_available(p, dy_ws)) {
    if (redo_pending) *redo_pending = 1;
    return launch_bwd_tile(p, states, dstates, dm, g_last, partA, partBias, redo, st);
  }
  ISSM_DISPATCH(p, {
    if (int e = launch_bwd_chunk_t<PT_, IOB_, DTB_, FULL_, MIXED_>(p, blocks, dy_ws, states, dstates, dm, g_last, partA,
                                                                  partBias, nullptr, 1, st))
      return e;
  });
  return (int)hipGetLastError();
}

// The level-hierarchy kernel over the heads the tile-base launches of directions p.dir0 .. p.dir0 + ndirs - 1 marked in
// `redo` (ordinary inputs mark none, and its workgroups return at once).
int launch_bwd_chunk_redo(const KP& p, int ndirs, const float* dy_ws, const float* states, const float* dstates,
                          const float* dm, const float* g_last, float* partA, float* partBias, const int* redo,
                          hipStream_t st) {
  const int blocks = p.B * p.nc * p.G * ((p.N + NS - 1) / NS);
  ISSM_DISPATCH(p, {
    if (int e = launch_bwd_chunk_t<PT_, IOB_, DTB_, FULL_, MIXED_>(p, blocks, dy_ws, states, dstates, dm, g_last, partA,
                                                                  partBias, redo, ndirs, st))
      return e;
  });
  return (int)hipGetLastError();
}

int launch_bwd_dx(const KP& p, const float* dy_ws, const float* dstates, const float* cabt, float* partD,
                  hipStream_t st) {
  const int units = p.B * p.ndir * p.nc * p.H;
  ISSM_DISPATCH(p, {
    const size_t sm = sizeof(BwdDxSmem<PT_, IOB_>);
    constexpr auto kern = MIXED_ ? &k_bwd_dx_mixed<PT_, IOB_, DTB_> : &k_bwd_dx<PT_, IOB_, DTB_, FULL_>;
    if (int e = set_lds(kern, sm)) return e;
    hipLaunchKernelGGL(kern, dim3(units), dim3(NTHREADS), sm, st, p, dy_ws, dstates, cabt, partD);
  });
  return (int)hipGetLastError();
}

int launch_bwd_reduce(const KP& p, const float* partA, const float* partBias, const float* partD,
                      const float* dh0_dir, float* dA, float* dbias, float* dD, float* dh0, hipStream_t st) {
  ReduceJobs j;
  j.partA = partA; j.partBias = partBias; j.partD = partD; j.dh0_dir = dh0_dir;
  j.dA = dA; j.dbias = dbias; j.dD = dD; j.dh0 = dh0;
  j.J = p.B * p.ndir * p.nc; j.nHN = p.H * p.N; j.H = p.H; j.P = p.P; j.ndir = p.ndir;
  j.d_hdim = (p.flags & F_D_HDIM) ? 1 : 0;
  j.n_h0 = (long)p.B * p.H * p.P * p.N;
  int nb = 0;
  j.b_A = nb; if (dA) nb += (j.nHN + 31) / 32;
  j.b_bias = nb; if (dbias) nb += (j.nHN + 31) / 32;
  j.b_D = nb; if (dD) nb += j.d_hdim ? (p.H * p.P + 31) / 32 : p.H;
  j.b_h0 = nb; if (dh0) nb += (int)((j.n_h0 + NTHREADS - 1) / NTHREADS);
  if (nb == 0) return 0;
  hipLaunchKernelGGL(k_bwd_reduce, dim3(nb), dim3(NTHREADS), 0, st, j);
  return (int)hipGetLastError();
}

}  // namespace issm
