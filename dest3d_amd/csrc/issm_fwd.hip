// Forward kernels of the ISSM chunked scan for gfx950.
//
//   k_chunk_local   dt transform + cumsum, chunk-local end states S_c and the intra-chunk
//                   matrix M_c = "C.A.B^T" in one pass over dt
//   k_state_fwd_full / k_state_fwd   inter-chunk recurrence (HBM streaming)
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
// ordinary product Cw . Bw^T of rescaled operands, restricted to its blocks.  Levels 32 and 16
// are products of whole 16-row tiles, levels 8 and 4 live inside a diagonal tile (there one
// operand t = C exp2(cs - ref) on upper rows, Bd exp2(ref - cs) on lower rows serves as both
// factors: t . t^T holds the wanted entries where the row is upper and the column lower), and
// the pairs of levels 2, 1 and the diagonal belong to a single lane of the column-lane layout,
// which evaluates them directly with one exp2 per pair.
#include "issm_dev.h"
#include "issm_fwd_local.h"

namespace issm {

template <int PT, bool IOB, bool DTB, bool FULL>
__global__ __launch_bounds__(NTHREADS, 2) void k_chunk_local(KP p, float* __restrict__ states, float* __restrict__ cs_last, float* __restrict__ cabt) {
  k_chunk_local_body<PT, IOB, DTB, FULL>(p, states, cs_last, cabt);
}
// One launch for a sequence whose last chunk is ragged: complete-tile code for the complete chunks, the general code
// for the last one (uniform per workgroup).
template <int PT, bool IOB, bool DTB>
__global__ __launch_bounds__(NTHREADS, 2) void k_chunk_local_mixed(KP p, float* __restrict__ states, float* __restrict__ cs_last, float* __restrict__ cabt) {
  if (decode_unit(p, xcd_remap(blockIdx.x, gridDim.x)).c == p.nc - 1) k_chunk_local_body<PT, IOB, DTB, false>(p, states, cs_last, cabt);
  else k_chunk_local_body<PT, IOB, DTB, true>(p, states, cs_last, cabt);
}


// ---------------------------------------------------------------- state passing
// One thread carries 4 adjacent state columns of one (bt, h, p) through all chunks.
// Slot c of `states` holds S_c on entry and H_c (state at the start of chunk c) on exit;
// slot nc receives the final state.
// The recurrence for N a multiple of 4, without any conditional access: thread = 4 adjacent columns of one state row,
// the operands of the next D chunks always requested (near the end the last chunk again: in range, unused), so the
// compiler can count the loads in flight and never waits for all of them; with loads inside branches it did, once
// per chunk.  D = 8 when few threads walk many chunks (memory latency sets the pace there), otherwise 4.
template <int D>
__global__ __launch_bounds__(NTHREADS) void k_state_fwd_full(KP p, float* __restrict__ states,
                                                             const float* __restrict__ cs_last) {
  const int nq = p.N >> 2;
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
  f4 st = {0, 0, 0, 0};
  if (p.h0.ptr) {
    const long o = (long)b * p.h0.s0 + (long)h * p.h0.s1 + (long)pp * p.h0.s2 + n;
#pragma unroll
    for (int j = 0; j < 4; ++j) st[j] = ldv(p.h0.ptr, o + j, p.h0_dt);
  }
  const long cstride = (long)p.H * p.P * p.N, dstride = (long)p.H * p.N;
  float* sp = states + st_off(p, bt, 0, h) + (long)pp * p.N + n;
  const float* cl = cs_last + vec_off(p, bt, 0, h) + n;
  // chunk c lives in slot c % D; the loop is unrolled over the D slots so that none is ever moved (a register copy
  // would have to wait for the load that fills it)
  const float* sp0 = sp;
  const float* cl0 = cl;
  f4 t[D], d[D];
#pragma unroll
  for (int i = 0; i < D; ++i) {
    const int ci = min(i, p.nc - 1);
    t[i] = *(const f4*)(sp0 + ci * cstride);
    d[i] = *(const f4*)(cl0 + ci * dstride);
  }
  int c = 0;
  for (; c + D <= p.nc; c += D) {
#pragma unroll
    for (int i = 0; i < D; ++i) {
      const f4 tt = t[i], dd = d[i];
      const int cn = min(c + i + D, p.nc - 1);
      t[i] = *(const f4*)(sp0 + cn * cstride);
      d[i] = *(const f4*)(cl0 + cn * dstride);
      *(f4*)sp = st;
#pragma unroll
      for (int j = 0; j < 4; ++j) st[j] = __expf(dd[j]) * st[j] + tt[j];
      sp += cstride;
    }
  }
#pragma unroll
  for (int i = 0; i < D - 1; ++i)
    if (c + i < p.nc) {  // uniform: the last nc % D chunks
      *(f4*)sp = st;
#pragma unroll
      for (int j = 0; j < 4; ++j) st[j] = __expf(d[i][j]) * st[j] + t[i][j];
      sp += cstride;
    }
  *(f4*)sp = st;  // slot nc keeps the final state for the backward pass
  if (p.final_states[dir]) *(f4*)(p.final_states[dir] + (((long)b * p.H + h) * p.P + pp) * p.N + n) = st;
}

// The recurrence for any N (launched when N is not a multiple of 4): element-wise guards, scalar accesses.
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
    for (int j = 0; j < 4; ++j) {
      const bool v = n + j < p.N;
      sv[j] = v ? sp[j] : 0.0f;
      dv[j] = v ? cl[j] : 0.0f;
      if (v) sp[j] = st[j];
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
// BF (bf16 inputs): the operands of the product over the state index are bf16 tiles read as matrix fragments of 8
// adjacent columns; fp32 inputs: (hi, lo) pairs of such tiles from two head tiles on, fp32 tiles for one.
#ifndef SCAN_SPLIT_FROM
#define SCAN_SPLIT_FROM 2
#endif
template <int PT, bool BF>
struct FwdScanSmem {
  static constexpr int LDPT = PT * 16 + 4;
  static constexpr int LDK = NS + 8;  // row stride of the bf16 tiles
  // fp32 inputs: the product over the state index on (hi, lo) bf16 tiles, hi.hi + hi.lo + lo.hi, instead of fp32
  // matrix instructions.  An fp32 matrix instruction takes the vector ALU's issue slots (the two never overlap on this
  // chip): they were 31 % of the kernel's issue cycles beside 46 % of vector work with two head tiles, 46 % beside
  // 39 % with four.  Three bf16 instructions per product take a fifth of that and run beside the vector ALU; the
  // splitting adds a quarter to the vector work.  (SCAN_SPLIT_FROM: head tiles from which this form is used.)
  static constexpr bool SPL = !BF && PT >= SCAN_SPLIT_FROM;
  static constexpr bool B16 = BF || SPL;
  static constexpr int NH = SPL ? 2 : 1;
  float xs[CS * LDPT];                                          // x [s][p]
  typename std::conditional<B16, uint16_t, float>::type ct[NH * CS * (B16 ? LDK : LDN)];       // C * exp2(cs) [l][n]
  typename std::conditional<B16, uint16_t, float>::type hs[NH * PT * 16 * (B16 ? LDK : LDN)];  // H [p][n]
};
// a (16 PT x 64) slab of fp32 values (layout of pn_load) rounded to bf16 into LDS dst[p][col], row stride LD
template <int PT, int LD>
__device__ __forceinline__ void pn_store_bf(const PnRegs<PT>& r, uint16_t* dst, int tid = threadIdx.x) {
  typedef PnRegs<PT> R;
#pragma unroll
  for (int i = 0; i < R::CNT; ++i) {
    const int e = tid + i * NTHREADS, pp = e / R::Q, c4 = (e % R::Q) * 4;
    if (e < R::TOT) *(uint2*)(dst + pp * LD + c4) = make_uint2(pack_bf16(r.v[i][0], r.v[i][1]), pack_bf16(r.v[i][2], r.v[i][3]));
  }
}
// the same slab as (hi, lo) bf16 pairs
template <int PT, int LD>
__device__ __forceinline__ void pn_store_split(const PnRegs<PT>& r, uint16_t* hi, uint16_t* lo, int tid = threadIdx.x) {
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
// the lane's 16 values of one column -> column `col` of a [64][LD] bf16 tile
template <int LD>
__device__ __forceinline__ void col_store_bf(const float (&v)[16], uint16_t* dst, int g4, int col) {
#pragma unroll
  for (int k = 0; k < 16; k += 2) {
    const unsigned h2 = pack_bf16(v[k], v[k + 1]);
    dst[lane_row(k, g4) * LD + col] = (uint16_t)h2;
    dst[lane_row(k + 1, g4) * LD + col] = (uint16_t)(h2 >> 16);
  }
}

template <int PT, bool IOB, bool DTB, bool FULL>
__device__ __forceinline__ void k_chunk_scan_body(const KP& p, const float* __restrict__ states, const float* __restrict__ cabt, float* __restrict__ out_x) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  typedef FwdScanSmem<PT, IOB> SM;
  SM& s = *reinterpret_cast<SM*>(smem_raw);
  constexpr int LDPT = SM::LDPT, LDK = SM::LDK;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int cm = lane & 15, g4 = lane >> 4;
  const Unit u = decode_unit(p, xcd_remap(blockIdx.x, gridDim.x));
  const float* hsrc = states + st_off(p, u.bt, u.c, u.h);

  int n = wave * 16 + cm;
  bool vn = FULL || n < p.N;
  RowMap rm;
  Coef cf;
  rm = make_rowmap<FULL>(p, u, g4, 0);
  float raw[16], cv[16];
  PnRegs<PT> hv;
  lane_load_ln<DTB>(p.dt, u.b, u.h, n, vn, g4, rm, raw);
  cf = lane_coef(p, u.h, n, vn);
  lane_load_ln<IOB>(p.Cm[u.dir], u.b, u.g, n, vn, g4, rm, cv);
  pn_load<PT>(p, hsrc, 0, hv);
  // M of this wave's 16 rows goes straight into matrix-operand registers (lane (row cm, group g4) holds columns
  // 16 kb + 4 g4 .. + 3 of the blocks kb <= wave, the upper triangle of the diagonal block zeroed): no LDS tile, which
  // lets a fourth workgroup live on the CU
  f4 mf[4];
  {
    const float* mrow = cabt + sq_off(p, u.bt, u.c, u.h) + (wave * 16 + cm) * CS + 4 * g4;
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) mf[kb] = *(const f4*)(mrow + 16 * min(kb, wave));  // no branch between the loads
#pragma unroll
    for (int kb = 0; kb < 4; ++kb)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (kb > wave || (kb == wave && 4 * g4 + j > cm)) mf[kb][j] = 0.0f;
  }
  {
    float xv[CS * PT * 16 / NTHREADS];
    lp_load<IOB, PT, FULL>(p, u, p.x[u.dir], xv);
    lp_store<PT>(xv, s.xs, LDPT);
  }
  f4 acc[PT];
#pragma unroll
  for (int pt = 0; pt < PT; ++pt) acc[pt] = (f4){0, 0, 0, 0};

  for (int n0 = 0; n0 < p.N; n0 += NS) {
    {
      float dtp[16], cs[16], dummy[16];
      lane_prep<false>(p, cf, vn, cm, g4, rm, raw, dtp, cs, dummy);
      if constexpr (IOB) {
        float ctv[16];
#pragma unroll
        for (int k = 0; k < 16; ++k) ctv[k] = cv[k] * ex2(cs[k]);
        col_store_bf<LDK>(ctv, s.ct, g4, wave * 16 + cm);
      } else if constexpr (SM::SPL) {
        float ctv[16];
#pragma unroll
        for (int k = 0; k < 16; ++k) ctv[k] = cv[k] * ex2(cs[k]);
        op_store<LDK, true>(ctv, s.ct, s.ct + CS * LDK, g4, wave * 16 + cm);
      } else {
#pragma unroll
        for (int k = 0; k < 16; ++k) s.ct[lane_row(k, g4) * LDN + wave * 16 + cm] = cv[k] * ex2(cs[k]);
      }
    }
    if constexpr (IOB) pn_store_bf<PT, LDK>(hv, s.hs);
    else if constexpr (SM::SPL) pn_store_split<PT, LDK>(hv, s.hs, s.hs + PT * 16 * LDK);
    else pn_store<PT>(hv, s.hs);
    if (n0 + NS < p.N) {
      n = n0 + NS + wave * 16 + cm;
      vn = FULL || n < p.N;
      rm = make_rowmap<FULL>(p, u, g4, n0 + NS);
      lane_load_ln<DTB>(p.dt, u.b, u.h, n, vn, g4, rm, raw);
      cf = lane_coef(p, u.h, n, vn);
      lane_load_ln<IOB>(p.Cm[u.dir], u.b, u.g, n, vn, g4, rm, cv);
      pn_load<PT>(p, hsrc, n0 + NS, hv);
    }
    __syncthreads();
    // y[l][p] += sum_n Ct[l][n] H[p][n]; wave owns 16 rows
    if constexpr (IOB) {
      // bf16 inputs: one rounding of C exp(cs) and of the entry state to bf16 (the reference stores the entry states
      // in the input dtype and casts its dot operands, issm_combined.py:87, issm_chunk_scan.py:149-190)
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const bf8 a = op_frag<LDK>(s.ct, wave * 16 + cm, g4, t);
#pragma unroll
        for (int pt = 0; pt < PT; ++pt) acc[pt] = mfma_bf(a, op_frag<LDK>(s.hs, pt * 16 + cm, g4, t), acc[pt]);
      }
    } else if constexpr (SM::SPL) {
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const bf8 ah = op_frag<LDK>(s.ct, wave * 16 + cm, g4, t), al = op_frag<LDK>(s.ct + CS * LDK, wave * 16 + cm, g4, t);
#pragma unroll
        for (int pt = 0; pt < PT; ++pt)
          acc[pt] = mfma_split(ah, al, op_frag<LDK>(s.hs, pt * 16 + cm, g4, t),
                               op_frag<LDK>(s.hs + PT * 16 * LDK, pt * 16 + cm, g4, t), acc[pt]);
      }
    } else {
#pragma unroll
      for (int kb = 0; kb < NS; kb += 16)
#pragma unroll
        for (int pt = 0; pt < PT; ++pt) mma16_mm(acc[pt], s.ct, LDN, wave * 16, s.hs, LDN, pt * 16, kb, lane);
    }
    __syncthreads();
  }
  // y[l][p] += sum_{s<=l} M[l][s] x[s][p]; rows of this wave only need s < 16(wave+1)
#pragma unroll
  for (int kb = 0; kb < 4; ++kb)
    if (kb <= wave) {  // uniform
      // the lane's four M values and four x values are the operands of one K = 16 bf16 instruction as they stand
      // (k-slot j of lane group g4 <-> row 16 kb + 4 g4 + j), M as a (hi, lo) pair and, for fp32 inputs, x too
      const float mw[4] = {mf[kb][0], mf[kb][1], mf[kb][2], mf[kb][3]};
      bf4 ah, al;
      split4(mw, ah, al);
#pragma unroll
      for (int pt = 0; pt < PT; ++pt) {
        const float* bp = s.xs + (16 * kb + 4 * g4) * LDPT + pt * 16 + cm;
        const float xw[4] = {bp[0], bp[LDPT], bp[2 * LDPT], bp[3 * LDPT]};
        bf4 bh, bl;
        split4(xw, bh, bl);
        acc[pt] = mfma_bf16k(al, bh, acc[pt]);
        if constexpr (!IOB) acc[pt] = mfma_bf16k(ah, bl, acc[pt]);  // (bf16 inputs: x is exact, its lo part zero)
        acc[pt] = mfma_bf16k(ah, bh, acc[pt]);
      }
    }

  const TensorD& to = p.out[u.dir];
  const TensorD& tz = p.z[u.dir];
#pragma unroll
  for (int pt = 0; pt < PT; ++pt) {
    int off[4];
    float v[4];
    // the skip coefficient of the lane's column, read once and without a lane-dependent branch (absent columns read
    // the head's last one; their results are not stored)
    float dcoef = 0.0f;
    if (p.D) dcoef = (p.flags & F_D_HDIM) ? p.D[u.h * p.P + min(pt * 16 + cm, p.P - 1)] : p.D[u.h];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int l = wave * 16 + 4 * g4 + r, pp = pt * 16 + cm;
      const int tt = u.c * CS + l;
      const bool ok = tt < p.L && pp < p.P;
      const int pr = ok ? phys_row(p, u.dir, tt) : 0;
      v[r] = fmaf(dcoef, s.xs[l * LDPT + pp], acc[pt][r]);
      if (tz.ptr && ok) {
        if (out_x) out_x[(((long)u.bt * p.L + pr) * p.H + u.h) * p.P + pp] = v[r];
        const float zz = ldv(tz.ptr, (long)u.b * tz.s0 + (long)pr * tz.s1 + (long)u.h * tz.s2 + pp, p.io_dt);
        v[r] *= zz * sigmoidf_(zz);
      }
      off[r] = ok ? pr * (int)to.s1 + pp : -1;
    }
    gstore<IOB, 4>(const_cast<void*>(to.ptr), (long)u.b * to.s0 + (long)u.h * to.s2, off, v);
  }
}
// fp32 inputs, two head tiles: 128 registers, so that a fourth workgroup lives on the CU (130 without the bound; the
// nine spilled dwords cost less than the fourth workgroup gives: 52 -> 48.5 us)
template <int PT, bool IOB, bool DTB, bool FULL>
__global__ __launch_bounds__(NTHREADS, (PT <= 2 && FULL && !IOB) ? 4 : 1) void k_chunk_scan(KP p, const float* __restrict__ states, const float* __restrict__ cabt, float* __restrict__ out_x) {
  k_chunk_scan_body<PT, IOB, DTB, FULL>(p, states, cabt, out_x);
}
// One launch for a sequence whose last chunk is ragged: complete-tile code for the complete chunks, the general code
// for the last one (uniform per workgroup).
template <int PT, bool IOB, bool DTB>
__global__ __launch_bounds__(NTHREADS) void k_chunk_scan_mixed(KP p, const float* __restrict__ states, const float* __restrict__ cabt, float* __restrict__ out_x) {
  if (decode_unit(p, xcd_remap(blockIdx.x, gridDim.x)).c == p.nc - 1) k_chunk_scan_body<PT, IOB, DTB, false>(p, states, cabt, out_x);
  else k_chunk_scan_body<PT, IOB, DTB, true>(p, states, cabt, out_x);
}


// ------------------------------------------------------------------- launchers
template <typename K>
static int set_lds(K kernel, size_t bytes) {
  return (int)hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
}

bool local_tile_available(const KP& p, const float* states, const float* cabt);
int launch_local_tile(const KP& p, float* states, float* cs_last, float* cabt, hipStream_t st);

// Launches made of complete tiles go to the row-lane kernel (which itself falls back to the level-hierarchy body for
// the chunks outside its range); everything else to the level-hierarchy kernel.
int launch_chunk_local(const KP& p, float* states, float* cs_last, float* cabt, hipStream_t st) {
  if (local_tile_available(p, states, cabt)) return launch_local_tile(p, states, cs_last, cabt, st);
  const int units = p.B * p.ndir * p.nc * p.H;
  ISSM_DISPATCH(p, {
    const size_t sm = sizeof(FwdLocalSmem<PT_, !IOB_>);
    constexpr auto kern = MIXED_ ? &k_chunk_local_mixed<PT_, IOB_, DTB_> : &k_chunk_local<PT_, IOB_, DTB_, FULL_>;
    if (int e = set_lds(kern, sm)) return e;
    hipLaunchKernelGGL(kern, dim3(units), dim3(NTHREADS), sm, st, p, states, cs_last, cabt);
  });
  return (int)hipGetLastError();
}

int launch_state_fwd(const KP& p, float* states, const float* cs_last, hipStream_t st) {
  const long total = (long)p.B * p.ndir * p.H * p.P * ((p.N + 3) / 4);
  const int blocks = (int)((total + NTHREADS - 1) / NTHREADS);
  if ((p.N & 3) == 0) {
    if (total < (1L << 17) && p.nc >= 16)
      hipLaunchKernelGGL(k_state_fwd_full<8>, dim3(blocks), dim3(NTHREADS), 0, st, p, states, cs_last);
    else
      hipLaunchKernelGGL(k_state_fwd_full<4>, dim3(blocks), dim3(NTHREADS), 0, st, p, states, cs_last);
  } else {
    hipLaunchKernelGGL(k_state_fwd, dim3(blocks), dim3(NTHREADS), 0, st, p, states, cs_last);
  }
  return (int)hipGetLastError();
}

int launch_chunk_scan(const KP& p, const float* states, const float* cabt, float* out_x, hipStream_t st) {
  const int units = p.B * p.ndir * p.nc * p.H;
  ISSM_DISPATCH(p, {
    const size_t sm = sizeof(FwdScanSmem<PT_, IOB_>);
    constexpr auto kern = MIXED_ ? &k_chunk_scan_mixed<PT_, IOB_, DTB_> : &k_chunk_scan<PT_, IOB_, DTB_, FULL_>;
    if (int e = set_lds(kern, sm)) return e;
    hipLaunchKernelGGL(kern, dim3(units), dim3(NTHREADS), sm, st, p, states, cabt, out_x);
  });
  return (int)hipGetLastError();
}

}  // namespace issm
