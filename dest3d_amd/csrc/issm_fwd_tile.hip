// k_local_tile: the chunk-local pass of the forward (dt transform, running sums, chunk end states S_c, intra-chunk
// matrix M_c, the chunk's total decay) for complete 64 x 64 tiles, in a ROW-lane layout.
//
// Lane (i, kg) of a wave owns row i of every 16-row tile of the chunk and four adjacent state columns
// n = n0 + 4 kg .. + 3: exactly the operand layout of v_mfma_f32_16x16x16_bf16 for a contraction over the state
// columns, and a 16-byte (fp32) or 8-byte (bf16) load per tensor and tile.  The four waves of a workgroup take the
// four 16-column quarters of each 64-column step.
//
//   running sums   down the 16 rows of a tile = across the 16 lanes of a DPP row: four shifted adds per value.
//                  pc[l] = sum of a = dt' A log2(e) over the rows of l's tile up to and including l.
//   decays         exp2(cs[l] - cs[s]) = up[l] . G . iup[s],  up = exp2(pc), iup = exp2(-pc), G = product of the whole-
//                  tile decays et[K] = exp2(tile sum K) of the tiles from s's tile up to (not including) l's tile
//   M (I, J)       = sum_n U_I[l][n] X_IJ[s][n],  U = C up,  X_JJ = W = dt' B iup,  X_(J+1)J = V = W et[J],
//                  X_(J+2)J = V et[J+1],  X_30 = V et[1] et[2]: ten plain 16 x 16 products per 16 columns with both
//                  operands taken from registers as they are.  Each wave sums over its columns; the four partial sums
//                  meet in LDS once per chunk.
//   S^T (n, p)     = sum_l V[l][n] (decay from the end of l's tile to the end of the chunk)[n] x[l][p].  This contracts
//                  over the ROWS, so V is needed with the roles of lane and register exchanged: one matrix instruction
//                  against a 16 x 16 identity moves a (bf16, hence exactly representable) tile into the accumulator
//                  layout, which is that exchanged layout.  x^T comes from LDS.  The decay to the end of the chunk depends
//                  on the OUTPUT row n only: the accumulator is multiplied by et[J+1] between the tiles (Horner).  The
//                  result holds four adjacent columns of a state row per lane: 16-byte stores.
//
// Everything but W is a product of factors <= 1.  W grows like 2^(span of a tile): a chunk with a tile whose sum of a is
// below -FWD_SPAN_LIMIT is computed once more, by the same workgroup, with the level-hierarchy body (k_chunk_local_body),
// which has no such limit and overwrites everything written for the chunk before.
#include "issm_dev.h"
#include "issm_fwd_local.h"

namespace issm {

constexpr float FWD_SPAN_LIMIT = 100.0f;

template <int PT, bool SPLIT>
struct FwdTileSmem {
  static constexpr int LDT = CS + 8;   // row stride of the transposed x tile
  uint16_t xt_hi[PT * 16 * LDT];       // x tile transposed, [p][l]
  uint16_t xt_lo[SPLIT ? PT * 16 * LDT : 8];
  f4 red[4 * 10 * 64];                 // the four waves' partial sums of the ten blocks of M
  int bad[4];
};
template <int PT, bool SPLIT>
constexpr size_t fwd_tile_lds() {     // the level-hierarchy body lays its own structure over the same memory
  return sizeof(FwdTileSmem<PT, SPLIT>) > sizeof(FwdLocalSmem<PT, SPLIT>) ? sizeof(FwdTileSmem<PT, SPLIT>)
                                                                          : sizeof(FwdLocalSmem<PT, SPLIT>);
}

// inclusive running sum over the 16 lanes of a DPP row (lanes sharing lane >> 4)
__device__ __forceinline__ float row_scan16(float v) {
#define ISSM_DPP_SHR(ctrl) \
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xf, 0xf, true))
  ISSM_DPP_SHR(0x111);  // row_shr:1, lanes without a source add 0
  ISSM_DPP_SHR(0x112);
  ISSM_DPP_SHR(0x114);
  ISSM_DPP_SHR(0x118);
#undef ISSM_DPP_SHR
  return v;
}

// four fp32 accumulator values that are exact bf16 numbers -> a bf16 fragment
__device__ __forceinline__ bf4 exact_bf4(f4 v) {
  // v_perm_b32: bytes 2, 3 of the second source below bytes 2, 3 of the first
  const uint2 r = make_uint2(__builtin_amdgcn_perm(__float_as_uint(v[1]), __float_as_uint(v[0]), 0x07060302u),
                             __builtin_amdgcn_perm(__float_as_uint(v[3]), __float_as_uint(v[2]), 0x07060302u));
  return __builtin_bit_cast(bf4, r);
}

template <bool SPLIT>
struct Frag {
  bf4 h, l;
};
template <bool SPLIT>
__device__ __forceinline__ Frag<SPLIT> make_frag(float a, float b, float c, float d) {
  Frag<SPLIT> f;
  const float v[4] = {a, b, c, d};
  if (SPLIT) {
    split4(v, f.h, f.l);
  } else {
    const uint2 r = make_uint2(pack_bf16(a, b), pack_bf16(c, d));
    f.h = __builtin_bit_cast(bf4, r);
    f.l = f.h;
  }
  return f;
}
// acc += A . B^T over the lane groups' columns: both operands (hi, lo) pairs when SPLIT, one bf16 rounding otherwise
template <bool SPLIT>
__device__ __forceinline__ f4 frag_product(const Frag<SPLIT>& a, const Frag<SPLIT>& b, f4 acc) {
  if (SPLIT) {
    acc = mfma_bf16k(a.l, b.h, acc);
    acc = mfma_bf16k(a.h, b.l, acc);
  }
  return mfma_bf16k(a.h, b.h, acc);
}

template <bool BF>
struct RawVec {
  typedef typename std::conditional<BF, uint2, f4>::type type;
};
template <bool BF>
__device__ __forceinline__ void unpack4(const typename RawVec<BF>::type& r, float* out) {
  if constexpr (BF) {
    out[0] = __uint_as_float(r.x << 16);
    out[1] = __uint_as_float(r.x & 0xffff0000u);
    out[2] = __uint_as_float(r.y << 16);
    out[3] = __uint_as_float(r.y & 0xffff0000u);
  } else {
    out[0] = r[0]; out[1] = r[1]; out[2] = r[2]; out[3] = r[3];
  }
}

template <int PT, bool IOB, bool DTB, bool FULLP>
__global__ __launch_bounds__(NTHREADS, 2) void k_local_tile(KP p, float* __restrict__ states, float* __restrict__ cs_last,
                                                            float* __restrict__ cabt) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  constexpr bool SPLIT = !IOB;
  typedef FwdTileSmem<PT, SPLIT> SM;
  SM& s = *reinterpret_cast<SM*>(smem_raw);
  constexpr int LDT = SM::LDT;
  typedef typename RawVec<DTB>::type RawDt;
  typedef typename RawVec<IOB>::type RawIo;
  typedef typename std::conditional<DTB, uint16_t, float>::type TDt;
  typedef typename std::conditional<IOB, uint16_t, float>::type TIo;
  typedef Frag<SPLIT> Fr;

  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int i = lane & 15, kg = lane >> 4;
  const int uidx = xcd_remap(blockIdx.x, gridDim.x);
  const Unit u = decode_unit(p, uidx);

  // addresses: uniform base + per-lane 32-bit element offset (the host checks that seqlen * stride fits in 31 bits);
  // tile J lies 16 J rows further along the scan, the step's columns 64 further along the row
  const int tl = u.dir ? p.L - 1 - u.c * CS - i : u.c * CS + i;   // the lane's token of tile 0
  const int sgn = u.dir ? -1 : 1;
  const int ncol = 16 * w + 4 * kg;                                // the lane's first column within a step
  const TDt* qdt = (const TDt*)p.dt.ptr + ((long)u.b * p.dt.s0 + (long)u.h * p.dt.s2);
  const TIo* qB = (const TIo*)p.Bm[u.dir].ptr + ((long)u.b * p.Bm[u.dir].s0 + (long)u.g * p.Bm[u.dir].s2);
  const TIo* qC = (const TIo*)p.Cm[u.dir].ptr + ((long)u.b * p.Cm[u.dir].s0 + (long)u.g * p.Cm[u.dir].s2);
  const unsigned odt = (unsigned)(tl * (int)p.dt.s1 + ncol), oB = (unsigned)(tl * (int)p.Bm[u.dir].s1 + ncol),
                 oC = (unsigned)(tl * (int)p.Cm[u.dir].s1 + ncol);
  const int jdt = sgn * 16 * (int)p.dt.s1, jB = sgn * 16 * (int)p.Bm[u.dir].s1, jC = sgn * 16 * (int)p.Cm[u.dir].s1;
  const float* qA = p.A + u.h * p.N + ncol;
  const float* qbias = (p.dt_bias ? p.dt_bias : p.A) + u.h * p.N + ncol;  // without a bias: any valid address, scaled by 0
  const float bias_on = p.dt_bias ? 1.0f : 0.0f;

  RawDt rdt[4];
  RawIo rB[4], rC[4];
  f4 rA, rbias;
#define ISSM_REQUEST(n0_)                                                              \
  {                                                                                    \
    _Pragma("unroll") for (int J = 0; J < 4; ++J) {                                    \
      rdt[J] = *(const RawDt*)(qdt + (int)(odt + (unsigned)(J * jdt + (n0_))));        \
      rB[J] = *(const RawIo*)(qB + (int)(oB + (unsigned)(J * jB + (n0_))));            \
      rC[J] = *(const RawIo*)(qC + (int)(oC + (unsigned)(J * jC + (n0_))));            \
    }                                                                                  \
    rA = *(const f4*)(qA + (n0_));                                                     \
    rbias = *(const f4*)(qbias + (n0_));                                               \
  }
  ISSM_REQUEST(0);

  // the unit's x tile, transposed, as bf16 (hi, lo) in LDS (its loads travel together with the first step's above)
  {
    float xv[CS * PT * 16 / NTHREADS];
    lp_load<IOB, PT, true>(p, u, p.x[u.dir], xv);
    lp_store_split_t<PT, LDT, SPLIT>(xv, s.xt_hi, s.xt_lo);
  }


  // identity operand of the exchange of lane and register roles: B[k = 4 kg + r][j = i] = (k == j)
  bf4 ident;
  {
    const unsigned one = 0x3F80u;
    const int r1 = i - 4 * kg;
    const uint2 idr = make_uint2((r1 == 0 ? one : 0u) | (r1 == 1 ? one << 16 : 0u), (r1 == 2 ? one : 0u) | (r1 == 3 ? one << 16 : 0u));
    ident = __builtin_bit_cast(bf4, idr);
  }
  const int last_lane = lane | 15;
  const float thr = ex2(-FWD_SPAN_LIMIT);

  f4 macc[10];
#pragma unroll
  for (int q = 0; q < 10; ++q) macc[q] = (f4){0.0f, 0.0f, 0.0f, 0.0f};
  float etmin = 1.0f;  // smallest whole-tile decay seen by the lane

  __syncthreads();  // x tile complete
  float* sdst = states + st_off(p, u.bt, u.c, u.h);
  float* cdst = cs_last + vec_off(p, u.bt, u.c, u.h);

#pragma unroll 1
  for (int n0 = 0; n0 < p.N; n0 += NS) {
    // ---- this step's values out of the request registers; the next step's request follows at once
    float dtv[16], bv[16], cv[16];
#pragma unroll
    for (int J = 0; J < 4; ++J) {
      unpack4<DTB>(rdt[J], dtv + 4 * J);
      unpack4<IOB>(rB[J], bv + 4 * J);
      unpack4<IOB>(rC[J], cv + 4 * J);
    }
    float A2[4], bias[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      A2[r] = rA[r] * LOG2E;
      bias[r] = rbias[r] * bias_on;
    }
    {  // branch-free: the last step asks for its own columns once more
      const int nn = min(n0 + NS, p.N - NS);
      ISSM_REQUEST(nn);
    }

    // ---- dt transform and the running sums of the tiles
    float dtp[16], dummy[16];
    {
      float pre[16];
#pragma unroll
      for (int k = 0; k < 16; ++k) pre[k] = dtv[k] + bias[k & 3];
      dt_transform<false, 16>(p, pre, dtp, dummy);
    }
    float pc[16], up[16], et[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) pc[k] = row_scan16(dtp[k] * A2[k & 3]);
#pragma unroll
    for (int k = 0; k < 16; ++k) up[k] = ex2(pc[k]);
#pragma unroll
    for (int k = 0; k < 16; ++k) et[k] = __shfl(up[k], last_lane, 64);  // whole-tile decay of the lane's columns
#pragma unroll
    for (int k = 0; k < 16; k += 2) etmin = fminf(etmin, fminf(et[k], et[k + 1]));
    {  // the chunk's total decay (natural logarithm), four adjacent columns per lane group.  All 16 lanes of a group
       // store the same values to the same place: a store under a lane condition sits behind a branch, and the waits
       // for the requests in flight -- counted in order with the stores -- would then have to assume it away and wait
       // for every store as well.
      f4 tot;
#pragma unroll
      for (int r = 0; r < 4; ++r)
        tot[r] = __shfl((((pc[r] + pc[4 + r]) + pc[8 + r]) + pc[12 + r]) * LN2, last_lane, 64);
      *(f4*)(cdst + n0 + ncol) = tot;
    }

    // ---- operands
    Fr U[4];
#pragma unroll
    for (int J = 0; J < 4; ++J)
      U[J] = make_frag<SPLIT>(cv[4 * J] * up[4 * J], cv[4 * J + 1] * up[4 * J + 1], cv[4 * J + 2] * up[4 * J + 2],
                              cv[4 * J + 3] * up[4 * J + 3]);
    f4 sacc[PT];
#pragma unroll
    for (int pt = 0; pt < PT; ++pt) sacc[pt] = (f4){0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int J = 0; J < 4; ++J) {
      float W[4], V[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int k = 4 * J + r;
        W[r] = dtp[k] * bv[k] * ex2(-pc[k]);
        V[r] = W[r] * et[k];
      }
      {
        const Fr f = make_frag<SPLIT>(W[0], W[1], W[2], W[3]);
        macc[J] = frag_product<SPLIT>(U[J], f, macc[J]);
      }
      // V serves the block below the diagonal one (J < 3) and the chunk state: always as a (hi, lo) pair
      const Frag<true> fv = make_frag<true>(V[0], V[1], V[2], V[3]);
      if (J < 3) {
        Fr f;
        f.h = fv.h;
        f.l = fv.l;
        macc[4 + J] = frag_product<SPLIT>(U[J + 1], f, macc[4 + J]);
      }
      if (J < 2) {
        float V2[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) V2[r] = V[r] * et[4 * (J + 1) + r];
        const Fr f = make_frag<SPLIT>(V2[0], V2[1], V2[2], V2[3]);
        macc[7 + J] = frag_product<SPLIT>(U[J + 2], f, macc[7 + J]);
        if (J == 0) {
          const Fr g = make_frag<SPLIT>(V2[0] * et[8], V2[1] * et[9], V2[2] * et[10], V2[3] * et[11]);
          macc[9] = frag_product<SPLIT>(U[3], g, macc[9]);
        }
      }
      // chunk state: what the earlier tiles have summed decays across tile J (accumulator r <-> the lane's column r),
      // then V of tile J, lane and register roles exchanged, meets x^T of tile J's rows
      {
        if (J > 0) {
#pragma unroll
          for (int pt = 0; pt < PT; ++pt)
#pragma unroll
            for (int r = 0; r < 4; ++r) sacc[pt][r] *= et[4 * J + r];
        }
        // (wider head dimensions: keep the scheduler from fetching every tile's x fragments ahead of time, which
        // costs more registers than there are)
        if (PT > 2) __builtin_amdgcn_sched_barrier(0);
        const f4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
        const bf4 th = exact_bf4(mfma_bf16k(fv.h, ident, zero)), tlo = exact_bf4(mfma_bf16k(fv.l, ident, zero));
#pragma unroll
        for (int pt = 0; pt < PT; ++pt) {
          const int xo = (16 * pt + i) * LDT + 16 * J + 4 * kg;
          const bf4 xh = *(const bf4*)(s.xt_hi + xo);
          sacc[pt] = mfma_bf16k(tlo, xh, sacc[pt]);
          if (SPLIT) {
            const bf4 xl = *(const bf4*)(s.xt_lo + xo);
            sacc[pt] = mfma_bf16k(th, xl, sacc[pt]);
          }
          sacc[pt] = mfma_bf16k(th, xh, sacc[pt]);
        }
      }
    }
    // S^T block: lane (p = i, kg) holds columns n0 + ncol .. + 3 of state row 16 pt + i
    if (FULLP) {  // every state row exists: plain stores (see the note at the chunk's total decay)
#pragma unroll
      for (int pt = 0; pt < PT; ++pt) *(f4*)(sdst + (16 * pt + i) * p.N + n0 + ncol) = sacc[pt];
    } else {
#pragma unroll
      for (int pt = 0; pt < PT; ++pt)
        if (16 * pt + i < p.P) *(f4*)(sdst + (16 * pt + i) * p.N + n0 + ncol) = sacc[pt];
    }
  }
#undef ISSM_REQUEST

  // ---- M: the waves' partial sums meet in LDS; wave w then finishes blocks w, w + 4, w + 8
#pragma unroll
  for (int q = 0; q < 10; ++q) s.red[(w * 10 + q) * 64 + lane] = macc[q];
  {
    const bool anybad = __ballot(!(etmin >= thr)) != 0ull;
    if (lane == 0) s.bad[w] = anybad ? 1 : 0;
  }
  __syncthreads();
  const int anybad = s.bad[0] | s.bad[1] | s.bad[2] | s.bad[3];  // uniform
  float* m = cabt + sq_off(p, u.bt, u.c, u.h);
#pragma unroll
  for (int t = 0; t < 3; ++t) {
    const int q = w + 4 * t;  // uniform
    if (q < 10) {
      f4 v = s.red[q * 64 + lane];
#pragma unroll
      for (int ww = 1; ww < 4; ++ww) {
        const f4 o = s.red[(ww * 10 + q) * 64 + lane];
        v[0] += o[0]; v[1] += o[1]; v[2] += o[2]; v[3] += o[3];
      }
      // block (I, J) of index q: 0..3 diagonal, 4..6 (J+1, J), 7..8 (J+2, J), 9 (3, 0)
      const int I = q < 4 ? q : q < 7 ? q - 3 : q < 9 ? q - 5 : 3, J = q < 4 ? q : q < 7 ? q - 4 : q < 9 ? q - 7 : 0;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int l = 4 * kg + r;  // accumulator r <-> (row 4 kg + r, column i) of the block
        m[(16 * I + l) * CS + 16 * J + i] = (I == J && i > l) ? 0.0f : v[r];
      }
    }
  }
  if (anybad) {
    // A tile of this chunk decays by more than 2^-FWD_SPAN_LIMIT: everything is computed once more in the form that has no
    // such limit.  The fence orders this workgroup's stores above before the ones the other form makes to the same places.
    __threadfence();
    __syncthreads();
    k_chunk_local_body<PT, IOB, DTB, true>(p, states, cs_last, cabt);
  }
}

// Whether the row-lane kernel can take the launch: complete tiles everywhere, both outputs wanted, and every operand
// addressable with 16-byte (fp32) / 8-byte (bf16) accesses.
bool local_tile_available(const KP& p, const float* states, const float* cabt) {
  if (p.full_tiles != 1 || !states || !cabt) return false;
  auto vec_ok = [](const TensorD& t, int bf) {
    return ((t.s0 | t.s1 | t.s2) & 3) == 0 && (((uintptr_t)t.ptr) & (bf ? 7 : 15)) == 0;
  };
  if (!vec_ok(p.dt, p.dt_dt)) return false;
  for (int d = 0; d < p.ndir; ++d)
    if (!vec_ok(p.Bm[d], p.io_dt) || !vec_ok(p.Cm[d], p.io_dt)) return false;
  if ((((uintptr_t)p.A) & 15) || (p.dt_bias && (((uintptr_t)p.dt_bias) & 15))) return false;
  if ((((uintptr_t)states) & 15) || (p.N & 63)) return false;
  return true;
}

template <typename K>
static int set_lds_tile(K kernel, size_t bytes) {
  return (int)hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
}

int launch_local_tile(const KP& p, float* states, float* cs_last, float* cabt, hipStream_t st) {
  const int units = p.B * p.ndir * p.nc * p.H;
  const int pt = (p.P + 15) / 16;
#define ISSM_LT(PT_, IOB_, DTB_)                                                                            \
  {                                                                                                         \
    const size_t sm = fwd_tile_lds<PT_, !IOB_>();                                                           \
    if (p.P == 16 * PT_) {                                                                                  \
      constexpr auto kern = &k_local_tile<PT_, IOB_, DTB_, true>;                                           \
      if (int e = set_lds_tile(kern, sm)) return e;                                                         \
      hipLaunchKernelGGL(kern, dim3(units), dim3(NTHREADS), sm, st, p, states, cs_last, cabt);              \
    } else {                                                                                                \
      constexpr auto kern = &k_local_tile<PT_, IOB_, DTB_, false>;                                          \
      if (int e = set_lds_tile(kern, sm)) return e;                                                         \
      hipLaunchKernelGGL(kern, dim3(units), dim3(NTHREADS), sm, st, p, states, cs_last, cabt);              \
    }                                                                                                       \
  }
#define ISSM_LT_DT(PT_)                                                      \
  {                                                                          \
    if (p.io_dt) {                                                           \
      if (p.dt_dt) ISSM_LT(PT_, true, true) else ISSM_LT(PT_, true, false)   \
    } else {                                                                 \
      if (p.dt_dt) ISSM_LT(PT_, false, true) else ISSM_LT(PT_, false, false) \
    }                                                                        \
  }
  if (pt <= 2) ISSM_LT_DT(2) else if (pt == 3) ISSM_LT_DT(3) else ISSM_LT_DT(4)
#undef ISSM_LT_DT
#undef ISSM_LT
  return (int)hipGetLastError();
}

}  // namespace issm
