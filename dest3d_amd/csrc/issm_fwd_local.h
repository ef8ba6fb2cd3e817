// The chunk-local pass of the forward in its level-hierarchy form (any tile shape, any decay): shared memory, helpers and
// the kernel body.  Included by the file that launches it as k_chunk_local and by the row-lane kernel for complete tiles,
// which calls the same body for the chunks outside its own range.
#pragma once
#include "issm_dev.h"

namespace issm {

// Shared memory of k_chunk_local.  Operands of the matrix instructions are bf16 tiles with the contraction index
// (the state column) contiguous: a lane's operand of one K = 32 step is 8 adjacent columns = one 16-byte read.
// SPLIT (fp32 inputs): every operand is kept as a (hi, lo) pair and a product is hi.hi + hi.lo + lo.hi; the four
// operand tiles then hold two levels at a time and a slice takes two passes.  Otherwise (bf16 inputs) one bf16
// rounding per operand is inside the bf16 tolerance and the four tiles hold the four levels.
template <int PT, bool SPLIT>
struct FwdLocalSmem {
  static constexpr int LDK = NS + 8;   // row stride of an operand tile, bf16 elements (conflict-free 16-byte fragment reads)
  static constexpr int LDT = CS + 8;   // row stride of the transposed x tile
  uint16_t xt_hi[PT * 16 * LDT];       // x tile transposed, [p][l]
  uint16_t xt_lo[SPLIT ? PT * 16 * LDT : 8];
  uint16_t op[4][CS * LDK];            // level operands [l][n]
};

// sum over the 16 lanes of a row (lanes sharing g4); the total is valid in the lane with cm == 15
__device__ __forceinline__ float row_sum16(float v) {
#define ISSM_DPP_ADD(ctrl) \
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xf, 0xf, true))
  ISSM_DPP_ADD(0x111);  // row_shr:1
  ISSM_DPP_ADD(0x112);  // row_shr:2
  ISSM_DPP_ADD(0x114);  // row_shr:4
  ISSM_DPP_ADD(0x118);  // row_shr:8
#undef ISSM_DPP_ADD
  return v;
}

// the lane's 16 values of one operand -> column `col` of a [64][LDK] bf16 tile (hi, and lo if wanted)
template <int LDK, bool SPLIT>
__device__ __forceinline__ void op_store(const float (&v)[16], uint16_t* hi, uint16_t* lo, int g4, int col) {
#pragma unroll
  for (int k = 0; k < 16; k += 2) {
    const unsigned h2 = pack_bf16(v[k], v[k + 1]);
    const int o0 = lane_row(k, g4) * LDK + col, o1 = lane_row(k + 1, g4) * LDK + col;
    hi[o0] = (uint16_t)h2;
    hi[o1] = (uint16_t)(h2 >> 16);
    if (SPLIT) {
      const unsigned l2 = pack_bf16(v[k] - __uint_as_float(h2 << 16), v[k + 1] - __uint_as_float(h2 & 0xffff0000u));
      lo[o0] = (uint16_t)l2;
      lo[o1] = (uint16_t)(l2 >> 16);
    }
  }
}
template <int LDK>
__device__ __forceinline__ bf8 op_frag(const uint16_t* tile, int row, int g4, int t) {
  return *(const bf8*)(tile + row * LDK + 32 * t + 8 * g4);
}

template <int PT, bool IOB, bool DTB, bool FULL>
__device__ __forceinline__ void k_chunk_local_body(const KP& p, float* __restrict__ states, float* __restrict__ cs_last, float* __restrict__ cabt) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  constexpr bool SPLIT = !IOB;
  typedef FwdLocalSmem<PT, SPLIT> SM;
  SM& s = *reinterpret_cast<SM*>(smem_raw);
  constexpr int LDT = SM::LDT, LDK = SM::LDK;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int cm = lane & 15, g4 = lane >> 4;
  const Unit u = decode_unit(p, xcd_remap(blockIdx.x, gridDim.x));
  const bool want_m = cabt != nullptr, want_s = states != nullptr;

  // column-lane operands of the first slice and the x tile are in flight together
  int n = wave * 16 + cm;
  bool vn = FULL || n < p.N;
  RowMap rm;
  Coef cf;
  rm = make_rowmap<FULL>(p, u, g4, 0);
  float raw[16], bv[16], cv[16];
  lane_load_ln<DTB>(p.dt, u.b, u.h, n, vn, g4, rm, raw);
  cf = lane_coef(p, u.h, n, vn);
  {
    float xv[CS * PT * 16 / NTHREADS];
    lp_load<IOB, PT, FULL>(p, u, p.x[u.dir], xv);
    lp_store_split_t<PT, LDT, SPLIT>(xv, s.xt_hi, s.xt_lo);
  }
  // Accumulators of M.  od: the off-diagonal 16x16 blocks (I, J) this wave owns -- (1,0) and (3,0) in wave 0, (3,2)
  // and (3,1) in wave 1, (2,0) in wave 2, (2,1) in wave 3; a8 / a4: levels 8 and 4 of the wave's diagonal block; sp:
  // the lane's in-group pairs (J, jl >= js) of its own column.
  f4 od[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}}, a8 = {0, 0, 0, 0}, a4 = {0, 0, 0, 0};
  float sp[40];
#pragma unroll
  for (int i = 0; i < 40; ++i) sp[i] = 0.0f;
  // roles of the lane's rows at the two levels that pair rows of one 16-row tile (the lane's rows are 4 g4 + j of
  // every tile): upper half of the 16-row block / of the 8-row block
  const bool up8 = (g4 & 2) != 0, up4 = (g4 & 1) != 0;
  const float sg8 = up8 ? 1.0f : -1.0f, sg4 = up4 ? 1.0f : -1.0f;

  __syncthreads();  // x tile complete
  for (int n0 = 0; n0 < p.N; n0 += NS) {
    // ---- column-lane phase, registers only
    lane_load_ln<IOB>(p.Bm[u.dir], u.b, u.g, n, vn, g4, rm, bv);
    lane_load_ln<IOB>(p.Cm[u.dir], u.b, u.g, n, vn, g4, rm, cv);
    float dtp[16], cs[16], dummy[16];
    const float last = lane_prep<false>(p, cf, vn, cm, g4, rm, raw, dtp, cs, dummy);
    float bd[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) bd[k] = bv[k] * dtp[k];
    if (g4 == 0 && vn) cs_last[vec_off(p, u.bt, u.c, u.h) + n] = last * LN2;
    if (n0 + NS < p.N) {  // the next slice's dt is requested as soon as this slice's has been consumed
      n = n0 + NS + wave * 16 + cm;
      vn = FULL || n < p.N;
      rm = make_rowmap<FULL>(p, u, g4, n0 + NS);
      lane_load_ln<DTB>(p.dt, u.b, u.h, n, vn, g4, rm, raw);
      cf = lane_coef(p, u.h, n, vn);
    }

    // Decays inside the lane's groups of four rows (rows 4J .. 4J+3 of tile J), from three exponentials per group:
    //   up[k] = 2^(cs[k] - cs[4J])  and  lo[k] = 2^(cs[4J+3] - cs[k]),  all <= 1.
    // Every other decay the slice needs is one of these times a factor that is the same for the four rows of a group
    // (2^(cs[4J] - ref) for rows after the reference row of a level, 2^(ref - cs[4J+3]) for rows up to it, again
    // <= 1): one exponential per group and level instead of one per element.
    float up[16], lo[16], d21[4];  // d21[J] = 2^(cs[4J+2] - cs[4J+1]), the one in-group decay that is neither
#pragma unroll
    for (int J = 0; J < 4; ++J) {
      const float d1 = ex2(cs[4 * J + 1] - cs[4 * J]), d2 = ex2(cs[4 * J + 2] - cs[4 * J + 1]);
      const float d3 = ex2(cs[4 * J + 3] - cs[4 * J + 2]);
      d21[J] = d2;
      up[4 * J] = 1.0f; up[4 * J + 1] = d1; up[4 * J + 2] = d1 * d2; up[4 * J + 3] = up[4 * J + 2] * d3;
      lo[4 * J + 3] = 1.0f; lo[4 * J + 2] = d3; lo[4 * J + 1] = d2 * d3; lo[4 * J] = up[4 * J + 3];
    }

    if (want_m) {
      // pairs inside the lane's groups of four rows (levels 2, 1 and the diagonal)
#pragma unroll
      for (int J = 0; J < 4; ++J)
#pragma unroll
        for (int jl = 0; jl < 4; ++jl)
#pragma unroll
          for (int js = 0; js <= jl; ++js) {
            const int kl = 4 * J + jl, ks = 4 * J + js;
            const float cb = cv[kl] * bd[ks];
            // 2^(cs[kl] - cs[ks]): pairs with the group's first row are entries of up, with its last row of lo
            const float dec = js == 0 ? up[kl] : jl == 3 ? lo[ks] : d21[J];
            sp[10 * J + jl * (jl + 1) / 2 + js] += jl == js ? cb : cb * dec;
          }
    }
    // What the levels (and the chunk state) multiply by their per-group factor: C * up for a row after a level's
    // reference row, Bd * lo for a row up to it.  C, Bd, up and lo themselves are not needed beyond this point.
    float pu[16], pl[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      pu[k] = cv[k] * up[k];
      pl[k] = bd[k] * lo[k];
    }

    if (want_s) {
      // S[p][n] = sum_l x[l][p] * Bd[l][n] exp2(last - cs[l][n]); B operand straight from registers
      f4 acc[PT];
#pragma unroll
      for (int pt = 0; pt < PT; ++pt) acc[pt] = (f4){0, 0, 0, 0};
      float tail[4];  // 2^(last - cs[4J+3])
#pragma unroll
      for (int J = 0; J < 4; ++J) tail[J] = ex2(last - cs[4 * J + 3]);
      rows_product_split<PT, LDT, SPLIT ? 1 : 2>(acc, s.xt_hi, s.xt_lo, [&](int k) { return pl[k] * tail[k >> 2]; }, cm, g4);
      float* dst = states + st_off(p, u.bt, u.c, u.h);
      const int nn = n0 + wave * 16 + cm;
      if (FULL && p.P == PT * 16) {  // uniform: nothing to mask
        float* d0 = dst + (4 * g4) * p.N + nn;
#pragma unroll
        for (int pt = 0; pt < PT; ++pt)
#pragma unroll
          for (int r = 0; r < 4; ++r) d0[(pt * 16 + r) * p.N] = acc[pt][r];
      } else {
#pragma unroll
        for (int pt = 0; pt < PT; ++pt)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int pp = pt * 16 + 4 * g4 + r;
            if (pp < p.P && nn < p.N) dst[(long)pp * p.N + nn] = acc[pt][r];
          }
      }
    }

    if (want_m) {
      // reference rows of the four levels: cross-lane fetches, all issued before the first is used
      const float r15 = __shfl(cs[3], cm + 48, 64), r31 = __shfl(cs[7], cm + 48, 64), r47 = __shfl(cs[11], cm + 48, 64);
      float ref8[4], ref4[4];
#pragma unroll
      for (int J = 0; J < 4; ++J) ref8[J] = __shfl(cs[4 * J + 3], cm + 16, 64);               // row 16 J + 7
#pragma unroll
      for (int J = 0; J < 4; ++J) ref4[J] = __shfl(cs[4 * J + 3], cm + 16 * (g4 & 2), 64);    // row 16 J + 8 (g4 / 2) + 3
      const int col = wave * 16 + cm;
      float v[16];
      // levels 16 and 32 pair rows of different tiles: the role of a row is fixed by its tile
      // rows after a level's reference row: (C * up) * 2^(cs[4J] - ref); rows up to it: (Bd * lo) * 2^(ref - cs[4J+3])
      auto big16 = [&]() {
#pragma unroll
        for (int J = 0; J < 4; ++J) {
          const float ref = (J & 2) ? r47 : r15;
          const float e = (J & 1) ? ex2(cs[4 * J] - ref) : ex2(ref - cs[4 * J + 3]);
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int k = 4 * J + j;
            v[k] = ((J & 1) ? pu[k] : pl[k]) * e;
          }
        }
      };
      auto big32 = [&]() {
#pragma unroll
        for (int J = 0; J < 4; ++J) {
          const float e = (J & 2) ? ex2(cs[4 * J] - r31) : ex2(r31 - cs[4 * J + 3]);
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int k = 4 * J + j;
            v[k] = ((J & 2) ? pu[k] : pl[k]) * e;
          }
        }
      };
      auto mid = [&](const float (&ref)[4], bool upper, float /*sg*/) {
#pragma unroll
        for (int J = 0; J < 4; ++J) {
          const float e = ex2(upper ? cs[4 * J] - ref[J] : ref[J] - cs[4 * J + 3]);
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int k = 4 * J + j;
            v[k] = (upper ? pu[k] : pl[k]) * e;
          }
        }
      };
      // products of one pass: T16 / T32 / T8 / T4 name the (hi, lo) tiles holding that level (nullptr = not in this pass)
      auto products = [&](const uint16_t* h16, const uint16_t* l16, const uint16_t* h32, const uint16_t* l32,
                          const uint16_t* h8, const uint16_t* l8, const uint16_t* h4, const uint16_t* l4) {
        auto prod = [&](f4& acc, const uint16_t* th, const uint16_t* tl, int ra, int rb) {
#pragma unroll
          for (int t = 0; t < 2; ++t) {
            const bf8 ah = op_frag<LDK>(th, ra + cm, g4, t), bh = op_frag<LDK>(th, rb + cm, g4, t);
            if (SPLIT) {
              const bf8 al = op_frag<LDK>(tl, ra + cm, g4, t), bl = op_frag<LDK>(tl, rb + cm, g4, t);
              acc = mfma_bf(al, bh, acc);
              acc = mfma_bf(ah, bl, acc);
            }
            acc = mfma_bf(ah, bh, acc);
          }
        };
        if (h8) prod(a8, h8, l8, wave * 16, wave * 16);
        if (h4) prod(a4, h4, l4, wave * 16, wave * 16);
        if (h16 && wave < 2) prod(od[0], h16, l16, wave ? 48 : 16, wave ? 32 : 0);       // (1,0) | (3,2)
        if (h32) {
          if (wave < 2) prod(od[1], h32, l32, 48, wave ? 16 : 0);                         // (3,0) | (3,1)
          else prod(od[0], h32, l32, 32, wave == 2 ? 0 : 16);                             // (2,0) | (2,1)
        }
      };
      if (n0 > 0) __syncthreads();  // every wave has finished reading the previous slice's tiles
      if (SPLIT) {
        big16(); op_store<LDK, true>(v, s.op[0], s.op[1], g4, col);
        big32(); op_store<LDK, true>(v, s.op[2], s.op[3], g4, col);
        __syncthreads();
        products(s.op[0], s.op[1], s.op[2], s.op[3], nullptr, nullptr, nullptr, nullptr);
        __syncthreads();
        mid(ref8, up8, sg8); op_store<LDK, true>(v, s.op[0], s.op[1], g4, col);
        mid(ref4, up4, sg4); op_store<LDK, true>(v, s.op[2], s.op[3], g4, col);
        __syncthreads();
        products(nullptr, nullptr, nullptr, nullptr, s.op[0], s.op[1], s.op[2], s.op[3]);
      } else {
        big16(); op_store<LDK, false>(v, s.op[0], nullptr, g4, col);
        big32(); op_store<LDK, false>(v, s.op[1], nullptr, g4, col);
        mid(ref8, up8, sg8); op_store<LDK, false>(v, s.op[2], nullptr, g4, col);
        mid(ref4, up4, sg4); op_store<LDK, false>(v, s.op[3], nullptr, g4, col);
        __syncthreads();
        products(s.op[0], nullptr, s.op[1], nullptr, s.op[2], nullptr, s.op[3], nullptr);
      }
    }
  }

  if (want_m) {
    float* m = cabt + sq_off(p, u.bt, u.c, u.h);
    // off-diagonal blocks: complete in the wave that owns them; accumulator r <-> (row 4 g4 + r, column cm)
    {
      const int I0 = wave == 0 ? 1 : wave == 1 ? 3 : 2, J0 = wave == 0 ? 0 : wave == 1 ? 2 : wave == 2 ? 0 : 1;
#pragma unroll
      for (int r = 0; r < 4; ++r) m[(I0 * 16 + 4 * g4 + r) * CS + J0 * 16 + cm] = od[0][r];
      if (wave < 2) {
#pragma unroll
        for (int r = 0; r < 4; ++r) m[(48 + 4 * g4 + r) * CS + wave * 16 + cm] = od[1][r];
      }
    }
    __syncthreads();  // all waves are done with the last slice's tiles
    // the in-lane pairs are sums over columns: over the 16 lanes of a row, then over the waves through LDS
    float* red_sp = reinterpret_cast<float*>(s.op[0]);   // [wave][g4][40]
    static_assert(4 * 4 * 40 * sizeof(float) <= sizeof(s.op[0]), "reduction scratch must fit in an operand tile");
#pragma unroll
    for (int i = 0; i < 40; ++i) {
      const float t = row_sum16(sp[i]);
      if (cm == 15) red_sp[(wave * 4 + g4) * 40 + i] = t;
    }
    __syncthreads();
    // diagonal block of this wave: row l = 4 g4 + r, column sc = cm
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int l = 4 * g4 + r, sc = cm, d = l ^ sc;
      float v;
      if (d >= 8) v = a8[r];
      else if (d >= 4) v = a4[r];
      else {  // same group of four rows: pair (jl, js) = (r, sc & 3) of group g4 in tile `wave`
        const int js = sc & 3, idx = 10 * wave + r * (r + 1) / 2 + (js <= r ? js : 0);
        v = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; ++w) v += red_sp[(w * 4 + g4) * 40 + idx];
      }
      if (sc > l) v = 0.0f;
      m[(wave * 16 + l) * CS + wave * 16 + sc] = v;
    }
  }
}

}  // namespace issm
