// Generation of the scan's dt / B / C from the pairwise distance encoding (gfx950).
//
// DEST builds the per-(token, query) scan parameters as tiny projections of `dist` (tokens, K, M):
//   base[r][k] = sum_m W[r][m] dist[k][m],   r = 0 .. R0-1,  R0 = H + 2G  (dt heads, B groups, C groups)
//   dt[h][k] = base[h][k] + bias[h],  B[g][k] = base[H+g][k] + bias[H+g],  C[g][k] = base[H+G+g][k] + bias[H+G+g]
// and, for the reversed-order scan, a second B / C pair from the same base rows with their own biases
// (models/dest_module.py:543-553).  As library GEMMs these are thousands of (R0 x M)(M x K) products with
// M = 16: launch- and layout-bound.  Here one pass reads `dist` once and writes every output; the backward is
// one pass as well (ddist, per-token bias gradients, per-workgroup partials of dW) plus a fixed-order
// reduction of the partials.  Everything is memory bound; arithmetic is fp32.
#include "issm_dev.h"

namespace issm {

constexpr int PG_MAXR0 = 12;  // largest H + 2G built (three 4-row steps of the matrix instruction)
constexpr int PG_M = 16;      // distance encoding width this kernel is built for
constexpr int PG_TOK = 4;     // tokens per workgroup in the backward (one per wave)
constexpr int PG_LDT = 20;    // row stride of the backward's 16 x 16 LDS tiles (column-wise reads of four row groups
                              // fall into different banks; rows stay 8- and 16-byte aligned)

// sum over the 16 lanes that share lane >> 4; valid in the lane with (lane & 15) == 15
__device__ __forceinline__ float row_sum16_(float v) {
#define ISSM_PG_DPP_ADD(ctrl) \
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xf, 0xf, true))
  ISSM_PG_DPP_ADD(0x111);  // row_shr:1
  ISSM_PG_DPP_ADD(0x112);  // row_shr:2
  ISSM_PG_DPP_ADD(0x114);  // row_shr:4
  ISSM_PG_DPP_ADD(0x118);  // row_shr:8
#undef ISSM_PG_DPP_ADD
  return v;
}

template <bool BF>
__device__ __forceinline__ void load_row16(const void* p, long off, float (&v)[PG_M]) {
  if (BF) {
    const uint4* q = (const uint4*)((const uint16_t*)p + off);
    const uint4 a = q[0], b = q[1];
    const unsigned w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      v[2 * i] = __uint_as_float(w[i] << 16);
      v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  } else {
    const f4* q = (const f4*)((const float*)p + off);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const f4 a = q[i];
      v[4 * i] = a.x; v[4 * i + 1] = a.y; v[4 * i + 2] = a.z; v[4 * i + 3] = a.w;
    }
  }
}
template <bool BF>
__device__ __forceinline__ void store_row16(void* p, long off, const float (&v)[PG_M]) {
  if (BF) {
    unsigned w[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) w[i] = (unsigned)f_to_bf16(v[2 * i]) | ((unsigned)f_to_bf16(v[2 * i + 1]) << 16);
    uint4* q = (uint4*)((uint16_t*)p + off);
    q[0] = make_uint4(w[0], w[1], w[2], w[3]);
    q[1] = make_uint4(w[4], w[5], w[6], w[7]);
  } else {
    f4* q = (f4*)((float*)p + off);
#pragma unroll
    for (int i = 0; i < 4; ++i) q[i] = (f4){v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]};
  }
}
template <bool BF>
__device__ __forceinline__ float ld1(const void* p, long i) {
  return BF ? bf16_to_f(((const uint16_t*)p)[i]) : ((const float*)p)[i];
}
template <bool BF>
__device__ __forceinline__ void st1(void* p, long i, float v) {
  if (BF) ((uint16_t*)p)[i] = f_to_bf16(v); else ((float*)p)[i] = v;
}

// KV adjacent outputs of one row as one store (4 bytes for two bf16, 8 / 16 bytes for two / four floats).
template <bool BF, int KV>
__device__ __forceinline__ void stv(void* p, long i, const float (&v)[KV]) {
  if constexpr (KV == 1) {
    st1<BF>(p, i, v[0]);
  } else if constexpr (BF) {
    unsigned w[KV / 2];
#pragma unroll
    for (int j = 0; j < KV / 2; ++j) w[j] = (unsigned)f_to_bf16(v[2 * j]) | ((unsigned)f_to_bf16(v[2 * j + 1]) << 16);
    uint16_t* q = (uint16_t*)p + i;
    if constexpr (KV == 4) *(uint2*)q = make_uint2(w[0], w[1]);
    else *(unsigned*)q = w[0];
  } else {
    float* q = (float*)p + i;
    if constexpr (KV == 4) *(f4*)q = (f4){v[0], v[1], v[2], v[3]};
    else *(float2*)q = make_float2(v[0], v[1]);
  }
}

// Forward: thread = (token, KV adjacent k) -- KV = 2 whenever K is even, so that every store instruction of a wave
// covers 256 (bf16) or 512 bytes instead of 128 / 256.  W and the token's biases are uniform across the lanes of a
// token: scalar operands.
template <bool BF, int KV>
__global__ __launch_bounds__(NTHREADS) void k_pgen_fwd(PGenP p) {
  const int R0 = p.H + 2 * p.G, R = R0 + (p.has_back ? 2 * p.G : 0);
  const int per_tok = (p.K + KV - 1) / KV;  // threads per token
  const long gid = (long)blockIdx.x * NTHREADS + threadIdx.x;
  const long t = gid / per_tok;
  const int k = (int)(gid % per_tok) * KV;
  if (t >= p.tokens) return;
  float d[KV][PG_M];
#pragma unroll
  for (int j = 0; j < KV; ++j) load_row16<BF>(p.dist, (t * p.K + k + j) * PG_M, d[j]);
  float wk[KV];
#pragma unroll
  for (int j = 0; j < KV; ++j) wk[j] = p.weights ? p.weights[t * p.K + k + j] : 1.0f;
  // the token's biases, all requested before the row loop (a load per row inside it would be waited for row by
  // row); bb: the reversed-order pair's bias of a B / C row
  const float* bias = p.bias + t * R;
  float bv[PG_MAXR0], bb[PG_MAXR0];
#pragma unroll
  for (int r = 0; r < PG_MAXR0; ++r) {
    bv[r] = bias[min(r, R - 1)];
    bb[r] = bias[min(max(R0 + r - p.H, 0), R - 1)];
  }
#pragma unroll
  for (int r = 0; r < PG_MAXR0; ++r) {
    if (r < R0) {  // uniform
      const float* w = p.W + r * PG_M;  // uniform: scalar loads
      float s[KV], v[KV];
#pragma unroll
      for (int j = 0; j < KV; ++j) {
        s[j] = 0.0f;
#pragma unroll
        for (int m = 0; m < PG_M; ++m) s[j] = fmaf(w[m], d[j][m], s[j]);
        v[j] = s[j] + bv[r];
      }
      if (r < p.H) {
        if (p.weights) {  // uniform: dt = softplus(raw) * weight, raw kept for the backward
          if (BF) {
#pragma unroll
            for (int j = 0; j < KV; ++j) v[j] = bf16_to_f(f_to_bf16(v[j]));  // the saved value is what the backward differentiates
          }
          stv<BF, KV>(p.dt_raw, (t * p.H + r) * p.K + k, v);
#pragma unroll
          for (int j = 0; j < KV; ++j) v[j] = softplus_(v[j]) * wk[j];
        }
        stv<BF, KV>(p.dt, (t * p.H + r) * p.K + k, v);
      } else {
        const bool isB = r < p.H + p.G;
        const int g = isB ? r - p.H : r - p.H - p.G;
        stv<BF, KV>(isB ? p.Bm : p.Cm, (t * p.G + g) * p.K + k, v);
        if (p.has_back) {
#pragma unroll
          for (int j = 0; j < KV; ++j) v[j] = s[j] + bb[r];
          stv<BF, KV>(isB ? p.Bb : p.Cb, (t * p.G + g) * p.K + k, v);
        }
      }
    }
  }
}

// Gradient row r of token t: dt heads, then B groups, then C groups (`back`: the reversed-order pair, which
// exists for the B / C rows only).  Returns the element offset of (t, row, k = 0), or -1 when there is none.
struct GradRows {
  const void *ddt, *dB, *dC, *dBb, *dCb;
  int H, G, K;
  __device__ __forceinline__ const void* base(int r, bool back) const {
    if (r < H) return back ? nullptr : ddt;
    if (r < H + G) return back ? dBb : dB;
    if (r < H + 2 * G) return back ? dCb : dC;
    return nullptr;
  }
  __device__ __forceinline__ long offset(long t, int r) const {
    if (r < H) return (t * H + r) * K;
    if (r < H + G) return (t * G + (r - H)) * K;
    return (t * G + (r - H - G)) * K;
  }
};

// Loads without branches: a lane with nothing to read (no such row, k past the end) reads element 0 of `safe`
// -- any readable buffer of at least 16 bytes -- and the value is replaced by zero afterwards.  Branch-free
// loads can all be in flight together; a branch per load would serialise them.
template <bool BF>
__device__ __forceinline__ float ld1_or0(const void* p, long off, bool ok, const void* safe) {
  const float v = ld1<BF>(ok ? p : safe, ok ? off : 0);
  return ok ? v : 0.0f;
}
// Four consecutive elements p[off .. off + 3] for k .. k + 3 (k >= kend reads as zero).  `vec`: the address is
// aligned for one wide load and kend is a multiple of 4.
template <bool BF>
__device__ __forceinline__ f4 load4(const void* p, long off, int k, int kend, bool vec, const void* safe) {
  f4 r;
  if (vec) {  // uniform
    const bool ok = p != nullptr && k < kend;
    const void* q = ok ? p : safe;
    const long o = ok ? off : 0;
    if (BF) {
      const uint2 w = *(const uint2*)((const uint16_t*)q + o);
      r.x = __uint_as_float(w.x << 16); r.y = __uint_as_float(w.x & 0xffff0000u);
      r.z = __uint_as_float(w.y << 16); r.w = __uint_as_float(w.y & 0xffff0000u);
    } else {
      r = *(const f4*)((const float*)q + o);
    }
    if (!ok) r = (f4){0.0f, 0.0f, 0.0f, 0.0f};
  } else {
#pragma unroll
    for (int v = 0; v < 4; ++v) r[v] = ld1_or0<BF>(p, off + v, p != nullptr && k + v < kend, safe);
  }
  return r;
}

// d softplus(x) / dx with torch's threshold: 1 above 20
__device__ __forceinline__ float dsoftplus_(float x) { return x <= 20.0f ? sigmoidf_(x) : 1.0f; }

// Backward on the matrix cores (v_mfma_f32_16x16x4_f32; lane = (i = lane & 15, q = lane >> 4)).
// Workgroup = PG_TOK consecutive tokens, a wave owns PG_TOK / 4 of them and walks k in blocks of 16:
//   ddist^T (m x k) = W^T (m x r) g (r x k)   -- A: lane (m, q) = W[4s + q][m], B: lane (k, q) = g[4s + q][k0 + k];
//                                                the result lane (k, q) holds ddist[k0 + k][4q .. 4q + 3]: one wide store
//   dW (r x m)     += g (r x k) dist (k x m)  -- A: lane (r, q) = g[r][k0 + 4q + v], B: lane (m, q) = dist[k0 + 4q + v][m],
//                                                v = 0..3 (the order of k inside the sum is free)
//   dbias[r]        = sum_k g[r][k]           -- from the second layout, reduced over q at the end of the token.
// g of a B / C row is the sum of its forward-order and reversed-order gradients wherever the shared base row is
// differentiated; the two bias gradients stay apart.  HASW (dt = softplus(raw) * weight): g of a dt row is
// ddt * weight * softplus'(raw), and dweight[k] = sum_h ddt[h][k] softplus(raw[h][k]).
// FULLK: K is a multiple of 64, so no load or store needs a bound on k, and every per-lane address is a
// pointer advanced once per trip plus a compile-time offset.  UNR blocks of 16 k have their loads in flight together.
template <bool BF, bool FULLK, bool HASW>
__global__ __launch_bounds__(NTHREADS, (BF || !HASW || !FULLK) ? 4 : 3) void k_pgen_bwd(PGenP p) {
  constexpr int UNR = 2;
  typedef typename std::conditional<BF, uint16_t, float>::type T;
  typedef typename std::conditional<BF, uint2, f4>::type T4;
  __shared__ float wred[4][16 * PG_M];
  // per-wave transposition tiles of the FULLK path: effective gradients [row][k] and the dist block [k][m]
  __shared__ __align__(16) float sg[FULLK ? 4 : 1][FULLK ? UNR : 1][FULLK ? 16 * PG_LDT : 4];
  __shared__ __align__(16) T sd[FULLK ? 4 : 1][FULLK ? UNR : 1][FULLK ? 16 * PG_LDT : 8];
  const int R0 = p.H + 2 * p.G, R = R0 + (p.has_back ? 2 * p.G : 0);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int i = lane & 15, q = lane >> 4;
  const int K = p.K;
  const bool vec = (K & 3) == 0;
  const GradRows gr{p.ddt, p.dB, p.dC, p.has_back ? p.dBb : nullptr, p.has_back ? p.dCb : nullptr, p.H, p.G, K};
  float wA[3];
#pragma unroll
  for (int s = 0; s < 3; ++s) wA[s] = (4 * s + q < R0) ? p.W[(4 * s + q) * PG_M + i] : 0.0f;
  // row-of-the-lane pointers: layout 2 (row i), layout 1 (rows 4s + q)
  const void* g2 = gr.base(i, false);
  const void* g2b = gr.base(i, true);
  const bool isdt2 = HASW && i < p.H && g2 != nullptr;
  const void *g1[3], *g1b[3];
  bool okg[3], okgb[3], isdt1[3];
#pragma unroll
  for (int s = 0; s < 3; ++s) {
    g1[s] = gr.base(4 * s + q, false);
    g1b[s] = gr.base(4 * s + q, true);
    okg[s] = g1[s] != nullptr;
    okgb[s] = g1b[s] != nullptr;
    isdt1[s] = HASW && 4 * s + q < p.H && okg[s];
  }
  const bool ok2 = g2 != nullptr, ok2b = g2b != nullptr;
  const bool any_back = gr.dBb != nullptr || gr.dCb != nullptr;  // uniform
  const f4 zero4 = {0.0f, 0.0f, 0.0f, 0.0f};
  auto widen = [](T4 w) -> f4 {
    if constexpr (BF) {
      return (f4){__uint_as_float(w.x << 16), __uint_as_float(w.x & 0xffff0000u), __uint_as_float(w.y << 16),
                  __uint_as_float(w.y & 0xffff0000u)};
    } else {
      return w;
    }
  };
  auto widen1 = [](T w) -> float {
    if constexpr (BF) return __uint_as_float((unsigned)w << 16);
    else return w;
  };
  // one block of 16 k, operands already in registers (a / ab / rw2 / ww2: layout 2; x*, raw1, w1: layout 1)
  f4 accW = zero4;
  float bs = 0.0f, bsb = 0.0f;
  auto block = [&](f4 a, f4 ab, f4 rw2, f4 ww2, const float (&dv)[4], const float (&x)[3], const float (&xb)[3],
                   const float (&raw1)[3], float w1, T* ddst, float* dwdst, bool in_k) {
    if constexpr (HASW) {
      if (isdt2) {
#pragma unroll
        for (int v = 0; v < 4; ++v) a[v] *= ww2[v] * dsoftplus_(rw2[v]);
      }
    }
    bs += (a.x + a.y) + (a.z + a.w);
    bsb += (ab.x + ab.y) + (ab.z + ab.w);
#pragma unroll
    for (int v = 0; v < 4; ++v) accW = mfma4(a[v] + ab[v], dv[v], accW);
    float gx[3], dws = 0.0f;
#pragma unroll
    for (int s = 0; s < 3; ++s) {
      gx[s] = x[s];
      if constexpr (HASW) {
        if (isdt1[s]) {
          dws += x[s] * softplus_(raw1[s]);
          gx[s] = x[s] * w1 * dsoftplus_(raw1[s]);
        }
      }
      gx[s] += xb[s];
    }
    if constexpr (HASW) {
      if (dwdst != nullptr) {  // uniform
        dws += __shfl_xor(dws, 16, 64);
        dws += __shfl_xor(dws, 32, 64);
        if (q == 0 && in_k) *dwdst = dws;
      }
    }
    if (ddst != nullptr) {  // uniform
      f4 dd = zero4;
#pragma unroll
      for (int s = 0; s < 3; ++s) dd = mfma4(wA[s], gx[s], dd);
      if (in_k) {
        if constexpr (BF) {
          uint2 w;
          w.x = pack_bf16(dd.x, dd.y);
          w.y = pack_bf16(dd.z, dd.w);
          *(uint2*)ddst = w;
        } else {
          *(f4*)ddst = dd;
        }
      }
    }
  };

  constexpr int TPW = PG_TOK / 4;
  for (int ti = 0; ti < TPW; ++ti) {
    const long t = (long)blockIdx.x * PG_TOK + wave * TPW + ti;
    if (t >= p.tokens) break;  // wave-uniform
    const long o2 = i < R0 ? gr.offset(t, i) : 0;
    long o1[3];
#pragma unroll
    for (int s = 0; s < 3; ++s) o1[s] = (4 * s + q < R0) ? gr.offset(t, 4 * s + q) : 0;
    bs = 0.0f;
    bsb = 0.0f;
    if constexpr (FULLK) {
      // Every operand is read once, with one 8- or 16-byte load per lane, in the layout whose lane index is the
      // gradient row (lane (i, q): row i, columns k0 + 4q .. + 3).  The second layout the products need -- lane index
      // = column -- comes out of a 16 x 16 tile per wave in LDS, written row-wise and read column-wise; so does the
      // block of dist (16 k x 16 m, loaded as 64 pieces of four adjacent m).  Reading both layouts from global memory
      // took fourteen 2-byte-per-lane loads per block, and the load pipe, not HBM, set the pace.
      const T* nil = (const T*)p.dist;  // what a lane with no row reads (at least 64 * 16 elements long)
      const T* pa = ok2 ? (const T*)g2 + o2 + 4 * q : nil;
      const T* pab = ok2b ? (const T*)g2b + o2 + 4 * q : nil;
      const T* pd = (const T*)p.dist + (t * K + 4 * q + (i >> 2)) * PG_M + 4 * (i & 3);
      const T* pr2 = isdt2 ? (const T*)p.dt_raw + o2 + 4 * q : nil;
      const float* pw2 = HASW ? p.weights + t * K + 4 * q : nullptr;
      T* pdd = p.ddist ? (T*)p.ddist + (t * K + i) * PG_M + 4 * q : nullptr;
      float* pdw = (HASW && p.dweights) ? p.dweights + t * K + 4 * q : nullptr;
      // Two sets of operand registers used in turn: while one set is worked on, the other set's loads are in flight
      // (K is a multiple of 64, so the number of 16 * UNR-column steps is even; the request after the last step reads
      // the last step's operands once more instead of sitting under a branch).
      constexpr int STEP = 16 * UNR;
      const int nstep = K / STEP;
      auto request = [&](int is, T4 (&ra)[UNR], T4 (&rab)[UNR], T4 (&rr2)[UNR], T4 (&rd)[UNR], f4 (&rw2)[UNR]) {
        const int k0 = min(is, nstep - 1) * STEP;
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
          ra[u] = *(const T4*)(pa + (ok2 ? k0 : 0) + 16 * u);
          if (any_back) rab[u] = *(const T4*)(pab + (ok2b ? k0 : 0) + 16 * u);
          rd[u] = *(const T4*)(pd + (long)(k0 + 16 * u) * PG_M);
          if constexpr (HASW) {
            rr2[u] = *(const T4*)(pr2 + (isdt2 ? k0 : 0) + 16 * u);
            rw2[u] = *(const f4*)(pw2 + k0 + 16 * u);
          }
        }
      };
      auto work = [&](int is, T4 (&ra)[UNR], T4 (&rab)[UNR], T4 (&rr2)[UNR], T4 (&rd)[UNR], f4 (&rw2)[UNR]) {
        const int k0 = is * STEP;
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
          float* S = sg[wave][u];
          T* D = sd[wave][u];
          f4 a = ok2 ? widen(ra[u]) : zero4;
          const f4 ab = (any_back && ok2b) ? widen(rab[u]) : zero4;
          f4 pw = zero4;  // ddt * softplus(raw): the weight's gradient once summed over the heads
          if constexpr (HASW) {
            if (isdt2) {
              const f4 raw = widen(rr2[u]);
#pragma unroll
              for (int v = 0; v < 4; ++v) {
                const float tt = ex2(raw[v] * LOG2E), uu = 1.0f + tt;
                const bool big = raw[v] > 20.0f;  // torch's softplus threshold
                pw[v] = a[v] * (big ? raw[v] : LN2 * __builtin_amdgcn_logf(uu));
                a[v] *= rw2[u][v] * (big ? 1.0f : tt * __builtin_amdgcn_rcpf(uu));
              }
            }
          }
          bs += (a.x + a.y) + (a.z + a.w);
          bsb += (ab.x + ab.y) + (ab.z + ab.w);
          const f4 g = a + ab;
          *(f4*)(S + i * PG_LDT + 4 * q) = g;
          *(T4*)(D + (4 * q + (i >> 2)) * PG_LDT + 4 * (i & 3)) = rd[u];
          // (LDS instructions of one wave are carried out in order: the reads below see the writes above)
          float dv[4], x[3];
#pragma unroll
          for (int v = 0; v < 4; ++v) dv[v] = widen1(D[(4 * q + v) * PG_LDT + i]);
#pragma unroll
          for (int s = 0; s < 3; ++s) x[s] = S[(4 * s + q) * PG_LDT + i];
#pragma unroll
          for (int v = 0; v < 4; ++v) accW = mfma4(g[v], dv[v], accW);
          if (pdd != nullptr) {  // uniform
            f4 dd = zero4;
#pragma unroll
            for (int s = 0; s < 3; ++s) dd = mfma4(wA[s], x[s], dd);
            T* dst = pdd + (long)(k0 + 16 * u) * PG_M;
            if constexpr (BF) {
              uint2 w;
              w.x = pack_bf16(dd.x, dd.y);
              w.y = pack_bf16(dd.z, dd.w);
              *(uint2*)dst = w;
            } else {
              *(f4*)dst = dd;
            }
          }
          if constexpr (HASW) {
            if (pdw != nullptr) {  // uniform: sum over the rows = over the 16 lanes that share q
#pragma unroll
              for (int v = 0; v < 4; ++v) pw[v] = row_sum16_(pw[v]);
              if (i == 15) *(f4*)(pdw + k0 + 16 * u) = pw;
            }
          }
        }
      };
      T4 ra0[UNR], rab0[UNR], rr20[UNR], rd0[UNR], ra1[UNR], rab1[UNR], rr21[UNR], rd1[UNR];
      f4 rw20[UNR], rw21[UNR];
      request(0, ra0, rab0, rr20, rd0, rw20);
      for (int is = 0; is < nstep; is += 2) {
        request(is + 1, ra1, rab1, rr21, rd1, rw21);
        work(is, ra0, rab0, rr20, rd0, rw20);
        request(is + 2, ra0, rab0, rr20, rd0, rw20);
        work(is + 1, ra1, rab1, rr21, rd1, rw21);
      }
    } else {
      const void* safe = p.W;
      for (int k0 = 0; k0 < K; k0 += 16) {
        const int kq = k0 + 4 * q;
        const bool in = k0 + i < K;
        const f4 a = load4<BF>(g2, o2 + kq, kq, K, vec, safe);
        const f4 ab = any_back ? load4<BF>(g2b, o2 + kq, kq, K, vec, safe) : zero4;
        f4 rw2 = zero4, ww2 = zero4;
        float dv[4], x[3], xb[3], raw1[3], w1 = 0.0f;
#pragma unroll
        for (int v = 0; v < 4; ++v) dv[v] = ld1_or0<BF>(p.dist, (t * K + kq + v) * PG_M + i, kq + v < K, safe);
#pragma unroll
        for (int s = 0; s < 3; ++s) {
          x[s] = ld1_or0<BF>(g1[s], o1[s] + k0 + i, in && okg[s], safe);
          xb[s] = any_back ? ld1_or0<BF>(g1b[s], o1[s] + k0 + i, in && okgb[s], safe) : 0.0f;
          raw1[s] = HASW ? ld1_or0<BF>(p.dt_raw, o1[s] + k0 + i, in && isdt1[s], safe) : 0.0f;
        }
        if constexpr (HASW) {
          rw2 = load4<BF>(isdt2 ? p.dt_raw : nullptr, o2 + kq, kq, K, vec, safe);
          ww2 = load4<false>(p.weights, t * K + kq, kq, K, vec, safe);
          w1 = ld1_or0<false>(p.weights, t * K + k0 + i, in, safe);
        }
        block(a, ab, rw2, ww2, dv, x, xb, raw1, w1,
              p.ddist ? (T*)p.ddist + (t * K + k0 + i) * PG_M + 4 * q : nullptr,
              (HASW && p.dweights) ? p.dweights + t * K + k0 + i : nullptr, in);
      }
    }
    bs += __shfl_xor(bs, 16, 64);
    bs += __shfl_xor(bs, 32, 64);
    bsb += __shfl_xor(bsb, 16, 64);
    bsb += __shfl_xor(bsb, 32, 64);
    if (p.dbias && q == 0 && i < R0) {
      p.dbias[t * R + i] = bs;
      if (p.has_back && i >= p.H) p.dbias[t * R + R0 + (i - p.H)] = bsb;
    }
  }
  // dW partial of the workgroup: the four waves in order.  Lane (m, q) holds rows 4q .. 4q + 3 of column m.
#pragma unroll
  for (int v = 0; v < 4; ++v) wred[wave][(4 * q + v) * PG_M + i] = accW[v];
  __syncthreads();
  for (int e = threadIdx.x; e < R0 * PG_M; e += NTHREADS)
    p.dw_partial[(long)blockIdx.x * R0 * PG_M + e] = (wred[0][e] + wred[1][e]) + (wred[2][e] + wred[3][e]);
}

// dW = fixed-order sum of the per-workgroup partials: one workgroup per entry of dW; the workgroups after those sum
// one column of dbias over the tokens each (same tree, so both are reproducible)
__global__ __launch_bounds__(NTHREADS) void k_pgen_dw(PGenP p) {
  __shared__ float red[NTHREADS];
  const int n = (p.H + 2 * p.G) * PG_M;
  const int c = blockIdx.x;
  float a0 = 0.0f, a1 = 0.0f;
  if (c < n) {
    int b = threadIdx.x;
    for (; b + NTHREADS < p.nblocks; b += 2 * NTHREADS) {
      a0 += p.dw_partial[(long)b * n + c];
      a1 += p.dw_partial[(long)(b + NTHREADS) * n + c];
    }
    if (b < p.nblocks) a0 += p.dw_partial[(long)b * n + c];
  } else {
    const int R = p.H + 2 * p.G + (p.has_back ? 2 * p.G : 0), r = c - n;
    long t = threadIdx.x;
    for (; t + NTHREADS < p.tokens; t += 2 * NTHREADS) {
      a0 += p.dbias[t * R + r];
      a1 += p.dbias[(t + NTHREADS) * R + r];
    }
    if (t < p.tokens) a0 += p.dbias[t * R + r];
  }
  red[threadIdx.x] = a0 + a1;
  __syncthreads();
#pragma unroll
  for (int w = NTHREADS / 2; w > 0; w >>= 1) {
    if ((int)threadIdx.x < w) red[threadIdx.x] += red[threadIdx.x + w];
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    if (c < n) p.dW[c] = red[0];
    else p.dbias_sum[c - n] = red[0];
  }
}

int pgen_bwd_blocks(long tokens) { return (int)((tokens + PG_TOK - 1) / PG_TOK); }

int launch_pgen_fwd(const PGenP& p, hipStream_t st) {
  // adjacent outputs go out as one store: K a multiple of the group and every output 16-byte aligned
  uintptr_t bits = 0;
  for (const void* q : {(const void*)p.dt, (const void*)p.dt_raw, (const void*)p.Bm, (const void*)p.Cm, (const void*)p.Bb,
                        (const void*)p.Cb})
    bits |= (uintptr_t)q;
  const bool al = (bits & 15) == 0;
  // (four adjacent k per thread, 8-byte bf16 stores, measured slower: 42 us against 39 at 8192 tokens x 256)
  const int kv = (p.K % 2 == 0 && al) ? 2 : 1;
  const long threads = p.tokens * ((p.K + kv - 1) / kv);
  const unsigned blocks = (unsigned)((threads + NTHREADS - 1) / NTHREADS);
  if (p.dtype) {
    if (kv == 2) hipLaunchKernelGGL((k_pgen_fwd<true, 2>), dim3(blocks), dim3(NTHREADS), 0, st, p);
    else hipLaunchKernelGGL((k_pgen_fwd<true, 1>), dim3(blocks), dim3(NTHREADS), 0, st, p);
  } else {
    if (kv == 2) hipLaunchKernelGGL((k_pgen_fwd<false, 2>), dim3(blocks), dim3(NTHREADS), 0, st, p);
    else hipLaunchKernelGGL((k_pgen_fwd<false, 1>), dim3(blocks), dim3(NTHREADS), 0, st, p);
  }
  return (int)hipGetLastError();
}

template <bool BF, bool HASW>
static void pgen_bwd_launch(const PGenP& p, hipStream_t st) {
  const dim3 g((unsigned)p.nblocks), b(NTHREADS);
  if (p.K % 64 == 0) hipLaunchKernelGGL((k_pgen_bwd<BF, true, HASW>), g, b, 0, st, p);
  else hipLaunchKernelGGL((k_pgen_bwd<BF, false, HASW>), g, b, 0, st, p);
}

int launch_pgen_bwd(const PGenP& p, hipStream_t st) {
  const int R0 = p.H + 2 * p.G;
  if (p.dtype) {
    if (p.weights) pgen_bwd_launch<true, true>(p, st);
    else pgen_bwd_launch<true, false>(p, st);
  } else {
    if (p.weights) pgen_bwd_launch<false, true>(p, st);
    else pgen_bwd_launch<false, false>(p, st);
  }
  int e = (int)hipGetLastError();
  if (e) return e;
  const int R = R0 + (p.has_back ? 2 * p.G : 0);
  hipLaunchKernelGGL(k_pgen_dw, dim3(R0 * PG_M + (p.dbias_sum ? R : 0)), dim3(NTHREADS), 0, st, p);
  return (int)hipGetLastError();
}

}  // namespace issm
