// Device-side building blocks shared by the ISSM kernels (gfx950 / CDNA4 only).
//
// Tiling conventions used by every kernel in this directory
//  * one workgroup = 256 threads = 4 wavefronts of 64 lanes;
//  * time is cut into chunks of CS = 64 tokens, the state dimension into slices of NS = 64
//    columns; a "unit" is one (batch*direction, chunk, head);
//  * every LDS tile is a row-major float array whose leading dimension is (width + 4): with
//    ld = 4 (mod 8) both fragment access patterns below are free of bank conflicts;
//  * matrix products run on v_mfma_f32_16x16x4_f32.  Lane (cm = lane & 15, g4 = lane >> 4)
//    feeds the j-th of four back-to-back MFMAs with k = kb + 4 g4 + j, so that an operand
//    stored with k contiguous ("M-major", tile[m][k]) is fetched with one 128-bit LDS read and
//    an operand stored with m contiguous ("K-major", tile[k][m]) with four 32-bit reads.  The
//    accumulator register r of that lane holds element (row = 4 g4 + r, col = cm) of the
//    16x16 result;
//  * "column-lane layout": a wave owns 16 state columns, lane (cm, g4) owns column cm and the
//    16 chunk rows {16J + 4 g4 + j : J, j = 0..3}, array index k = 4J + j.  A lane then holds
//    exactly the elements it feeds as the K-major B operand of a product that contracts over
//    rows, and exactly the accumulator rows it gets back from a product whose output rows are
//    chunk rows, so cumulative sums, decays and all elementwise work stay in registers.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

// A wave-uniform value made opaque to the optimizer (its multiples are then formed next to their use instead of being
// hoisted out of loops into scarce scalar registers).  A translation unit may define its own form before including this.
#ifndef ISSM_OPAQUE_S
#define ISSM_OPAQUE_S(x) asm volatile("" : "+s"(x))
#endif

namespace issm {

constexpr int CS = 64;         // tokens per chunk
constexpr int NS = 64;         // state columns per slice
constexpr int LDN = NS + 4;    // leading dimension of [*][NS] tiles
constexpr int LDC = CS + 4;    // leading dimension of [*][CS] tiles
constexpr int MAXP = 64;       // largest head dimension built
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
  int dir0;  // direction handled by this launch (kernels launched per direction)
  int io_dt, dt_dt, h0_dt;  // 0 = f32, 1 = bf16
  unsigned flags;
  float dt_min, dt_max;
  TensorD x[2], Bm[2], Cm[2], z[2], out[2], dout[2], dx[2], dB[2], dC[2], dz[2];
  TensorD dt, ddt, h0;
  // Two directions with a bf16 ddt: the first direction's share of ddt travels in fp32 through this (B, L, H, N) buffer
  // instead of through ddt itself, so that the sum of the two is rounded to bf16 once (null: it travels through ddt).
  TensorD ddt_part;
  const float* A;
  const float* D;
  const float* dt_bias;
  float* final_states[2];
  const float* dfinal[2];
  const int* seq_idx;   // (B, L) sequence ids of packed rows, or null
  long seq_s0, seq_s1;
  // Chunks [c_lo, c_lo + ncl) are the ones a launch of a per-chunk kernel covers (all nc of them).  full_tiles picks
  // the kernel variants: 1 = every chunk has 64 rows and every column slice 64 columns (complete-tile code, no
  // masks); 2 = that holds for all chunks but the last in scan order (the sequence length is not a multiple of 64):
  // one launch whose workgroups take the complete-tile code except those of the last chunk, which take the general
  // code -- the general code alone runs 1.5 - 2x longer; 0 = general code everywhere (ragged column slices, packed
  // sequences, a single chunk).
  int c_lo, ncl, full_tiles;
};

enum : unsigned { F_SOFTPLUS = 1u, F_D_HDIM = 2u, F_NOCLAMP = 4u };
// What the running sum of dt' A log2(e) takes where the sequence id changes: decays across the change become 2^-128.
constexpr float SEQ_CUT = 128.0f;

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
  int ln;           // LayerNorm statistics (mean subtracted) instead of RMS
  const void* b;    // bias in the weight's dtype, or null
  float* mean;
  float* db_partial;
  float* db;
};

// parameters of the serialization-code kernel (hilbert.hip)
struct HilbertP {
  int B, N, bits;
  int perm[3];          // grid coordinate used as first / second / third curve coordinate
  float cell;
  const float* points;  // (B, N, 3)
  const float* mins;    // (B, 3) per-sample minimum corner
  long* codes;          // (B, N)
};

// the whole serialization in one launch (hilbert.hip): index / inverse (norder, B, N), NP = N rounded up to a power of two
struct HilbertOrderP {
  int B, N, NP, bits, norder;
  int perm[6][3];
  float cell;
  const float* points;
  long* index;
  long* inverse;  // may be null
};

// parameters of the box-to-point distance encoding kernels (box_dist.hip)
struct BoxDistP {
  int B, L, K, D, H, W, dtype, nwg, nwg_bwd;
  const float* key;      // (B, L, 3)
  const float* corners;  // (B, K, 8, 3), or NULL with boxes given
  const float* boxes;    // (B, K, 7) centre, size, heading: corners (and the weight's centre / radius) derived from it
  float min_radius;
  const float* angle;    // (B, K) or NULL (zero)
  const float* table;    // (16, D, H, W)
  float log_scale, max_value;
  void* dist;            // (B, L, K, 16) io dtype, or NULL
  const float* qcenter;  // (B, K, 3), with radius (B, K): inputs of the locality weight
  const float* radius;
  float weight_dist;
  float* weights;        // (B, L, K) fp32, or NULL
  const void* ddist;     // (B, L, K, 16) io dtype
  void* partial;         // 2 words (scale) + (nwg_bwd, D*H*W, 16) 64-bit fixed-point words
  float* dtable;         // (16, D, H, W) fp32
};

// parameters of the depthwise conv + SiLU kernels (dwconv_silu.hip)
struct DwConvP {
  int B, L, C, nsets, dtype;
  int chain;           // nsets == 2: set 1 convolves set 0's output instead of u
  const void* u;       // (B, L, C) io dtype, element strides u_bs (batch), u_ls (token), channels contiguous
  long u_bs, u_ls;
  const float* w;      // (nsets, C, 7) fp32
  const float* bias;   // (nsets, C) fp32
  void* y;             // (nsets, B, L, C) io dtype; with split > 0: (nsets, B, L, split), channels [0, split)
  void* y_tail;        // split > 0: (nsets, B, L, C - split), channels [split, C)
  int split;
  void* pre;           // (nsets, B, L, C) io dtype: convolution output before SiLU (saved for the backward)
  const void* dy[2];   // (B, L, C) io dtype per set, or NULL; with split > 0: (B, L, split)
  const void* dy_tail[2];  // split > 0: (B, L, C - split) per set, or NULL
  void* du;            // (B, L, C) io dtype, element strides du_bs, du_ls, channels contiguous
  long du_bs, du_ls;
  float* partial;      // (nrows, nsets, 8, C) fp32
  int nrows;
  float* dw;           // (nsets, C, 7) fp32
  float* dbias;        // (nsets, C) fp32
};

// parameters of the dt / B / C generation kernels (param_gen.hip)
struct PGenP {
  long tokens;
  int K, H, G, dtype, has_back;
  const void* dist;      // (tokens, K, M) io dtype
  const float* W;        // (R0, M) fp32
  const float* bias;     // (tokens, R) fp32, R = R0 + (has_back ? 2G : 0)
  void *dt, *Bm, *Cm, *Bb, *Cb;                    // (tokens, H|G, K) io dtype
  const float* weights;  // (tokens, K) fp32 or NULL: dt = softplus(raw) * weights instead of raw
  void* dt_raw;          // (tokens, H, K) io dtype: raw dt, written by the forward when weights is given
  float* dweights;       // (tokens, K) fp32 or NULL
  const void *ddt, *dB, *dC, *dBb, *dCb;           // gradients of the outputs
  void* ddist;           // (tokens, K, M) io dtype
  float* dbias;          // (tokens, R) fp32
  float* dbias_sum;      // (R) fp32 or NULL: dbias summed over the tokens
  float* dw_partial;     // (nblocks, R0, M) fp32
  float* dW;             // (R0, M) fp32
  int nblocks;
};

// two floats -> two bf16 (round to nearest even) in one dword
__device__ __forceinline__ unsigned pack_bf16(float lo, float hi) {
  typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
  typedef float fl2 __attribute__((ext_vector_type(2)));
  const bf2 h = __builtin_convertvector((fl2){lo, hi}, bf2);
  return __builtin_bit_cast(unsigned, h);
}

__device__ __forceinline__ float bf16_to_f(uint16_t v) { return __uint_as_float(((uint32_t)v) << 16); }
// round to nearest even; the hardware conversion (v_cvt_pk_bf16_f32), one instruction per two values
__device__ __forceinline__ uint16_t f_to_bf16(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }
// a float rounded to bf16 (nearest even) and back
__device__ __forceinline__ float bf16_round(float f) { return (float)(__bf16)f; }
// runtime-dtype element access (used only outside hot loops)
__device__ __forceinline__ float ldv(const void* p, long i, int dt) {
  return dt ? bf16_to_f(((const uint16_t*)p)[i]) : ((const float*)p)[i];
}
__device__ __forceinline__ void stv(void* p, long i, int dt, float v) {
  if (dt) ((uint16_t*)p)[i] = f_to_bf16(v); else ((float*)p)[i] = v;
}
__device__ __forceinline__ float ex2(float x) { return __builtin_amdgcn_exp2f(x); }
// (the hardware exp2 / log2 directly: the arguments here need none of the library's range fix-ups --
// 1 + exp(x) >= 1 is never denormal and an exp that underflows to 0 is the right answer)
__device__ __forceinline__ float sigmoidf_(float x) { return __builtin_amdgcn_rcpf(1.0f + ex2(-x * LOG2E)); }
// softplus as the reference evaluates it: log(exp(x) + 1) for x <= 20, identity above
__device__ __forceinline__ float softplus_(float x) {
  return x <= 20.0f ? LN2 * __builtin_amdgcn_logf(1.0f + ex2(x * LOG2E)) : x;
}

// Batched global loads / stores of one element type: all CNT accesses are issued before any
// value is consumed.  The address is (uniform element offset ubase) + (per-lane 32-bit element
// offset off[i]), which lets the compiler keep the base in scalar registers; off[i] < 0 marks an
// absent element (load: reads as 0, the access itself goes to offset 0; store: skipped).
template <bool BF, int CNT>
__device__ __forceinline__ void gload(const void* p, long ubase, const int (&off)[CNT], float (&out)[CNT]) {
  if (BF) {
    const uint16_t* q = (const uint16_t*)p + ubase;
    uint16_t r[CNT];
#pragma unroll
    for (int i = 0; i < CNT; ++i) r[i] = q[off[i] < 0 ? 0 : off[i]];
#pragma unroll
    for (int i = 0; i < CNT; ++i) out[i] = off[i] < 0 ? 0.0f : bf16_to_f(r[i]);
  } else {
    const float* q = (const float*)p + ubase;
    float r[CNT];
#pragma unroll
    for (int i = 0; i < CNT; ++i) r[i] = q[off[i] < 0 ? 0 : off[i]];
#pragma unroll
    for (int i = 0; i < CNT; ++i) out[i] = off[i] < 0 ? 0.0f : r[i];
  }
}
template <bool BF, int CNT>
__device__ __forceinline__ void gstore(void* p, long ubase, const int (&off)[CNT], const float (&v)[CNT]) {
  if (BF) {
    uint16_t* q = (uint16_t*)p + ubase;
#pragma unroll
    for (int i = 0; i < CNT; ++i)
      if (off[i] >= 0) q[off[i]] = f_to_bf16(v[i]);
  } else {
    float* q = (float*)p + ubase;
#pragma unroll
    for (int i = 0; i < CNT; ++i)
      if (off[i] >= 0) q[off[i]] = v[i];
  }
}

// Opaque pass-through of registers: everything that depends on the values is ordered after this
// point and everything that produces them before, which keeps the phases of a long straight-line
// kernel from being interleaved by the scheduler (and their temporaries from being live together).
__device__ __forceinline__ void pin16(float (&a)[16]) {
  asm volatile("" : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]), "+v"(a[5]), "+v"(a[6]), "+v"(a[7]),
               "+v"(a[8]), "+v"(a[9]), "+v"(a[10]), "+v"(a[11]), "+v"(a[12]), "+v"(a[13]), "+v"(a[14]), "+v"(a[15]));
}
__device__ __forceinline__ void pin4(f4& a) { asm volatile("" : "+v"(a)); }
// Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous range of logical
// ids so that units sharing B/C tiles (the heads of one chunk) share an L2.
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

// ------------------------------------------------------------------ split-bf16 products
// v_mfma_f32_16x16x4_f32 shares the vector ALU's issue slots (measured: its time adds to the VALU time
// instead of overlapping it), while v_mfma_f32_16x16x32_bf16 does 8x the multiply-adds in about half the
// time.  Where both operands of a product are reused often enough to amortise the conversion, an fp32
// product a.b is therefore evaluated as  ah.bh + ah.bl + al.bh  with a = ah + al, ah = bf16(a),
// al = bf16(a - ah) (16 significand bits per operand; the dropped al.bl term is <= 2^-16 |a.b|) and fp32
// accumulation.  One instruction contracts over K = 32: lane (cm, g4) supplies k-slots 0..7 of group g4.
typedef __bf16 bf8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ f4 mfma_bf(bf8 a, bf8 b, f4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
// acc += A.B with both operands given as (hi, lo) pairs
__device__ __forceinline__ f4 mfma_split(bf8 ah, bf8 al, bf8 bh, bf8 bl, f4 c) {
  c = mfma_bf(al, bh, c);
  c = mfma_bf(ah, bl, c);
  return mfma_bf(ah, bh, c);
}
__device__ __forceinline__ void split4(const float (&v)[4], bf4& hi, bf4& lo) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const __bf16 h = (__bf16)v[j];
    hi[j] = h;
    lo[j] = (__bf16)(v[j] - (float)h);
  }
}
// eight fp32 values of a lane (k-slots 0..7) -> (hi, lo) fragments
__device__ __forceinline__ void split8(const float (&v)[8], bf8& hi, bf8& lo) {
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const __bf16 h = (__bf16)v[j];
    hi[j] = h;
    lo[j] = (__bf16)(v[j] - (float)h);
  }
}
// Row-major bf16 tiles [rows][SplitLd] holding the hi and the lo halves of an fp32 (rows x KW) tile, KW a
// multiple of 16.  Fragment of K-step t for lane (row, g4): columns 32t + 4 g4 .. +3 and 32t + 16 + 4 g4 .. +3,
// i.e. k-slot s <-> column 32t + 16 (s >> 2) + 4 g4 + (s & 3).
template <int KW>
struct SplitTile {
  static constexpr int LD = KW + 8;
  uint16_t hi[CS * LD];
  uint16_t lo[CS * LD];
};
// (HALF: the tile has no columns 32t + 16 .. 32t + 31; those k-slots read as zero.)
template <int LD, bool HALF = false>
__device__ __forceinline__ bf8 split_frag(const uint16_t* tile, int row, int g4, int t) {
  const uint16_t* q = tile + row * LD + 32 * t + 4 * g4;
  const bf4 a = *(const bf4*)q;
  bf4 b = {0, 0, 0, 0};
  if (!HALF) b = *(const bf4*)(q + 16);
  return __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
}
// Store of a cooperative (64 x 16 PT) register tile (layout of lp_load) as split bf16 tiles.
template <int PT, int LD>
__device__ __forceinline__ void lp_store_split(const float (&v)[CS * PT * 16 / NTHREADS], uint16_t* hi, uint16_t* lo,
                                               int tid = threadIdx.x) {
  constexpr int G4 = 4 * PT;
#pragma unroll
  for (int i = 0; i < PT; ++i) {
    const int e4 = tid + i * NTHREADS, o = (e4 / G4) * LD + (e4 % G4) * 4;
    const float w[4] = {v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]};
    bf4 h, l;
    split4(w, h, l);
    *(bf4*)(hi + o) = h;
    *(bf4*)(lo + o) = l;
  }
}

// Same register tile stored transposed, [p][l] (rows = head dimension, KW = CS columns), for products that
// contract over the rows of the chunk.
template <int PT, int LD, bool SPLIT = true>
__device__ __forceinline__ void lp_store_split_t(const float (&v)[CS * PT * 16 / NTHREADS], uint16_t* hi,
                                                 uint16_t* lo, int tid = threadIdx.x) {
  constexpr int G4 = 4 * PT;
#pragma unroll
  for (int i = 0; i < PT; ++i) {
    const int e4 = tid + i * NTHREADS, l = e4 / G4, p4 = (e4 % G4) * 4;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float w = v[4 * i + j];
      const __bf16 h = (__bf16)w;
      const __bf16 lw = (__bf16)(w - (float)h);
      hi[(p4 + j) * LD + l] = __builtin_bit_cast(uint16_t, h);
      if (SPLIT) lo[(p4 + j) * LD + l] = __builtin_bit_cast(uint16_t, lw);
    }
  }
}
// acc[pt] += (tile^T)(16 pt .. +15, :) . b  for a product over the 64 chunk rows whose B operand is the lane's
// 16 column-lane values (k = 4J + j <-> row 16J + 4 g4 + j): two K = 32 steps, step t <-> values 8t .. 8t+7.
// `b(k)` yields the lane's value k (evaluated step by step, so that only eight are live at a time).
// MODE 1: both operands as (hi, lo) pairs, three instructions per step.  MODE 0: both operands rounded to bf16, one
// instruction.  MODE 2: the tile is exact in bf16 (bf16 inputs), only b is split: two instructions.
template <int PT, int LD, int MODE = 1, typename F>
__device__ __forceinline__ void rows_product_split(f4 (&acc)[PT], const uint16_t* thi, const uint16_t* tlo, F b,
                                                   int cm, int g4) {
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    float w[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) w[j] = b(8 * t + j);
    bf8 bh, bl;
    if (MODE != 0) {
      split8(w, bh, bl);
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) bh[j] = (__bf16)w[j];
    }
#pragma unroll
    for (int pt = 0; pt < PT; ++pt) {
      const bf8 ah = split_frag<LD>(thi, pt * 16 + cm, g4, t);
      if (MODE == 1) {
        const bf8 al = split_frag<LD>(tlo, pt * 16 + cm, g4, t);
        acc[pt] = mfma_split(ah, al, bh, bl, acc[pt]);
      } else if (MODE == 2) {
        acc[pt] = mfma_bf(ah, bl, acc[pt]);
        acc[pt] = mfma_bf(ah, bh, acc[pt]);
      } else {
        acc[pt] = mfma_bf(ah, bh, acc[pt]);
      }
    }
  }
}

// a (64 x 16 PT) register tile (layout of lp_load) as bf16 into LDS dst[l][p]
template <int PT, int LD>
__device__ __forceinline__ void lp_store_bf(const float (&v)[CS * PT * 16 / NTHREADS], uint16_t* dst, int tid) {
  constexpr int G4 = 4 * PT;
#pragma unroll
  for (int i = 0; i < PT; ++i) {
    const int e4 = tid + i * NTHREADS;
    *(uint2*)(dst + (e4 / G4) * LD + (e4 % G4) * 4) =
        make_uint2(pack_bf16(v[4 * i], v[4 * i + 1]), pack_bf16(v[4 * i + 2], v[4 * i + 3]));
  }
}

// Decode a unit id -> (b, dir, c, h); h is fastest so that the heads of one chunk run back to
// back and share the B/C tiles in cache.
struct Unit {
  int b, dir, bt, c, h, g;
};
// Order of the units: heads fastest.  With two directions the next index is the direction, and chunk j of the
// forward direction is paired with chunk nc - 1 - j of the reversed one: the same block of tokens, so the two
// workgroups that read one head's dt tile (the largest operand, shared by the directions) run side by side on one
// XCD and the second read is served by its L2.
__device__ __forceinline__ Unit decode_unit(const KP& p, int u) {
  Unit r;
  r.h = u % p.H;
  u /= p.H;
  if (p.ndir == 2) {
    r.dir = u & 1;
    u >>= 1;
    const int j = u % p.ncl;
    r.b = u / p.ncl;
    r.c = p.c_lo + (r.dir ? p.ncl - 1 - j : j);
    r.bt = r.b * 2 + r.dir;
  } else {
    r.c = p.c_lo + u % p.ncl;
    r.bt = u / p.ncl;
    r.dir = r.bt % p.ndir;
    r.b = r.bt / p.ndir;
  }
  r.g = r.h / p.hpg;
  return r;
}
// physical row of logical time t for a direction
__device__ __forceinline__ int phys_row(const KP& p, int dir, int t) { return dir ? p.L - 1 - t : t; }

// ---------------------------------------------------------------- column-lane layout helpers
// chunk row of array index k for lane group g4
__device__ __forceinline__ int lane_row(int k, int g4) { return 16 * (k >> 2) + 4 * g4 + (k & 3); }

// inclusive prefix / suffix over the four lane groups g4 = 0..3 (lanes cm, cm+16, cm+32, cm+48)
__device__ __forceinline__ float scan_g_incl(float v, int g4) {
  float t = __shfl_up(v, 16, 64);
  if (g4 >= 1) v += t;
  t = __shfl_up(v, 32, 64);
  if (g4 >= 2) v += t;
  return v;
}
__device__ __forceinline__ float scan_g_incl_rev(float v, int g4) {
  float t = __shfl_down(v, 16, 64);
  if (g4 <= 2) v += t;
  t = __shfl_down(v, 32, 64);
  if (g4 <= 1) v += t;
  return v;
}

// Where the lane's 16 chunk rows live in memory.  Element k = 4J + j is chunk row 16J + 4 g4 + j,
// i.e. physical row base + step * (16J + j): a per-lane part (base) plus a part that is the same
// for the whole wave, so that in a full chunk the address of every element is a scalar base
// plus ONE per-lane offset.  `full` (a compile-time constant of the kernel variant) says that all 64
// rows and all 64 columns of every slice exist (the head dimension is checked separately at run time); otherwise rows >= nvalid and lanes with !vn read as zero.
struct RowMap {
  int base, step, nvalid;
  bool full;
  unsigned long long cut;  // bit r: the sequence id changes between rows r - 1 and r of the chunk (scan order; the initial states count as id 0); uniform
};
template <bool FULL>
__device__ __forceinline__ RowMap make_rowmap(const KP& p, const Unit& u, int g4, int n0) {
  RowMap r;
  const int t0 = u.c * CS + 4 * g4;
  r.base = u.dir ? p.L - 1 - t0 : t0;
  r.step = u.dir ? -1 : 1;
  r.nvalid = min(CS, p.L - u.c * CS);
  // FULL kernels are only launched when every chunk and every column slice is complete
  r.full = FULL;
  r.cut = 0;
  if (!FULL && p.seq_idx) {  // packed sequences take the kernels' general variants
    // lane = row of the chunk in scan order; its predecessor in scan order may be the previous chunk's last row
    const int row = u.c * CS + (int)(threadIdx.x & 63);
    // The initial states belong to sequence id 0 (issm_chunk_scan.py:123 and issm_state_passing.py:91 start from id 0):
    // a row whose first id is not 0 is cut off from them, like a row from a predecessor of another id.
    bool changes = false;
    if (row < p.L) {
      const long t = u.dir ? p.L - 1 - row : row, tp = u.dir ? t + 1 : t - 1;
      const int* q = p.seq_idx + (long)u.b * p.seq_s0;
      changes = q[t * p.seq_s1] != (row > 0 ? q[tp * p.seq_s1] : 0);
    }
    r.cut = __ballot(changes);
  }
  return r;
}
// Lane's 16 values of column n of a (B,L,G|H,N)-shaped tensor.
template <bool BF>
__device__ __forceinline__ void lane_load_ln(const TensorD& t, int b, int third, int n, bool vn, int g4,
                                             const RowMap& rm, float (&out)[16]) {
  typedef typename std::conditional<BF, uint16_t, float>::type T;
  const T* q = (const T*)t.ptr + ((long)b * t.s0 + (long)third * t.s2);
  const long ss = (long)rm.step * t.s1;  // uniform
  T r[16];
  if (rm.full) {
    // 32-bit offsets (the host checks that seqlen * stride fits): address = scalar base + per-lane offset.
    // ks is made opaque so that its multiples are formed here, next to their use, instead of being
    // hoisted out of an enclosing loop into (scarce) scalar registers.
    // BYTE offsets in 32 bits, so that the access is "scalar base + 32-bit per-lane offset" and costs one
    // integer add per element.
    const unsigned lo = (unsigned)(rm.base * (int)t.s1 + n) * (unsigned)sizeof(T);
    unsigned ks = (unsigned)(rm.step * (int)t.s1) * (unsigned)sizeof(T);
    ISSM_OPAQUE_S(ks);
    const char* qb = (const char*)q;
#pragma unroll
    for (int k = 0; k < 16; ++k) r[k] = *(const T*)(qb + (lo + (unsigned)(16 * (k >> 2) + (k & 3)) * ks));
#pragma unroll
    for (int k = 0; k < 16; ++k) out[k] = BF ? bf16_to_f((uint16_t)r[k]) : (float)r[k];
  } else {
    // The same 32-bit addressing with the row clamped to the chunk's last existing row and the column to 0: every
    // lane reads an address inside the tensor, and what it read is replaced by zero where the row or column is absent
    // (64-bit per-element offsets and a mask array held across the loads cost the general variants some forty
    // registers per call site).
    (void)ss;
    const int rmax = rm.nvalid - 1 - 4 * g4;  // last existing row, relative to the lane's row 0 (may be negative)
    const unsigned lo = (unsigned)(rm.base * (int)t.s1 + (vn ? n : 0)) * (unsigned)sizeof(T);
    unsigned ks = (unsigned)(rm.step * (int)t.s1) * (unsigned)sizeof(T);
    ISSM_OPAQUE_S(ks);
    const char* qb = (const char*)q;
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const int rk = 16 * (k >> 2) + (k & 3);
      r[k] = *(const T*)(qb + (lo + (unsigned)min(rk, rmax) * ks));  // a negative row wraps like the base does
    }
#pragma unroll
    for (int k = 0; k < 16; ++k)
      out[k] = (vn && 16 * (k >> 2) + (k & 3) <= rmax) ? (BF ? bf16_to_f((uint16_t)r[k]) : (float)r[k]) : 0.0f;
  }
}
// Store of the lane's 16 values to column n of a (B,L,G|H,N)-shaped tensor (absent rows / columns skipped).
template <bool BF>
__device__ __forceinline__ void lane_store_ln(const TensorD& t, int b, int third, int n, bool vn, int g4,
                                              const RowMap& rm, const float (&v)[16]) {
  typedef typename std::conditional<BF, uint16_t, float>::type T;
  T* q = (T*)const_cast<void*>(t.ptr) + ((long)b * t.s0 + (long)third * t.s2);
  const long ss = (long)rm.step * t.s1;
  if (rm.full) {
    const unsigned lo = (unsigned)(rm.base * (int)t.s1 + n) * (unsigned)sizeof(T);
    unsigned ks = (unsigned)(rm.step * (int)t.s1) * (unsigned)sizeof(T);
    ISSM_OPAQUE_S(ks);
    char* qb = (char*)q;
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      T* d = (T*)(qb + (lo + (unsigned)(16 * (k >> 2) + (k & 3)) * ks));
      if (BF) *d = (T)f_to_bf16(v[k]); else *d = (T)v[k];
    }
  } else {
    (void)ss;
    const int rmax = rm.nvalid - 1 - 4 * g4;
    const unsigned lo = (unsigned)(rm.base * (int)t.s1 + n) * (unsigned)sizeof(T);
    unsigned ks = (unsigned)(rm.step * (int)t.s1) * (unsigned)sizeof(T);
    ISSM_OPAQUE_S(ks);
    char* qb = (char*)q;
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const int rk = 16 * (k >> 2) + (k & 3);
      if (vn && rk <= rmax) {
        T* d = (T*)(qb + (lo + (unsigned)rk * ks));
        if (BF) *d = (T)f_to_bf16(v[k]); else *d = (T)v[k];
      }
    }
  }
}
// Lane's values of column n of a (P x N) fp32 slab: index q <-> row 16 (q >> 2) + 4 g4 + (q & 3).
template <int CNT>
__device__ __forceinline__ void lane_load_pn(const float* __restrict__ src, int P, int N, int n, bool vn, int g4,
                                             bool full, float (&out)[CNT]) {
  if (full) {
    const unsigned lo = (unsigned)(4 * g4 * N + n) * 4u;
    unsigned nb = (unsigned)N * 4u;
    ISSM_OPAQUE_S(nb);
    const char* sb = (const char*)src;
#pragma unroll
    for (int q = 0; q < CNT; ++q) out[q] = *(const float*)(sb + (lo + (unsigned)(16 * (q >> 2) + (q & 3)) * nb));
  } else {
    // rows clamped to the last one of the head, the column to 0; absent values replaced by zero afterwards
    float r[CNT];
    const int pmax = P - 1 - 4 * g4;
    const unsigned lo = (unsigned)(4 * g4 * N + (vn ? n : 0)) * 4u;
    unsigned nb = (unsigned)N * 4u;
    ISSM_OPAQUE_S(nb);
    const char* sb = (const char*)src;
#pragma unroll
    for (int q = 0; q < CNT; ++q)
      r[q] = *(const float*)(sb + (lo + (unsigned)min(16 * (q >> 2) + (q & 3), pmax) * nb));
#pragma unroll
    for (int q = 0; q < CNT; ++q) out[q] = (vn && 16 * (q >> 2) + (q & 3) <= pmax) ? r[q] : 0.0f;
  }
}
// dt transform (bias -> softplus -> clamp) of the lane's rows and the inclusive running sum of
// dt' * A * log2(e) down the chunk (so decays are exp2 of differences).  `raw` holds the loaded
// dt values.  dfac (if WANT_DFAC) receives d dt' / d dt: the softplus derivative times the clamp
// mask.  Returns the chunk total (running sum at row 63), the same on all lanes of the column.
// Per-column coefficients of the dt transform; loaded together with the column's dt values so that
// their latency is covered by the same prefetch.
struct Coef {
  float A, bias;
};
__device__ __forceinline__ Coef lane_coef(const KP& p, int h, int n, bool vn) {
  Coef c;
  c.A = vn ? p.A[h * p.N + n] : 0.0f;
  c.bias = (vn && p.dt_bias) ? p.dt_bias[h * p.N + n] : 0.0f;
  return c;
}
// dt transform of CNT values that already include the bias: softplus -> clamp; dfac (if WANT_DFAC) receives
// d dt' / d dt.  Softplus and its derivative share one exponential: with t = e^pre, softplus = log(1 + t) and
// sigmoid = t / (1 + t); above the reference's threshold of 20 both are replaced (identity, 1).  F_NOCLAMP: the limits
// are (0, inf) and softplus is on, so the clamp and its mask cannot act and are skipped.
template <bool WANT_DFAC, int CNT>
__device__ __forceinline__ void dt_transform(const KP& p, const float (&pre_)[CNT], float (&dtp)[CNT], float (&dfac)[CNT]) {
  if (p.flags & F_SOFTPLUS) {
    if (p.flags & F_NOCLAMP) {
#pragma unroll
      for (int k = 0; k < CNT; ++k) {
        const float pre = pre_[k];
        const float t = ex2(pre * LOG2E), u = 1.0f + t;
        const bool big = pre > 20.0f;
        dtp[k] = big ? pre : LN2 * __builtin_amdgcn_logf(u);
        if (WANT_DFAC) dfac[k] = big ? 1.0f : t * __builtin_amdgcn_rcpf(u);
      }
    } else {
#pragma unroll
      for (int k = 0; k < CNT; ++k) {
        const float pre = pre_[k];
        const float t = ex2(pre * LOG2E), u = 1.0f + t;
        const bool big = pre > 20.0f;
        const float sp = big ? pre : LN2 * __builtin_amdgcn_logf(u);
        dtp[k] = __builtin_amdgcn_fmed3f(sp, p.dt_min, p.dt_max);
        if (WANT_DFAC) dfac[k] = (sp < p.dt_min || sp > p.dt_max) ? 0.0f : (big ? 1.0f : t * __builtin_amdgcn_rcpf(u));
      }
    }
  } else {
#pragma unroll
    for (int k = 0; k < CNT; ++k) {
      const float sp = pre_[k];
      dtp[k] = __builtin_amdgcn_fmed3f(sp, p.dt_min, p.dt_max);
      if (WANT_DFAC) dfac[k] = (sp < p.dt_min || sp > p.dt_max) ? 0.0f : 1.0f;
    }
  }
}
// dt transform (bias -> softplus -> clamp) of the lane's 16 rows.  Rows past the end of the sequence and absent columns
// come out as dt' = 0.
template <bool WANT_DFAC>
__device__ __forceinline__ void lane_dt(const KP& p, const Coef& cf, bool vn, int g4, const RowMap& rm,
                                        const float (&raw)[16], float (&dtp)[16], float (&dfac)[16]) {
  float pre[16];
#pragma unroll
  for (int k = 0; k < 16; ++k) pre[k] = raw[k] + cf.bias;
  dt_transform<WANT_DFAC, 16>(p, pre, dtp, dfac);
  if (!rm.full) {  // rows past the end of the sequence and absent columns behave as dt' = 0
#pragma unroll
    for (int k = 0; k < 16; ++k)
      if (!(vn && lane_row(k, g4) < rm.nvalid)) dtp[k] = 0.0f;
  }
}
template <bool WANT_DFAC>
__device__ __forceinline__ float lane_prep(const KP& p, const Coef& cf, bool vn, int cm, int g4, const RowMap& rm,
                                           const float (&raw)[16], float (&dtp)[16], float (&cs)[16],
                                           float (&dfac)[16]) {
  const float A2 = cf.A * LOG2E;
  lane_dt<WANT_DFAC>(p, cf, vn, g4, rm, raw, dtp, dfac);
  // Running sum down the 64 rows: in the lane over its four rows of each tile, then across the four lane groups
  // of a tile, then across the tiles.  The cross-lane steps of the four tiles do not depend on each other, so each
  // step is issued for all four before any result is used (a cross-lane fetch goes through the LDS pipe: taken tile
  // by tile, twelve latencies would line up instead of three).  Same operations in the same order as tile by tile.
  float c[4], v[4], t[4];
  if (rm.full || rm.cut == 0) {  // uniform (and the only form the complete-tile variants contain)
#pragma unroll
    for (int J = 0; J < 4; ++J) {
      float a = 0.0f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        a += dtp[4 * J + j] * A2;
        cs[4 * J + j] = a;
      }
      c[J] = a;
    }
  } else {  // packed sequences: the sum drops by SEQ_CUT at every row where the sequence id changes
#pragma unroll
    for (int J = 0; J < 4; ++J) {
      const unsigned bits = (unsigned)(rm.cut >> (16 * J + 4 * g4)) & 15u;
      float a = 0.0f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        a += dtp[4 * J + j] * A2 - (((bits >> j) & 1u) ? SEQ_CUT : 0.0f);
        cs[4 * J + j] = a;
      }
      c[J] = a;
    }
  }
#pragma unroll
  for (int J = 0; J < 4; ++J) t[J] = __shfl_up(c[J], 16, 64);
#pragma unroll
  for (int J = 0; J < 4; ++J) v[J] = g4 >= 1 ? c[J] + t[J] : c[J];
#pragma unroll
  for (int J = 0; J < 4; ++J) t[J] = __shfl_up(v[J], 32, 64);
#pragma unroll
  for (int J = 0; J < 4; ++J) v[J] = g4 >= 2 ? v[J] + t[J] : v[J];  // inclusive over the lane groups
#pragma unroll
  for (int J = 0; J < 4; ++J) t[J] = __shfl(v[J], cm + 48, 64);      // tile totals
  float carry = 0.0f;
#pragma unroll
  for (int J = 0; J < 4; ++J) {
    const float add = carry + (v[J] - c[J]);
#pragma unroll
    for (int j = 0; j < 4; ++j) cs[4 * J + j] += add;
    carry += t[J];
  }
  return carry;
}

// Running sums of a = dt' A log2(e) restarted at every 16-row tile: pc[k] = sum of a over the rows of k's tile up to and
// including k's row, tt[J] = the whole tile's sum (the same on the four lanes of a column).  Used by the kernels that
// write a decay exp2(cs[l] - cs[s]) as  exp2(pc[l]) . exp2(base(tile of l) - base(tile of s)) . exp2(-pc[s])  with
// base(J) = tt[0] + .. + tt[J-1]: two exponentials per element and ten per column serve every pair of rows of the chunk.
__device__ __forceinline__ void lane_tile_sums(float A2, int cm, int g4, const RowMap& rm, const float (&dtp)[16],
                                               float (&pc)[16], float (&tt)[4]) {
  float c[4], v[4], t[4];
  if (rm.full || rm.cut == 0) {
#pragma unroll
    for (int J = 0; J < 4; ++J) {
      float a = 0.0f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        a += dtp[4 * J + j] * A2;
        pc[4 * J + j] = a;
      }
      c[J] = a;
    }
  } else {  // packed sequences: the sum drops by SEQ_CUT at every row where the sequence id changes
#pragma unroll
    for (int J = 0; J < 4; ++J) {
      const unsigned bits = (unsigned)(rm.cut >> (16 * J + 4 * g4)) & 15u;
      float a = 0.0f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        a += dtp[4 * J + j] * A2 - (((bits >> j) & 1u) ? SEQ_CUT : 0.0f);
        pc[4 * J + j] = a;
      }
      c[J] = a;
    }
  }
#pragma unroll
  for (int J = 0; J < 4; ++J) t[J] = __shfl_up(c[J], 16, 64);
#pragma unroll
  for (int J = 0; J < 4; ++J) v[J] = g4 >= 1 ? c[J] + t[J] : c[J];
#pragma unroll
  for (int J = 0; J < 4; ++J) t[J] = __shfl_up(v[J], 32, 64);
#pragma unroll
  for (int J = 0; J < 4; ++J) v[J] = g4 >= 2 ? v[J] + t[J] : v[J];  // inclusive over the lane groups
#pragma unroll
  for (int J = 0; J < 4; ++J) tt[J] = __shfl(v[J], cm + 48, 64);    // tile totals
#pragma unroll
  for (int J = 0; J < 4; ++J) {
    const float add = v[J] - c[J];
#pragma unroll
    for (int j = 0; j < 4; ++j) pc[4 * J + j] += add;
  }
}

// v_mfma_f32_16x16x16_bf16: lane (m, g4) supplies k = 4 g4 .. 4 g4 + 3 -- in the column-lane layout exactly the lane's
// four rows of one 16-row tile.
typedef short sh4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ f4 mfma_bf16k(bf4 a, bf4 b, f4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(sh4, a), __builtin_bit_cast(sh4, b), c, 0, 0, 0);
}
// an fp32 value cut to 16 significand bits (towards zero): it then splits into two bf16 numbers exactly
__device__ __forceinline__ float trunc16(float v) { return __uint_as_float(__float_as_uint(v) & 0xffffff00u); }

// ------------------------------------------------------------------ cooperative tile loaders
// The unit's (64 x P) tile of a (B,L,H,P) tensor, zero padded to 16*PT columns: registers, then
// LDS dst[l][p] (leading dimension ld).  Element e = tid + 256 i is (l, p) = (e / 16PT, e % 16PT).
// Thread `tid` owns PT groups of four adjacent columns: group i is element e4 = tid + 256 i, i.e.
// (l, p) = (e4 / 4PT, 4 (e4 % 4PT)).  When the tensor allows it (uniform test) a group is one 8- or 16-byte
// access.
__device__ __forceinline__ bool lp_vec_ok(const KP& p, const TensorD& t, int esize) {
  return ((p.P & 3) == 0) && (((t.s0 | t.s1 | t.s2) & 3) == 0) && ((((uintptr_t)t.ptr) & (4 * esize - 1)) == 0);
}
template <bool BF, int PT, bool FULL = false>
__device__ __forceinline__ void lp_load(const KP& p, const Unit& u, const TensorD& t,
                                        float (&v)[CS * PT * 16 / NTHREADS], int tid = threadIdx.x) {
  constexpr int G4 = 4 * PT;  // groups per row
  typedef typename std::conditional<BF, uint16_t, float>::type T;
  const T* q = (const T*)t.ptr + ((long)u.b * t.s0 + (long)u.h * t.s2);
  const int nvalid = min(CS, p.L - u.c * CS);
  const long ss = (long)(u.dir ? -1 : 1) * t.s1;
  const long r0 = (long)(u.dir ? p.L - 1 - u.c * CS : u.c * CS) * t.s1;
  if (lp_vec_ok(p, t, sizeof(T))) {
    typedef typename std::conditional<BF, uint2, f4>::type V;
    V r[PT];
    bool ok[PT];
#pragma unroll
    for (int i = 0; i < PT; ++i) {
      const int e4 = tid + i * NTHREADS, l = e4 / G4, p4 = (e4 % G4) * 4;
      ok[i] = p4 < p.P && (FULL || l < nvalid);
      r[i] = *(const V*)(q + (ok[i] ? r0 + l * ss + p4 : 0));
    }
#pragma unroll
    for (int i = 0; i < PT; ++i) {
      if (BF) {
        const uint2 w = *(const uint2*)&r[i];
        v[4 * i + 0] = ok[i] ? __uint_as_float(w.x << 16) : 0.0f;
        v[4 * i + 1] = ok[i] ? __uint_as_float(w.x & 0xffff0000u) : 0.0f;
        v[4 * i + 2] = ok[i] ? __uint_as_float(w.y << 16) : 0.0f;
        v[4 * i + 3] = ok[i] ? __uint_as_float(w.y & 0xffff0000u) : 0.0f;
      } else {
        const f4 w = *(const f4*)&r[i];
#pragma unroll
        for (int j = 0; j < 4; ++j) v[4 * i + j] = ok[i] ? w[j] : 0.0f;
      }
    }
  } else {
    T r[4 * PT];
    bool ok[4 * PT];
#pragma unroll
    for (int i = 0; i < PT; ++i) {
      const int e4 = tid + i * NTHREADS, l = e4 / G4, p4 = (e4 % G4) * 4;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        ok[4 * i + j] = p4 + j < p.P && (FULL || l < nvalid);
        r[4 * i + j] = q[ok[4 * i + j] ? r0 + l * ss + p4 + j : 0];
      }
    }
#pragma unroll
    for (int e = 0; e < 4 * PT; ++e) v[e] = ok[e] ? (BF ? bf16_to_f((uint16_t)r[e]) : (float)r[e]) : 0.0f;
  }
}
template <int PT>
__device__ __forceinline__ void lp_store(const float (&v)[CS * PT * 16 / NTHREADS], float* dst, int ld,
                                         int tid = threadIdx.x) {
  constexpr int G4 = 4 * PT;
#pragma unroll
  for (int i = 0; i < PT; ++i) {
    const int e4 = tid + i * NTHREADS;
    *(f4*)(dst + (e4 / G4) * ld + (e4 % G4) * 4) = (f4){v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]};
  }
}
// dy tile: from the caller's dout (io dtype) or from the gated fp32 (Bt,L,H,P) workspace copy.
template <bool BF, int PT, bool FULL = false>
__device__ __forceinline__ void dy_load(const KP& p, const Unit& u, const float* dy_ws,
                                        float (&v)[CS * PT * 16 / NTHREADS], int tid = threadIdx.x) {
  if (dy_ws) {
    TensorD t;
    t.ptr = dy_ws + (long)(u.bt - u.b) * p.L * p.H * p.P;  // so that b * s0 lands on row block bt
    t.s0 = (long)p.L * p.H * p.P;
    t.s1 = (long)p.H * p.P;
    t.s2 = p.P;
    lp_load<false, PT, FULL>(p, u, t, v, tid);
  } else {
    lp_load<BF, PT, FULL>(p, u, p.dout[u.dir], v, tid);
  }
}

// The same tiles for bf16 tensors as raw pairs of bf16 (no trip through fp32): group i of thread `tid` (lp_load's
// layout) in r[i], zeros where the row or the columns do not exist.  dy from the gated fp32 workspace is rounded here.
template <int PT, bool FULL>
__device__ __forceinline__ void lp_load_bf(const KP& p, const Unit& u, const TensorD& t, uint2 (&r)[PT], int tid) {
  if (lp_vec_ok(p, t, 2)) {
    constexpr int G4 = 4 * PT;
    const uint16_t* q = (const uint16_t*)t.ptr + ((long)u.b * t.s0 + (long)u.h * t.s2);
    const int nvalid = min(CS, p.L - u.c * CS);
    const long ss = (long)(u.dir ? -1 : 1) * t.s1;
    const long r0 = (long)(u.dir ? p.L - 1 - u.c * CS : u.c * CS) * t.s1;
#pragma unroll
    for (int i = 0; i < PT; ++i) {
      const int e4 = tid + i * NTHREADS, l = e4 / G4, p4 = (e4 % G4) * 4;
      const bool ok = p4 < p.P && (FULL || l < nvalid);
      const uint2 w = *(const uint2*)(q + (ok ? r0 + l * ss + p4 : 0));
      r[i] = ok ? w : make_uint2(0u, 0u);
    }
  } else {
    float v[CS * PT * 16 / NTHREADS];
    lp_load<true, PT, FULL>(p, u, t, v, tid);
#pragma unroll
    for (int i = 0; i < PT; ++i)  // exact: the values are bf16
      r[i] = make_uint2(pack_bf16(v[4 * i], v[4 * i + 1]), pack_bf16(v[4 * i + 2], v[4 * i + 3]));
  }
}
template <int PT, bool FULL>
__device__ __forceinline__ void dy_load_bf(const KP& p, const Unit& u, const float* dy_ws, uint2 (&r)[PT], int tid) {
  if (dy_ws) {
    float v[CS * PT * 16 / NTHREADS];
    dy_load<true, PT, FULL>(p, u, dy_ws, v, tid);
#pragma unroll
    for (int i = 0; i < PT; ++i)
      r[i] = make_uint2(pack_bf16(v[4 * i], v[4 * i + 1]), pack_bf16(v[4 * i + 2], v[4 * i + 3]));
  } else {
    lp_load_bf<PT, FULL>(p, u, p.dout[u.dir], r, tid);
  }
}
template <int PT, int LD>
__device__ __forceinline__ void lp_store_raw(const uint2 (&r)[PT], uint16_t* dst, int tid) {
  constexpr int G4 = 4 * PT;
#pragma unroll
  for (int i = 0; i < PT; ++i) {
    const int e4 = tid + i * NTHREADS;
    *(uint2*)(dst + (e4 / G4) * LD + (e4 % G4) * 4) = r[i];
  }
}

// Lower triangle (s <= l, rest zero) of a 64x64 fp32 block: registers, then LDS dst[l][s] (ld = LDC).
__device__ __forceinline__ void tril_load(const float* __restrict__ src, f4 (&v)[4], int tid = threadIdx.x) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int e = tid + i * NTHREADS, l = e >> 4, s4 = (e & 15) * 4;
    v[i] = (s4 <= l) ? *(const f4*)(src + l * CS + s4) : (f4){0, 0, 0, 0};
  }
}
// The same lower triangle from the pair of symmetric bf16 matrices (hi at src, lo 8 KB behind it, each 64 x 64) that
// k_bwd_dstates writes for fp32 inputs: dM = hi + lo.
__device__ __forceinline__ void tril_load_hl(const float* __restrict__ src, f4 (&v)[4], int tid = threadIdx.x) {
  const uint16_t* hi = reinterpret_cast<const uint16_t*>(src);
  const uint16_t* lo = hi + CS * CS;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int e = tid + i * NTHREADS, l = e >> 4, s4 = (e & 15) * 4;
    const uint2 a = *(const uint2*)(hi + l * CS + s4), b = *(const uint2*)(lo + l * CS + s4);
    const f4 w = {__uint_as_float(a.x << 16) + __uint_as_float(b.x << 16),
                  __uint_as_float(a.x & 0xffff0000u) + __uint_as_float(b.x & 0xffff0000u),
                  __uint_as_float(a.y << 16) + __uint_as_float(b.y << 16),
                  __uint_as_float(a.y & 0xffff0000u) + __uint_as_float(b.y & 0xffff0000u)};
    v[i] = (s4 <= l) ? w : (f4){0, 0, 0, 0};
  }
}
__device__ __forceinline__ void tril_store(const f4 (&v)[4], float* dst, int tid = threadIdx.x) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int e = tid + i * NTHREADS, l = e >> 4, s4 = (e & 15) * 4;
    f4 w = v[i];
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (s4 + j > l) w[j] = 0.0f;
    *(f4*)(dst + l * LDC + s4) = w;
  }
}

// Columns n0..n0+63 of a (P x N) fp32 slab, zero padded to 16*PT rows and past N: registers, then
// LDS dst[p][col] (leading dimension LDN).
template <int PT>
struct PnRegs {
  static constexpr int Q = NS / 4, TOT = PT * 16 * Q, CNT = (TOT + NTHREADS - 1) / NTHREADS;
  f4 v[CNT];
};
template <int PT>
__device__ __forceinline__ void pn_load(const KP& p, const float* __restrict__ src, int n0, PnRegs<PT>& r,
                                        int tid = threadIdx.x) {
  typedef PnRegs<PT> R;
  const bool vec = (p.N & 3) == 0;
#pragma unroll
  for (int i = 0; i < R::CNT; ++i) {
    const int e = tid + i * NTHREADS, pp = e / R::Q, c4 = (e % R::Q) * 4;
    const bool ok = e < R::TOT && pp < p.P;
    const long o = (long)pp * p.N + n0 + c4;
    // absent rows / columns read the slab's first elements and count as zero: a conditional load would become a
    // branch, and a branch per load makes each wait for the one before
    if (vec) {
      const bool in = ok && n0 + c4 < p.N;
      const f4 w = *(const f4*)(src + (in ? o : 0));
      r.v[i] = in ? w : (f4){0, 0, 0, 0};
    } else {
      f4 w;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const bool in = ok && n0 + c4 + j < p.N;
        const float t = src[in ? o + j : 0];
        w[j] = in ? t : 0.0f;
      }
      r.v[i] = w;
    }
  }
}
template <int PT>
__device__ __forceinline__ void pn_store(const PnRegs<PT>& r, float* dst, int tid = threadIdx.x) {
  typedef PnRegs<PT> R;
#pragma unroll
  for (int i = 0; i < R::CNT; ++i) {
    const int e = tid + i * NTHREADS, pp = e / R::Q, c4 = (e % R::Q) * 4;
    if (e < R::TOT) *(f4*)(dst + pp * LDN + c4) = r.v[i];
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

// Kernel dispatch on (P tiles, io dtype, dt dtype, complete / mixed tiles): the statement sees PT_, IOB_, DTB_, FULL_, MIXED_
// as constants.
#define ISSM_DISPATCH_FULL(full, ...)                                                                       \
  if ((full) == 1) { constexpr bool FULL_ = true; constexpr bool MIXED_ = false; (void)MIXED_; __VA_ARGS__ }        \
  else if ((full) == 2) { constexpr bool FULL_ = false; constexpr bool MIXED_ = true; (void)FULL_; __VA_ARGS__ }    \
  else { constexpr bool FULL_ = false; constexpr bool MIXED_ = false; (void)MIXED_; __VA_ARGS__ }
#define ISSM_DISPATCH_DT(iob, dtb, full, ...)                          \
  if (iob) {                                                           \
    constexpr bool IOB_ = true;                                        \
    if (dtb) { constexpr bool DTB_ = true; ISSM_DISPATCH_FULL(full, __VA_ARGS__) }  \
    else { constexpr bool DTB_ = false; ISSM_DISPATCH_FULL(full, __VA_ARGS__) }     \
  } else {                                                             \
    constexpr bool IOB_ = false;                                       \
    if (dtb) { constexpr bool DTB_ = true; ISSM_DISPATCH_FULL(full, __VA_ARGS__) }  \
    else { constexpr bool DTB_ = false; ISSM_DISPATCH_FULL(full, __VA_ARGS__) }     \
  }
#define ISSM_DISPATCH(p, ...)                                                                        \
  do {                                                                                               \
    const int pt_ = ((p).P + 15) / 16;                                                               \
    const bool iob_ = (p).io_dt != 0, dtb_ = (p).dt_dt != 0;                                         \
    const int full_ = (p).full_tiles;                                                                \
    if (pt_ <= 2) { constexpr int PT_ = 2; ISSM_DISPATCH_DT(iob_, dtb_, full_, __VA_ARGS__) }        \
    else if (pt_ == 3) { constexpr int PT_ = 3; ISSM_DISPATCH_DT(iob_, dtb_, full_, __VA_ARGS__) }   \
    else { constexpr int PT_ = 4; ISSM_DISPATCH_DT(iob_, dtb_, full_, __VA_ARGS__) }                 \
  } while (0)

}  // namespace issm
