// Table gradient of the box-to-point distance encoding without a scatter (gfx950).
//
// dtable[node][ch] = sum over (point, box) pairs of weight[pair][node] * ddist[pair][ch].  Scattering that into an
// LDS copy of the table is bound by the LDS atomic rate (about one add per three cycles per CU).  Here the pairs are
// first sorted by where they land: a pair contributes one *entry* per window of 3 x 3 x 3 nodes it touches (one if
// its corners are on one side of the point, two if it straddles the point along one axis, ...), entries are binned
// by window anchor with a counting sort, and then all entries of a bin share their 27 nodes, so the gradient of a
// bin is a dense (27 x entries) . (entries x 16) product, taken exactly on the int8 matrix cores.  Passes:
//   gmax, boxes   max|ddist| (scale of the fixed point); corners and rotations of every box, once
//   count   workgroup histograms of the entries' bins (LDS integer atomics, one per entry)
//   plan    bin offsets and the list of work items (bin, range of at most BDS_SEG entries); then each counting
//           workgroup's base inside each bin (a scan over workgroups, so the ranges do not depend on timing)
//   fill    the same walk again, writing each entry's record (pair index, corner mask) into its bin
//   accum   one workgroup per work item: 256 entries at a time, lane = entry recomputes the window weights of its
//           corners and stages them with ddist in LDS as fixed-point values split into signed base-256 digits; each
//           wave then multiplies its 64 entries' digits with v_mfma_i32_16x16x64_i8 (integer sums: order-independent,
//           hence reproducible)
//   scatter / finish   work-item results into the table (integer atomics in global memory, a few 10^5), then float.
#include "box_dist_dev.h"

namespace issm {

typedef int i4 __attribute__((ext_vector_type(4)));

constexpr int BDS_SEG = 2048;      // entries per work item
constexpr int BDS_MAXBINS = 9280;  // (D + 2)(H + 2)(W + 2) for D*H*W <= 1024 is at most 1026 * 3 * 3
constexpr int BDS_NWG = 512;       // workgroups of the count and fill passes (they must walk identically)
constexpr int BDS_OUT = 27 * BD_C; // results per work item

struct SortP {
  unsigned* scal;               // [0] bits of max|ddist|, [1] number of work items
  int* counts;                  // [nbins] entries per bin
  int* binoff;                  // [nbins] first entry of each bin
  int* wgbase;                  // [BDS_NWG][nbins] counts per workgroup, turned into base positions by the plan
  int* items;                   // [maxitems][3] bin, first entry, one past the last entry
  unsigned long long* records;  // [maxrecords] pair index | corner mask << 32
  long long* item_out;          // [maxitems][BDS_OUT]
  float* boxtab;                // [B * K][40] corners x, y, z and rotations cos, sin of every box, 8 values each
  long long* dtab;              // [2][cells][16]: sums of the low 32 bits of the items' results, sums of the rest
  int nbins, maxitems;
  long maxrecords;
};

// Fixed point: weights in units of 2^-24, ddist in units of max|ddist| * 2^-22.  A term is at most 8 * 2^24 * 2^22 =
// 2^49 and a work item's sum at most 2^60; the table takes the items' sums as two 64-bit halves (low 32 bits and
// the rest), each far from overflow for the 2^26 pairs the launcher admits.
constexpr float BDS_W_SCALE = 16777216.0f;
__device__ __forceinline__ float bds_scale(const unsigned* scal) {
  const float gmax = __uint_as_float(scal[0]);
  return gmax > 1e-30f ? 4194304.0f / gmax : 1.0f;  // below that the quotient could overflow; such gradients round to 0
}

__device__ __forceinline__ int bds_bin(const BoxDistP& p, int mx, int my, int mz) {
  if (mx < -2 || mx > p.W - 1 || my < -2 || my > p.H - 1 || mz < -2 || mz > p.D - 1) return -1;  // no node inside
  return ((mz + 2) * (p.H + 2) + (my + 2)) * (p.W + 2) + (mx + 2);
}

__global__ __launch_bounds__(NTHREADS) void k_bds_clear(BoxDistP p, SortP s) {
  const int cells = p.D * p.H * p.W;
  const int i = blockIdx.x * NTHREADS + threadIdx.x;
  if (i < 4) s.scal[i] = 0u;
  if (i < s.nbins) s.counts[i] = 0;
  if (i < cells * BD_C) s.dtab[i] = s.dtab[cells * BD_C + i] = 0;
}

// Corners and rotations of every box, once: the accumulation pass visits a box from many lanes, and evaluating the
// sines and cosines there again for every entry cost more than everything else in it.
__global__ __launch_bounds__(NTHREADS) void k_bds_boxes(BoxDistP p, SortP s) {
  const int i = blockIdx.x * NTHREADS + threadIdx.x;
  if (i >= p.B * p.K) return;
  BoxLane bx;
  load_box(p, i / p.K, i % p.K, bx);
  float* o = s.boxtab + (long)i * 40;
#pragma unroll
  for (int c = 0; c < 8; ++c) {
    o[c] = bx.cx[c]; o[8 + c] = bx.cy[c]; o[16 + c] = bx.cz[c]; o[24 + c] = bx.cs[c]; o[32 + c] = bx.sn[c];
  }
}

// The walk shared by count and fill: thread = (b, l, k) as in the forward, f(bin, pair index, corner mask).
template <class F>
__device__ __forceinline__ void bds_walk(const BoxDistP& p, F f) {
  const Items it = my_items(p);
  const float scale = 1.0f / (3.0f * p.max_value);
  BoxLane bx;
  long cur = -1;
  for (long item = it.i0; item < it.i1; ++item) {
    const int l = (int)(item % p.L);
    const long bk = item / p.L;
    const int b = (int)(bk / it.kchunks), k = (int)(bk % it.kchunks) * NTHREADS + threadIdx.x;
    if (k >= p.K) continue;
    if (bk != cur) {
      load_box(p, b, k, bx);
      cur = bk;
    }
    const float* key = p.key + ((long)b * p.L + l) * 3;
    CornerGrid cg;
    corner_grid(p, bx, key[0], key[1], key[2], scale, cg);
    const unsigned pid = (unsigned)(((long)b * p.L + l) * p.K + k);
    for_entries(cg, [&](int mx, int my, int mz, unsigned mask) {
      const int bin = bds_bin(p, mx, my, mz);
      if (bin >= 0) f(bin, pid, mask);
    });
  }
}

__global__ __launch_bounds__(NTHREADS) void k_bds_count(BoxDistP p, SortP s) {
  __shared__ int hist[BDS_MAXBINS];
  for (int e = threadIdx.x; e < s.nbins; e += NTHREADS) hist[e] = 0;
  __syncthreads();
  bds_walk(p, [&](int bin, unsigned, unsigned) { atomicAdd(&hist[bin], 1); });
  __syncthreads();
  for (int e = threadIdx.x; e < s.nbins; e += NTHREADS) {
    const int c = hist[e];
    s.wgbase[(long)blockIdx.x * s.nbins + e] = c;
    if (c) atomicAdd(&s.counts[e], c);
  }
}

// exclusive scan of v[0..n) into out (one workgroup; v and out may alias); returns the total to every thread
__device__ int bds_scan(const int* v, int* out, int n, int* part) {
  const int per = (n + NTHREADS - 1) / NTHREADS;
  const int e0 = min(threadIdx.x * per, n), e1 = min(e0 + per, n);
  int sum = 0;
  for (int e = e0; e < e1; ++e) sum += v[e];
  part[threadIdx.x] = sum;
  __syncthreads();
  if (threadIdx.x < 64) {  // exclusive scan of the 256 partial sums by one wave: 4 per lane, then across the lanes
    const int t0 = threadIdx.x * 4;
    const int c0 = part[t0], c1 = part[t0 + 1], c2 = part[t0 + 2], c3 = part[t0 + 3];
    const int mine = c0 + c1 + c2 + c3;
    int incl = mine;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int v = __shfl_up(incl, o, 64);
      if ((int)threadIdx.x >= o) incl += v;
    }
    const int excl = incl - mine;
    part[t0] = excl; part[t0 + 1] = excl + c0; part[t0 + 2] = excl + c0 + c1; part[t0 + 3] = excl + c0 + c1 + c2;
    if (threadIdx.x == 63) part[NTHREADS] = incl;
  }
  __syncthreads();
  int run = part[threadIdx.x];
  for (int e = e0; e < e1; ++e) {
    const int c = v[e];
    out[e] = run;
    run += c;
  }
  const int total = part[NTHREADS];
  __syncthreads();
  return total;
}

__global__ __launch_bounds__(NTHREADS) void k_bds_plan(SortP s) {
  __shared__ int off[BDS_MAXBINS];
  __shared__ int ibase[BDS_MAXBINS];
  __shared__ int part[NTHREADS + 1];
  bds_scan(s.counts, off, s.nbins, part);
  for (int e = threadIdx.x; e < s.nbins; e += NTHREADS) {
    s.binoff[e] = off[e];
    ibase[e] = (s.counts[e] + BDS_SEG - 1) / BDS_SEG;
  }
  __syncthreads();
  // work items: ranges of at most BDS_SEG entries of one bin
  const int nitems = bds_scan(ibase, ibase, s.nbins, part);
  for (int e = threadIdx.x; e < s.nbins; e += NTHREADS) {
    const int c = s.counts[e], first = off[e];
    int it = ibase[e];
    for (int a = 0; a < c; a += BDS_SEG, ++it) {
      if (it < s.maxitems) {
        s.items[3 * it] = e;
        s.items[3 * it + 1] = first + a;
        s.items[3 * it + 2] = first + min(a + BDS_SEG, c);
      }
    }
  }
  if (threadIdx.x == 0) s.scal[1] = (unsigned)min(nitems, s.maxitems);
}

// Base position of every counting workgroup inside every bin: a running sum over the workgroups, in order (thread
// = bin; 64 loads in flight at a time).
__global__ __launch_bounds__(64) void k_bds_wgbase(SortP s) {
  const int e = blockIdx.x * 64 + threadIdx.x;
  if (e >= s.nbins) return;
  int run = s.binoff[e];
  for (int w0 = 0; w0 < BDS_NWG; w0 += 64) {
    int c[64];
#pragma unroll
    for (int j = 0; j < 64; ++j) c[j] = s.wgbase[(long)(w0 + j) * s.nbins + e];
#pragma unroll
    for (int j = 0; j < 64; ++j) {
      s.wgbase[(long)(w0 + j) * s.nbins + e] = run;
      run += c[j];
    }
  }
}

__global__ __launch_bounds__(NTHREADS) void k_bds_fill(BoxDistP p, SortP s) {
  __shared__ int cur[BDS_MAXBINS];
  for (int e = threadIdx.x; e < s.nbins; e += NTHREADS) cur[e] = s.wgbase[(long)blockIdx.x * s.nbins + e];
  __syncthreads();
  bds_walk(p, [&](int bin, unsigned pid, unsigned mask) {
    const int pos = atomicAdd(&cur[bin], 1);
    if (pos >= 0 && pos < s.maxrecords) s.records[pos] = (unsigned long long)pid | ((unsigned long long)mask << 32);
  });
}

// Trilinear weights of one axis over the window's three nodes m, m + 1, m + 2 for a sample at node position x: the
// hat function max(0, 1 - |x - node|), which is (1 - f, f) on the two nodes around x and zero on the third -- no
// floor, no case distinction.  (An entry only holds corners whose base node is m or m + 1.)
__device__ __forceinline__ void axis3(float x, float m, float (&a)[3]) {
  const float t = x - m;
#pragma unroll
  for (int j = 0; j < 3; ++j) a[j] = fmaxf(1.0f - fabsf(t - (float)j), 0.0f);
}

// 4 x 4 transpose of bytes: in q[0..3] byte d of q[r] is digit d of entry r; out t[d] holds digit d of the four
// entries.
__device__ __forceinline__ void digits4(const unsigned (&q)[4], unsigned (&t)[4]) {
  const unsigned x0 = __builtin_amdgcn_perm(q[1], q[0], 0x05010400u), x1 = __builtin_amdgcn_perm(q[1], q[0], 0x07030602u);
  const unsigned y0 = __builtin_amdgcn_perm(q[3], q[2], 0x05010400u), y1 = __builtin_amdgcn_perm(q[3], q[2], 0x07030602u);
  t[0] = __builtin_amdgcn_perm(y0, x0, 0x05040100u);
  t[1] = __builtin_amdgcn_perm(y0, x0, 0x07060302u);
  t[2] = __builtin_amdgcn_perm(y1, x1, 0x05040100u);
  t[3] = __builtin_amdgcn_perm(y1, x1, 0x07060302u);
}
// 16 entries' fixed-point values (one dword each, four signed digits) -> per digit the 16 bytes of a matrix operand
__device__ __forceinline__ void digit_operands(const unsigned* row, i4 (&op)[4]) {
  unsigned t[4][4];
#pragma unroll
  for (int m = 0; m < 4; ++m) {
    const uint4 v = *(const uint4*)(row + 4 * m);
    const unsigned q[4] = {v.x, v.y, v.z, v.w};
    digits4(q, t[m]);
  }
#pragma unroll
  for (int d = 0; d < 4; ++d) op[d] = (i4){(int)t[0][d], (int)t[1][d], (int)t[2][d], (int)t[3][d]};
}
// A 32-bit integer as four signed base-256 digits, one per byte: v = sum d_i 256^i with d_i in [-128, 127].
__device__ __forceinline__ unsigned signed_digits(int v) { return ((unsigned)v + 0x80808080u) ^ 0x80808080u; }

// One work item: out[node][ch] = sum over the item's entries of weight[entry][node] * ddist[entry][ch], exactly, in
// integers, on the matrix cores.  Weights are taken to 2^-24 and ddist to 2^-22 of its largest magnitude; both are
// written as signed base-256 digits, and the product of two values is the sum of the products of their digits,
// 256^(i+j) apart: twelve int8 products (v_mfma_i32_16x16x64_i8: 16 nodes x 16 channels x 64 entries) that add into
// six 32-bit accumulators, one per power of 256.  Integer sums do not depend on the order of the entries, which the
// fill pass does not fix, so the result is reproducible bit for bit.  Wave w of a batch of 256 entries owns entries
// 64 w .. 64 w + 63: it stages their values as Wq[node][entry], Gq[channel][entry] and reads back 16 entries per lane.
constexpr int BDS_ROW = 64 + 4;  // dwords per staged row: lanes of one 16-lane group start 4 banks apart
template <bool BF>
__global__ __launch_bounds__(NTHREADS) void k_bds_accum(BoxDistP p, SortP s) {
  __shared__ __attribute__((aligned(16))) unsigned Wq[4][27][BDS_ROW];
  __shared__ __attribute__((aligned(16))) unsigned Gq[4][BD_C][BDS_ROW];
  const int item = blockIdx.x;
  if (item >= (int)s.scal[1]) return;  // uniform
  const int bin = s.items[3 * item], first = s.items[3 * item + 1], last = s.items[3 * item + 2];
  const int mx = bin % (p.W + 2) - 2, my = (bin / (p.W + 2)) % (p.H + 2) - 2, mz = bin / ((p.W + 2) * (p.H + 2)) - 2;
  const float fmx = (float)mx, fmy = (float)my, fmz = (float)mz;
  const float scale = 1.0f / (3.0f * p.max_value);
  const float g_scale = bds_scale(s.scal);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r = lane & 15, kg = lane >> 4;
  i4 acc[2][6];
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int c = 0; c < 6; ++c) acc[t][c] = (i4){0, 0, 0, 0};
  for (int base = first; base < last; base += NTHREADS) {
    const int e = base + threadIdx.x;
    float w[27];
#pragma unroll
    for (int j = 0; j < 27; ++j) w[j] = 0.0f;
    f4 g[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) g[j] = (f4){0.0f, 0.0f, 0.0f, 0.0f};
    if (e < last) {
      const unsigned long long rec = s.records[e];
      unsigned pid = (unsigned)rec, mask = (unsigned)(rec >> 32);
      if (pid >= (unsigned)((long)p.B * p.L * p.K) || mask > 255u) { pid = 0u; mask = 0u; }  // never index with a stray record
      const int k = (int)(pid % (unsigned)p.K);
      const unsigned bl = pid / (unsigned)p.K;
      const int l = (int)(bl % (unsigned)p.L), b = (int)(bl / (unsigned)p.L);
      const float* key = p.key + ((long)b * p.L + l) * 3;
      const float kx = key[0], ky = key[1], kz = key[2];
      // ddist of the pair: requested before the corner loop (and unpacked after it) so that its latency runs under it
      uint4 graw[4];
      {
        const uint4* src = (const uint4*)((const char*)p.ddist + (long)pid * BD_C * (BF ? 2 : 4));
#pragma unroll
        for (int j = 0; j < (BF ? 2 : 4); ++j) graw[j] = src[j];
      }
      f4 bt[10];  // the box: x[8], y[8], z[8], cos[8], sin[8]
#pragma unroll
      for (int j = 0; j < 10; ++j) bt[j] = *(const f4*)(s.boxtab + ((long)b * p.K + k) * 40 + 4 * j);
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        if (mask & (1u << c)) {
          float x, y, z;
          corner_pos(p, bt[c >> 2][c & 3], bt[2 + (c >> 2)][c & 3], bt[4 + (c >> 2)][c & 3], bt[6 + (c >> 2)][c & 3],
                     bt[8 + (c >> 2)][c & 3], kx, ky, kz, scale, x, y, z);
          float ax[3], ay[3], az[3];
          axis3(x, fmx, ax);
          axis3(y, fmy, ay);
          axis3(z, fmz, az);
#pragma unroll
          for (int i = 0; i < 3; ++i)
#pragma unroll
            for (int j = 0; j < 3; ++j) {
              const float yx = ay[i] * ax[j];
#pragma unroll
              for (int kk = 0; kk < 3; ++kk) w[kk * 9 + i * 3 + j] = fmaf(az[kk], yx, w[kk * 9 + i * 3 + j]);
            }
        }
      }
      if (BF) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const uint4 v = graw[j];
          g[2 * j] = (f4){__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u), __uint_as_float(v.y << 16),
                          __uint_as_float(v.y & 0xffff0000u)};
          g[2 * j + 1] = (f4){__uint_as_float(v.z << 16), __uint_as_float(v.z & 0xffff0000u), __uint_as_float(v.w << 16),
                              __uint_as_float(v.w & 0xffff0000u)};
        }
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) g[j] = __builtin_bit_cast(f4, graw[j]);
      }
    }
    // a weight is at most 8 (eight corners on one node): 2^27 as an integer; |ddist * g_scale| <= 2^22 (three digits)
#pragma unroll
    for (int j = 0; j < 27; ++j) Wq[wave][j][lane] = signed_digits(__float2int_rn(w[j] * BDS_W_SCALE));
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      Gq[wave][4 * j + 0][lane] = signed_digits(__float2int_rn(g[j].x * g_scale));
      Gq[wave][4 * j + 1][lane] = signed_digits(__float2int_rn(g[j].y * g_scale));
      Gq[wave][4 * j + 2][lane] = signed_digits(__float2int_rn(g[j].z * g_scale));
      Gq[wave][4 * j + 3][lane] = signed_digits(__float2int_rn(g[j].w * g_scale));
    }
    __syncthreads();
    if (base + wave * 64 < last) {  // uniform per wave: the wave's 64 entries hold something
      i4 bop[4];
      digit_operands(&Gq[wave][r][16 * kg], bop);
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const int node = 16 * t + r;
        i4 aop[4];
        digit_operands(&Wq[wave][node < 27 ? node : 0][16 * kg], aop);
#pragma unroll
        for (int d = 0; d < 4; ++d)
          if (node >= 27) aop[d] = (i4){0, 0, 0, 0};
#pragma unroll
        for (int dw = 0; dw < 4; ++dw)
#pragma unroll
          for (int dg = 0; dg < 3; ++dg)
            acc[t][dw + dg] = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop[dw], bop[dg], acc[t][dw + dg], 0, 0, 0);
      }
    }
    __syncthreads();
  }
  // 256^c apart, in 64 bits; then the four waves' sums.  The lane holds nodes 16 t + 4 kg + i, channel r.
  long long* red = (long long*)&Wq[0][0][0];  // [wave][t * 4 + i][lane]: 16 KB of the staging area
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      long long v = 0;
#pragma unroll
      for (int c = 5; c >= 0; --c) v = v * 256 + (long long)acc[t][c][i];
      red[(wave * 8 + t * 4 + i) * 64 + lane] = v;
    }
  __syncthreads();
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int ti = h * 4 + wave, node = 16 * (ti >> 2) + 4 * kg + (ti & 3);
    if (node < 27) {
      long long v = 0;
#pragma unroll
      for (int w2 = 0; w2 < 4; ++w2) v += red[(w2 * 8 + ti) * 64 + lane];
      s.item_out[(long)item * BDS_OUT + node * BD_C + r] = v;
    }
  }
}

__global__ __launch_bounds__(NTHREADS) void k_bds_scatter(BoxDistP p, SortP s) {
  const long id = (long)blockIdx.x * NTHREADS + threadIdx.x;
  const int item = (int)(id / BDS_OUT);
  if (item >= (int)s.scal[1]) return;
  const int r = (int)(id % BDS_OUT), slot = r >> 4, ch = r & 15;
  const int bin = s.items[3 * item];
  const int jx = bin % (p.W + 2) - 2 + slot % 3, jy = (bin / (p.W + 2)) % (p.H + 2) - 2 + (slot / 3) % 3,
            jz = bin / ((p.W + 2) * (p.H + 2)) - 2 + slot / 9;
  if (jx < 0 || jx >= p.W || jy < 0 || jy >= p.H || jz < 0 || jz >= p.D) return;
  const long long v = s.item_out[id];
  if (v == 0) return;
  const long e = ((long)(jz * p.H + jy) * p.W + jx) * BD_C + ch;
  atomicAdd((unsigned long long*)&s.dtab[e], (unsigned long long)v & 0xffffffffull);                      // low half, >= 0
  atomicAdd((unsigned long long*)&s.dtab[(long)p.D * p.H * p.W * BD_C + e], (unsigned long long)(v >> 32));  // the rest, signed
}

__global__ __launch_bounds__(NTHREADS) void k_bds_finish(BoxDistP p, SortP s) {
  const int cells = p.D * p.H * p.W;
  const int e = blockIdx.x * NTHREADS + threadIdx.x;  // e = cell * 16 + ch
  if (e >= cells * BD_C) return;
  const double v = (double)s.dtab[cells * BD_C + e] * 4294967296.0 + (double)s.dtab[e];
  p.dtable[(long)(e % BD_C) * cells + e / BD_C] = (float)(v / ((double)BDS_W_SCALE * (double)bds_scale(s.scal)));
}

// max |ddist|, four wide loads in flight per lane (n is a multiple of 16)
template <bool BF>
__global__ __launch_bounds__(NTHREADS) void k_bds_gmax(BoxDistP p, unsigned* scal) {
  const long n = (long)p.B * p.L * p.K * BD_C;
  const long per = BF ? 8 : 4, step = (long)gridDim.x * NTHREADS * per;  // elements per 16-byte load; per sweep
  unsigned m = 0u;  // largest magnitude as a bit pattern: orders like the float for non-negative values
  for (long e = ((long)blockIdx.x * NTHREADS + threadIdx.x) * per; e < n; e += 4 * step) {
    uint4 v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const long ej = e + j * step;
      v[j] = *(const uint4*)((const char*)p.ddist + (ej < n ? ej : e) * (BF ? 2 : 4));
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const unsigned w[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (BF) {
          const unsigned lo = (w[i] << 16) & 0x7fffffffu, hi = w[i] & 0x7fff0000u;
          m = max(m, (lo <= 0x7f800000u ? lo : 0u));  // NaN patterns are left out
          m = max(m, (hi <= 0x7f800000u ? hi : 0u));
        } else {
          const unsigned a = w[i] & 0x7fffffffu;
          m = max(m, (a <= 0x7f800000u ? a : 0u));
        }
      }
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) m = max(m, (unsigned)__shfl_xor((int)m, o, 64));
  __shared__ unsigned wm[NTHREADS / 64];
  if ((threadIdx.x & 63) == 0) wm[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) {  // one atomic per workgroup: thousands on one address would take longer than the sweep
#pragma unroll
    for (int w = 1; w < NTHREADS / 64; ++w) m = max(m, wm[w]);
    if (m > 0u) atomicMax(scal, m);
  }
}

static long bds_align(long v) { return (v + 15) & ~15L; }

struct BdsLayout {
  long scal, counts, binoff, wgbase, items, records, item_out, dtab, boxtab, total;
  int nbins, maxitems;
  long maxrecords;
};
static BdsLayout bds_layout(int B, int L, int K, int D, int H, int W) {
  BdsLayout y;
  const long pairs = (long)B * L * K, maxrec = pairs * 8;
  y.nbins = (D + 2) * (H + 2) * (W + 2);
  y.maxitems = (int)(y.nbins + maxrec / BDS_SEG + 1);
  long o = 0;
  y.scal = o; o = bds_align(o + 16);
  y.counts = o; o = bds_align(o + (long)y.nbins * 4);
  y.binoff = o; o = bds_align(o + (long)y.nbins * 4);
  y.wgbase = o; o = bds_align(o + (long)BDS_NWG * y.nbins * 4);
  y.items = o; o = bds_align(o + (long)y.maxitems * 12);
  y.records = o; o = bds_align(o + maxrec * 8);
  y.item_out = o; o = bds_align(o + (long)y.maxitems * BDS_OUT * 8);
  y.dtab = o; o = bds_align(o + (long)D * H * W * BD_C * 16);  // two halves
  y.boxtab = o; o = bds_align(o + (long)B * K * 40 * 4);
  y.total = o;
  return y;
}

long box_dist_sorted_scratch_bytes(int B, int L, int K, int D, int H, int W) { return bds_layout(B, L, K, D, H, W).total; }

int launch_box_dist_bwd_sorted(const BoxDistP& p, hipStream_t st) {
  const BdsLayout y = bds_layout(p.B, p.L, p.K, p.D, p.H, p.W);
  if (y.nbins > BDS_MAXBINS) return (int)hipErrorInvalidValue;
  char* base = (char*)p.partial;
  SortP s;
  s.scal = (unsigned*)(base + y.scal);
  s.counts = (int*)(base + y.counts);
  s.binoff = (int*)(base + y.binoff);
  s.wgbase = (int*)(base + y.wgbase);
  s.items = (int*)(base + y.items);
  s.records = (unsigned long long*)(base + y.records);
  s.item_out = (long long*)(base + y.item_out);
  s.dtab = (long long*)(base + y.dtab);
  s.boxtab = (float*)(base + y.boxtab);
  s.nbins = y.nbins;
  s.maxitems = y.maxitems;
  s.maxrecords = (long)p.B * p.L * p.K * 8;
  const dim3 b(NTHREADS);
  const int cells16 = p.D * p.H * p.W * BD_C;
  const int nclear = cells16 > y.nbins ? cells16 : y.nbins;
  hipLaunchKernelGGL(k_bds_clear, dim3((nclear + NTHREADS - 1) / NTHREADS), b, 0, st, p, s);
  if (p.dtype) hipLaunchKernelGGL(k_bds_gmax<true>, dim3(512), b, 0, st, p, s.scal);
  else hipLaunchKernelGGL(k_bds_gmax<false>, dim3(512), b, 0, st, p, s.scal);
  hipLaunchKernelGGL(k_bds_boxes, dim3((p.B * p.K + NTHREADS - 1) / NTHREADS), b, 0, st, p, s);
  hipLaunchKernelGGL(k_bds_count, dim3(BDS_NWG), b, 0, st, p, s);
  hipLaunchKernelGGL(k_bds_plan, dim3(1), b, 0, st, s);
  hipLaunchKernelGGL(k_bds_wgbase, dim3((y.nbins + 63) / 64), dim3(64), 0, st, s);
  hipLaunchKernelGGL(k_bds_fill, dim3(BDS_NWG), b, 0, st, p, s);
  int e = (int)hipGetLastError();
  if (e) return e;
  if (p.dtype) hipLaunchKernelGGL(k_bds_accum<true>, dim3(y.maxitems), b, 0, st, p, s);
  else hipLaunchKernelGGL(k_bds_accum<false>, dim3(y.maxitems), b, 0, st, p, s);
  const long nscat = (long)y.maxitems * BDS_OUT;
  hipLaunchKernelGGL(k_bds_scatter, dim3((unsigned)((nscat + NTHREADS - 1) / NTHREADS)), b, 0, st, p, s);
  hipLaunchKernelGGL(k_bds_finish, dim3((cells16 + NTHREADS - 1) / NTHREADS), b, 0, st, p, s);
  return (int)hipGetLastError();
}

}  // namespace issm
