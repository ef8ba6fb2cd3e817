// Depthwise 7-tap convolution along the token order + SiLU, on (B, L, C) tensors as they are (gfx950).
//
// DEST's PointLiteConv (models/dest_module.py:400-423) is nn.Conv1d(C, C, 7, padding=3, groups=C) + SiLU applied
// to feature.transpose(1, 2).  A library convolution sees (B, C, L) and pays for two transposes and an
// im2col-style lowering; here channels stay innermost (lanes run over c: every access is coalesced) and a thread
// owns DW_TL consecutive tokens of one channel, with the 3 + 3 halo rows in registers.  `nsets` weight sets are applied in one pass:
//   pre[s][b][l][c] = bias[s][c] + sum_j w[s][c][j] in_s[b][l + j - 3][c]      (zero outside [0, L))
//   y[s] = pre[s] * sigmoid(pre[s])
// with in_s = u for every set, or -- `chain` -- in_0 = u and in_1 = y[0]: the module's reversed-order branch convolves the
// forward-order branch's OUTPUT (dest_module.py:530 reassigns xbc = key_conv(xbc) before :534 calls key_conv_back on it).
// The chained kernels keep a 6 + 6 halo of u so that y[0] is at hand on the 3 + 3 halo the second convolution needs
// (y[0] outside [0, L) is the second convolution's zero padding, not the first one applied to padding).
// The backward reads dy and the saved pre: dpre = dy * sigmoid(pre) * (1 + pre * (1 - sigmoid(pre))),
//   du[b][l][c] = sum_s sum_j w[s][c][j] dpre[s][b][l + 3 - j][c],
//   dw[s][c][j] = sum_{b,l} dpre[s][b][l][c] u[b][l + j - 3][c],   dbias[s][c] = sum_{b,l} dpre[s][b][l][c],
// the last two as per-thread partials (one per (b, token tile)) summed in fixed order by a second kernel.
// Everything is memory bound; arithmetic is fp32.
#include "issm_dev.h"

namespace issm {

constexpr int DW_TAPS = 7;
constexpr int DW_TL = 16;     // tokens per thread

template <bool BF>
__device__ __forceinline__ float dw_ld(const void* p, long i) {
  return BF ? bf16_to_f(((const uint16_t*)p)[i]) : ((const float*)p)[i];
}
template <bool BF>
__device__ __forceinline__ void dw_st(void* p, long i, float v) {
  if (BF) ((uint16_t*)p)[i] = f_to_bf16(v); else ((float*)p)[i] = v;
}

// thread -> (b, tile, c), c fastest
__device__ __forceinline__ bool dw_item(const DwConvP& p, int& b, int& l0, int& c) {
  const long id = (long)blockIdx.x * NTHREADS + threadIdx.x;
  const int ntile = (p.L + DW_TL - 1) / DW_TL;
  if (id >= (long)p.B * ntile * p.C) return false;
  c = (int)(id % p.C);
  const long r = id / p.C;
  l0 = (int)(r % ntile) * DW_TL;
  b = (int)(r / ntile);
  return true;
}

template <bool BF, int S>
__global__ __launch_bounds__(NTHREADS) void k_dwconv_fwd(DwConvP p) {
  int b, l0, c;
  if (!dw_item(p, b, l0, c)) return;
  float w[S][DW_TAPS], bias[S];
#pragma unroll
  for (int s = 0; s < S; ++s) {
#pragma unroll
    for (int j = 0; j < DW_TAPS; ++j) w[s][j] = p.w[((long)s * p.C + c) * DW_TAPS + j];
    bias[s] = p.bias[(long)s * p.C + c];
  }
  const long ub = (long)b * p.u_bs + c;
  // rows outside [0, L) read row 0 or L - 1 and are replaced by zero: loads without branches stay in flight together
  auto u_at = [&](int l) -> float {
    const float v = dw_ld<BF>(p.u, ub + (long)min(max(l, 0), p.L - 1) * p.u_ls);
    return (l >= 0 && l < p.L) ? v : 0.0f;
  };
  float ub_[DW_TL + DW_TAPS - 1];  // u[l0 - 3 .. l0 + DW_TL + 2]: every load is issued before the first use
#pragma unroll
  for (int j = 0; j < DW_TL + DW_TAPS - 1; ++j) ub_[j] = u_at(l0 + j - 3);
#pragma unroll
  for (int i = 0; i < DW_TL; ++i) {
    const int l = l0 + i;
    if (l < p.L) {
#pragma unroll
      for (int s = 0; s < S; ++s) {
        float a = bias[s];
#pragma unroll
        for (int j = 0; j < DW_TAPS; ++j) a = fmaf(w[s][j], ub_[i + j], a);
        const long o = (((long)s * p.B + b) * p.L + l) * p.C + c;
        if (BF) a = bf16_to_f(f_to_bf16(a));  // the saved pre-activation is what the backward differentiates
        dw_st<BF>(p.pre, o, a);
        const float yv = a * sigmoidf_(a);
        if (p.split > 0) {  // uniform: channels [0, split) and [split, C) go to two dense tensors
          const long row = ((long)s * p.B + b) * p.L + l;
          if (c < p.split) dw_st<BF>(p.y, row * p.split + c, yv);
          else dw_st<BF>(p.y_tail, row * (p.C - p.split) + (c - p.split), yv);
        } else {
          dw_st<BF>(p.y, o, yv);
        }
      }
    }
  }
}

// partial layout: [(b * ntile + tile)][s][j (0..6: taps, 7: bias)][c]
template <bool BF, int S>
__global__ __launch_bounds__(NTHREADS) void k_dwconv_bwd(DwConvP p) {
  int b, l0, c;
  if (!dw_item(p, b, l0, c)) return;
  float w[S][DW_TAPS];
#pragma unroll
  for (int s = 0; s < S; ++s)
#pragma unroll
    for (int j = 0; j < DW_TAPS; ++j) w[s][j] = p.w[((long)s * p.C + c) * DW_TAPS + j];
  const long ub = (long)b * p.u_bs + c;
  constexpr int W = DW_TL + DW_TAPS - 1;
  float ub_[W], dyb[S][W], prb[S][W];  // rows l0 - 3 .. l0 + DW_TL + 2, loaded before the first use
#pragma unroll
  for (int j = 0; j < W; ++j) {
    // rows outside [0, L) read row 0 or L - 1 and are replaced by zero: loads without branches stay in flight together
    const int l = l0 + j - 3, lc = min(max(l, 0), p.L - 1);
    const bool in = l >= 0 && l < p.L;
    const float uv = dw_ld<BF>(p.u, ub + (long)lc * p.u_ls);
    ub_[j] = in ? uv : 0.0f;
#pragma unroll
    for (int s = 0; s < S; ++s) {
      const long o = ((long)b * p.L + lc) * p.C + c;
      // with a split the gradient arrives as the two dense tensors of the forward: which one a lane reads is chosen
      // by selecting the address, not by a branch (an absent tensor reads `pre` and counts as zero), so that all
      // loads of the thread stay in flight together
      const bool head = p.split <= 0 || c < p.split;
      const void* src = head ? p.dy[s] : p.dy_tail[s];
      const long row = (long)b * p.L + lc;
      long off = o;
      if (p.split > 0) off = head ? row * p.split + c : row * (p.C - p.split) + (c - p.split);  // uniform condition
      const bool have = src != nullptr;
      const float dyv = dw_ld<BF>(have ? src : p.pre, have ? off : o);
      const float pv = dw_ld<BF>(p.pre, (long)s * p.B * p.L * p.C + o);
      dyb[s][j] = (in && have) ? dyv : 0.0f;
      prb[s][j] = in ? pv : 0.0f;
    }
  }
  // dpre in place of dy
#pragma unroll
  for (int s = 0; s < S; ++s)
#pragma unroll
    for (int j = 0; j < W; ++j) {
      const float x = prb[s][j], sg = sigmoidf_(x);
      dyb[s][j] *= sg * (1.0f + x * (1.0f - sg));
    }
  float gw[S][DW_TAPS], gb[S];
#pragma unroll
  for (int s = 0; s < S; ++s) {
    gb[s] = 0.0f;
#pragma unroll
    for (int j = 0; j < DW_TAPS; ++j) gw[s][j] = 0.0f;
  }
#pragma unroll
  for (int i = 0; i < DW_TL; ++i) {
    const int l = l0 + i;
    if (l < p.L) {
      float du = 0.0f;
#pragma unroll
      for (int s = 0; s < S; ++s) {
        // u[l] feeds pre[l + 3 - j] through tap j: buffer slot i + 6 - j
#pragma unroll
        for (int j = 0; j < DW_TAPS; ++j) du = fmaf(w[s][j], dyb[s][i + DW_TAPS - 1 - j], du);
        const float d0 = dyb[s][i + 3];  // dpre[s][l]
        gb[s] += d0;
#pragma unroll
        for (int j = 0; j < DW_TAPS; ++j) gw[s][j] = fmaf(d0, ub_[i + j], gw[s][j]);
      }
      if (p.du) dw_st<BF>(p.du, (long)b * p.du_bs + (long)l * p.du_ls + c, du);
    }
  }
  const int ntile = (p.L + DW_TL - 1) / DW_TL;
  const long row = (long)b * ntile + l0 / DW_TL;
#pragma unroll
  for (int s = 0; s < S; ++s) {
    float* dst = p.partial + ((row * S + s) * 8) * p.C + c;
#pragma unroll
    for (int j = 0; j < DW_TAPS; ++j) dst[(long)j * p.C] = gw[s][j];
    dst[(long)DW_TAPS * p.C] = gb[s];
  }
}

// ---- chained pair: set 1 convolves set 0's output (rounded to the I/O dtype, as it is stored)
template <bool BF>
__device__ __forceinline__ float dw_round(float v) { return BF ? bf16_to_f(f_to_bf16(v)) : v; }

// output / gradient address of (set s, row, channel c) with or without the channel split
__device__ __forceinline__ long dw_out_off(const DwConvP& p, long row, int c, bool& head) {
  head = p.split <= 0 || c < p.split;
  if (p.split <= 0) return row * p.C + c;
  return head ? row * p.split + c : row * (p.C - p.split) + (c - p.split);
}

template <bool BF>
__global__ __launch_bounds__(NTHREADS) void k_dwconv_chain_fwd(DwConvP p) {
  int b, l0, c;
  if (!dw_item(p, b, l0, c)) return;
  float w[2][DW_TAPS], bias[2];
#pragma unroll
  for (int s = 0; s < 2; ++s) {
#pragma unroll
    for (int j = 0; j < DW_TAPS; ++j) w[s][j] = p.w[((long)s * p.C + c) * DW_TAPS + j];
    bias[s] = p.bias[(long)s * p.C + c];
  }
  const long ub = (long)b * p.u_bs + c;
  constexpr int W1 = DW_TL + DW_TAPS - 1, W2 = W1 + DW_TAPS - 1;
  float ub_[W2];  // u[l0 - 6 .. l0 + DW_TL + 5]
#pragma unroll
  for (int j = 0; j < W2; ++j) {
    const int l = l0 + j - 6;
    const float v = dw_ld<BF>(p.u, ub + (long)min(max(l, 0), p.L - 1) * p.u_ls);
    ub_[j] = (l >= 0 && l < p.L) ? v : 0.0f;
  }
  float pre0[W1], y0[W1];  // rows l0 - 3 .. l0 + DW_TL + 2
#pragma unroll
  for (int j = 0; j < W1; ++j) {
    const int l = l0 + j - 3;
    float a = bias[0];
#pragma unroll
    for (int t = 0; t < DW_TAPS; ++t) a = fmaf(w[0][t], ub_[j + t], a);
    a = dw_round<BF>(a);
    pre0[j] = a;
    y0[j] = (l >= 0 && l < p.L) ? dw_round<BF>(a * sigmoidf_(a)) : 0.0f;
  }
#pragma unroll
  for (int i = 0; i < DW_TL; ++i) {
    const int l = l0 + i;
    if (l < p.L) {
      float a = bias[1];
#pragma unroll
      for (int t = 0; t < DW_TAPS; ++t) a = fmaf(w[1][t], y0[i + t], a);
      a = dw_round<BF>(a);
      const float y1 = a * sigmoidf_(a);
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const long row = ((long)s * p.B + b) * p.L + l;
        dw_st<BF>(p.pre, row * p.C + c, s ? a : pre0[i + 3]);
        bool head;
        const long o = dw_out_off(p, row, c, head);
        dw_st<BF>(head ? p.y : p.y_tail, o, s ? y1 : y0[i + 3]);
      }
    }
  }
}

template <bool BF>
__global__ __launch_bounds__(NTHREADS) void k_dwconv_chain_bwd(DwConvP p) {
  int b, l0, c;
  if (!dw_item(p, b, l0, c)) return;
  float w[2][DW_TAPS];
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int j = 0; j < DW_TAPS; ++j) w[s][j] = p.w[((long)s * p.C + c) * DW_TAPS + j];
  const long ub = (long)b * p.u_bs + c;
  constexpr int W1 = DW_TL + DW_TAPS - 1, W2 = W1 + DW_TAPS - 1;
  const long set1 = (long)p.B * p.L * p.C;
  // every load is issued before the first use; rows outside [0, L) read a clamped row and count as zero
  float d1[W2], p1[W2];          // dy[1], pre[1] on rows l0 - 6 .. l0 + DW_TL + 5
  float d0[W1], p0[W1], ub_[W1]; // dy[0], pre[0], u on rows l0 - 3 .. l0 + DW_TL + 2
  auto grad_at = [&](int s, int lc, bool in) -> float {
    bool head;
    const long o = dw_out_off(p, (long)b * p.L + lc, c, head);
    const void* src = head ? p.dy[s] : p.dy_tail[s];
    const bool have = src != nullptr;
    const float v = dw_ld<BF>(have ? src : p.pre, have ? o : ((long)b * p.L + lc) * p.C + c);
    return (in && have) ? v : 0.0f;
  };
#pragma unroll
  for (int j = 0; j < W2; ++j) {
    const int l = l0 + j - 6, lc = min(max(l, 0), p.L - 1);
    const bool in = l >= 0 && l < p.L;
    d1[j] = grad_at(1, lc, in);
    const float pv = dw_ld<BF>(p.pre, set1 + ((long)b * p.L + lc) * p.C + c);
    p1[j] = in ? pv : 0.0f;
  }
#pragma unroll
  for (int j = 0; j < W1; ++j) {
    const int l = l0 + j - 3, lc = min(max(l, 0), p.L - 1);
    const bool in = l >= 0 && l < p.L;
    d0[j] = grad_at(0, lc, in);
    const float pv = dw_ld<BF>(p.pre, ((long)b * p.L + lc) * p.C + c);
    const float uv = dw_ld<BF>(p.u, ub + (long)lc * p.u_ls);
    p0[j] = in ? pv : 0.0f;
    ub_[j] = in ? uv : 0.0f;
  }
  // dpre[1] in place of dy[1]
#pragma unroll
  for (int j = 0; j < W2; ++j) {
    const float x = p1[j], sg = sigmoidf_(x);
    d1[j] *= sg * (1.0f + x * (1.0f - sg));
  }
  // y[0] (the second convolution's input) and dpre[0] = (dy[0] + what flows back through set 1) * silu'(pre[0])
  float y0[W1];
#pragma unroll
  for (int j = 0; j < W1; ++j) {
    const int l = l0 + j - 3;
    const bool in = l >= 0 && l < p.L;
    const float x = p0[j], sg = sigmoidf_(x);
    y0[j] = in ? dw_round<BF>(x * sg) : 0.0f;
    float g = d0[j];
    // y0[l] feeds pre1[l + 3 - t] through tap t: d1 slot (j + 3) + 3 - t
#pragma unroll
    for (int t = 0; t < DW_TAPS; ++t) g = fmaf(w[1][t], d1[j + DW_TAPS - 1 - t], g);
    d0[j] = in ? g * sg * (1.0f + x * (1.0f - sg)) : 0.0f;
  }
  float gw[2][DW_TAPS], gb[2] = {0.0f, 0.0f};
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int j = 0; j < DW_TAPS; ++j) gw[s][j] = 0.0f;
#pragma unroll
  for (int i = 0; i < DW_TL; ++i) {
    const int l = l0 + i;
    if (l < p.L) {
      float du = 0.0f;
#pragma unroll
      for (int t = 0; t < DW_TAPS; ++t) du = fmaf(w[0][t], d0[i + DW_TAPS - 1 - t], du);
      const float g0 = d0[i + 3], g1 = d1[i + 6];  // dpre[0][l], dpre[1][l]
      gb[0] += g0;
      gb[1] += g1;
#pragma unroll
      for (int t = 0; t < DW_TAPS; ++t) {
        gw[0][t] = fmaf(g0, ub_[i + t], gw[0][t]);
        gw[1][t] = fmaf(g1, y0[i + t], gw[1][t]);
      }
      if (p.du) dw_st<BF>(p.du, (long)b * p.du_bs + (long)l * p.du_ls + c, du);
    }
  }
  const int ntile = (p.L + DW_TL - 1) / DW_TL;
  const long row = (long)b * ntile + l0 / DW_TL;
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    float* dst = p.partial + ((row * 2 + s) * 8) * p.C + c;
#pragma unroll
    for (int j = 0; j < DW_TAPS; ++j) dst[(long)j * p.C] = gw[s][j];
    dst[(long)DW_TAPS * p.C] = gb[s];
  }
}

// dw[s][c][j], dbias[s][c] = fixed-order sums over the partial rows: workgroup = 32 columns x 8 row groups
__global__ __launch_bounds__(NTHREADS) void k_dwconv_dw(DwConvP p) {
  __shared__ float red[NTHREADS];
  const int ncol = p.nsets * 8 * p.C;  // column = (s * 8 + j) * C + c
  const int col = blockIdx.x * 32 + (threadIdx.x & 31), g = threadIdx.x >> 5;
  float a0 = 0.0f, a1 = 0.0f;
  if (col < ncol) {
    int r = g;
    for (; r + 8 < p.nrows; r += 16) {
      a0 += p.partial[(long)r * ncol + col];
      a1 += p.partial[(long)(r + 8) * ncol + col];
    }
    if (r < p.nrows) a0 += p.partial[(long)r * ncol + col];
  }
  red[threadIdx.x] = a0 + a1;
  __syncthreads();
  if (g == 0 && col < ncol) {
    float t = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) t += red[i * 32 + (threadIdx.x & 31)];
    const int c = col % p.C, sj = col / p.C, s = sj >> 3, j = sj & 7;
    if (j < DW_TAPS) p.dw[((long)s * p.C + c) * DW_TAPS + j] = t;
    else p.dbias[(long)s * p.C + c] = t;
  }
}

int dwconv_partial_rows(int B, int L) { return B * ((L + DW_TL - 1) / DW_TL); }

static unsigned dw_blocks(const DwConvP& p) {
  const long items = (long)p.B * ((p.L + DW_TL - 1) / DW_TL) * p.C;
  return (unsigned)((items + NTHREADS - 1) / NTHREADS);
}

int launch_dwconv_fwd(const DwConvP& p, hipStream_t st) {
  const dim3 g(dw_blocks(p)), b(NTHREADS);
  if (p.chain) {
    if (p.dtype) hipLaunchKernelGGL(k_dwconv_chain_fwd<true>, g, b, 0, st, p);
    else hipLaunchKernelGGL(k_dwconv_chain_fwd<false>, g, b, 0, st, p);
  } else if (p.dtype) {
    if (p.nsets == 1) hipLaunchKernelGGL((k_dwconv_fwd<true, 1>), g, b, 0, st, p);
    else hipLaunchKernelGGL((k_dwconv_fwd<true, 2>), g, b, 0, st, p);
  } else {
    if (p.nsets == 1) hipLaunchKernelGGL((k_dwconv_fwd<false, 1>), g, b, 0, st, p);
    else hipLaunchKernelGGL((k_dwconv_fwd<false, 2>), g, b, 0, st, p);
  }
  return (int)hipGetLastError();
}

int launch_dwconv_bwd(const DwConvP& p, hipStream_t st) {
  const dim3 g(dw_blocks(p)), b(NTHREADS);
  if (p.chain) {
    if (p.dtype) hipLaunchKernelGGL(k_dwconv_chain_bwd<true>, g, b, 0, st, p);
    else hipLaunchKernelGGL(k_dwconv_chain_bwd<false>, g, b, 0, st, p);
  } else if (p.dtype) {
    if (p.nsets == 1) hipLaunchKernelGGL((k_dwconv_bwd<true, 1>), g, b, 0, st, p);
    else hipLaunchKernelGGL((k_dwconv_bwd<true, 2>), g, b, 0, st, p);
  } else {
    if (p.nsets == 1) hipLaunchKernelGGL((k_dwconv_bwd<false, 1>), g, b, 0, st, p);
    else hipLaunchKernelGGL((k_dwconv_bwd<false, 2>), g, b, 0, st, p);
  }
  int e = (int)hipGetLastError();
  if (e) return e;
  hipLaunchKernelGGL(k_dwconv_dw, dim3((p.nsets * 8 * p.C + 31) / 32), b, 0, st, p);
  return (int)hipGetLastError();
}

}  // namespace issm
