// Device helpers shared by the box-to-point distance encoding kernels (box_dist.hip, box_dist_sorted.hip).
#pragma once
#include "issm_dev.h"

namespace issm {

constexpr int BD_C = 16;          // channels of the table
constexpr int BD_MAXCELLS = 1024; // D * H * W nodes that fit the 64 KB LDS copy

struct BoxLane {
  float cx[8], cy[8], cz[8];  // corners of the lane's box
  float cs[8], sn[8];         // rotation of flattened corner j = k * 8 + c: angle of query j mod K (as the reference)
  float qx, qy, qz, radius;
};

// Corner c of box k: from the corner tensor, or from the box itself -- boxes (B, K, 7) = centre, size (l, w, h),
// heading -- with the reference's corner order (dest_module.py:62-70 after the axis changes of :26-38):
//   x = cx + sx l/2 cos + sz w/2 sin,  y = cy - sx l/2 sin + sz w/2 cos,  z = cz - sy h/2,
//   sx = + + - - + + - -,  sy = + + + + - - - -,  sz = + - - + + - - +.
__device__ __forceinline__ void box_corner(const BoxDistP& p, int b, int k, int c, float& x, float& y, float& z) {
  if (p.boxes) {  // uniform
    const float* q = p.boxes + ((long)b * p.K + k) * 7;
    const float lx = ((c & 2) ? -0.5f : 0.5f) * q[3];
    const float hy = ((c & 4) ? -0.5f : 0.5f) * q[5];
    const float wz = (((c ^ (c >> 1)) & 1) ? -0.5f : 0.5f) * q[4];
    const float cs = cosf(q[6]), sn = sinf(q[6]);
    x = q[0] + lx * cs + wz * sn;
    y = q[1] - lx * sn + wz * cs;
    z = q[2] - hy;
  } else {
    const float* q = p.corners + (((long)b * p.K + k) * 8 + c) * 3;
    x = q[0]; y = q[1]; z = q[2];
  }
}
// rotation applied to the deltas of corner c of box k: the angle of query (8k + c) mod K, as the reference's tiling
__device__ __forceinline__ void corner_rotation(const BoxDistP& p, int b, int k, int c, float& cs, float& sn) {
  cs = 1.0f;
  sn = 0.0f;
  if (p.angle) {  // uniform
    const float a = p.angle[(long)b * p.K + (k * 8 + c) % p.K];
    cs = cosf(a);
    sn = sinf(a);
  }
}

__device__ __forceinline__ void load_box(const BoxDistP& p, int b, int k, BoxLane& bx) {
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    box_corner(p, b, k, j, bx.cx[j], bx.cy[j], bx.cz[j]);
    corner_rotation(p, b, k, j, bx.cs[j], bx.sn[j]);
  }
  if (p.qcenter) {
    const float* q = p.qcenter + ((long)b * p.K + k) * 3;
    bx.qx = q[0]; bx.qy = q[1]; bx.qz = q[2];
    bx.radius = p.radius[(long)b * p.K + k];
  } else if (p.boxes) {  // locality weight from the box: centre, radius = max(|size|, min_radius)
    const float* q = p.boxes + ((long)b * p.K + k) * 7;
    bx.qx = q[0]; bx.qy = q[1]; bx.qz = q[2];
    bx.radius = fmaxf(sqrtf(q[3] * q[3] + q[4] * q[4] + q[5] * q[5]), p.min_radius);
  }
}

// corner slot j takes the values of slot j + 1, slot 7 those of slot 0 (after 8 calls the box is as it was)
__device__ __forceinline__ void rotate_box(BoxLane& bx) {
  const float x0 = bx.cx[0], y0 = bx.cy[0], z0 = bx.cz[0], c0 = bx.cs[0], s0 = bx.sn[0];
#pragma unroll
  for (int j = 0; j < 7; ++j) {
    bx.cx[j] = bx.cx[j + 1]; bx.cy[j] = bx.cy[j + 1]; bx.cz[j] = bx.cz[j + 1];
    bx.cs[j] = bx.cs[j + 1]; bx.sn[j] = bx.sn[j + 1];
  }
  bx.cx[7] = x0; bx.cy[7] = y0; bx.cz[7] = z0; bx.cs[7] = c0; bx.sn[7] = s0;
}

// signed log compression and grid_sample's un-normalisation (align_corners False) in one: position in node units
__device__ __forceinline__ float node_pos(float v, float log_scale, float scale, int n) {
  const float m = __log2f(fabsf(v) * log_scale + 1.0f) * scale;  // scale = 1 / (log2(8) * max_value)
  const float g = v < 0.0f ? -m : m;
  return (g + 1.0f) * (0.5f * n) - 0.5f;
}

// The 8 neighbours of one sampling position: LDS offset of the node (node index * stride) and its weight (0 outside).
struct Tri {
  int off[8];
  float w[8];
};
__device__ __forceinline__ void trilinear(const BoxDistP& p, float x, float y, float z, Tri& t, int stride = BD_C) {
  const float fx = floorf(x), fy = floorf(y), fz = floorf(z);
  const float ax = x - fx, ay = y - fy, az = z - fz;
  const int ix = (int)fx, iy = (int)fy, iz = (int)fz;
#pragma unroll
  for (int n = 0; n < 8; ++n) {
    const int dx = n & 1, dy = (n >> 1) & 1, dz = n >> 2;
    const int jx = ix + dx, jy = iy + dy, jz = iz + dz;
    const bool ok = jx >= 0 && jx < p.W && jy >= 0 && jy < p.H && jz >= 0 && jz < p.D;
    const float w = (dx ? ax : 1.0f - ax) * (dy ? ay : 1.0f - ay) * (dz ? az : 1.0f - az);
    t.w[n] = ok ? w : 0.0f;
    t.off[n] = ok ? ((jz * p.H + jy) * p.W + jx) * stride : 0;
  }
}

// The 8 corners of a box usually fall into the same or adjacent table cells (a box is small next to the spacing
// of the log-compressed lattice), so their 8 x 8 node weights are first merged, in registers, over a 3 x 3 x 3 window
// of nodes anchored at the smallest base node: up to 27 -- typically 8 to 12 non-zero -- table accesses per
// (point, box) pair instead of 64.  Possible when the corners' base nodes differ by at most one along every axis;
// otherwise the caller walks the corners one by one.
struct Window {
  int mx, my, mz;
  float w[27];  // [dz][dy][dx]
};
__device__ __forceinline__ bool corner_window(const BoxDistP& p, const BoxLane& bx, float kx, float ky, float kz,
                                              float scale, Window& win) {
  float fx[8], fy[8], fz[8];
  int ix[8], iy[8], iz[8];
#pragma unroll
  for (int c = 0; c < 8; ++c) {
    const float dx = bx.cx[c] - kx, dy = bx.cy[c] - ky, dz = bx.cz[c] - kz;
    const float rx = dx * bx.cs[c] - dy * bx.sn[c], ry = dx * bx.sn[c] + dy * bx.cs[c];
    const float x = node_pos(rx, p.log_scale, scale, p.W), y = node_pos(ry, p.log_scale, scale, p.H),
                z = node_pos(dz, p.log_scale, scale, p.D);
    const float gx = floorf(x), gy = floorf(y), gz = floorf(z);
    fx[c] = x - gx; fy[c] = y - gy; fz[c] = z - gz;
    ix[c] = (int)gx; iy[c] = (int)gy; iz[c] = (int)gz;
  }
  int mx = ix[0], my = iy[0], mz = iz[0], Mx = ix[0], My = iy[0], Mz = iz[0];
#pragma unroll
  for (int c = 1; c < 8; ++c) {
    mx = min(mx, ix[c]); Mx = max(Mx, ix[c]);
    my = min(my, iy[c]); My = max(My, iy[c]);
    mz = min(mz, iz[c]); Mz = max(Mz, iz[c]);
  }
  if (Mx - mx > 1 || My - my > 1 || Mz - mz > 1) return false;
  win.mx = mx; win.my = my; win.mz = mz;
#pragma unroll
  for (int e = 0; e < 27; ++e) win.w[e] = 0.0f;
#pragma unroll
  for (int c = 0; c < 8; ++c) {
    const bool sx = ix[c] != mx, sy = iy[c] != my, sz = iz[c] != mz;
    const float ax[3] = {sx ? 0.0f : 1.0f - fx[c], sx ? 1.0f - fx[c] : fx[c], sx ? fx[c] : 0.0f};
    const float ay[3] = {sy ? 0.0f : 1.0f - fy[c], sy ? 1.0f - fy[c] : fy[c], sy ? fy[c] : 0.0f};
    const float az[3] = {sz ? 0.0f : 1.0f - fz[c], sz ? 1.0f - fz[c] : fz[c], sz ? fz[c] : 0.0f};
#pragma unroll
    for (int i = 0; i < 3; ++i)
#pragma unroll
      for (int j = 0; j < 3; ++j) {
        const float yx = ay[i] * ax[j];
#pragma unroll
        for (int k = 0; k < 3; ++k) win.w[k * 9 + i * 3 + j] = fmaf(az[k], yx, win.w[k * 9 + i * 3 + j]);
      }
  }
  return true;
}
// visit the window's nodes that lie inside the table and carry weight: f(LDS offset in floats, weight)
template <class F>
__device__ __forceinline__ void for_window(const BoxDistP& p, const Window& win, F f, int stride = BD_C) {
#pragma unroll
  for (int k = 0; k < 3; ++k)
#pragma unroll
    for (int i = 0; i < 3; ++i)
#pragma unroll
      for (int j = 0; j < 3; ++j) {
        const int jx = win.mx + j, jy = win.my + i, jz = win.mz + k;
        const bool ok = jx >= 0 && jx < p.W && jy >= 0 && jy < p.H && jz >= 0 && jz < p.D;
        const float w = win.w[k * 9 + i * 3 + j];
        if (ok && w != 0.0f) f(((jz * p.H + jy) * p.W + jx) * stride, w);
      }
}

// work split: items = (b, k chunk of 256, l), l fastest; workgroup w takes a contiguous range
struct Items {
  long i0, i1;
  int kchunks;
};
__device__ __forceinline__ Items my_items(const BoxDistP& p) {
  Items it;
  it.kchunks = (p.K + NTHREADS - 1) / NTHREADS;
  const long n = (long)p.B * it.kchunks * p.L;
  it.i0 = n * blockIdx.x / gridDim.x;
  it.i1 = n * (blockIdx.x + 1) / gridDim.x;
  return it;
}

// Fixed-point scale of the table gradient.  A pair's node weights sum to 8 (one per corner), so a node of one
// workgroup's copy collects at most 8 * pairs-per-workgroup * max|ddist|; with 2^34 / max|ddist| that stays below
// 2^63 for 2^26 pairs per workgroup, and the sum over all workgroups is taken in 64 bits as well (2^26 pairs in total
// is the bound the launcher checks).
__device__ __forceinline__ float bd_scale(const unsigned* scal) {
  const float gmax = __uint_as_float(scal[0]);
  return gmax > 1e-27f ? 17179869184.0f / gmax : 1.0f;  // below that the quotient could overflow; such gradients round to 0
}


// ---- corner clusters ---------------------------------------------------------------------------------------
// A box that straddles the point along an axis has corners on both sides of zero, which the signed log sends to
// opposite ends of the lattice: one 3 x 3 x 3 window cannot hold them, but one per side can.  Per axis the corners
// are split into the cluster of the smallest base node (base <= min + 1) and the rest, which must again span at most
// two nodes; a corner then belongs to one of 8 combinations of clusters, each with its own window anchor.  `ok` is
// false when some axis needs a third cluster: then every corner is its own entry, anchored at its base node.
struct CornerGrid {
  float fx[8], fy[8], fz[8];
  int ix[8], iy[8], iz[8];
  int ax[2], ay[2], az[2];  // anchors of the two clusters per axis
  unsigned combo[8];        // cluster combination of each corner: bit 0 x, bit 1 y, bit 2 z
  bool ok;
};
__device__ __forceinline__ bool split_axis(const int (&i)[8], int (&anchor)[2], unsigned (&combo)[8], unsigned bit) {
  int m0 = i[0];
#pragma unroll
  for (int c = 1; c < 8; ++c) m0 = min(m0, i[c]);
  int m1 = 0x7fffffff, M1 = m0;
#pragma unroll
  for (int c = 0; c < 8; ++c) {
    const bool far = i[c] > m0 + 1;
    combo[c] |= far ? bit : 0u;
    m1 = far ? min(m1, i[c]) : m1;
    M1 = far ? max(M1, i[c]) : M1;
  }
  anchor[0] = m0;
  anchor[1] = m1 == 0x7fffffff ? m0 : m1;
  return m1 == 0x7fffffff || M1 - m1 <= 1;
}
// position of corner (cx, cy, cz) relative to the key, in node units
__device__ __forceinline__ void corner_pos(const BoxDistP& p, float cx, float cy, float cz, float cs, float sn, float kx,
                                           float ky, float kz, float scale, float& x, float& y, float& z) {
  const float dx = cx - kx, dy = cy - ky, dz = cz - kz;
  const float rx = dx * cs - dy * sn, ry = dx * sn + dy * cs;
  x = node_pos(rx, p.log_scale, scale, p.W);
  y = node_pos(ry, p.log_scale, scale, p.H);
  z = node_pos(dz, p.log_scale, scale, p.D);
}
__device__ __forceinline__ void corner_grid(const BoxDistP& p, const BoxLane& bx, float kx, float ky, float kz,
                                            float scale, CornerGrid& cg) {
#pragma unroll
  for (int c = 0; c < 8; ++c) {
    float x, y, z;
    corner_pos(p, bx.cx[c], bx.cy[c], bx.cz[c], bx.cs[c], bx.sn[c], kx, ky, kz, scale, x, y, z);
    const float gx = floorf(x), gy = floorf(y), gz = floorf(z);
    cg.fx[c] = x - gx; cg.fy[c] = y - gy; cg.fz[c] = z - gz;
    cg.ix[c] = (int)gx; cg.iy[c] = (int)gy; cg.iz[c] = (int)gz;
    cg.combo[c] = 0u;
  }
  const bool okx = split_axis(cg.ix, cg.ax, cg.combo, 1u);
  const bool oky = split_axis(cg.iy, cg.ay, cg.combo, 2u);
  const bool okz = split_axis(cg.iz, cg.az, cg.combo, 4u);
  cg.ok = okx && oky && okz;
}
// The pair's entries: f(anchor x, y, z, mask of the corners that the window anchored there holds)
template <class F>
__device__ __forceinline__ void for_entries(const CornerGrid& cg, F f) {
  if (cg.ok) {
#pragma unroll 1
    for (unsigned combo = 0; combo < 8; ++combo) {
      unsigned mask = 0;
#pragma unroll
      for (int c = 0; c < 8; ++c) mask |= (cg.combo[c] == combo) ? (1u << c) : 0u;
      if (mask) f((combo & 1u) ? cg.ax[1] : cg.ax[0], (combo & 2u) ? cg.ay[1] : cg.ay[0],
                  (combo & 4u) ? cg.az[1] : cg.az[0], mask);
    }
  } else {
#pragma unroll
    for (int c = 0; c < 8; ++c) f(cg.ix[c], cg.iy[c], cg.iz[c], 1u << c);
  }
}

}  // namespace issm
