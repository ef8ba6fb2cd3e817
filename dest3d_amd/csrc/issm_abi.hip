// C ABI of libissm_hip.so: argument validation, workspace carving and stage sequencing.
// All device work lives in issm_fwd.hip / issm_bwd.hip / rmsnorm_gated.hip.
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <atomic>
#include <mutex>

#include "../../include/issm.h"
#include "issm_dev.h"

namespace issm {
int launch_chunk_local(const KP& p, float* states, float* cs_last, float* cabt, hipStream_t st);
bool bwd_tile_available(const KP& p, const float* dy_ws);
int launch_state_fwd(const KP& p, float* states, const float* cs_last, hipStream_t st);
int launch_chunk_scan(const KP& p, const float* states, const float* cabt, float* out_x, hipStream_t st);
int launch_bwd_gate(const KP& p, const float* out_x, float* dy_ws, hipStream_t st);
int launch_bwd_dstates(const KP& p, const float* dy_ws, float* dstates, float* dm, hipStream_t st);
int launch_state_bwd(const KP& p, const float* states, const float* cs_last, float* dstates, float* g_last,
                     float* dh0_dir, hipStream_t st);
int launch_bwd_chunk(const KP& p, const float* dy_ws, const float* states, const float* dstates, const float* dm,
                     const float* g_last, float* partA, float* partBias, int* redo, int* redo_pending, hipStream_t st);
int launch_bwd_chunk_redo(const KP& p, int ndirs, const float* dy_ws, const float* states, const float* dstates,
                          const float* dm, const float* g_last, float* partA, float* partBias, const int* redo,
                          hipStream_t st);
int launch_bwd_dx(const KP& p, const float* dy_ws, const float* dstates, const float* cabt, float* partD,
                  hipStream_t st);
int launch_bwd_reduce(const KP& p, const float* partA, const float* partBias, const float* partD,
                      const float* dh0_dir, float* dA, float* dbias, float* dD, float* dh0, hipStream_t st);

int launch_rmsnorm_fwd(const NormP& p, hipStream_t st);
int launch_rmsnorm_bwd(const NormP& p, hipStream_t st);
int launch_hilbert_codes(const HilbertP& p, hipStream_t st);
int launch_hilbert_order(const HilbertOrderP& p, hipStream_t st);
struct TrP {
  int B, R, C, in_dt, out_dt;
  const void* in0;
  const void* in1;
  void* out;
  float alpha;
};
int launch_transpose_states(const TrP& p, hipStream_t st);
int launch_fps(int b, int n, int npoint, const float* xyz, float* temp, int* idxs, hipStream_t st);
int launch_ball_query(int b, int n, int m, float radius, int nsample, const float* new_xyz, const float* xyz, int* idx,
                      hipStream_t st);
int launch_group_points(int b, int c, int n, int ms, const float* points, const int* idx, float* out, hipStream_t st);
int launch_group_points_grad(int b, int c, int n, int ms, const float* grad_out, const int* idx, float* grad_points,
                             hipStream_t st);
int launch_three_nn(int b, int n, int m, const float* unknown, const float* known, float* dist2, int* idx, hipStream_t st);
int launch_three_interpolate(int b, int c, int m, int n, const float* points, const int* idx, const float* weight, float* out,
                             hipStream_t st);
int launch_three_interpolate_grad(int b, int c, int n, int m, const float* grad_out, const int* idx, const float* weight,
                                  float* grad_points, hipStream_t st);
int launch_scatter_channel_last(bool k3, int b, int c, int n, int ne, const float* grad_out, const int* idx,
                                const float* weight, float* out_cl, hipStream_t st);
int box_dist_workgroups(int B, int L, int K);
int box_dist_bwd_workgroups(int B, int L, int K);
long box_dist_bwd_scratch_bytes(int B, int L, int K, int D, int H, int W);
int launch_box_dist_fwd(const BoxDistP& p, hipStream_t st);
int launch_box_dist_bwd(const BoxDistP& p, hipStream_t st);
int dwconv_partial_rows(int B, int L);
int launch_dwconv_fwd(const DwConvP& p, hipStream_t st);
int launch_dwconv_bwd(const DwConvP& p, hipStream_t st);
int pgen_bwd_blocks(long tokens);
int launch_pgen_fwd(const PGenP& p, hipStream_t st);
int launch_pgen_bwd(const PGenP& p, hipStream_t st);
}  // namespace issm

using namespace issm;

static thread_local char g_err[512] = "";

static int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

static TensorD td(const issm_tensor& t) {
  TensorD r;
  r.ptr = t.ptr;
  r.s0 = t.stride[0];
  r.s1 = t.stride[1];
  r.s2 = t.stride[2];
  return r;
}

static size_t align64(size_t nfloats) { return (nfloats + 63) & ~(size_t)63; }

struct FwdWs {
  size_t states, cs_last, cabt, out_x, total;  // offsets in floats
};
struct BwdWs {
  size_t dstates, dm, g_last, dh0_dir, partA, partBias, partD, redo, dy_ws, ddt_part, total;
};

static int nchunks(const issm_dims& d) { return (d.seqlen + ISSM_CHUNK - 1) / ISSM_CHUNK; }

static FwdWs fwd_layout(const issm_dims& d, bool has_z) {
  const size_t Bt = (size_t)d.batch * d.ndir, nc = nchunks(d), H = d.nheads, P = d.headdim, N = d.dstate;
  FwdWs w;
  size_t o = 0;
  w.states = o; o += align64(Bt * (nc + 1) * H * P * N);
  w.cs_last = o; o += align64(Bt * nc * H * N);
  w.cabt = o; o += align64(Bt * nc * H * ISSM_CHUNK * ISSM_CHUNK);
  w.out_x = o; if (has_z) o += align64(Bt * d.seqlen * H * P);
  w.total = o;
  return w;
}

// ddt_part: with two directions and a bf16 ddt, the first direction's share of ddt in fp32 ((B, L, H, N))
static BwdWs bwd_layout(const issm_dims& d, bool has_z, bool ddt_part) {
  const size_t Bt = (size_t)d.batch * d.ndir, nc = nchunks(d), H = d.nheads, P = d.headdim, N = d.dstate;
  BwdWs w;
  size_t o = 0;
  w.dstates = o; o += align64(Bt * nc * H * P * N);
  w.dm = o; o += align64(Bt * nc * H * ISSM_CHUNK * ISSM_CHUNK);
  w.g_last = o; o += align64(Bt * nc * H * N);
  w.dh0_dir = o; o += align64((size_t)d.ndir * d.batch * H * P * N);
  w.partA = o; o += align64(Bt * nc * H * N);
  w.partBias = o; o += align64(Bt * nc * H * N);
  w.partD = o; o += align64(Bt * nc * H * P);
  w.redo = o; o += align64(Bt * nc * H * ((N + ISSM_CHUNK - 1) / ISSM_CHUNK));  // one int per direction, workgroup and head
  w.dy_ws = o; if (has_z) o += align64(Bt * d.seqlen * H * P);
  w.ddt_part = o; if (ddt_part) o += align64((size_t)d.batch * d.seqlen * H * N);
  w.total = o;
  return w;
}
static bool wants_ddt_part(const issm_scan_args* a) { return a->dims.ndir == 2 && a->dt_dtype == ISSM_BF16; }

static int check_dims(const issm_scan_args* a) {
  if (!a) return fail(ISSM_E_NULL, "args is NULL");
  const issm_dims& d = a->dims;
  if (d.batch <= 0 || d.seqlen <= 0 || d.nheads <= 0 || d.headdim <= 0 || d.dstate <= 0 || d.ngroups <= 0)
    return fail(ISSM_E_SHAPE, "non-positive dimension (B=%d L=%d H=%d P=%d N=%d G=%d)", d.batch, d.seqlen, d.nheads,
                d.headdim, d.dstate, d.ngroups);
  if (d.chunk_size <= 0) return fail(ISSM_E_SHAPE, "chunk_size must be positive, got %d", d.chunk_size);
  if (d.nheads % d.ngroups) return fail(ISSM_E_SHAPE, "nheads %d not divisible by ngroups %d", d.nheads, d.ngroups);
  if (d.ndir != 1 && d.ndir != 2) return fail(ISSM_E_SHAPE, "ndir must be 1 or 2, got %d", d.ndir);
  if (d.headdim > MAXP) return fail(ISSM_E_UNSUPPORTED, "headdim %d > %d is not built", d.headdim, MAXP);
  if ((long)d.batch * d.ndir * nchunks(d) * d.nheads > 0x7fffffffL) return fail(ISSM_E_SHAPE, "too many chunk units");
  return ISSM_OK;
}

static int check_strides(const issm_scan_args* a);

static int check_common(const issm_scan_args* a) {
  int rc = check_dims(a);
  if (rc) return rc;
  if ((unsigned)a->io_dtype > 1u || (unsigned)a->dt_dtype > 1u || (unsigned)a->h0_dtype > 1u)
    return fail(ISSM_E_DTYPE, "unknown dtype code (io=%d dt=%d h0=%d)", a->io_dtype, a->dt_dtype, a->h0_dtype);
  if (a->flags & ISSM_FLAG_SEQ_IDX) {
    if (!a->seq_idx) return fail(ISSM_E_NULL, "ISSM_FLAG_SEQ_IDX is set and seq_idx is NULL");
    if (a->dims.ndir != 1) return fail(ISSM_E_UNSUPPORTED, "seq_idx with ndir = %d (one direction only)", a->dims.ndir);
    if (a->seq_idx_stride[0] < 0 || a->seq_idx_stride[1] < 0 ||
        a->seq_idx_stride[1] * (int64_t)a->dims.seqlen >= ((int64_t)1 << 31))
      return fail(ISSM_E_STRIDE, "seq_idx strides (%lld, %lld)", (long long)a->seq_idx_stride[0], (long long)a->seq_idx_stride[1]);
  }
  if (!(a->dt_min >= 0.0f)) return fail(ISSM_E_UNSUPPORTED, "dt_limit[0] = %g < 0 is not supported", a->dt_min);
  if (!(a->dt_max >= a->dt_min)) return fail(ISSM_E_SHAPE, "dt_limit is empty (%g, %g)", a->dt_min, a->dt_max);
  if (!a->A) return fail(ISSM_E_NULL, "A is NULL");
  if (!a->dt.ptr) return fail(ISSM_E_NULL, "dt is NULL");
  for (int dir = 0; dir < a->dims.ndir; ++dir) {
    if (!a->x[dir].ptr || !a->Bm[dir].ptr || !a->Cm[dir].ptr)
      return fail(ISSM_E_NULL, "x/B/C of direction %d is NULL", dir);
    if ((a->z[0].ptr != nullptr) != (a->z[dir].ptr != nullptr))
      return fail(ISSM_E_NULL, "z must be given for all directions or none");
  }
  return check_strides(a);
}

// The kernels address a row of a caller tensor as a 64-bit (batch, head) base plus a 32-bit BYTE
// offset (time row * stride[1] + column) * element size: that offset must fit (2^30 elements), and
// strides may not be negative.
static int check_td(const issm_tensor& t, const char* name, int dir, long rows, long inner) {
  if (!t.ptr) return ISSM_OK;
  for (int i = 0; i < 3; ++i)
    if (t.stride[i] < 0) return fail(ISSM_E_STRIDE, "%s[%d]: negative stride %ld", name, dir, (long)t.stride[i]);
  if ((rows - 1) * (long)t.stride[1] + inner > 0x3fffffffL)
    return fail(ISSM_E_STRIDE, "%s[%d]: seqlen * stride[1] = %ld * %ld exceeds the 32-bit row offset range", name, dir,
                rows, (long)t.stride[1]);
  return ISSM_OK;
}

static int check_strides(const issm_scan_args* a) {
  const issm_dims& d = a->dims;
  int rc;
  for (int i = 0; i < d.ndir; ++i) {
    if ((rc = check_td(a->x[i], "x", i, d.seqlen, d.headdim))) return rc;
    if ((rc = check_td(a->z[i], "z", i, d.seqlen, d.headdim))) return rc;
    if ((rc = check_td(a->out[i], "out", i, d.seqlen, d.headdim))) return rc;
    if ((rc = check_td(a->dout[i], "dout", i, d.seqlen, d.headdim))) return rc;
    if ((rc = check_td(a->dx[i], "dx", i, d.seqlen, d.headdim))) return rc;
    if ((rc = check_td(a->dz[i], "dz", i, d.seqlen, d.headdim))) return rc;
    if ((rc = check_td(a->Bm[i], "B", i, d.seqlen, d.dstate))) return rc;
    if ((rc = check_td(a->Cm[i], "C", i, d.seqlen, d.dstate))) return rc;
    if ((rc = check_td(a->dB[i], "dB", i, d.seqlen, d.dstate))) return rc;
    if ((rc = check_td(a->dC[i], "dC", i, d.seqlen, d.dstate))) return rc;
  }
  if ((rc = check_td(a->dt, "dt", 0, d.seqlen, d.dstate))) return rc;
  if ((rc = check_td(a->ddt, "ddt", 0, d.seqlen, d.dstate))) return rc;
  if ((rc = check_td(a->h0, "initial_states", 0, d.nheads, d.dstate))) return rc;
  return ISSM_OK;
}

static KP make_kp(const issm_scan_args* a) {
  KP p;
  memset(&p, 0, sizeof(p));
  const issm_dims& d = a->dims;
  p.B = d.batch; p.L = d.seqlen; p.H = d.nheads; p.P = d.headdim; p.N = d.dstate; p.G = d.ngroups;
  p.ndir = d.ndir; p.nc = nchunks(d); p.hpg = d.nheads / d.ngroups; p.dir0 = 0;
  p.io_dt = a->io_dtype; p.dt_dt = a->dt_dtype; p.h0_dt = a->h0_dtype;
  p.flags = ((a->flags & ISSM_FLAG_DT_SOFTPLUS) ? F_SOFTPLUS : 0u) | ((a->flags & ISSM_FLAG_D_HAS_HDIM) ? F_D_HDIM : 0u);
  p.dt_min = a->dt_min; p.dt_max = a->dt_max;
  // softplus is positive: limits of (<= 0, >= 3e38 or inf) cannot act on it
  if ((p.flags & F_SOFTPLUS) && a->dt_min <= 0.0f && a->dt_max >= 3.0e38f) p.flags |= F_NOCLAMP;
  for (int i = 0; i < 2; ++i) {
    p.x[i] = td(a->x[i]); p.Bm[i] = td(a->Bm[i]); p.Cm[i] = td(a->Cm[i]); p.z[i] = td(a->z[i]);
    p.out[i] = td(a->out[i]); p.dout[i] = td(a->dout[i]); p.dx[i] = td(a->dx[i]); p.dB[i] = td(a->dB[i]);
    p.dC[i] = td(a->dC[i]); p.dz[i] = td(a->dz[i]);
    p.final_states[i] = a->final_states[i];
    p.dfinal[i] = a->dfinal[i];
  }
  p.dt = td(a->dt); p.ddt = td(a->ddt); p.h0 = td(a->h0);
  p.A = a->A; p.D = a->D; p.dt_bias = a->dt_bias;
  if (a->flags & ISSM_FLAG_SEQ_IDX) {
    p.seq_idx = a->seq_idx; p.seq_s0 = a->seq_idx_stride[0]; p.seq_s1 = a->seq_idx_stride[1];
  }
  p.c_lo = 0; p.ncl = p.nc;
  if (p.N % 64 == 0 && !p.seq_idx) p.full_tiles = p.L % ISSM_CHUNK == 0 ? 1 : (p.nc > 1 ? 2 : 0);
  return p;
}

static int launched(int hip_err, const char* what) {
  if (hip_err == 0) return ISSM_OK;
  return fail(ISSM_E_LAUNCH, "%s: %s", what, hipGetErrorString((hipError_t)hip_err));
}

static void norm_scratch_warm(hipStream_t stream);  // further down, with the allocation-free backward it serves

extern "C" {

int issm_abi_version(void) { return ISSM_ABI_VERSION; }
const char* issm_last_error(void) { return g_err; }

int issm_fwd_workspace_bytes(const issm_scan_args* a, size_t* out) {
  int rc = check_dims(a);
  if (rc) return rc;
  if (!out) return fail(ISSM_E_NULL, "out is NULL");
  *out = fwd_layout(a->dims, a->z[0].ptr != nullptr).total * sizeof(float);
  return ISSM_OK;
}

int issm_bwd_workspace_bytes(const issm_scan_args* a, size_t* out) {
  int rc = check_dims(a);
  if (rc) return rc;
  if (!out) return fail(ISSM_E_NULL, "out is NULL");
  *out = bwd_layout(a->dims, a->z[0].ptr != nullptr, wants_ddt_part(a)).total * sizeof(float);
  return ISSM_OK;
}

int issm_stage_chunk_local(const issm_scan_args* a, float* states, float* cs_last, float* cabt) {
  int rc = check_common(a);
  if (rc) return rc;
  if (!cs_last) return fail(ISSM_E_NULL, "cs_last is NULL");
  KP p = make_kp(a);
  return launched(launch_chunk_local(p, states, cs_last, cabt, (hipStream_t)a->stream), "chunk_local");
}

int issm_stage_state_passing_fwd(const issm_scan_args* a, float* states, const float* cs_last) {
  int rc = check_dims(a);
  if (rc) return rc;
  if (!states || !cs_last) return fail(ISSM_E_NULL, "states/cs_last is NULL");
  KP p = make_kp(a);
  return launched(launch_state_fwd(p, states, cs_last, (hipStream_t)a->stream), "state_passing_fwd");
}

int issm_stage_chunk_scan(const issm_scan_args* a, const float* states, const float* cabt, float* out_x) {
  int rc = check_common(a);
  if (rc) return rc;
  if (!states || !cabt) return fail(ISSM_E_NULL, "states/cabt is NULL");
  for (int dir = 0; dir < a->dims.ndir; ++dir)
    if (!a->out[dir].ptr) return fail(ISSM_E_NULL, "out of direction %d is NULL", dir);
  if (a->z[0].ptr && !out_x) return fail(ISSM_E_NULL, "out_x is required when z is given");
  KP p = make_kp(a);
  return launched(launch_chunk_scan(p, states, cabt, out_x, (hipStream_t)a->stream), "chunk_scan");
}

int issm_scan_fwd(const issm_scan_args* a) {
  int rc = check_common(a);
  if (rc) return rc;
  const bool has_z = a->z[0].ptr != nullptr;
  const FwdWs w = fwd_layout(a->dims, has_z);
  if (!a->workspace || a->workspace_bytes < w.total * sizeof(float))
    return fail(ISSM_E_WORKSPACE, "forward workspace: need %zu bytes, got %zu", w.total * sizeof(float),
                a->workspace ? a->workspace_bytes : (size_t)0);
  for (int dir = 0; dir < a->dims.ndir; ++dir)
    if (!a->out[dir].ptr) return fail(ISSM_E_NULL, "out of direction %d is NULL", dir);
  float* ws = (float*)a->workspace;
  KP p = make_kp(a);
  hipStream_t st = (hipStream_t)a->stream;
  if ((rc = launched(launch_chunk_local(p, ws + w.states, ws + w.cs_last, ws + w.cabt, st), "chunk_local"))) return rc;
  if ((rc = launched(launch_state_fwd(p, ws + w.states, ws + w.cs_last, st), "state_passing_fwd"))) return rc;
  return launched(launch_chunk_scan(p, ws + w.states, ws + w.cabt, has_z ? ws + w.out_x : nullptr, st), "chunk_scan");
}

int issm_stage_bwd_gate(const issm_scan_args* a, const float* out_x, float* dy_gated) {
  int rc = check_common(a);
  if (rc) return rc;
  if (!out_x || !dy_gated || !a->z[0].ptr) return fail(ISSM_E_NULL, "out_x/dy_gated/z is NULL");
  KP p = make_kp(a);
  return launched(launch_bwd_gate(p, out_x, dy_gated, (hipStream_t)a->stream), "bwd_gate");
}

static int check_dout(const issm_scan_args* a, const float* dy_gated) {
  if (dy_gated) return ISSM_OK;
  for (int dir = 0; dir < a->dims.ndir; ++dir)
    if (!a->dout[dir].ptr) return fail(ISSM_E_NULL, "dout of direction %d is NULL", dir);
  return ISSM_OK;
}

int issm_stage_bwd_dstates(const issm_scan_args* a, const float* dy_gated, float* dstates, float* dm) {
  int rc = check_common(a);
  if (rc) return rc;
  if ((rc = check_dout(a, dy_gated))) return rc;
  KP p = make_kp(a);
  return launched(launch_bwd_dstates(p, dy_gated, dstates, dm, (hipStream_t)a->stream), "bwd_dstates");
}

int issm_stage_state_passing_bwd(const issm_scan_args* a, const float* states, const float* cs_last, float* dstates,
                                 float* g_last, float* dh0_dir) {
  int rc = check_dims(a);
  if (rc) return rc;
  if (!states || !cs_last || !dstates || !g_last || !dh0_dir) return fail(ISSM_E_NULL, "state_passing_bwd: NULL buffer");
  KP p = make_kp(a);
  return launched(launch_state_bwd(p, states, cs_last, dstates, g_last, dh0_dir, (hipStream_t)a->stream),
                  "state_passing_bwd");
}

size_t issm_bwd_chunk_redo_ints(const issm_scan_args* a) {
  if (check_dims(a)) return 0;
  const issm_dims& d = a->dims;
  return (size_t)d.batch * d.ndir * nchunks(d) * d.nheads * ((d.dstate + ISSM_CHUNK - 1) / ISSM_CHUNK);
}

int issm_stage_bwd_chunk(const issm_scan_args* a, int dir, const float* dy_gated, const float* states,
                         const float* dstates, const float* dm, const float* g_last, float* part_a,
                         float* part_bias, int32_t* redo) {
  int rc = check_common(a);
  if (rc) return rc;
  if ((rc = check_dout(a, dy_gated))) return rc;
  if (dir < 0 || dir >= a->dims.ndir) return fail(ISSM_E_SHAPE, "dir %d out of range", dir);
  if (!states || !dstates || !dm || !g_last || !part_a || !part_bias) return fail(ISSM_E_NULL, "bwd_chunk: NULL buffer");
  KP p = make_kp(a);
  p.dir0 = dir;
  int pending = 0;
  if ((rc = launched(launch_bwd_chunk(p, dy_gated, states, dstates, dm, g_last, part_a, part_bias, redo, &pending,
                                      (hipStream_t)a->stream),
                     "bwd_chunk")))
    return rc;
  if (!pending) return ISSM_OK;
  return launched(launch_bwd_chunk_redo(p, 1, dy_gated, states, dstates, dm, g_last, part_a, part_bias, redo,
                                        (hipStream_t)a->stream),
                  "bwd_chunk (redo)");
}

int issm_stage_bwd_dx(const issm_scan_args* a, const float* dy_gated, const float* dstates, const float* cabt,
                      float* part_d) {
  int rc = check_common(a);
  if (rc) return rc;
  if ((rc = check_dout(a, dy_gated))) return rc;
  if (!dstates || !cabt) return fail(ISSM_E_NULL, "bwd_dx: NULL buffer");
  if (a->D && a->dD && !part_d) return fail(ISSM_E_NULL, "bwd_dx: part_d is NULL");
  KP p = make_kp(a);
  return launched(launch_bwd_dx(p, dy_gated, dstates, cabt, part_d, (hipStream_t)a->stream), "bwd_dx");
}

int issm_stage_bwd_reduce(const issm_scan_args* a, const float* part_a, const float* part_bias, const float* part_d,
                          const float* dh0_dir) {
  int rc = check_dims(a);
  if (rc) return rc;
  KP p = make_kp(a);
  return launched(launch_bwd_reduce(p, part_a, part_bias, part_d, dh0_dir, part_a ? a->dA : nullptr,
                                    (part_bias && a->dt_bias) ? a->ddt_bias : nullptr,
                                    (part_d && a->D) ? a->dD : nullptr, dh0_dir ? a->dh0 : nullptr,
                                    (hipStream_t)a->stream),
                  "bwd_reduce");
}

int issm_scan_bwd(const issm_scan_args* a) {
  int rc = check_common(a);
  if (rc) return rc;
  const bool has_z = a->z[0].ptr != nullptr;
  const FwdWs fw = fwd_layout(a->dims, has_z);
  const BwdWs bw = bwd_layout(a->dims, has_z, wants_ddt_part(a));
  if (!a->saved) return fail(ISSM_E_WORKSPACE, "saved forward workspace is NULL");
  if (!a->bwd_workspace || a->bwd_workspace_bytes < bw.total * sizeof(float))
    return fail(ISSM_E_WORKSPACE, "backward workspace: need %zu bytes, got %zu", bw.total * sizeof(float),
                a->bwd_workspace ? a->bwd_workspace_bytes : (size_t)0);
  for (int dir = 0; dir < a->dims.ndir; ++dir)
    if (!a->dout[dir].ptr) return fail(ISSM_E_NULL, "dout of direction %d is NULL", dir);
  const float* sv = (const float*)a->saved;
  float* ws = (float*)a->bwd_workspace;
  KP p = make_kp(a);
  hipStream_t st = (hipStream_t)a->stream;
  const float* dy = nullptr;
  if (has_z) {
    if ((rc = launched(launch_bwd_gate(p, sv + fw.out_x, ws + bw.dy_ws, st), "bwd_gate"))) return rc;
    dy = ws + bw.dy_ws;
  }
  if ((rc = launched(launch_bwd_dstates(p, dy, ws + bw.dstates, ws + bw.dm, st), "bwd_dstates"))) return rc;
  if ((rc = launched(launch_state_bwd(p, sv + fw.states, sv + fw.cs_last, ws + bw.dstates, ws + bw.g_last,
                                      ws + bw.dh0_dir, st),
                     "state_passing_bwd")))
    return rc;
  int* redo = reinterpret_cast<int*>(ws + bw.redo);
  int pending = 0;
  KP pc = p;
  if (wants_ddt_part(a) && bwd_tile_available(p, dy)) {
    // both directions go through the tile-base kernel: the first one's share of the bf16 ddt travels in fp32
    pc.ddt_part.ptr = ws + bw.ddt_part;
    pc.ddt_part.s2 = p.N;
    pc.ddt_part.s1 = (long)p.H * p.N;
    pc.ddt_part.s0 = (long)p.L * p.H * p.N;
  }
  for (int dir = 0; dir < p.ndir; ++dir) {
    KP pd = pc;
    pd.dir0 = dir;
    if ((rc = launched(launch_bwd_chunk(pd, dy, sv + fw.states, ws + bw.dstates, ws + bw.dm, ws + bw.g_last,
                                        ws + bw.partA, ws + bw.partBias, redo, &pending, st),
                       "bwd_chunk")))
      return rc;
  }
  if (pending &&
      (rc = launched(launch_bwd_chunk_redo(p, p.ndir, dy, sv + fw.states, ws + bw.dstates, ws + bw.dm, ws + bw.g_last,
                                           ws + bw.partA, ws + bw.partBias, redo, st),
                     "bwd_chunk (redo)")))
    return rc;
  if ((rc = launched(launch_bwd_dx(p, dy, ws + bw.dstates, sv + fw.cabt, ws + bw.partD, st), "bwd_dx"))) return rc;
  return launched(launch_bwd_reduce(p, ws + bw.partA, ws + bw.partBias, ws + bw.partD, ws + bw.dh0_dir, a->dA,
                                    a->dt_bias ? a->ddt_bias : nullptr, a->D ? a->dD : nullptr, a->dh0, st),
                  "bwd_reduce");
}

// ------------------------------------------------------------------ gated RMSNorm
int issm_rmsnorm_bwd_blocks(int64_t rows) {
  if (rows <= 0) return 0;
  return (int)(rows < 2048 ? rows : 2048);
}

static int norm_params(const issm_norm_args* a, NormP* p, bool bwd) {
  if (!a) return fail(ISSM_E_NULL, "args is NULL");
  if (a->rows <= 0 || a->ncols <= 0) return fail(ISSM_E_SHAPE, "rmsnorm: rows=%lld ncols=%d", (long long)a->rows, a->ncols);
  const int gs = a->group_size > 0 ? a->group_size : a->ncols;
  if (a->ncols % gs) return fail(ISSM_E_SHAPE, "rmsnorm: ncols %d not divisible by group_size %d", a->ncols, gs);
  if ((unsigned)a->dtype > 1u || (unsigned)a->weight_dtype > 1u) return fail(ISSM_E_DTYPE, "rmsnorm: unknown dtype");
  if (!a->x || !a->w || !a->rstd) return fail(ISSM_E_NULL, "rmsnorm: x/w/rstd is NULL");
  if (a->ncols > 16384) return fail(ISSM_E_UNSUPPORTED, "rmsnorm: ncols %d > 16384", a->ncols);
  if (!bwd && !a->y) return fail(ISSM_E_NULL, "rmsnorm: y is NULL");
  if (bwd && (!a->dy || !a->dx || !a->dw_partial || !a->dw)) return fail(ISSM_E_NULL, "rmsnorm bwd: NULL buffer");
  if (bwd && a->z && !a->dz) return fail(ISSM_E_NULL, "rmsnorm bwd: dz is NULL");
  if (a->layer_norm && !a->mean) return fail(ISSM_E_NULL, "layernorm: mean is NULL");
  if (bwd && a->bias && (!a->db_partial || !a->db)) return fail(ISSM_E_NULL, "norm bwd with bias: db_partial/db is NULL");
  // only the backward stages the bias partial sums next to the weight's in LDS; the forward has no such limit
  if (bwd && a->bias && a->ncols > 8192 && !(a->ncols / gs == 1 && (a->ncols & 3) == 0 && a->ncols <= 1024))
    return fail(ISSM_E_UNSUPPORTED, "norm bwd with bias: ncols %d > 8192", a->ncols);
  p->rows = a->rows; p->ncols = a->ncols; p->gs = gs; p->ngroups = a->ncols / gs;
  p->dt = a->dtype; p->wdt = a->weight_dtype; p->nbg = a->norm_before_gate; p->eps = a->eps;
  p->x = a->x; p->z = a->z; p->w = a->w; p->xs = a->x_row_stride; p->zs = a->z_row_stride;
  p->y = a->y; p->ys = a->y_row_stride; p->rstd = a->rstd;
  p->dy = a->dy; p->dys = a->dy_row_stride; p->dx = a->dx; p->dz = a->dz; p->dxs = a->dx_row_stride;
  p->dzs = a->dz_row_stride; p->dw_partial = a->dw_partial; p->dw = a->dw;
  p->nblocks = issm_rmsnorm_bwd_blocks(a->rows);
  p->ln = a->layer_norm ? 1 : 0; p->b = a->bias; p->mean = a->mean; p->db_partial = a->db_partial; p->db = a->db;
  return ISSM_OK;
}

int issm_gated_rmsnorm_fwd(const issm_norm_args* a) {
  NormP p;
  int rc = norm_params(a, &p, false);
  if (rc) return rc;
  norm_scratch_warm((hipStream_t)a->stream);
  return launched(launch_rmsnorm_fwd(p, (hipStream_t)a->stream), "rmsnorm_fwd");
}

int issm_gated_rmsnorm_bwd(const issm_norm_args* a) {
  NormP p;
  int rc = norm_params(a, &p, true);
  if (rc) return rc;
  norm_scratch_warm((hipStream_t)a->stream);
  return launched(launch_rmsnorm_bwd(p, (hipStream_t)a->stream), "rmsnorm_bwd");
}

}  // extern "C"

// ---- the same backward on a scratch buffer that belongs to the library: no allocation by anyone
// The per-block partial sums of dw (nblocks x ncols floats) normally arrive as args->dw_partial.  For callers that
// cannot allocate, they go into this array instead; every GPU the library runs on holds its own copy (8 MiB) at
// its own address until the process ends.  In host code the array's name is only a handle for
// hipGetSymbolAddress: the device address is looked up once per device and kept, and it is that pointer -- never
// the name -- that the kernels receive.  (No `used` attribute on the array: the compiler gives a file-scope device
// variable that host code refers to an external symbol, which is what the runtime's lookup needs; `used` keeps it local
// and the lookup then aborts the process.)
static __device__ __align__(256) float g_norm_scratch[ISSM_NORM_SCRATCH_FLOATS];
static constexpr int kMaxDevices = 64;
static std::mutex g_norm_scratch_mutex;
static float* g_norm_scratch_ptr[kMaxDevices];  // [device]: address of that device's copy, once looked up
static std::atomic<bool> g_norm_scratch_known[kMaxDevices];  // set after the pointer: a cheap test for norm_scratch_warm

// The look-up may load the code object and so must not run while `stream` records a graph: a first call on a device
// that arrives under capture is refused (one eager call per device, of this entry point or of any other of the
// library's normalisation calls, comes first -- those resolve the address on the way, see norm_scratch_warm).
static int norm_scratch_ptr(float** out, hipStream_t stream) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(ISSM_E_LAUNCH, "hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return fail(ISSM_E_UNSUPPORTED, "device index %d outside 0..%d", dev, kMaxDevices - 1);
  std::lock_guard<std::mutex> lock(g_norm_scratch_mutex);
  if (!g_norm_scratch_ptr[dev]) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone)
      return fail(ISSM_E_UNSUPPORTED,
                  "rmsnorm bwd without allocation: the first call on device %d came while its stream records a graph; "
                  "make one eager call of a normalisation entry point on this device before the capture", dev);
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_norm_scratch));  // of the current device's copy
    if (e != hipSuccess || !ptr)
      return fail(ISSM_E_LAUNCH, "hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
    g_norm_scratch_ptr[dev] = (float*)ptr;
    g_norm_scratch_known[dev].store(true, std::memory_order_release);
  }
  *out = g_norm_scratch_ptr[dev];
  return ISSM_OK;
}
// Called by the other normalisation entry points: resolves the current device's address when that is possible now
// (not under capture), silently otherwise, so that a model whose forward ran eagerly once can capture the
// allocation-free backward without a warm-up call of its own.
static void norm_scratch_warm(hipStream_t stream) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    (void)hipGetLastError();
    return;
  }
  if (g_norm_scratch_known[dev].load(std::memory_order_acquire)) return;
  float* unused = nullptr;
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) {
    (void)hipGetLastError();
    return;
  }
  if (norm_scratch_ptr(&unused, stream) != ISSM_OK) g_err[0] = 0;
}

extern "C" {

int issm_gated_rmsnorm_bwd_noalloc(const issm_norm_args* a) {
  if (!a) return fail(ISSM_E_NULL, "args is NULL");
  issm_norm_args b = *a;
  float* scratch = nullptr;
  // sizes are checked before anything touches the device
  const int64_t part = b.rows > 0 && b.ncols > 0 ? (int64_t)issm_rmsnorm_bwd_blocks(b.rows) * b.ncols : 0;
  const int64_t need = part * (b.bias ? 2 : 1);  // the partial sums of dw, then those of db
  if (need > (int64_t)ISSM_NORM_SCRATCH_FLOATS)
    return fail(ISSM_E_WORKSPACE,
                "rmsnorm bwd without allocation: %d row blocks x %d columns%s = %lld floats of partial sums exceed the "
                "library's %d-float scratch array; use issm_gated_rmsnorm_bwd with a dw_partial buffer",
                issm_rmsnorm_bwd_blocks(b.rows), b.ncols, b.bias ? " x 2 (weight and bias)" : "", (long long)need,
                (int)ISSM_NORM_SCRATCH_FLOATS);
  // placeholders so that the shared validation sees buffers; replaced below
  b.dw_partial = (float*)(uintptr_t)256;
  b.db_partial = (float*)(uintptr_t)256;
  NormP p;
  int rc = norm_params(&b, &p, true);
  if (rc) return rc;
  if ((rc = norm_scratch_ptr(&scratch, (hipStream_t)a->stream))) return rc;
  p.dw_partial = scratch;  // every launched block writes its whole row of partials before the sum reads it
  p.db_partial = scratch + part;
  return launched(launch_rmsnorm_bwd(p, (hipStream_t)a->stream), "rmsnorm_bwd_noalloc");
}

static int pgen_params(const issm_pgen_args* a, PGenP* p, bool bwd) {
  if (!a) return fail(ISSM_E_NULL, "param_gen: args is NULL");
  if (a->tokens < 0 || a->K < 0 || a->H < 1 || a->G < 1) return fail(ISSM_E_SHAPE, "param_gen: bad shape");
  if (a->M != 16) return fail(ISSM_E_UNSUPPORTED, "param_gen: M = %d (only 16 is built)", a->M);
  if (a->H + 2 * a->G > 12) return fail(ISSM_E_UNSUPPORTED, "param_gen: H + 2G = %d > 12", a->H + 2 * a->G);
  if (a->dtype != ISSM_F32 && a->dtype != ISSM_BF16) return fail(ISSM_E_DTYPE, "param_gen: dtype %d", a->dtype);
  if (a->tokens * (int64_t)a->K * 16 >= ((int64_t)1 << 40)) return fail(ISSM_E_SHAPE, "param_gen: too large");
  if (!a->dist || !a->W) return fail(ISSM_E_NULL, "param_gen: dist/W is NULL");
  if (a->weights && !a->dt_raw) return fail(ISSM_E_NULL, "param_gen: weights given but dt_raw is NULL");
  if (!bwd) {
    if (!a->bias || !a->dt || !a->Bm || !a->Cm) return fail(ISSM_E_NULL, "param_gen: bias/dt/Bm/Cm is NULL");
    if (a->has_back && (!a->Bm_back || !a->Cm_back)) return fail(ISSM_E_NULL, "param_gen: Bm_back/Cm_back is NULL");
  } else {
    if (!a->dw_partial || !a->dW) return fail(ISSM_E_NULL, "param_gen bwd: dw_partial/dW is NULL");
  }
  p->tokens = a->tokens; p->K = a->K; p->H = a->H; p->G = a->G; p->dtype = a->dtype; p->has_back = a->has_back ? 1 : 0;
  p->dist = a->dist; p->W = a->W; p->bias = a->bias;
  p->dt = a->dt; p->Bm = a->Bm; p->Cm = a->Cm; p->Bb = a->Bm_back; p->Cb = a->Cm_back;
  p->ddt = a->ddt; p->dB = a->dBm; p->dC = a->dCm; p->dBb = a->dBm_back; p->dCb = a->dCm_back;
  p->weights = a->weights; p->dt_raw = a->dt_raw; p->dweights = a->weights ? a->dweights : nullptr;
  if (a->dbias_sum && !a->dbias) return fail(ISSM_E_NULL, "param_gen: dbias_sum needs dbias");
  p->dbias_sum = a->dbias_sum;
  p->ddist = a->ddist; p->dbias = a->dbias; p->dw_partial = a->dw_partial; p->dW = a->dW;
  p->nblocks = pgen_bwd_blocks(a->tokens);
  return ISSM_OK;
}

int issm_param_gen_bwd_blocks(int64_t tokens) { return tokens > 0 ? pgen_bwd_blocks(tokens) : 0; }

int issm_param_gen_fwd(const issm_pgen_args* a) {
  PGenP p;
  int rc = pgen_params(a, &p, false);
  if (rc) return rc;
  if (p.tokens == 0 || p.K == 0) return ISSM_OK;
  return launched(launch_pgen_fwd(p, (hipStream_t)a->stream), "param_gen_fwd");
}

int issm_param_gen_bwd(const issm_pgen_args* a) {
  PGenP p;
  int rc = pgen_params(a, &p, true);
  if (rc) return rc;
  if (p.tokens == 0) return ISSM_OK;
  return launched(launch_pgen_bwd(p, (hipStream_t)a->stream), "param_gen_bwd");
}

static int dwconv_params(const issm_dwconv_args* a, DwConvP* p, bool bwd) {
  if (!a) return fail(ISSM_E_NULL, "dwconv: args is NULL");
  if (a->batch < 0 || a->seqlen < 0 || a->channels < 1) return fail(ISSM_E_SHAPE, "dwconv: bad shape");
  if (a->taps != 7) return fail(ISSM_E_UNSUPPORTED, "dwconv: %d taps (only 7 is built)", a->taps);
  if (a->nsets < 1 || a->nsets > 2) return fail(ISSM_E_UNSUPPORTED, "dwconv: nsets = %d (1 or 2)", a->nsets);
  if (a->chain && a->nsets != 2) return fail(ISSM_E_SHAPE, "dwconv: chain needs nsets = 2, got %d", a->nsets);
  if (a->dtype != ISSM_F32 && a->dtype != ISSM_BF16) return fail(ISSM_E_DTYPE, "dwconv: dtype %d", a->dtype);
  if (!a->u || !a->w || !a->pre) return fail(ISSM_E_NULL, "dwconv: u/w/pre is NULL");
  if (a->u_token_stride < a->channels || a->u_batch_stride < 0)
    return fail(ISSM_E_STRIDE, "dwconv: u strides (%lld, %lld)", (long long)a->u_batch_stride, (long long)a->u_token_stride);
  if (!bwd && (!a->bias || !a->y)) return fail(ISSM_E_NULL, "dwconv: bias/y is NULL");
  if (bwd && (!a->partial || !a->dw || !a->dbias)) return fail(ISSM_E_NULL, "dwconv bwd: partial/dw/dbias is NULL");
  p->B = a->batch; p->L = a->seqlen; p->C = a->channels; p->nsets = a->nsets; p->dtype = a->dtype;
  p->chain = a->chain ? 1 : 0;
  p->u = a->u; p->u_bs = a->u_batch_stride; p->u_ls = a->u_token_stride;
  if (a->split < 0 || a->split >= a->channels) return fail(ISSM_E_SHAPE, "dwconv: split %d outside [0, channels)", a->split);
  if (a->split > 0 && !bwd && !a->y_tail) return fail(ISSM_E_NULL, "dwconv: y_tail is NULL");
  p->split = a->split; p->y_tail = a->y_tail;
  p->dy_tail[0] = a->dy_tail[0]; p->dy_tail[1] = a->nsets > 1 ? a->dy_tail[1] : nullptr;
  p->w = a->w; p->bias = a->bias; p->y = a->y; p->pre = a->pre;
  p->dy[0] = a->dy[0]; p->dy[1] = a->nsets > 1 ? a->dy[1] : nullptr;
  if ((a->du_batch_stride || a->du_token_stride) && (a->du_token_stride < a->channels || a->du_batch_stride < 0))
    return fail(ISSM_E_STRIDE, "dwconv: du strides (%lld, %lld)", (long long)a->du_batch_stride, (long long)a->du_token_stride);
  p->du = a->du; p->partial = a->partial; p->nrows = dwconv_partial_rows(a->batch, a->seqlen);
  p->du_ls = a->du_token_stride ? a->du_token_stride : a->channels;
  p->du_bs = a->du_token_stride ? a->du_batch_stride : (long)a->seqlen * a->channels;
  p->dw = a->dw; p->dbias = a->dbias;
  return ISSM_OK;
}

int issm_dwconv_partial_rows(int32_t batch, int32_t seqlen) {
  return (batch > 0 && seqlen > 0) ? dwconv_partial_rows(batch, seqlen) : 0;
}

int issm_dwconv_silu_fwd(const issm_dwconv_args* a) {
  DwConvP p;
  int rc = dwconv_params(a, &p, false);
  if (rc) return rc;
  if (p.B == 0 || p.L == 0) return ISSM_OK;
  return launched(launch_dwconv_fwd(p, (hipStream_t)a->stream), "dwconv_silu_fwd");
}

int issm_dwconv_silu_bwd(const issm_dwconv_args* a) {
  DwConvP p;
  int rc = dwconv_params(a, &p, true);
  if (rc) return rc;
  return launched(launch_dwconv_bwd(p, (hipStream_t)a->stream), "dwconv_silu_bwd");
}

static int box_dist_params(const issm_box_dist_args* a, BoxDistP* p, bool bwd) {
  if (!a) return fail(ISSM_E_NULL, "box_dist: args is NULL");
  if (a->batch < 0 || a->seqlen < 0 || a->nquery < 0 || a->D < 1 || a->H < 1 || a->W < 1)
    return fail(ISSM_E_SHAPE, "box_dist: bad shape");
  if ((int64_t)a->D * a->H * a->W > 1024)
    return fail(ISSM_E_UNSUPPORTED, "box_dist: table of %d x %d x %d nodes (at most 1024 fit)", a->D, a->H, a->W);
  if (a->dtype != ISSM_F32 && a->dtype != ISSM_BF16) return fail(ISSM_E_DTYPE, "box_dist: dtype %d", a->dtype);
  if (!a->key || (!a->corners && !a->boxes)) return fail(ISSM_E_NULL, "box_dist: key or corners/boxes is NULL");
  if (!bwd) {
    if (a->dist && !a->table) return fail(ISSM_E_NULL, "box_dist: table is NULL");
    if (a->weights && !a->boxes && (!a->qcenter || !a->radius)) return fail(ISSM_E_NULL, "box_dist: qcenter/radius is NULL");
    if (a->qcenter && !a->radius) return fail(ISSM_E_NULL, "box_dist: radius is NULL");
  } else if (!a->ddist || !a->partial || !a->dtable) {
    return fail(ISSM_E_NULL, "box_dist bwd: ddist/partial/dtable is NULL");
  }
  p->B = a->batch; p->L = a->seqlen; p->K = a->nquery; p->D = a->D; p->H = a->H; p->W = a->W; p->dtype = a->dtype;
  p->nwg = box_dist_workgroups(a->batch, a->seqlen, a->nquery);
  p->nwg_bwd = box_dist_bwd_workgroups(a->batch, a->seqlen, a->nquery);
  if (bwd && (int64_t)a->batch * a->seqlen * a->nquery > ((int64_t)1 << 26))
    return fail(ISSM_E_UNSUPPORTED, "box_dist bwd: more than 2^26 (point, box) pairs");
  p->key = a->key; p->corners = a->corners; p->boxes = a->corners ? nullptr : a->boxes; p->min_radius = a->min_radius;
  p->angle = a->angle; p->table = a->table;
  p->log_scale = a->log_scale; p->max_value = a->max_value; p->dist = a->dist;
  p->qcenter = a->qcenter; p->radius = a->radius; p->weight_dist = a->weight_dist; p->weights = a->weights;
  p->ddist = a->ddist; p->partial = a->partial; p->dtable = a->dtable;
  return ISSM_OK;
}

int64_t issm_box_dist_bwd_scratch_bytes(int32_t batch, int32_t seqlen, int32_t nquery, int32_t D, int32_t H, int32_t W) {
  if (batch <= 0 || seqlen <= 0 || nquery <= 0 || D <= 0 || H <= 0 || W <= 0) return 16;
  return box_dist_bwd_scratch_bytes(batch, seqlen, nquery, D, H, W);
}

int issm_box_dist_fwd(const issm_box_dist_args* a) {
  BoxDistP p;
  int rc = box_dist_params(a, &p, false);
  if (rc) return rc;
  if (p.nwg == 0 || (!p.dist && !p.weights)) return ISSM_OK;
  return launched(launch_box_dist_fwd(p, (hipStream_t)a->stream), "box_dist_fwd");
}

int issm_box_dist_bwd(const issm_box_dist_args* a) {
  BoxDistP p;
  int rc = box_dist_params(a, &p, true);
  if (rc) return rc;
  if (p.nwg_bwd == 0) return ISSM_OK;
  return launched(launch_box_dist_bwd(p, (hipStream_t)a->stream), "box_dist_bwd");
}

int issm_transpose_states(const issm_transpose_args* a) {
  if (!a) return fail(ISSM_E_NULL, "transpose: args is NULL");
  if (a->batch < 0 || a->rows < 0 || a->cols < 0) return fail(ISSM_E_SHAPE, "transpose: bad shape");
  if ((a->in_dtype != ISSM_F32 && a->in_dtype != ISSM_BF16) || (a->out_dtype != ISSM_F32 && a->out_dtype != ISSM_BF16))
    return fail(ISSM_E_DTYPE, "transpose: dtypes %d -> %d", a->in_dtype, a->out_dtype);
  if (a->batch == 0 || a->rows == 0 || a->cols == 0) return ISSM_OK;
  if (!a->in0 || !a->out) return fail(ISSM_E_NULL, "transpose: in0/out is NULL");
  if (a->batch > 65535 || (a->rows + 63) / 64 > 65535) return fail(ISSM_E_SHAPE, "transpose: batch / rows too large for one launch");
  TrP p;
  p.B = a->batch; p.R = a->rows; p.C = a->cols; p.in_dt = a->in_dtype; p.out_dt = a->out_dtype;
  p.in0 = a->in0; p.in1 = a->in1; p.out = a->out; p.alpha = a->alpha;
  return launched(launch_transpose_states(p, (hipStream_t)a->stream), "transpose_states");
}

int issm_hilbert_codes(const issm_hilbert_args* a) {
  if (!a) return fail(ISSM_E_NULL, "hilbert: args is NULL");
  if (a->batch < 0 || a->npoint < 0) return fail(ISSM_E_SHAPE, "hilbert: bad shape");
  if (a->bits < 1 || a->bits > 20) return fail(ISSM_E_UNSUPPORTED, "hilbert: bits = %d (1..20)", a->bits);
  if (!(a->cell > 0.0f)) return fail(ISSM_E_SHAPE, "hilbert: cell must be positive");
  int seen = 0;
  for (int i = 0; i < 3; ++i) {
    if (a->order[i] < 0 || a->order[i] > 2) return fail(ISSM_E_SHAPE, "hilbert: order[%d] = %d", i, a->order[i]);
    seen |= 1 << a->order[i];
  }
  if (seen != 7) return fail(ISSM_E_SHAPE, "hilbert: order is not a permutation of 0, 1, 2");
  if ((int64_t)a->batch * a->npoint == 0) return ISSM_OK;
  if (!a->points || !a->mins || !a->codes) return fail(ISSM_E_NULL, "hilbert: points/mins/codes is NULL");
  HilbertP p;
  p.B = a->batch; p.N = a->npoint; p.bits = a->bits; p.cell = a->cell;
  for (int i = 0; i < 3; ++i) p.perm[i] = a->order[i];
  p.points = a->points; p.mins = a->mins; p.codes = (long*)a->codes;
  return launched(launch_hilbert_codes(p, (hipStream_t)a->stream), "hilbert_codes");
}

int issm_hilbert_order(const issm_hilbert_order_args* a) {
  if (!a) return fail(ISSM_E_NULL, "hilbert_order: args is NULL");
  if (a->batch < 0 || a->npoint < 0) return fail(ISSM_E_SHAPE, "hilbert_order: bad shape");
  if (a->norder < 1 || a->norder > 6) return fail(ISSM_E_SHAPE, "hilbert_order: norder = %d (1..6)", a->norder);
  if (a->bits < 1 || a->bits > 17) return fail(ISSM_E_UNSUPPORTED, "hilbert_order: bits = %d (1..17)", a->bits);
  if (a->npoint > ISSM_HILBERT_ORDER_MAX_POINTS)
    return fail(ISSM_E_UNSUPPORTED, "hilbert_order: %d points (at most %d per sample; use issm_hilbert_codes and a sort)",
                a->npoint, ISSM_HILBERT_ORDER_MAX_POINTS);
  if (!(a->cell > 0.0f)) return fail(ISSM_E_SHAPE, "hilbert_order: cell must be positive");
  for (int o = 0; o < a->norder; ++o) {
    int seen = 0;
    for (int i = 0; i < 3; ++i) {
      if (a->order[o][i] < 0 || a->order[o][i] > 2) return fail(ISSM_E_SHAPE, "hilbert_order: order[%d][%d] = %d", o, i, a->order[o][i]);
      seen |= 1 << a->order[o][i];
    }
    if (seen != 7) return fail(ISSM_E_SHAPE, "hilbert_order: order %d is not a permutation of 0, 1, 2", o);
  }
  if ((int64_t)a->batch * a->npoint == 0) return ISSM_OK;
  if (!a->points || !a->index) return fail(ISSM_E_NULL, "hilbert_order: points/index is NULL");
  if ((int64_t)a->batch * a->norder > 0x7fffffff) return fail(ISSM_E_SHAPE, "hilbert_order: too many samples");
  HilbertOrderP p;
  p.B = a->batch; p.N = a->npoint; p.bits = a->bits; p.norder = a->norder; p.cell = a->cell;
  p.NP = 2;
  while (p.NP < p.N) p.NP <<= 1;
  for (int o = 0; o < a->norder; ++o)
    for (int i = 0; i < 3; ++i) p.perm[o][i] = a->order[o][i];
  p.points = a->points; p.index = (long*)a->index; p.inverse = (long*)a->inverse;
  return launched(launch_hilbert_order(p, (hipStream_t)a->stream), "hilbert_order");
}

// shared checks of the point-set operators: non-negative sizes, work present, pointers given
#define PN2_SIZES(what, ...)                                                              \
  do {                                                                                    \
    const long long dims_[] = {__VA_ARGS__};                                              \
    for (long long d_ : dims_)                                                            \
      if (d_ < 0) return fail(ISSM_E_SHAPE, what ": negative size");                      \
  } while (0)
#define PN2_PTRS(what, ...)                                                               \
  do {                                                                                    \
    const void* ptrs_[] = {__VA_ARGS__};                                                  \
    for (const void* q_ : ptrs_)                                                          \
      if (!q_) return fail(ISSM_E_NULL, what ": NULL pointer");                           \
  } while (0)

int issm_pn2_furthest_point_sampling(int32_t b, int32_t n, int32_t npoint, const float* xyz, float* temp, int32_t* idxs,
                                     void* stream) {
  PN2_SIZES("furthest_point_sampling", b, n, npoint);
  if (b == 0 || npoint == 0) return ISSM_OK;
  if (n == 0) return fail(ISSM_E_SHAPE, "furthest_point_sampling: no points to draw from");
  if (b > 65535) return fail(ISSM_E_UNSUPPORTED, "furthest_point_sampling: batch %d > 65535", b);
  PN2_PTRS("furthest_point_sampling", xyz, idxs);
  if (n > 24576 && !temp) return fail(ISSM_E_NULL, "furthest_point_sampling: temp is NULL (needed above 24576 points)");
  return launched(launch_fps(b, n, npoint, xyz, temp, idxs, (hipStream_t)stream), "furthest_point_sampling");
}

int issm_pn2_ball_query(int32_t b, int32_t n, int32_t m, float radius, int32_t nsample, const float* new_xyz,
                        const float* xyz, int32_t* idx, void* stream) {
  PN2_SIZES("ball_query", b, n, m, nsample);
  if (b == 0 || m == 0 || nsample == 0) return ISSM_OK;
  if (b > 65535) return fail(ISSM_E_UNSUPPORTED, "ball_query: batch %d > 65535", b);
  PN2_PTRS("ball_query", new_xyz, idx);
  if (n > 0 && !xyz) return fail(ISSM_E_NULL, "ball_query: xyz is NULL");
  return launched(launch_ball_query(b, n, m, radius, nsample, new_xyz, xyz, idx, (hipStream_t)stream), "ball_query");
}

int issm_pn2_group_points(int32_t b, int32_t c, int32_t n, int32_t npoints, int32_t nsample, const float* points,
                          const int32_t* idx, float* out, void* stream) {
  PN2_SIZES("group_points", b, c, n, npoints, nsample);
  if ((int64_t)b * c * npoints * nsample == 0) return ISSM_OK;
  if (n == 0) return fail(ISSM_E_SHAPE, "group_points: no points to index");
  if ((int64_t)npoints * nsample > 0x7fffffff) return fail(ISSM_E_SHAPE, "group_points: too many indices per sample");
  PN2_PTRS("group_points", points, idx, out);
  return launched(launch_group_points(b, c, n, npoints * nsample, points, idx, out, (hipStream_t)stream), "group_points");
}

int issm_pn2_group_points_grad(int32_t b, int32_t c, int32_t n, int32_t npoints, int32_t nsample, const float* grad_out,
                               const int32_t* idx, float* grad_points, void* stream) {
  PN2_SIZES("group_points_grad", b, c, n, npoints, nsample);
  if ((int64_t)b * c * npoints * nsample == 0) return ISSM_OK;
  if (n == 0) return fail(ISSM_E_SHAPE, "group_points_grad: no points to index");
  if ((int64_t)npoints * nsample > 0x7fffffff) return fail(ISSM_E_SHAPE, "group_points_grad: too many indices per sample");
  PN2_PTRS("group_points_grad", grad_out, idx, grad_points);
  return launched(launch_group_points_grad(b, c, n, npoints * nsample, grad_out, idx, grad_points, (hipStream_t)stream),
                  "group_points_grad");
}

int issm_pn2_gather_points(int32_t b, int32_t c, int32_t n, int32_t npoints, const float* points, const int32_t* idx,
                           float* out, void* stream) {
  return issm_pn2_group_points(b, c, n, npoints, 1, points, idx, out, stream);
}

int issm_pn2_gather_points_grad(int32_t b, int32_t c, int32_t n, int32_t npoints, const float* grad_out,
                                const int32_t* idx, float* grad_points, void* stream) {
  return issm_pn2_group_points_grad(b, c, n, npoints, 1, grad_out, idx, grad_points, stream);
}

int issm_pn2_three_nn(int32_t b, int32_t n, int32_t m, const float* unknown, const float* known, float* dist2,
                      int32_t* idx, void* stream) {
  PN2_SIZES("three_nn", b, n, m);
  if (b == 0 || n == 0) return ISSM_OK;
  if (b > 65535) return fail(ISSM_E_UNSUPPORTED, "three_nn: batch %d > 65535", b);
  PN2_PTRS("three_nn", unknown, dist2, idx);
  if (m > 0 && !known) return fail(ISSM_E_NULL, "three_nn: known is NULL");
  return launched(launch_three_nn(b, n, m, unknown, known, dist2, idx, (hipStream_t)stream), "three_nn");
}

int issm_pn2_three_interpolate(int32_t b, int32_t c, int32_t m, int32_t n, const float* points, const int32_t* idx,
                               const float* weight, float* out, void* stream) {
  PN2_SIZES("three_interpolate", b, c, m, n);
  if ((int64_t)b * c * n == 0) return ISSM_OK;
  if (m == 0) return fail(ISSM_E_SHAPE, "three_interpolate: no points to index");
  PN2_PTRS("three_interpolate", points, idx, weight, out);
  return launched(launch_three_interpolate(b, c, m, n, points, idx, weight, out, (hipStream_t)stream), "three_interpolate");
}

int issm_pn2_three_interpolate_grad(int32_t b, int32_t c, int32_t n, int32_t m, const float* grad_out, const int32_t* idx,
                                    const float* weight, float* grad_points, void* stream) {
  PN2_SIZES("three_interpolate_grad", b, c, n, m);
  if ((int64_t)b * c * n == 0) return ISSM_OK;
  if (m == 0) return fail(ISSM_E_SHAPE, "three_interpolate_grad: no points to index");
  PN2_PTRS("three_interpolate_grad", grad_out, idx, weight, grad_points);
  return launched(launch_three_interpolate_grad(b, c, n, m, grad_out, idx, weight, grad_points, (hipStream_t)stream),
                  "three_interpolate_grad");
}

int issm_pn2_group_points_grad_cl(int32_t b, int32_t c, int32_t n, int32_t npoints, int32_t nsample, const float* grad_out,
                                  const int32_t* idx, float* grad_points_cl, void* stream) {
  PN2_SIZES("group_points_grad_cl", b, c, n, npoints, nsample);
  if ((int64_t)b * c * npoints * nsample == 0) return ISSM_OK;
  if (n == 0) return fail(ISSM_E_SHAPE, "group_points_grad_cl: no points to index");
  if ((int64_t)npoints * nsample > 0x7fffffff || b > 65535)
    return fail(ISSM_E_UNSUPPORTED, "group_points_grad_cl: too many indices per sample or batch > 65535");
  PN2_PTRS("group_points_grad_cl", grad_out, idx, grad_points_cl);
  return launched(launch_scatter_channel_last(false, b, c, n, npoints * nsample, grad_out, idx, nullptr, grad_points_cl,
                                              (hipStream_t)stream), "group_points_grad_cl");
}

int issm_pn2_three_interpolate_grad_cl(int32_t b, int32_t c, int32_t n, int32_t m, const float* grad_out,
                                       const int32_t* idx, const float* weight, float* grad_points_cl, void* stream) {
  PN2_SIZES("three_interpolate_grad_cl", b, c, n, m);
  if ((int64_t)b * c * n == 0) return ISSM_OK;
  if (m == 0) return fail(ISSM_E_SHAPE, "three_interpolate_grad_cl: no points to index");
  if (b > 65535) return fail(ISSM_E_UNSUPPORTED, "three_interpolate_grad_cl: batch %d > 65535", b);
  PN2_PTRS("three_interpolate_grad_cl", grad_out, idx, weight, grad_points_cl);
  return launched(launch_scatter_channel_last(true, b, c, m, n, grad_out, idx, weight, grad_points_cl, (hipStream_t)stream),
                  "three_interpolate_grad_cl");
}

}  // extern "C"
