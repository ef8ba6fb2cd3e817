/*
 * issm.h -- C ABI of libissm_hip.so: the interactive-SSM (ISSM) chunked scan of DEST,
 * forward and backward, plus the gated RMSNorm epilogue, as hand-written gfx950 HIP
 * kernels.
 *
 * The reference has no native code on this path (it launches Triton kernels from
 * Python); the entry points below are what a ctypes/cffi binding inside the
 * reference's issm_triton/ package would call instead of those launchers.  Each
 * declaration cites the reference function it replaces (paths relative to the
 * reference checkout).
 *
 * Conventions
 *  - Every pointer is a DEVICE pointer owned by the caller.  The library never
 *    allocates, frees or retains memory; all work is enqueued on `stream` and is
 *    asynchronous with respect to the host.
 *  - Every function returns ISSM_OK (0) or a negative issm_status; the message for
 *    the calling thread's last failure is returned by issm_last_error().  Nothing
 *    throws and nothing calls exit().
 *  - Tensors with an issm_tensor descriptor may be strided in their first three
 *    dimensions (element strides); the innermost dimension must be contiguous.
 *  - Layouts: x,z,out,dout,dx,dz (B,L,H,P); dt,ddt (B,L,H,N); Bm,Cm,dB,dC (B,L,G,N);
 *    A,dt_bias,dA,ddt_bias (H,N) fp32 contiguous; D,dD (H) or (H,P) fp32 contiguous;
 *    h0 (B,H,P,N); final_states,dfinal,dh0 (B,H,P,N) fp32 contiguous.
 *  - Time is split into chunks of ISSM_CHUNK tokens inside the library whatever
 *    `chunk_size` the caller names: the result of the scan does not depend on the
 *    chunk length.  nc = ceil(L / ISSM_CHUNK); tail rows behave as dt' = 0
 *    (issm_triton/issm_chunk_state.py:81-100).
 *  - ndir = 2 runs the module's bidirectional pair (models/dest_module.py:565-575) in
 *    one call: direction 1 walks the same dt / A / D / h0 backwards in time with its
 *    own x / Bm / Cm and writes its outputs back in natural (un-flipped) time order.
 *  - Numerics: cumulative sums, decays, dt', states and all accumulation are fp32 for every
 *    I/O dtype.  With io_dtype = ISSM_F32 the products x^T.(B dt' decay), dy^T.(C decay),
 *    x.dS, dy.H and the within-chunk matrix M of the forward are evaluated as three bf16
 *    matrix products with fp32 accumulation on operands split into bf16 high and low parts
 *    (16 significand bits per operand; relative error of a product <= 2^-16); every other
 *    product is fp32.  With io_dtype = ISSM_BF16 every matrix product takes its operands
 *    rounded once to bf16 (as the reference's kernels cast their dot operands to the input
 *    dtype, issm_triton/issm_cabt_bmm.py:42-43), except x.dS, dy.H and the chunk state
 *    x^T.(B dt' decay), whose fp32 operands enter as high and low parts; the gradient of
 *    the running sum of dt'.A is assembled from identically rounded products, so that dA and
 *    ddt_bias carry no accumulated rounding bias.  Results are bit-reproducible from run to
 *    run (fixed-order reductions, no atomics).
 *  - Strides: stride[1] * seqlen must stay below 2^30 elements (row byte offsets are 32-bit).
 */
#ifndef ISSM_H
#define ISSM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ISSM_ABI_VERSION 5
#define ISSM_CHUNK 64 /* tokens per internal chunk */

typedef enum issm_status {
  ISSM_OK = 0,
  ISSM_E_NULL = -1,        /* a required pointer is NULL */
  ISSM_E_SHAPE = -2,       /* a dimension is non-positive / inconsistent (issm_combined.py:58-83) */
  ISSM_E_STRIDE = -3,      /* a stride is unusable */
  ISSM_E_DTYPE = -4,       /* unknown dtype code */
  ISSM_E_UNSUPPORTED = -5, /* legal in the reference but not built (dt_min < 0, headdim > 64) */
  ISSM_E_WORKSPACE = -6,   /* workspace missing or too small */
  ISSM_E_LAUNCH = -7       /* hipGetLastError() != hipSuccess after a launch */
} issm_status;

typedef enum issm_dtype { ISSM_F32 = 0, ISSM_BF16 = 1 } issm_dtype;

enum {
  ISSM_FLAG_DT_SOFTPLUS = 1u << 0, /* apply softplus to dt + dt_bias (softplus.py:7-16) */
  ISSM_FLAG_D_HAS_HDIM = 1u << 1,  /* D is (H,P) instead of (H) */
  ISSM_FLAG_SEQ_IDX = 1u << 2      /* args->seq_idx is given (packed sequences, issm_combined.py:29) */
};

typedef struct issm_dims {
  int32_t batch, seqlen, nheads, headdim, dstate, ngroups;
  int32_t chunk_size; /* the caller's chunk_size, validated (> 0) and otherwise unused */
  int32_t ndir;       /* 1 = one scan, 2 = forward + time-reversed scan */
} issm_dims;

typedef struct issm_tensor {
  void* ptr;         /* NULL = absent */
  int64_t stride[3]; /* element strides of dims 0,1,2 */
} issm_tensor;

/* One argument block for the forward, the backward and the stage entry points.
 * Fields that an entry point does not use may be zero. */
typedef struct issm_scan_args {
  issm_dims dims;
  int32_t io_dtype; /* issm_dtype of x, Bm, Cm, z, out, dout, dx, dB, dC, dz */
  int32_t dt_dtype; /* issm_dtype of dt, ddt */
  int32_t h0_dtype; /* issm_dtype of h0 */
  uint32_t flags;
  float dt_min, dt_max; /* dt_limit; dt_min >= 0 required */
  /* inputs ([dir]) */
  issm_tensor x[2];
  issm_tensor dt;
  issm_tensor Bm[2], Cm[2];
  issm_tensor z[2]; /* optional gate */
  const float* A;
  const float* D;       /* optional */
  const float* dt_bias; /* optional */
  issm_tensor h0;       /* optional; strides of dims B,H,P */
  /* forward outputs */
  issm_tensor out[2];
  float* final_states[2]; /* optional */
  /* Forward workspace, issm_fwd_workspace_bytes() bytes, 256-byte aligned.  After
   * issm_scan_fwd it holds what issm_scan_bwd needs (per-chunk entry states, the
   * intra-chunk C.A.B^T blocks, chunk decay totals, the pre-gate output if z is given)
   * and is passed unchanged to issm_scan_bwd as `saved`. */
  void* workspace;
  size_t workspace_bytes;
  /* backward inputs */
  const void* saved;
  issm_tensor dout[2];
  const float* dfinal[2]; /* optional */
  /* backward outputs (NULL pointer = not wanted, where the math allows skipping) */
  issm_tensor dx[2], dB[2], dC[2], dz[2];
  issm_tensor ddt;
  float* dA;
  float* dD;
  float* ddt_bias;
  float* dh0;
  /* backward scratch, issm_bwd_workspace_bytes() bytes, 256-byte aligned */
  void* bwd_workspace;
  size_t bwd_workspace_bytes;
  void* stream; /* hipStream_t */
  /* seq_idx (issm_triton/issm_combined.py:29, ndir = 1 only): (batch, seqlen) int32, read when ISSM_FLAG_SEQ_IDX is
   * set.  Tokens of a batch row whose values differ belong to different sequences packed into that row, and no
   * state passes from one to the next: wherever seq_idx changes from a token to its successor the running sum of
   * dt'.A takes an extra -128 ln 2, i.e. every decay across the change is multiplied by 2^-128 (3e-39: zero at fp32
   * resolution, where the reference's kernels multiply by an exact 0).  The backward must be given the same array.
   * Contract: the ids of a row must not decrease.  The initial states count as id 0, as in the reference
   * (issm_chunk_scan.py:123 takes 0 as the id before the first chunk, issm_state_passing.py:91 starts from 0): they
   * feed the first sequence of a row whose ids start at 0 and nothing in a row whose ids start higher (dh0 of that
   * row is then 0).  Ids that decrease are not rejected; the reference's equality masks would reconnect equal ids
   * inside a chunk but not across chunks, and that mix is not reproduced: here every change of id is a cut. */
  const int32_t* seq_idx;
  int64_t seq_idx_stride[2]; /* element strides of (batch, seqlen) */
} issm_scan_args;

/* Version of this header the library was built against. */
int issm_abi_version(void);
/* Message of the calling thread's most recent failure ("" if none). */
const char* issm_last_error(void);

/* Workspace sizes for a problem (only args->dims, args->z[0].ptr and args->dt_dtype are read: with two directions and
 * a bf16 ddt the backward workspace also holds the first direction's share of ddt in fp32, so that the sum of the two
 * directions is rounded to bf16 once). */
int issm_fwd_workspace_bytes(const issm_scan_args* args, size_t* out);
int issm_bwd_workspace_bytes(const issm_scan_args* args, size_t* out);

/* Whole operator.
 * issm_scan_fwd  replaces _issm_chunk_scan_combined_fwd (issm_triton/issm_combined.py:57-92),
 *                called from ISSMChunkScanCombinedFn.forward (issm_combined.py:38-47).
 * issm_scan_bwd  replaces _issm_chunk_scan_combined_bwd (issm_combined.py:95-179),
 *                called from ISSMChunkScanCombinedFn.backward (issm_combined.py:49-54).
 *                Unlike the reference it does not recompute the forward: it reads `saved`. */
int issm_scan_fwd(const issm_scan_args* args);
int issm_scan_bwd(const issm_scan_args* args);

/* Stage entry points (used by the operator above; exported for tests and profiling).
 * Intermediates, all fp32 contiguous, Bt = batch*ndir with index b*ndir+dir:
 *   states  (Bt, nc+1, H, P, N) chunk-local end states, then (in place) slot c = state entering
 *                               chunk c and slot nc = final state
 *   cs_last (Bt, nc, H, N)      per-chunk total of dt'*A
 *   cabt    (Bt, nc, H, 64, 64) intra-chunk matrix M[l][s], valid for l >= s
 *
 * issm_stage_chunk_local: dt transform + cumsum, chunk states and C.A.B^T in one pass
 *   over dt.  Replaces _chunk_cumsum_fwd (issm_chunk_state.py:11-104), _chunk_state_fwd
 *   (issm_chunk_state.py:234-356) and _bmm_CABT_chunk_fwd (issm_cabt_bmm.py:7-153).
 *   states / cabt may be NULL to skip that product.
 *   Launches made of complete 64 x 64 tiles run a kernel that writes every decay as a product of per-tile factors
 *   (valid while no 16-row tile's sum of dt'.A.log2(e) falls below -100) and computes the chunks outside that range
 *   with the general formulation in the same launch. */
int issm_stage_chunk_local(const issm_scan_args* args, float* states, float* cs_last, float* cabt);
/* issm_stage_state_passing_fwd: H_0 = h0, H_{c+1} = exp(cs_last_c) * H_c + S_c, in place
 *   (states[c] becomes H_c); final = H_nc.  Replaces _state_passing_fwd
 *   (issm_state_passing.py:5-107). */
int issm_stage_state_passing_fwd(const issm_scan_args* args, float* states, const float* cs_last);
/* issm_stage_chunk_scan: out = (C*exp(cs)) . H^T + tril(M) . x + D*x, optional silu(z) gate.
 *   Replaces _chunk_scan_fwd (issm_chunk_scan.py:10-214).  out_x (optional, fp32
 *   (Bt,L,H,P) contiguous) receives the pre-gate value when z is given. */
int issm_stage_chunk_scan(const issm_scan_args* args, const float* states, const float* cabt,
                          float* out_x);
/* issm_stage_bwd_gate: z-gate backward: dz and dy = dout*silu(z) (fp32 (Bt,L,H,P) contiguous,
 *   physical time order) from the saved pre-gate output.  Replaces _chunk_scan_bwd_dz
 *   (issm_chunk_scan.py:217-377); its dD part is produced by issm_stage_bwd_dx. */
int issm_stage_bwd_gate(const issm_scan_args* args, const float* out_x, float* dy_gated);
/* issm_stage_bwd_dstates: dH_c = dy^T . (C*exp(cs)) into dstates (Bt,nc,H,P,N) and
 *   dM = tril(dy . x^T) into dm (Bt,nc,H,64,64); either output may be NULL.  `dy` is args->dout
 *   unless dy_gated is given.  A 16 KB block of dm holds the symmetric 64 x 64 bf16 matrix
 *   T[i][j] = dM[max(i,j)][min(i,j)] in its first 8 KB (the form issm_stage_bwd_chunk reads: the sums over rows and
 *   over columns of dM both become row reads) and, for io_dtype = ISSM_F32, a second such matrix in the other 8 KB
 *   holding the bf16 rounding of what the first left: dM = hi + lo to 16 significand bits.  Replaces _chunk_scan_bwd_dstates (issm_chunk_scan.py:380-512) and
 *   _chunk_scan_bwd_dcb (issm_chunk_scan.py:790-900). */
int issm_stage_bwd_dstates(const issm_scan_args* args, const float* dy_gated, float* dstates, float* dm);
/* issm_stage_state_passing_bwd: reverse recurrence in place (dstates[c] becomes dS_c, the gradient
 *   of the chunk-local end state), g_last (Bt,nc,H,N) = sum_p dS_c * H_{c+1} (the total gradient
 *   reaching the chunk's last cumulative sum through the states), and dh0_dir (ndir,B,H,P,N).
 *   `states` is (Bt,nc+1,H,P,N) as left by issm_stage_state_passing_fwd.  Replaces
 *   _state_passing_bwd (issm_state_passing.py:110-278) and the sum over P at issm_combined.py:159. */
int issm_stage_state_passing_bwd(const issm_scan_args* args, const float* states,
                                 const float* cs_last, float* dstates, float* g_last,
                                 float* dh0_dir);
/* issm_stage_bwd_chunk: ddt, dB, dC of direction `dir` and the per-unit partial sums
 *   part_a / part_bias (Bt*nc,H,N) of dA / ddt_bias.  ddt accumulates into args->ddt when
 *   dir > 0.  Replaces _chunk_state_bwd_db (issm_chunk_state.py:493-652), _chunk_scan_bwd_dc
 *   (issm_chunk_scan.py:515-657), _chunk_scan_chunk_state_bwd_dt (issm_combined.py:398-557),
 *   _bmm_CABT_dbc_chunk_bwd (issm_cabt_bmm.py:454-673), _chunk_scan_bwd_ddAcs_stable
 *   (issm_chunk_scan.py:903-1031) and the elementwise part of _chunk_cumsum_bwd
 *   (issm_chunk_state.py:107-231).
 *   `redo` (issm_bwd_chunk_redo_ints(args) ints, contents irrelevant on entry, or NULL): with it the sums with the
 *   decay inside run in tile-base form (two exponentials per element, every block of the chunk a plain matrix
 *   product) wherever a 16-row tile's total decay stays below 2^96, and the level-hierarchy kernel, which has no such
 *   limit, evaluates only the (workgroup, head) pairs the buffer then marks; NULL: the level-hierarchy kernel
 *   evaluates everything.  Same results to rounding either way. */
int issm_stage_bwd_chunk(const issm_scan_args* args, int dir, const float* dy_gated,
                         const float* states, const float* dstates, const float* dm,
                         const float* g_last, float* part_a, float* part_bias, int32_t* redo);
/* Number of ints issm_stage_bwd_chunk's `redo` buffer needs (batch * directions * chunks * heads * 64-column slices;
 *   each direction uses its own part); 0 on bad dimensions.  No counterpart in the reference. */
size_t issm_bwd_chunk_redo_ints(const issm_scan_args* args);
/* issm_stage_bwd_dx: dx and the per-unit partial sums part_d (Bt*nc*H,P) of dD.  Replaces
 *   _chunk_scan_chunk_state_bwd_dx (issm_combined.py:183-395). */
int issm_stage_bwd_dx(const issm_scan_args* args, const float* dy_gated, const float* dstates,
                      const float* cabt, float* part_d);
/* issm_stage_bwd_reduce: fixed-order sums of the partials into args->dA, ddt_bias, dD and of
 *   dh0_dir over directions into args->dh0.  Replaces the atomics of _chunk_cumsum_bwd
 *   (issm_chunk_state.py:224-231) and the host-side sums at issm_combined.py:236-240. */
int issm_stage_bwd_reduce(const issm_scan_args* args, const float* part_a, const float* part_bias,
                          const float* part_d, const float* dh0_dir);

/* Gated RMSNorm epilogue: y = rmsnorm(x * silu(z)) * w  (norm_before_gate = 0, what DEST
 * uses) or rmsnorm(x) * w * silu(z) (norm_before_gate = 1); z may be NULL.
 * Replaces _layer_norm_fwd / _layer_norm_bwd with is_rms_norm=True, bias=None
 * (issm_triton/layernorm_gated.py:98-137, 261-325).  x,z,y,dy,dx,dz are (rows, ncols) with
 * a row stride in elements; ncols is split into groups of group_size (0 = one group);
 * rstd (ngroups*rows) fp32; dw_partial (nblocks, ncols) fp32 scratch where
 * nblocks = issm_rmsnorm_bwd_blocks(rows); dw (ncols) fp32. */
typedef struct issm_norm_args {
  int64_t rows;
  int32_t ncols, group_size;
  int32_t dtype;        /* issm_dtype of x, z, y, dy, dx, dz */
  int32_t weight_dtype; /* issm_dtype of w */
  int32_t norm_before_gate;
  float eps;
  const void *x, *z, *w;
  int64_t x_row_stride, z_row_stride;
  void* y;
  int64_t y_row_stride;
  float* rstd;
  /* backward */
  const void* dy;
  int64_t dy_row_stride;
  void *dx, *dz;
  int64_t dx_row_stride, dz_row_stride;
  float* dw_partial;
  float* dw;
  void* stream;
  /* LayerNorm statistics and bias (HAS_BIAS / IS_RMS_NORM = False of issm_triton/layernorm_gated.py:35-97, 145-260):
   * layer_norm = 0 normalises with x * rstd, rstd = 1/sqrt(mean(x^2) + eps); layer_norm = 1 with (x - mean) * rstd,
   * rstd = 1/sqrt(mean((x - mean)^2) + eps), and `mean` (ngroups*rows, fp32) is then required: written by the forward,
   * read by the backward.  bias (ncols, weight_dtype), optional, is added after the weight and before the gate; the
   * backward then needs db_partial (nblocks, ncols) fp32 scratch and writes db (ncols) fp32.  With a bias and more than
   * one group per row or more than 1024 columns, ncols <= 8192. */
  int32_t layer_norm;
  const void* bias;
  float* mean;
  float* db_partial;
  float* db;
} issm_norm_args;

int issm_rmsnorm_bwd_blocks(int64_t rows);
int issm_gated_rmsnorm_fwd(const issm_norm_args* args);
int issm_gated_rmsnorm_bwd(const issm_norm_args* args);

/* issm_gated_rmsnorm_bwd for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments and the same
 * results, bit for bit, as issm_gated_rmsnorm_bwd, except that args->dw_partial is ignored: the per-block partial
 * sums of dw go into a scratch array inside the library (ISSM_NORM_SCRATCH_FLOATS floats = 8 MiB per GPU the library
 * runs on, held until the process ends).  Problems with issm_rmsnorm_bwd_blocks(rows) * ncols >
 * ISSM_NORM_SCRATCH_FLOATS return ISSM_E_WORKSPACE (rows of up to 1024 columns always fit; with a bias db_partial is
 * ignored as well, its partial sums follow those of dw in the array, and the bound holds for twice the product:
 * up to 512 columns always fit).  The function calls no
 * hipMalloc / hipFree or other allocating routine.  All calls on one GPU share that GPU's array: two calls that
 * overlap in time on one GPU (different streams or host threads) race; calls on one stream are ordered and safe.
 * Nothing in the array has to be cleared between calls (every partial that is read was written by the same call).
 * The array's device address is looked up once per device, on the first eager call there of this function or of
 * issm_gated_rmsnorm_fwd / issm_gated_rmsnorm_bwd; that look-up may load code and is kept out of graph capture: if the
 * very first normalisation call on a device arrives while args->stream is recording, this function returns
 * ISSM_E_UNSUPPORTED and launches nothing.  Make one eager call per device before capturing. */
#define ISSM_NORM_SCRATCH_FLOATS (2048 * 1024)
int issm_gated_rmsnorm_bwd_noalloc(const issm_norm_args* args);

/* ---- generation of the scan parameters from the distance encoding -------------------
 * Replaces the bc_proj / dt_proj Linear layers, their transposes and the broadcast bias
 * additions of MultiHeadISSMScan.forward (models/dest_module.py:541-553) by one pass:
 *   base[r][k] = sum_m W[r][m] dist[t][k][m]        r < R0 = H + 2G, rows ordered dt heads, B groups, C groups
 *   dt[t][h][k] = base[h][k] + bias[t][h]           (pre-softplus; bias = token bias + dt_bias parameter)
 *   Bm[t][g][k] = base[H+g][k] + bias[t][H+g]       Cm[t][g][k] = base[H+G+g][k] + bias[t][H+G+g]
 *   Bm_back / Cm_back: the same base rows with bias columns R0+g and R0+G+g (has_back).
 * t runs over the B*L tokens, M must be 16 and R0 <= 12.  dist, the outputs and their gradients
 * are contiguous in `dtype`; W (R0, M), bias (tokens, R) with R = R0 + (has_back ? 2G : 0), dbias
 * (tokens, R) and dW (R0, M) are fp32 contiguous.  dw_partial: issm_param_gen_bwd_blocks(tokens)
 * * R0 * M floats of scratch.  Absent output gradients may be NULL (treated as zero).
 * weights (tokens, K) fp32, optional -- the per-(token, query) locality weight or 0/1 keep mask that
 * MultiHeadISSMScan multiplies into dt (dest_module.py:553-559): when given, dt = softplus(raw) * weights
 * (softplus with torch's threshold 20), the raw values go to dt_raw (tokens, H, K, `dtype`; required then, and
 * read back by the backward), and dweights (tokens, K) fp32, if not NULL, receives
 * sum_h ddt[t][h][k] * softplus(raw[t][h][k]).  dbias_sum needs dbias (it is summed in a fixed order after it
 * is written). */
typedef struct issm_pgen_args {
  int64_t tokens;
  int32_t K, M, H, G;
  int32_t dtype; /* issm_dtype of dist, dt, Bm, Cm, their gradients and ddist */
  int32_t has_back;
  const void* dist;
  const float* W;
  const float* bias;
  void *dt, *Bm, *Cm, *Bm_back, *Cm_back;
  const float* weights;
  void* dt_raw;
  /* backward */
  const void *ddt, *dBm, *dCm, *dBm_back, *dCm_back;
  void* ddist;
  float* dbias;
  float* dweights;
  float* dw_partial;
  float* dW;
  void* stream;
  float* dbias_sum; /* optional, (R) fp32: dbias summed over the tokens (the dt_bias parameter's gradient is its first H) */
} issm_pgen_args;

int issm_param_gen_bwd_blocks(int64_t tokens);
int issm_param_gen_fwd(const issm_pgen_args* args);
int issm_param_gen_bwd(const issm_pgen_args* args);

/* ---- depthwise 7-tap convolution along the token order + SiLU -------------------------
 * PointLiteConv (models/dest_module.py:400-423): nn.Conv1d(C, C, 7, padding=3, groups=C) on
 * feature.transpose(1, 2), then SiLU, transposed back.  Here on (B, L, C) as it lies, for up to two
 * weight sets in one pass:
 *   pre[s][b][l][c] = bias[s][c] + sum_j w[s][c][j] in_s[b][l+j-3][c]   (zero outside [0, L)),  y[s] = silu(pre[s]).
 * chain = 0: in_s = u for every set.  chain = 1 (nsets = 2): in_0 = u and in_1 = y[0] (as stored, i.e. rounded to
 * `dtype`) -- MultiHeadISSMScan's pair: dest_module.py:530 reassigns xbc = key_conv(xbc), and :534 applies
 * key_conv_back to that result, not to the key_proj output; du is then the gradient through both convolutions.
 * u: `dtype`, channels contiguous, element strides u_batch_stride / u_token_stride.  w (nsets, C, 7) and
 * bias (nsets, C): fp32 contiguous.  y and pre: (nsets, B, L, C) contiguous in `dtype`; pre is the
 * convolution output before SiLU, which the backward reads.  With 0 < split < C the output is written as two dense
 * tensors instead, y (nsets, B, L, split) for channels [0, split) and y_tail (nsets, B, L, C - split) for the rest
 * (MultiHeadISSMScan splits the result into x and the B / C biases, dest_module.py:532), and the backward takes
 * dy[s] (B, L, split) and dy_tail[s] (B, L, C - split).  Backward: dy[s] (B, L, C) contiguous or NULL
 * (zero); du (B, L, C), contiguous unless the du strides say otherwise; dw (nsets, C, 7), dbias (nsets, C) fp32; partial:
 * issm_dwconv_partial_rows(B, L) * nsets * 8 * C floats of scratch. */
typedef struct issm_dwconv_args {
  int32_t batch, seqlen, channels, nsets, taps; /* taps must be 7 */
  int32_t dtype;
  const void* u;
  int64_t u_batch_stride, u_token_stride;
  const float* w;
  const float* bias;
  void* y;
  void* pre;
  /* backward */
  const void* dy[2];
  void* du;
  float* partial;
  float* dw;
  float* dbias;
  void* stream;
  /* optional split of the output channels (0 = none) */
  int32_t split;
  void* y_tail;
  const void* dy_tail[2];
  /* element strides of du (0, 0 = contiguous (B, L, C)): lets the gradient land inside a wider row */
  int64_t du_batch_stride, du_token_stride;
  int32_t chain; /* 1: set 1 convolves set 0's output (needs nsets = 2) */
} issm_dwconv_args;

int issm_dwconv_partial_rows(int32_t batch, int32_t seqlen);
int issm_dwconv_silu_fwd(const issm_dwconv_args* args);
int issm_dwconv_silu_bwd(const issm_dwconv_args* args);

/* ---- queries <-> scan states -----------------------------------------------------------------
 * The rearrangements around the scan in MultiHeadISSMScan.forward: queries become initial states
 * ("b l (h hd) -> b h hd l", models/dest_module.py:537-538) and the two directions' final states become the query
 * output ("(last + last_back) / 2", "b h p l -> b l (h p)", :575 and :582); the backward needs the same two the
 * other way round.  One batched transpose with the sum, the scale and the dtype conversion folded in:
 *   out[b][c][r] = alpha * (in0[b][r][c] + in1[b][r][c]),   in0 / in1 (B, R, C), out (B, C, R), all contiguous;
 * in1 may be NULL.  in_dtype applies to in0 and in1, out_dtype to out (issm_dtype). */
typedef struct issm_transpose_args {
  int32_t batch, rows, cols;
  int32_t in_dtype, out_dtype;
  const void* in0;
  const void* in1;
  void* out;
  float alpha;
  void* stream;
} issm_transpose_args;

int issm_transpose_states(const issm_transpose_args* args);

/* ---- box-to-point distance encoding and locality weight ----------------------------------
 * BoxDistFun.forward (models/dest_module.py:174-195) and ISSMDecoderLayer.local_weight (:240-249), the two
 * (B, L, K) fields computed right before MultiHeadISSMScan:
 *   dist[b][l][k][0..15] = sum over the 8 corners c of box k of trilinear(table, f(R_j (corner - key_l)))
 *     f(v) = sign(v) log2(|v| log_scale + 1) / log2(8) / max_value per component, R_j the x-y rotation by
 *     angle[b][(8k + c) mod K] (the reference tiles the angles that way; NULL = no rotation), trilinear =
 *     grid_sample(mode bilinear, padding zeros, align_corners False) with x indexing W, y H, z D;
 *   weights[b][l][k] = exp(weight_dist * min(radius[b][k] - |key_l - qcenter[b][k]|, 0)).
 * key (B, L, 3), corners (B, K, 8, 3), angle (B, K), table (16, D, H, W) with D*H*W <= 1024, qcenter (B, K, 3),
 * radius (B, K), weights (B, L, K), dtable (16, D, H, W): fp32 contiguous.  Instead of corners (and of qcenter /
 * radius) the boxes themselves may be given: boxes (B, K, 7) = centre, size (l, w, h), heading; the corners are
 * then those of box_parametrization_to_corners (dest_module.py:99-103) and, for the weights, the centre is the
 * box's and radius = max(|size|, min_radius).  dist and ddist: (B, L, K, 16)
 * contiguous in `dtype`.  Either output of the forward may be NULL (skipped).  The backward produces the table
 * gradient only (the reference detaches the corners; key positions and angles are inputs); partial:
 * issm_box_dist_bwd_scratch_bytes(...) bytes of scratch, 16-byte aligned (about 64 bytes per pair for large
 * problems: the pairs are sorted by the table cells they touch).  The gradient is accumulated in integers -- for
 * large problems weights in units of 2^-24 and ddist in units of 2^-22 max|ddist|, exact products and sums -- so it
 * does not depend on the order of the adds (reproducible bit for bit); at most 2^26 (point, box) pairs per call. */
typedef struct issm_box_dist_args {
  int32_t batch, seqlen, nquery, D, H, W;
  int32_t dtype;
  const float* key;
  const float* corners;
  const float* boxes;
  float min_radius;
  const float* angle;
  const float* table;
  float log_scale, max_value;
  void* dist;
  const float* qcenter;
  const float* radius;
  float weight_dist;
  float* weights;
  /* backward */
  const void* ddist;
  void* partial;
  float* dtable;
  void* stream;
} issm_box_dist_args;

int64_t issm_box_dist_bwd_scratch_bytes(int32_t batch, int32_t seqlen, int32_t nquery, int32_t D, int32_t H, int32_t W);
int issm_box_dist_fwd(const issm_box_dist_args* args);
int issm_box_dist_bwd(const issm_box_dist_args* args);

/* ---- serialization codes of the key points ------------------------------------------------
 * Serialization.forward / encode (models/dest_module.py:307-356): grid = trunc((point - min of the sample) / cell)
 * clamped to 2^bits - 1, coordinates permuted by `order` (order[i] = which of x, y, z is the i-th curve
 * coordinate: "yxz" is {1, 0, 2}), mapped to its position on the 3-D Hilbert curve.  The reference looks the
 * position up in a table file it does not ship; this entry point computes it (Skilling's algorithm), so the curve's
 * orientation may differ from that table's.  points (B, N, 3), mins (B, 3): fp32 contiguous; codes (B, N) int64.
 * 1 <= bits <= 20. */
typedef struct issm_hilbert_args {
  int32_t batch, npoint, bits;
  int32_t order[3];
  float cell;
  const float* points;
  const float* mins;
  int64_t* codes;
  void* stream;
} issm_hilbert_args;

int issm_hilbert_codes(const issm_hilbert_args* args);

/* Serialization.forward as a whole (models/dest_module.py:319-345), all orders in one launch: for every order o and
 * sample b, index[o][b][:] lists the points of the sample along the curve (what torch.argsort of the codes above
 * returns; points of one cell keep their input order) and inverse[o][b][:] is the inverse permutation (the
 * reference's second argsort).  The minimum corner is taken inside.  points (B, N, 3) fp32 contiguous; index,
 * inverse (norder, B, N) int64 contiguous, inverse may be NULL.  N <= ISSM_HILBERT_ORDER_MAX_POINTS and bits <= 17
 * (ISSM_E_UNSUPPORTED beyond: take issm_hilbert_codes and a library sort). */
#define ISSM_HILBERT_ORDER_MAX_POINTS 4096
typedef struct issm_hilbert_order_args {
  int32_t batch, npoint, bits;
  int32_t norder; /* 1..6 */
  int32_t order[6][3];
  float cell;
  const float* points;
  int64_t* index;
  int64_t* inverse;
  void* stream;
} issm_hilbert_order_args;

int issm_hilbert_order(const issm_hilbert_order_args* args);

/* ---- point-set operators of the PointNet++ backbone ---------------------------------------
 * The functions of the reference's `pointnet2._ext` (pointnet2/_ext_src/src/bindings.cpp:8-24), same argument
 * meaning as its C++ wrappers; fp32 / int32, contiguous, device pointers.  Outputs that the reference allocates
 * with torch::zeros and then accumulates into (the *_grad functions) must be zeroed by the caller.
 *   furthest_point_sampling  sampling.cpp:70-91     xyz (b, n, 3) -> idxs (b, npoint); temp (b, n) scratch, used
 *                            only when n > 24576.  Starts at point 0; points with |p|^2 <= 1e-3 are never drawn;
 *                            equal distances go to the smaller index.
 *   ball_query               ball_query.cpp:13-37   new_xyz (b, m, 3), xyz (b, n, 3) -> idx (b, m, nsample)
 *   group_points(_grad)      group_points.cpp:17-65 points (b, c, n), idx (b, npoints, nsample) -> (b, c, npoints, nsample)
 *   gather_points(_grad)     sampling.cpp:20-68     points (b, c, n), idx (b, npoints) -> (b, c, npoints)
 *   three_nn                 interpolate.cpp:19-45  unknown (b, n, 3), known (b, m, 3) -> dist2, idx (b, n, 3)
 *   three_interpolate(_grad) interpolate.cpp:47-104 points (b, c, m), idx, weight (b, n, 3) -> (b, c, n)
 * Distances are evaluated in plain fp32 steps (no fused multiply-add), so index choices follow a straightforward
 * fp32 evaluation. */
int issm_pn2_furthest_point_sampling(int32_t b, int32_t n, int32_t npoint, const float* xyz, float* temp, int32_t* idxs,
                                     void* stream);
int issm_pn2_ball_query(int32_t b, int32_t n, int32_t m, float radius, int32_t nsample, const float* new_xyz,
                        const float* xyz, int32_t* idx, void* stream);
int issm_pn2_group_points(int32_t b, int32_t c, int32_t n, int32_t npoints, int32_t nsample, const float* points,
                          const int32_t* idx, float* out, void* stream);
int issm_pn2_group_points_grad(int32_t b, int32_t c, int32_t n, int32_t npoints, int32_t nsample, const float* grad_out,
                               const int32_t* idx, float* grad_points, void* stream);
int issm_pn2_gather_points(int32_t b, int32_t c, int32_t n, int32_t npoints, const float* points, const int32_t* idx,
                           float* out, void* stream);
int issm_pn2_gather_points_grad(int32_t b, int32_t c, int32_t n, int32_t npoints, const float* grad_out,
                                const int32_t* idx, float* grad_points, void* stream);
int issm_pn2_three_nn(int32_t b, int32_t n, int32_t m, const float* unknown, const float* known, float* dist2,
                      int32_t* idx, void* stream);
int issm_pn2_three_interpolate(int32_t b, int32_t c, int32_t m, int32_t n, const float* points, const int32_t* idx,
                               const float* weight, float* out, void* stream);
int issm_pn2_three_interpolate_grad(int32_t b, int32_t c, int32_t n, int32_t m, const float* grad_out, const int32_t* idx,
                                    const float* weight, float* grad_points, void* stream);
/* The same two gradients accumulated into a channel-last buffer, grad_points_cl (b, n, c) resp. (b, m, c), zeroed by
 * the caller: its transpose is the reference's result.  No counterpart in the reference; the atomics then touch
 * 64 consecutive floats per instruction instead of 64 scattered cache lines (about 10x faster at C = 128). */
int issm_pn2_group_points_grad_cl(int32_t b, int32_t c, int32_t n, int32_t npoints, int32_t nsample, const float* grad_out,
                                  const int32_t* idx, float* grad_points_cl, void* stream);
int issm_pn2_three_interpolate_grad_cl(int32_t b, int32_t c, int32_t n, int32_t m, const float* grad_out,
                                       const int32_t* idx, const float* weight, float* grad_points_cl, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* ISSM_H */
