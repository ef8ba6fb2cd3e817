// Issue-rate probe for gfx950: does a matrix instruction run beside the vector ALU?
//
// One workgroup of 256 threads per CU slot; every wave runs a loop whose body is, per variant,
//   - 4 x v_mfma_f32_16x16x4_f32 on independent accumulators,
//   - 4 x v_mfma_f32_16x16x32_bf16,
//   - 32 x v_fma_f32 in 8 independent chains,
//   - 32 x v_exp_f32,
//   - the matrix and the vector work together, either one block after the other or interleaved
//     (one matrix instruction, then 8 vector instructions, enforced with sched_group_barrier).
// It prints the time per loop iteration and wave in cycles of a nominal 2.4 GHz clock, with one and with two
// waves per SIMD.  If matrix and vector work overlapped, "together" would cost the larger of the two parts;
// if they share issue slots it costs their sum.
//
// Build and run (not part of libissm_hip.so):
//   python -m dest3d_amd.build --probe && ./dest3d_amd/probe_mfma_valu
#include <hip/hip_runtime.h>
#include <cstdio>

typedef float f4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf8 __attribute__((ext_vector_type(8)));
constexpr int ITERS = 2000;

enum Mode { MFMA32 = 0, VALU = 1, MFMA32_THEN_VALU = 2, MFMA16 = 3, MFMA16_THEN_VALU = 4, EXP = 5,
            MFMA32_INTERLEAVED = 6, MFMA16_INTERLEAVED = 7, NMODES = 8 };

#define VBLK                                                                                      \
  v0 = __builtin_fmaf(v0, 1.0001f, 0.5f); v1 = __builtin_fmaf(v1, 1.0001f, 0.5f);                 \
  v2 = __builtin_fmaf(v2, 1.0001f, 0.5f); v3 = __builtin_fmaf(v3, 1.0001f, 0.5f);                 \
  v4 = __builtin_fmaf(v4, 1.0001f, 0.5f); v5 = __builtin_fmaf(v5, 1.0001f, 0.5f);                 \
  v6 = __builtin_fmaf(v6, 1.0001f, 0.5f); v7 = __builtin_fmaf(v7, 1.0001f, 0.5f);
#define ONE_MFMA_THEN_8_VALU                              \
  __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);      \
  __builtin_amdgcn_sched_group_barrier(0x002, 8, 0);

template <int MODE>
__global__ __launch_bounds__(256) void k(float* out, float seed) {
  f4 a0 = {0, 0, 0, 0}, a1 = a0, a2 = a0, a3 = a0;
  const float x = threadIdx.x * 1e-3f + seed, y = seed;
  float v0 = x, v1 = x + 1, v2 = x + 2, v3 = x + 3, v4 = x + 4, v5 = x + 5, v6 = x + 6, v7 = x + 7;
  bf8 ba, bb;
  for (int i = 0; i < 8; ++i) { ba[i] = (__bf16)(x + i); bb[i] = (__bf16)(y + i); }
  for (int it = 0; it < ITERS; ++it) {
    if (MODE == MFMA32 || MODE == MFMA32_THEN_VALU) {
      a0 = __builtin_amdgcn_mfma_f32_16x16x4f32(x, y, a0, 0, 0, 0);
      a1 = __builtin_amdgcn_mfma_f32_16x16x4f32(x, y, a1, 0, 0, 0);
      a2 = __builtin_amdgcn_mfma_f32_16x16x4f32(x, y, a2, 0, 0, 0);
      a3 = __builtin_amdgcn_mfma_f32_16x16x4f32(x, y, a3, 0, 0, 0);
    }
    if (MODE == MFMA16 || MODE == MFMA16_THEN_VALU) {
      a0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ba, bb, a0, 0, 0, 0);
      a1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ba, bb, a1, 0, 0, 0);
      a2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ba, bb, a2, 0, 0, 0);
      a3 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ba, bb, a3, 0, 0, 0);
    }
    if (MODE == VALU || MODE == MFMA32_THEN_VALU || MODE == MFMA16_THEN_VALU) {
      VBLK VBLK VBLK VBLK
    }
    if (MODE == MFMA32_INTERLEAVED) {
      a0 = __builtin_amdgcn_mfma_f32_16x16x4f32(x, y, a0, 0, 0, 0); VBLK
      a1 = __builtin_amdgcn_mfma_f32_16x16x4f32(x, y, a1, 0, 0, 0); VBLK
      a2 = __builtin_amdgcn_mfma_f32_16x16x4f32(x, y, a2, 0, 0, 0); VBLK
      a3 = __builtin_amdgcn_mfma_f32_16x16x4f32(x, y, a3, 0, 0, 0); VBLK
      ONE_MFMA_THEN_8_VALU ONE_MFMA_THEN_8_VALU ONE_MFMA_THEN_8_VALU ONE_MFMA_THEN_8_VALU
    }
    if (MODE == MFMA16_INTERLEAVED) {
      a0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ba, bb, a0, 0, 0, 0); VBLK
      a1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ba, bb, a1, 0, 0, 0); VBLK
      a2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ba, bb, a2, 0, 0, 0); VBLK
      a3 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ba, bb, a3, 0, 0, 0); VBLK
      ONE_MFMA_THEN_8_VALU ONE_MFMA_THEN_8_VALU ONE_MFMA_THEN_8_VALU ONE_MFMA_THEN_8_VALU
    }
    if (MODE == EXP) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        v0 = __builtin_amdgcn_exp2f(v0); v1 = __builtin_amdgcn_exp2f(v1); v2 = __builtin_amdgcn_exp2f(v2);
        v3 = __builtin_amdgcn_exp2f(v3); v4 = __builtin_amdgcn_exp2f(v4); v5 = __builtin_amdgcn_exp2f(v5);
        v6 = __builtin_amdgcn_exp2f(v6); v7 = __builtin_amdgcn_exp2f(v7);
      }
    }
  }
  out[blockIdx.x * 256 + threadIdx.x] = a0[0] + a1[1] + a2[2] + a3[3] + v0 + v1 + v2 + v3 + v4 + v5 + v6 + v7;
}

#define CHECK(e) do { hipError_t r_ = (e); if (r_ != hipSuccess) { printf("HIP error %s at line %d\n", hipGetErrorString(r_), __LINE__); return -1.0f; } } while (0)

template <int MODE>
float run(float* d, int blocks) {
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  hipLaunchKernelGGL(k<MODE>, dim3(blocks), dim3(256), 0, 0, d, 1.0f);  // warm-up
  CHECK(hipEventRecord(e0));
  hipLaunchKernelGGL(k<MODE>, dim3(blocks), dim3(256), 0, 0, d, 1.0f);
  CHECK(hipEventRecord(e1));
  CHECK(hipEventSynchronize(e1));
  float ms = 0;
  CHECK(hipEventElapsedTime(&ms, e0, e1));
  return ms;
}

int main() {
  float* d = nullptr;
  if (hipMalloc(&d, 1024 * 256 * sizeof(float)) != hipSuccess) { printf("hipMalloc failed\n"); return 1; }
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, 0) != hipSuccess) return 1;
  const int cus = prop.multiProcessorCount;
  const char* names[NMODES] = {"4 x mfma_f32_16x16x4_f32", "32 x v_fma_f32", "fp32 mfma block, then fma block",
                               "4 x mfma_f32_16x16x32_bf16", "bf16 mfma block, then fma block", "32 x v_exp_f32",
                               "fp32 mfma interleaved with fma", "bf16 mfma interleaved with fma"};
  printf("%s, %d CUs; cycles per loop iteration and wave at a nominal 2.4 GHz\n", prop.gcnArchName, cus);
  for (int occ = 1; occ <= 2; ++occ) {
    const int blocks = cus * occ;  // occ workgroups of 4 waves per CU = occ waves per SIMD
    const float t[NMODES] = {run<0>(d, blocks), run<1>(d, blocks), run<2>(d, blocks), run<3>(d, blocks),
                             run<4>(d, blocks), run<5>(d, blocks), run<6>(d, blocks), run<7>(d, blocks)};
    for (int m = 0; m < NMODES; ++m)
      printf("waves/SIMD=%d  %-34s %8.3f ms  %7.1f cycles\n", occ, names[m], t[m], t[m] * 1e-3 * 2.4e9 / ITERS / occ);
  }
  (void)hipFree(d);
  return 0;
}
