// bench_mfma_probe.hip — what the matrix pipe of this board sustains with no memory access at
// all: every wave of a full grid (8 waves per block, 4 blocks per compute unit) issues
// v_mfma_f32_16x16x32_bf16 on operands it keeps in registers, sixteen independent accumulators
// deep. bench.py --gemm-study times it on all-zero and on random operands beside the library's
// batched GEMM and the vendor library's, because the board holds its power limit by lowering the
// shader clock and the bits that toggle set the power: the published 2.5 PFLOP/s assumes 2.4 GHz.
// Not part of libnxhip; built by __graft_entry__.build() into bench_mfma_probe.so.
#include <hip/hip_runtime.h>

#include <cstdint>

typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

__global__ __launch_bounds__(512) void mfma_only(float *out, const uint32_t *in, int iters) {
  bf16x8 aa[4], bb[4];
  for (int q = 0; q < 4; q++) {
    const uint32_t *p = in + (threadIdx.x & 255) * 4 + q * 2048;
    aa[q] = __builtin_bit_cast(bf16x8, u32x4{p[0], p[1], p[2], p[3]});
    bb[q] = __builtin_bit_cast(bf16x8, u32x4{p[1024], p[1025], p[1026], p[1027]});
  }
  f32x4 acc[16];
  for (int t = 0; t < 16; t++)
    for (int e = 0; e < 4; e++) acc[t][e] = 0;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int t = 0; t < 16; t++) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(aa[t & 3], bb[t >> 2], acc[t], 0, 0, 0);
  }
  float r = 0;
  for (int t = 0; t < 16; t++)
    for (int e = 0; e < 4; e++) r += acc[t][e];
  out[(size_t)blockIdx.x * 512 + threadIdx.x] = r;
}

// Runs `reps` launches of `iters` rounds of sixteen MFMAs per wave on the current device's
// default stream; returns the flops of one launch (0 on a HIP error), the mean time in *ms.
// `in` holds 8192 words (bf16 pairs), `out` blocks * 512 floats.
extern "C" __attribute__((visibility("default"))) double mfma_probe_run(const uint32_t *in, float *out, int blocks, int iters,
                                                                        int reps, float *ms) {
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return 0;
  hipLaunchKernelGGL(mfma_only, dim3(blocks), dim3(512), 0, 0, out, in, 8);
  (void)hipEventRecord(e0, 0);
  for (int r = 0; r < reps; r++) hipLaunchKernelGGL(mfma_only, dim3(blocks), dim3(512), 0, 0, out, in, iters);
  (void)hipEventRecord(e1, 0);
  const bool ok = hipEventSynchronize(e1) == hipSuccess && hipGetLastError() == hipSuccess;
  float t = 0;
  (void)hipEventElapsedTime(&t, e0, e1);
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  *ms = t / (float)reps;
  return ok ? (double)blocks * 8.0 * (double)iters * 16.0 * 16384.0 : 0.0;
}
