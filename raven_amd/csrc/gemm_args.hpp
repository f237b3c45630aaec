// Arguments every GEMM kernel of the library takes: one product's operands and strides, and the
// batch dims that are decoded on the device.
#pragma once

#include <cstdint>

#include "nxh_common.hpp"

constexpr int MM_MAXB = 8;  // batch dims decoded on the device

struct BatchDims {
  int n;
  uint32_t shape[MM_MAXB];
  int64_t a[MM_MAXB], b[MM_MAXB], c[MM_MAXB];
};
__device__ __forceinline__ void batch_decode(const BatchDims &d, uint32_t idx, int64_t &ao, int64_t &bo,
                                             int64_t &co) {
  ao = bo = co = 0;
  for (int i = d.n - 1; i >= 0; i--) {
    uint32_t q = idx / d.shape[i], c = idx - q * d.shape[i];
    idx = q;
    ao += (int64_t)c * d.a[i];
    bo += (int64_t)c * d.b[i];
    co += (int64_t)c * d.c[i];
  }
}

struct GemmArgs {
  const void *A, *B;
  void *C;
  int64_t M, N, K;
  int64_t ars, acs, brs, bcs, crs, ccs;  // element strides: row, col
  BatchDims batch;
  uint32_t batch0;   // first batch index of this launch
  int a_vec, b_vec;  // 16-byte loads allowed (alignment + stride multiple)
  // tiled kernels only: extents that may be loaded along M / N (a padded copy's row length)
  int64_t m_ld, n_ld;
};

// The register-blocked kernel for the dtypes without a matrix-instruction path (gemm_block.hip):
// NXH_OK, an error status, or -1 when the shape is better left to the one-lane-per-output kernel.
int nxh_gemm_block(nxh_context *ctx, int dtype, GemmArgs &a, uint32_t nbatch);
