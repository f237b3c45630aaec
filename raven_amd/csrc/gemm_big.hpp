// gemm_big.hpp — the large-tile MFMA GEMM for 16-bit inputs (bf16 / f16) with
// f32 accumulation: the kernel behind batched [.., M, K] x [.., K, N] when M and
// N are multiples of 256 and K of 64.
//
// Shape of the kernel (one block per CU, WM x WN wave64s; 4 x 2 in production):
//   block tile 256 x 256, K-slab 64, LDS double-buffered (2 x 72 KiB);
//   each wave owns (256/WM) x (256/WN) outputs as 32x32 tiles of
//   v_mfma_f32_32x32x16 (64 x 128 = 2 x 4 tiles, 128 accumulator registers);
//   global -> registers -> LDS with the loads for slab t+2 in flight while slab
//   t is multiplied; one barrier per slab. Inside a slab the work is software-
//   pipelined by hand: the LDS fragment reads of k-step s+1, a quarter of the
//   register -> LDS stores of slab t+1 and a quarter of the global loads of slab
//   t+2 are issued in front of the 8 MFMAs of k-step s (scheduling barriers keep
//   the compiler from regrouping them), so memory instructions never queue up
//   in front of the matrix pipe.
// An operand that is contiguous along K sits in LDS as [row][k] (+16 B pad) and
// is fetched with ds_read_b128. An operand that is contiguous along M / N (a
// row-major B) stays in its memory order, [k][row] (+64 B pad), and the
// k-contiguous fragments MFMA wants are produced by the transposing LDS read
// ds_read_b64_tr_b16: within each group of 16 lanes, result element j of lane L
// is element (L & 3) of the 8 bytes addressed by lane 4*j + (L >> 2). No 2-byte
// scatter into LDS, no transposed copy in HBM.
// Block ids are remapped so that the 32 blocks resident on one XCD (ids equal
// modulo 8) cover a compact patch of tiles and share A / B panels in that XCD's
// L2.
#pragma once

#include "nxh_common.hpp"

#include <type_traits>

namespace gemm_big {

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int PK = BK + 8;    // pitch (elements) of a [row][k] tile
constexpr int PR = 256 + 32;  // pitch (elements) of a [k][row] tile
constexpr int TILE_ELEMS = 256 * PK;  // == BK * PR == 18432
static_assert(256 * PK == BK * PR, "both tile layouts occupy the same LDS space");
constexpr int STAGE_ELEMS = 2 * TILE_ELEMS;
constexpr size_t LDS_BYTES = 2 * STAGE_ELEMS * sizeof(uint16_t);  // 147456

typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
typedef __attribute__((ext_vector_type(4))) uint32_t V16;  // one 16-byte register quad

struct Args {
  const uint16_t *A, *B;
  uint16_t *C;
  int64_t lda, ldb, ldc;  // the non-unit stride of each matrix (elements)
  int64_t K;
  uint32_t tiles_m, tiles_n, nbatch;
  // batch offsets: up to 4 broadcastable batch dims
  int nbd;
  uint32_t bshape[4];
  int64_t ba[4], bb[4], bc[4];
};

template <bool BF16>
__device__ __forceinline__ void mfma16(f32x16 &acc, const V16 &a, const V16 &b) {
  if constexpr (BF16)
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), acc, 0, 0, 0);
  else
    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), acc, 0, 0, 0);
}

// Global -> registers -> LDS, one 16-byte vector at a time: vector i of this lane
// (of 2048 / THREADS) of one operand's 256 x 64 slab. KC: rows are 128 B apart in
// the slab (8 vectors per row); otherwise the slab is 64 k-rows of 512 B (32
// vectors per k-row).
template <bool KC, int THREADS>
__device__ __forceinline__ V16 slab_load1(int i, const uint16_t *p, int64_t ld) {
  const int v = threadIdx.x + i * THREADS;
  const uint16_t *q = KC ? p + (int64_t)(v >> 3) * ld + (v & 7) * 8 : p + (int64_t)(v >> 5) * ld + (v & 31) * 8;
  return *reinterpret_cast<const V16 *>(q);
}
template <bool KC, int THREADS>
__device__ __forceinline__ void slab_store1(int i, const V16 &r, uint16_t *lds) {
  const int v = threadIdx.x + i * THREADS;
  uint16_t *q = KC ? lds + (v >> 3) * PK + (v & 7) * 8 : lds + (v >> 5) * PR + (v & 31) * 8;
  *reinterpret_cast<V16 *>(q) = r;
}
template <bool KC, int THREADS>
__device__ __forceinline__ void slab_load(V16 (&r)[2048 / THREADS], const uint16_t *p, int64_t ld) {
#pragma unroll
  for (int i = 0; i < 2048 / THREADS; i++) r[i] = slab_load1<KC, THREADS>(i, p, ld);
}
template <bool KC, int THREADS>
__device__ __forceinline__ void slab_store(const V16 (&r)[2048 / THREADS], uint16_t *lds) {
#pragma unroll
  for (int i = 0; i < 2048 / THREADS; i++) slab_store1<KC, THREADS>(i, r[i], lds);
}

// One MFMA operand fragment (8 k-values for this lane's row) for k-step `ks`
// (16 k-values per step) and the 32-row group starting at `row0`.
template <bool KC>
__device__ __forceinline__ V16 frag_load(const uint16_t *lds, int row0, int ks, int lane) {
  if constexpr (KC) {
    return *reinterpret_cast<const V16 *>(lds + (row0 + (lane & 31)) * PK + ks * 16 + (lane >> 5) * 8);
  } else {
    // source address of this lane for the transposing read (see the header)
    const int k = ks * 16 + (lane >> 5) * 8 + ((lane & 15) >> 2);
    const int r = row0 + ((lane >> 4) & 1) * 16 + (lane & 3) * 4;
    const uint16_t *q = lds + k * PR + r;
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)q);
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(q + 4 * PR));
    typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
    const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
    return V16{l2[0], l2[1], h2[0], h2[1]};
  }
}

// Tile order: blocks with the same id modulo 8 run on the same XCD. Give each
// XCD a contiguous run of the tile sequence, and make that sequence walk the
// output in 4-tile-tall column strips so neighbouring tiles share panels.
__device__ __forceinline__ void tile_of_block(const Args &a, uint32_t bid, uint32_t &batch, uint32_t &tm,
                                              uint32_t &tn) {
  const uint32_t total = a.tiles_m * a.tiles_n * a.nbatch;
  uint32_t t = bid;
  if ((total & 7u) == 0) {
    const uint32_t per_xcd = total >> 3;
    t = (bid & 7u) * per_xcd + (bid >> 3);
  }
  const uint32_t per_batch = a.tiles_m * a.tiles_n;
  batch = t / per_batch;
  uint32_t r = t - batch * per_batch;
  constexpr uint32_t G = 4;
  const uint32_t strip = r / (G * a.tiles_n);
  const uint32_t first_m = strip * G;
  const uint32_t gsz = a.tiles_m - first_m < G ? a.tiles_m - first_m : G;
  const uint32_t in_strip = r - strip * G * a.tiles_n;
  tm = first_m + in_strip % gsz;
  tn = in_strip / gsz;
}

// WM x WN waves per block; each wave owns (256 / WM) x (256 / WN) outputs.
template <bool BF16, bool A_KC, bool B_KC, int WM, int WN>
__global__ __launch_bounds__(64 * WM * WN) void kernel(Args a) {
  constexpr int THREADS = 64 * WM * WN;
  constexpr int TM = 256 / WM / 32, TN = 256 / WN / 32;  // MFMA tiles per wave
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  uint32_t batch, tm, tn;
  tile_of_block(a, blockIdx.x, batch, tm, tn);
  int64_t ao = 0, bo = 0, co = 0;
  {
    uint32_t idx = batch;
#pragma unroll
    for (int i = 3; i >= 0; i--) {  // constant indices keep the arguments out of scratch
      if (i < a.nbd) {
        uint32_t q = idx / a.bshape[i], c = idx - q * a.bshape[i];
        idx = q;
        ao += (int64_t)c * a.ba[i];
        bo += (int64_t)c * a.bb[i];
        co += (int64_t)c * a.bc[i];
      }
    }
  }
  const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;
  // slab origin and per-slab advance of each operand
  const uint16_t *gA = a.A + ao + (A_KC ? m0 * a.lda : m0);
  const uint16_t *gB = a.B + bo + (B_KC ? n0 * a.ldb : n0);
  const int64_t stepA = A_KC ? BK : (int64_t)BK * a.lda;
  const int64_t stepB = B_KC ? BK : (int64_t)BK * a.ldb;

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = (wave / WN) * (TM * 32), wn = (wave % WN) * (TN * 32);

  f32x16 acc[TM][TN];
#pragma unroll
  for (int t = 0; t < TM; t++)
#pragma unroll
    for (int u = 0; u < TN; u++)
#pragma unroll
      for (int e = 0; e < 16; e++) acc[t][u][e] = 0.0f;

  V16 ra[2048 / THREADS], rb[2048 / THREADS];
  const int nk = (int)(a.K / BK);
  slab_load<A_KC, THREADS>(ra, gA, a.lda);
  slab_load<B_KC, THREADS>(rb, gB, a.ldb);
  slab_store<A_KC, THREADS>(ra, smem);
  slab_store<B_KC, THREADS>(rb, smem + TILE_ELEMS);
  if (nk > 1) {
    // same issue order as in the main loop, so its in-order wait counts hold
#pragma unroll
    for (int i = 0; i < 2048 / THREADS; i++) {
      ra[i] = slab_load1<A_KC, THREADS>(i, gA + stepA, a.lda);
      rb[i] = slab_load1<B_KC, THREADS>(i, gB + stepB, a.ldb);
    }
  }
  __syncthreads();

  constexpr int NV = 2048 / THREADS, KSTEPS = BK / 16, VPS = NV / KSTEPS;  // staged vectors per k-step
  static_assert(NV % KSTEPS == 0, "staging is spread evenly over the k-steps");
  // One K-slab: multiply slab kt out of LDS; when STAGE, move slab kt+1 from
  // registers to the other LDS stage; when FETCH, start the loads of slab kt+2.
  // Fragments for step ks+1 are fetched while step ks multiplies, and the
  // staging traffic is spread over the k-steps, a few vectors between each group
  // of MFMAs, so no wave sits behind a full memory-instruction queue when it
  // could be issuing MFMAs. The steady state (both true) is free of branches.
  auto slab = [&](int kt, auto stage_c, auto fetch_c) {
    constexpr bool STAGE = decltype(stage_c)::value, FETCH = decltype(fetch_c)::value;
    const uint16_t *sA = smem + (kt & 1) * STAGE_ELEMS;
    const uint16_t *sB = sA + TILE_ELEMS;
    uint16_t *nA = smem + ((kt + 1) & 1) * STAGE_ELEMS;
    uint16_t *nB = nA + TILE_ELEMS;
    const uint16_t *pA = gA + (int64_t)(kt + 2) * stepA, *pB = gB + (int64_t)(kt + 2) * stepB;
    V16 fa[2][TM], fb[2][TN];
#pragma unroll
    for (int t = 0; t < TM; t++) fa[0][t] = frag_load<A_KC>(sA, wm + t * 32, 0, lane);
#pragma unroll
    for (int u = 0; u < TN; u++) fb[0][u] = frag_load<B_KC>(sB, wn + u * 32, 0, lane);
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) {
      const int cur = ks & 1, nxt = cur ^ 1;
      if (ks + 1 < KSTEPS) {
#pragma unroll
        for (int t = 0; t < TM; t++) fa[nxt][t] = frag_load<A_KC>(sA, wm + t * 32, ks + 1, lane);
#pragma unroll
        for (int u = 0; u < TN; u++) fb[nxt][u] = frag_load<B_KC>(sB, wn + u * 32, ks + 1, lane);
      }
      if constexpr (STAGE) {
#pragma unroll
        for (int j = 0; j < VPS; j++) {
          slab_store1<A_KC, THREADS>(ks * VPS + j, ra[ks * VPS + j], nA);
          slab_store1<B_KC, THREADS>(ks * VPS + j, rb[ks * VPS + j], nB);
        }
      }
      if constexpr (FETCH) {
#pragma unroll
        for (int j = 0; j < VPS; j++) {
          ra[ks * VPS + j] = slab_load1<A_KC, THREADS>(ks * VPS + j, pA, a.lda);
          rb[ks * VPS + j] = slab_load1<B_KC, THREADS>(ks * VPS + j, pB, a.ldb);
        }
      }
      // keep the order written here (LDS returns in order, so the wait before
      // the first MFMA only covers the current fragments)
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int t = 0; t < TM; t++)
#pragma unroll
        for (int u = 0; u < TN; u++) mfma16<BF16>(acc[t][u], fa[cur][t], fb[cur][u]);
      __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
  };
  using yes = std::integral_constant<bool, true>;
  using no = std::integral_constant<bool, false>;
  int kt = 0;
  for (; kt + 2 < nk; kt++) slab(kt, yes{}, yes{});
  if (kt + 1 < nk) slab(kt++, yes{}, no{});
  slab(kt, no{}, no{});

  // accumulator element e of lane l is C[(e/4)*8 + (l/32)*4 + e%4][l%32]
  uint16_t *C = a.C + co;
  const int r32 = lane & 31, kg = lane >> 5;
#pragma unroll
  for (int t = 0; t < TM; t++)
#pragma unroll
    for (int u = 0; u < TN; u++) {
      const int64_t col = n0 + wn + u * 32 + r32;
#pragma unroll
      for (int e = 0; e < 16; e++) {
        const int64_t row = m0 + wm + t * 32 + (e >> 2) * 8 + kg * 4 + (e & 3);
        C[row * a.ldc + col] = BF16 ? f32_to_bf16(acc[t][u][e]) : f32_to_f16(acc[t][u][e]);
      }
    }
}

}  // namespace gemm_big
