// gemm_tile.hpp — the LDS-tiled MFMA GEMM family for 16-bit inputs (bf16 / f16)
// with f32 accumulation, behind batched [.., M, K] x [.., K, N] whenever K is a
// multiple of 64 and the operands are 16-byte aligned.
//
// One kernel template, three block shapes (BM x BN outputs per block, each of
// the WM x WN wave64s owning TM x TN tiles of v_mfma_f32_32x32x16):
//   256 x 256  8 waves of 64 x 128   large products: most reuse per byte
//   128 x 128  4 waves of 64 x 64    products whose 256-tiles would not fill
//                                    the chip (GPT-2 linears: N = 768)
//   256 x  64  4 waves of 64 x 64    narrow outputs (probs x V: N = 64), bound
//                                    by streaming A
// Common structure: K-slab 64, LDS double-buffered, global -> registers -> LDS
// with the loads for slab t+2 in flight while slab t is multiplied, one barrier
// per slab. Inside a slab the work is software-pipelined by hand: the LDS
// fragment reads of k-step s+1, a share of the register -> LDS stores of slab
// t+1 and of the global loads of slab t+2 are issued in front of the MFMAs of
// k-step s (scheduling barriers keep the compiler from regrouping them), so
// memory instructions never queue up in front of the matrix pipe.
// An operand that is contiguous along K sits in LDS as [row][k] (+16 B pad) and
// is fetched with ds_read_b128. An operand that is contiguous along M / N (a
// row-major B) stays in its memory order, [k][row] (+32 or 64 B pad), and the
// k-contiguous fragments MFMA wants are produced by the transposing LDS read
// ds_read_b64_tr_b16: within each group of 16 lanes, result element j of lane L
// is element (L & 3) of the 8 bytes addressed by lane 4*j + (L >> 2). No 2-byte
// scatter into LDS, no transposed copy in HBM.
// Ragged M / N (EDGE): loads of rows past the edge are redirected to the last
// valid row (or, along a contiguous M / N, to the last whole 8-element vector),
// which only feeds outputs that are never stored; stores are bounds-checked.
// Block ids are remapped so that the blocks resident on one XCD (ids equal
// modulo 8) cover a compact patch of tiles and share A / B panels in that XCD's
// L2.
#pragma once

#include "nxh_common.hpp"

#include <type_traits>

namespace gemm_tile {

constexpr int BK = 64;
constexpr int PK = BK + 8;  // pitch (elements) of a [row][k] tile
// pad (elements) of a [k][row] tile's pitch: 64 B for 256-row tiles, 32 B for
// the smaller ones (two 128x128 blocks then fit one CU's LDS)
constexpr int padr(int rows) { return rows >= 256 ? 32 : 16; }

typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
typedef __attribute__((ext_vector_type(4))) uint32_t V16;  // one 16-byte register quad

template <int WM_, int WN_, int TM_, int TN_>
struct Shape {
  static constexpr int WM = WM_, WN = WN_, TM = TM_, TN = TN_;
  static constexpr int BM = WM * TM * 32, BN = WN * TN * 32, THREADS = 64 * WM * WN;
  // LDS elements of one operand tile: [rows][PK] or [BK][rows + pad]
  static constexpr int tile_elems(int rows) { return rows * PK > BK * (rows + padr(rows)) ? rows * PK : BK * (rows + padr(rows)); }
  static constexpr int A_ELEMS = tile_elems(BM), B_ELEMS = tile_elems(BN);
  static constexpr int STAGE_ELEMS = A_ELEMS + B_ELEMS;
  static constexpr size_t LDS_BYTES = 2 * (size_t)STAGE_ELEMS * sizeof(uint16_t);
  static constexpr int NVA = BM * BK / 8 / THREADS, NVB = BN * BK / 8 / THREADS;  // staged vectors per lane
  static_assert(NVA >= 1 && NVB >= 1 && NVA * THREADS * 8 == BM * BK && NVB * THREADS * 8 == BN * BK, "staging");
};
using Shape256x256 = Shape<4, 2, 2, 4>;
using Shape128x128 = Shape<2, 2, 2, 2>;
using Shape256x64 = Shape<4, 1, 2, 2>;

struct Args {
  const uint16_t *A, *B;
  uint16_t *C;
  int64_t lda, ldb, ldc;  // the non-unit stride of each matrix (elements)
  int64_t M, N, K;
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
// of one operand's ROWS x 64 slab. KC: rows are 128 B apart in the slab (8
// vectors per row); otherwise the slab is 64 k-rows of ROWS elements (ROWS / 8
// vectors per k-row). `edge` is the number of valid rows from the slab's
// origin (EDGE only).
template <bool KC, int ROWS, int THREADS, bool EDGE>
__device__ __forceinline__ V16 slab_load1(int i, const uint16_t *p, int64_t ld, int edge) {
  const int v = threadIdx.x + i * THREADS;
  if constexpr (KC) {
    int row = v >> 3;
    if constexpr (EDGE) row = row < edge ? row : edge - 1;
    return *reinterpret_cast<const V16 *>(p + (int64_t)row * ld + (v & 7) * 8);
  } else {
    constexpr int VPR = ROWS / 8;
    int c = (v % VPR) * 8;
    if constexpr (EDGE) c = c + 8 <= edge ? c : edge - 8;
    return *reinterpret_cast<const V16 *>(p + (int64_t)(v / VPR) * ld + c);
  }
}
template <bool KC, int ROWS, int THREADS>
__device__ __forceinline__ void slab_store1(int i, const V16 &r, uint16_t *lds) {
  const int v = threadIdx.x + i * THREADS;
  constexpr int VPR = ROWS / 8;
  uint16_t *q = KC ? lds + (v >> 3) * PK + (v & 7) * 8 : lds + (v / VPR) * (ROWS + padr(ROWS)) + (v % VPR) * 8;
  *reinterpret_cast<V16 *>(q) = r;
}

// One MFMA operand fragment (8 k-values for this lane's row) for k-step `ks`
// (16 k-values per step) and the 32-row group starting at `row0`.
template <bool KC, int ROWS>
__device__ __forceinline__ V16 frag_load(const uint16_t *lds, int row0, int ks, int lane) {
  if constexpr (KC) {
    return *reinterpret_cast<const V16 *>(lds + (row0 + (lane & 31)) * PK + ks * 16 + (lane >> 5) * 8);
  } else {
    // source address of this lane for the transposing read (see the header)
    constexpr int PR = ROWS + padr(ROWS);
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

template <bool BF16, bool A_KC, bool B_KC, class SH, bool EDGE>
__global__ __launch_bounds__(SH::THREADS) void kernel(Args a) {
  constexpr int THREADS = SH::THREADS, BM = SH::BM, BN = SH::BN, TM = SH::TM, TN = SH::TN;
  constexpr int NVA = SH::NVA, NVB = SH::NVB, KSTEPS = BK / 16;
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
  const int edge_m = EDGE ? (int)(a.M - m0 < BM ? a.M - m0 : BM) : BM;
  const int edge_n = EDGE ? (int)(a.N - n0 < BN ? a.N - n0 : BN) : BN;
  // slab origin and per-slab advance of each operand
  const uint16_t *gA = a.A + ao + (A_KC ? m0 * a.lda : m0);
  const uint16_t *gB = a.B + bo + (B_KC ? n0 * a.ldb : n0);
  const int64_t stepA = A_KC ? BK : (int64_t)BK * a.lda;
  const int64_t stepB = B_KC ? BK : (int64_t)BK * a.ldb;

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = (wave / SH::WN) * (TM * 32), wn = (wave % SH::WN) * (TN * 32);

  f32x16 acc[TM][TN];
#pragma unroll
  for (int t = 0; t < TM; t++)
#pragma unroll
    for (int u = 0; u < TN; u++)
#pragma unroll
      for (int e = 0; e < 16; e++) acc[t][u][e] = 0.0f;

  V16 ra[NVA], rb[NVB];
  const int nk = (int)(a.K / BK);
  // Staged vector i of an operand moves at k-step i % KSTEPS; the prologue uses
  // the same issue order, so the loop's in-order wait counts hold from the start.
  auto fetch_step = [&](int ks, const uint16_t *pA, const uint16_t *pB) {
#pragma unroll
    for (int i = 0; i < (NVA > NVB ? NVA : NVB); i++) {
      if (i % KSTEPS != ks) continue;
      if (i < NVA) ra[i] = slab_load1<A_KC, BM, THREADS, EDGE>(i, pA, a.lda, edge_m);
      if (i < NVB) rb[i] = slab_load1<B_KC, BN, THREADS, EDGE>(i, pB, a.ldb, edge_n);
    }
  };
  auto stage_step = [&](int ks, uint16_t *nA, uint16_t *nB) {
#pragma unroll
    for (int i = 0; i < (NVA > NVB ? NVA : NVB); i++) {
      if (i % KSTEPS != ks) continue;
      if (i < NVA) slab_store1<A_KC, BM, THREADS>(i, ra[i], nA);
      if (i < NVB) slab_store1<B_KC, BN, THREADS>(i, rb[i], nB);
    }
  };
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ks++) fetch_step(ks, gA, gB);
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ks++) stage_step(ks, smem, smem + SH::A_ELEMS);
  if (nk > 1) {
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) fetch_step(ks, gA + stepA, gB + stepB);
  }
  __syncthreads();

  // One K-slab: multiply slab kt out of LDS; when STAGE, move slab kt+1 from
  // registers to the other LDS stage; when FETCH, start the loads of slab kt+2.
  // The steady state (both true) is free of branches.
  auto slab = [&](int kt, auto stage_c, auto fetch_c) {
    constexpr bool STAGE = decltype(stage_c)::value, FETCH = decltype(fetch_c)::value;
    const uint16_t *sA = smem + (kt & 1) * SH::STAGE_ELEMS;
    const uint16_t *sB = sA + SH::A_ELEMS;
    uint16_t *nA = smem + ((kt + 1) & 1) * SH::STAGE_ELEMS;
    uint16_t *nB = nA + SH::A_ELEMS;
    const uint16_t *pA = gA + (int64_t)(kt + 2) * stepA, *pB = gB + (int64_t)(kt + 2) * stepB;
    V16 fa[2][TM], fb[2][TN];
#pragma unroll
    for (int t = 0; t < TM; t++) fa[0][t] = frag_load<A_KC, BM>(sA, wm + t * 32, 0, lane);
#pragma unroll
    for (int u = 0; u < TN; u++) fb[0][u] = frag_load<B_KC, BN>(sB, wn + u * 32, 0, lane);
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) {
      const int cur = ks & 1, nxt = cur ^ 1;
      if (ks + 1 < KSTEPS) {
#pragma unroll
        for (int t = 0; t < TM; t++) fa[nxt][t] = frag_load<A_KC, BM>(sA, wm + t * 32, ks + 1, lane);
#pragma unroll
        for (int u = 0; u < TN; u++) fb[nxt][u] = frag_load<B_KC, BN>(sB, wn + u * 32, ks + 1, lane);
      }
      if constexpr (STAGE) stage_step(ks, nA, nB);
      if constexpr (FETCH) fetch_step(ks, pA, pB);
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
      const int cl = wn + u * 32 + r32;
      if (EDGE && cl >= edge_n) continue;
#pragma unroll
      for (int e = 0; e < 16; e++) {
        const int rl = wm + t * 32 + (e >> 2) * 8 + kg * 4 + (e & 3);
        if (EDGE && rl >= edge_m) continue;
        C[(m0 + rl) * a.ldc + n0 + cl] = BF16 ? f32_to_bf16(acc[t][u][e]) : f32_to_f16(acc[t][u][e]);
      }
    }
}

}  // namespace gemm_tile
