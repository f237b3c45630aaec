// gemm_tile.hpp — the LDS-tiled MFMA GEMM family: bf16 / f16 inputs
// (v_mfma_f32_32x32x16) and f32 inputs (v_mfma_f32_32x32x2, true f32), f32
// accumulation, behind batched [.., M, K] x [.., K, N] whenever K is a multiple
// of one slab (128 bytes of k: 64 / 32 elements) and the operands are 16-byte
// aligned.
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
// per slab, placed so that the next slab's first fragment reads overlap the
// current slab's last MFMAs. Inside a slab the work is software-pipelined by hand: the LDS
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
// scatter into LDS, no transposed copy in HBM. For f32 the [k][row] order is
// already what the 32x32x2 MFMA wants (one float per lane): four ds_read_b32.
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

// Element traits. VE = elements per 16-byte vector; a K-slab is 8 vectors (128
// bytes of k) per row, a k-step is 2 vectors: lanes 0-31 multiply the first VE
// k-values of a step, lanes 32-63 the second (any fixed assignment of k to
// lanes is valid as long as A and B agree).
struct ElBF16 {
  using S = uint16_t;
  static constexpr int VE = 8;
  static constexpr bool F32 = false, BF16 = true;
};
struct ElF16 {
  using S = uint16_t;
  static constexpr int VE = 8;
  static constexpr bool F32 = false, BF16 = false;
};
struct ElF32 {
  using S = float;
  static constexpr int VE = 4;
  static constexpr bool F32 = true, BF16 = false;
};
constexpr int KSTEPS = 4;

typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
typedef __attribute__((ext_vector_type(4))) uint32_t V16;  // one 16-byte register quad

// Tile geometry in elements of EL. PK: pitch of a [row][k] tile (+16 B). The
// [k][row] pitch adds 64 B for 16-bit tiles: the four k-rows a half-wave's
// transposing read touches then start 16 banks apart and its 32 lanes cover all 64
// banks once (with 32 B a 128-row tile's k-rows were 8 banks apart and met the
// lanes 16 rows further on: a fifth of its LDS cycles were bank conflicts); two
// 128x128 blocks still fit one CU's LDS. For f32 it adds 32 B, which puts the two
// k-rows a wave reads at once 32 banks apart.
template <class EL>
struct Geo {
  static constexpr int VE = EL::VE, BK = 8 * VE, PK = BK + VE;
  static constexpr int padr(int) { return EL::F32 ? 2 * VE : 4 * VE; }
  static constexpr int tile_elems(int rows) {
    return rows * PK > BK * (rows + padr(rows)) ? rows * PK : BK * (rows + padr(rows));
  }
};

template <int WM_, int WN_, int TM_, int TN_>
struct Shape {
  static constexpr int WM = WM_, WN = WN_, TM = TM_, TN = TN_;
  static constexpr int BM = WM * TM * 32, BN = WN * TN * 32, THREADS = 64 * WM * WN;
  // staged 16-byte vectors per lane and slab: rows x 8 vectors / THREADS
  static constexpr int NVA = BM * 8 / THREADS, NVB = BN * 8 / THREADS;
  static_assert(NVA >= 1 && NVB >= 1 && NVA * THREADS == BM * 8 && NVB * THREADS == BN * 8, "staging");
  // Two blocks of a four-wave shape fit a compute unit's LDS; they also fit its register
  // file when a wave stays within 256 registers (accumulators included), which the
  // kernel asks the compiler for: the second block hides the first one's load latency.
  static constexpr int WAVES_PER_SIMD = THREADS <= 256 ? 2 : 1;
  template <class EL>
  static constexpr int a_elems() { return Geo<EL>::tile_elems(BM); }
  template <class EL>
  static constexpr int stage_elems() { return Geo<EL>::tile_elems(BM) + Geo<EL>::tile_elems(BN); }
  template <class EL>
  static constexpr size_t lds_bytes() { return 2 * (size_t)stage_elems<EL>() * sizeof(typename EL::S); }
};
using Shape256x256 = Shape<4, 2, 2, 4>;
using Shape128x128 = Shape<2, 2, 2, 2>;
using Shape256x64 = Shape<4, 1, 2, 2>;
using Shape128x64 = Shape<2, 2, 2, 1>;
using Shape64x64 = Shape<2, 2, 1, 1>;

struct Args {
  const void *A, *B;
  void *C;
  int64_t lda, ldb, ldc;  // the non-unit stride of each matrix (elements)
  int64_t M, N, K;
  // Extents that may be LOADED along M / N (>= M / N, whole 16-byte vectors): an operand
  // contiguous along that dim may be padded past the logical edge.
  int64_t Mld, Nld;
  uint32_t tiles_m, tiles_n, nbatch;
  // batch offsets: up to 4 broadcastable batch dims
  int nbd;
  uint32_t bshape[4];
  int64_t ba[4], bb[4], bc[4];
  // EPI kernels only: out = round(round(round(A B) + bias[col]) + R), each step
  // skipped when its pointer is null. R has C's shape, unit column stride.
  const void *bias, *R;
  int64_t ldr, br[4];
  // EPI kernels, 16-bit dtypes, whole tiles, no R: then the tanh GELU of kaun/lib/fn.ml:31-38 on
  // the biased product, step by step with the roundings of its nine primitives
  // (c0..c3 = 0.044715, sqrt(2/pi), 1, 0.5 as the dtype holds them).
  int gelu;
  float gc[4];
  // bfloat16, direct-to-LDS kernels with room for it: the GELU by table. 2 * lut_n results
  // for the inputs with magnitude bits [lut_lo, lut_lo + lut_n) of either sign; below that
  // range the result is narrow(x * c3), above it x or -0, as the host has verified for every
  // input; infinities, NaN and the last finite binade take the arithmetic.
  const void *gelu_lut;
  uint32_t lut_lo, lut_n;
  // direct-to-LDS kernels without an epilogue: C is stored past the memory-side cache
  int stream_c;
  // EPI kernels: up to three products that share A and differ in (B, bias, C) of one shape and
  // layout, as one launch (the q / k / v linears of an attention layer): tile column tn of
  // the launch belongs to member tn / gtn. Offsets of members 1 and 2 from member 0, in elements.
  uint32_t ngroup, gtn;
  int64_t goff_b[2], goff_c[2], goff_bias[2];
};

// The arithmetic of the fused linear's epilogue on 16-bit results, two neighbours per
// register (low half first): every step is rounded to the dtype, as a primitive's store
// and the next primitive's load would. bf16 is widened by a shift and a mask and
// narrowed by one conversion of the pair.
template <class EL>
__device__ __forceinline__ void epi_widen2(uint32_t x, float &lo, float &hi) {
  if constexpr (EL::BF16) {
    lo = __builtin_bit_cast(float, x << 16);
    hi = __builtin_bit_cast(float, x & 0xffff0000u);
  } else {
    lo = f16_to_f32((uint16_t)(x & 0xffffu));
    hi = f16_to_f32((uint16_t)(x >> 16));
  }
}
template <class EL>
__device__ __forceinline__ uint32_t epi_narrow2(float lo, float hi) {
  if constexpr (EL::BF16) return f32x2_to_bf16x2(lo, hi);
  else return (uint32_t)f32_to_f16(lo) | ((uint32_t)f32_to_f16(hi) << 16);
}
template <class EL>
__device__ __forceinline__ void epi_rnd2(float &lo, float &hi) {
  epi_widen2<EL>(epi_narrow2<EL>(lo, hi), lo, hi);
}
template <class EL>
__device__ __forceinline__ uint32_t epi_add2(uint32_t x, uint32_t y) {
  float x0, x1, y0, y1;
  epi_widen2<EL>(x, x0, x1);
  epi_widen2<EL>(y, y0, y1);
  return epi_narrow2<EL>(x0 + y0, x1 + y1);
}
// The tanh GELU of kaun/lib/fn.ml:31-38, primitive by primitive; c0..c3 = 0.044715,
// sqrt(2/pi), 1, 0.5 as the dtype holds them.
template <class EL>
__device__ __forceinline__ uint32_t epi_gelu2(uint32_t x, float c0, float c1, float c2, float c3) {
  float v0, v1;
  epi_widen2<EL>(x, v0, v1);
  float a0 = v0 * v0, a1 = v1 * v1;  // x * x
  epi_rnd2<EL>(a0, a1);
  a0 = v0 * a0, a1 = v1 * a1;        // x * (x * x)
  epi_rnd2<EL>(a0, a1);
  a0 = a0 * c0, a1 = a1 * c0;
  epi_rnd2<EL>(a0, a1);
  a0 = v0 + a0, a1 = v1 + a1;
  epi_rnd2<EL>(a0, a1);
  a0 = a0 * c1, a1 = a1 * c1;
  epi_rnd2<EL>(a0, a1);
  a0 = tanh_for_16bit(a0), a1 = tanh_for_16bit(a1);
  epi_rnd2<EL>(a0, a1);
  a0 = a0 + c2, a1 = a1 + c2;
  epi_rnd2<EL>(a0, a1);
  a0 = v0 * a0, a1 = v1 * a1;
  epi_rnd2<EL>(a0, a1);
  a0 = a0 * c3, a1 = a1 * c3;
  return epi_narrow2<EL>(a0, a1);
}

// The same function for two bfloat16 neighbours through the LDS copy of the table
// (Args::gelu_lut). The caller has sent registers holding an input of the last finite
// binade, an infinity or a NaN (magnitude bits >= 0x7f00) to epi_gelu2 instead.
__device__ __forceinline__ uint32_t epi_gelu_lut2(uint32_t x, const uint16_t *lut, uint32_t lo, uint32_t n, float c3) {
  float v0, v1;
  v0 = __builtin_bit_cast(float, x << 16);
  v1 = __builtin_bit_cast(float, x & 0xffff0000u);
  const uint32_t small = f32x2_to_bf16x2(v0 * c3, v1 * c3);
  uint32_t out = 0;
#pragma unroll
  for (int h = 0; h < 2; h++) {
    const uint32_t e = h ? x >> 16 : x & 0xffffu;
    const uint32_t m = e & 0x7fffu, neg = e >> 15;
    const uint32_t idx = m - lo;  // (wraps below the range)
    const uint32_t at = (idx < n ? idx : n - 1) + neg * n;
    const uint32_t t = lut[at];
    const uint32_t big = neg ? 0x8000u : e;
    const uint32_t sm = h ? small >> 16 : small & 0xffffu;
    const uint32_t r = m < lo ? sm : (idx < n ? t : big);
    out |= r << (16 * h);
  }
  return out;
}

// One k-step of one 32x32 tile: a, b hold this lane's VE k-values of its row.
template <class EL>
__device__ __forceinline__ void mfma_step(f32x16 &acc, const V16 &a, const V16 &b) {
  if constexpr (EL::F32) {
    const f32x4 x = __builtin_bit_cast(f32x4, a), y = __builtin_bit_cast(f32x4, b);
#pragma unroll
    for (int s = 0; s < 4; s++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(x[s], y[s], acc, 0, 0, 0);
  } else if constexpr (EL::BF16) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), acc, 0, 0, 0);
  } else {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), acc, 0, 0, 0);
  }
}

// Global -> registers -> LDS, one 16-byte vector at a time: vector i of this lane
// of one operand's ROWS x BK slab. KC: rows are 128 B apart in the slab (8
// vectors per row); otherwise the slab is BK k-rows of ROWS elements (ROWS / VE
// vectors per k-row). `edge` is the number of valid rows from the slab's
// origin (EDGE only).
template <class EL, bool KC, int ROWS, int THREADS, bool EDGE>
__device__ __forceinline__ V16 slab_load1(int i, const typename EL::S *p, int64_t ld, int edge) {
  constexpr int VE = EL::VE;
  const int v = threadIdx.x + i * THREADS;
  if constexpr (KC) {
    int row = v >> 3;
    if constexpr (EDGE) row = row < edge ? row : edge - 1;
    return *reinterpret_cast<const V16 *>(p + (int64_t)row * ld + (v & 7) * VE);
  } else {
    constexpr int VPR = ROWS / VE;
    int c = (v % VPR) * VE;
    if constexpr (EDGE) c = c + VE <= edge ? c : edge - VE;
    return *reinterpret_cast<const V16 *>(p + (int64_t)(v / VPR) * ld + c);
  }
}
template <class EL, bool KC, int ROWS, int THREADS>
__device__ __forceinline__ void slab_store1(int i, const V16 &r, typename EL::S *lds) {
  using G = Geo<EL>;
  constexpr int VE = EL::VE, VPR = ROWS / VE;
  const int v = threadIdx.x + i * THREADS;
  typename EL::S *q = KC ? lds + (v >> 3) * G::PK + (v & 7) * VE : lds + (v / VPR) * (ROWS + G::padr(ROWS)) + (v % VPR) * VE;
  *reinterpret_cast<V16 *>(q) = r;
}

// One MFMA operand fragment (VE k-values for this lane's row) for k-step `ks`
// (2 * VE k-values per step) and the 32-row group starting at `row0`.
template <class EL, bool KC, int ROWS>
__device__ __forceinline__ V16 frag_load(const typename EL::S *lds, int row0, int ks, int lane) {
  using G = Geo<EL>;
  constexpr int VE = EL::VE;
  if constexpr (KC) {
    return *reinterpret_cast<const V16 *>(lds + (row0 + (lane & 31)) * G::PK + ks * 2 * VE + (lane >> 5) * VE);
  } else if constexpr (EL::F32) {
    constexpr int PR = ROWS + G::padr(ROWS);
    const float *q = lds + (ks * 2 * VE + (lane >> 5) * VE) * PR + row0 + (lane & 31);
    const f32x4 x = {q[0], q[PR], q[2 * PR], q[3 * PR]};
    return __builtin_bit_cast(V16, x);
  } else {
    // source address of this lane for the transposing read (see the header)
    constexpr int PR = ROWS + G::padr(ROWS);
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

// OUT32: the f32 sums are stored as they are (C is float, `ldc` and the batch strides in floats):
// the partial sums of a product cut along K, added up by a second kernel.
template <class EL, bool A_KC, bool B_KC, class SH, bool EDGE, bool EPI = false, bool OUT32 = false>
__global__ __launch_bounds__(SH::THREADS) __attribute__((amdgpu_waves_per_eu(SH::WAVES_PER_SIMD))) void kernel(Args a) {
  constexpr int THREADS = SH::THREADS, BM = SH::BM, BN = SH::BN, TM = SH::TM, TN = SH::TN;
  constexpr int NVA = SH::NVA, NVB = SH::NVB, BK = Geo<EL>::BK;
  constexpr int A_ELEMS = SH::template a_elems<EL>(), STAGE_ELEMS = SH::template stage_elems<EL>();
  using S = typename EL::S;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  S *smem = reinterpret_cast<S *>(smem_raw);
  uint32_t batch, tm, tn;
  // tiles are walked from the end: an operand the previous kernel has just written
  // front to back still has its tail in the memory-side cache
  tile_of_block(a, gridDim.x - 1 - blockIdx.x, batch, tm, tn);
  int64_t ao = 0, bo = 0, co = 0, ro = 0;
  if constexpr (EPI) {
    if (a.ngroup > 1) {
      const uint32_t member = tn / a.gtn;
      tn -= member * a.gtn;
      if (member) {
        bo = member == 1 ? a.goff_b[0] : a.goff_b[1];
        co = member == 1 ? a.goff_c[0] : a.goff_c[1];
        if (a.bias) a.bias = (const S *)a.bias + (member == 1 ? a.goff_bias[0] : a.goff_bias[1]);
      }
    }
  }
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
        if constexpr (EPI) ro += (int64_t)c * a.br[i];
      }
    }
  }
  const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;
  const int edge_m = EDGE ? (int)(a.M - m0 < BM ? a.M - m0 : BM) : BM;
  const int edge_n = EDGE ? (int)(a.N - n0 < BN ? a.N - n0 : BN) : BN;
  // a k-contiguous operand clamps its rows to the logical edge; one contiguous along M / N
  // clamps its vectors to the loadable extent
  const int ledge_m = EDGE && !A_KC ? (int)(a.Mld - m0 < BM ? a.Mld - m0 : BM) : edge_m;
  const int ledge_n = EDGE && !B_KC ? (int)(a.Nld - n0 < BN ? a.Nld - n0 : BN) : edge_n;
  // slab origin and per-slab advance of each operand
  const S *gA = (const S *)a.A + ao + (A_KC ? m0 * a.lda : m0);
  const S *gB = (const S *)a.B + bo + (B_KC ? n0 * a.ldb : n0);
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
  auto fetch_step = [&](int ks, const S *pA, const S *pB) {
#pragma unroll
    for (int i = 0; i < (NVA > NVB ? NVA : NVB); i++) {
      if (i % KSTEPS != ks) continue;
      if (i < NVA) ra[i] = slab_load1<EL, A_KC, BM, THREADS, EDGE>(i, pA, a.lda, ledge_m);
      if (i < NVB) rb[i] = slab_load1<EL, B_KC, BN, THREADS, EDGE>(i, pB, a.ldb, ledge_n);
    }
  };
  auto stage_step = [&](int ks, S *nA, S *nB) {
#pragma unroll
    for (int i = 0; i < (NVA > NVB ? NVA : NVB); i++) {
      if (i % KSTEPS != ks) continue;
      if (i < NVA) slab_store1<EL, A_KC, BM, THREADS>(i, ra[i], nA);
      if (i < NVB) slab_store1<EL, B_KC, BN, THREADS>(i, rb[i], nB);
    }
  };
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ks++) fetch_step(ks, gA, gB);
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ks++) stage_step(ks, smem, smem + A_ELEMS);
  if (nk > 1) {
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) fetch_step(ks, gA + stepA, gB + stepB);
  }
  __syncthreads();

  // One K-slab: multiply slab kt out of LDS; when STAGE, move slab kt+1 from
  // registers to the other LDS stage; when FETCH, start the loads of slab kt+2.
  // The steady state (both true) is free of branches. The block's one barrier per
  // slab sits in the LAST k-step, after this wave's share of slab kt+1 has been
  // written: by then every wave has also issued (and waited for) its last
  // fragment reads of slab kt, so the next slab's first fragments can be fetched
  // right behind the barrier, under the MFMAs of the last k-step, and no LDS
  // latency is exposed at the slab boundary.
  V16 fa[2][TM], fb[2][TN];
#pragma unroll
  for (int t = 0; t < TM; t++) fa[0][t] = frag_load<EL, A_KC, BM>(smem, wm + t * 32, 0, lane);
#pragma unroll
  for (int u = 0; u < TN; u++) fb[0][u] = frag_load<EL, B_KC, BN>(smem + A_ELEMS, wn + u * 32, 0, lane);
  auto slab = [&](int kt, auto stage_c, auto fetch_c) {
    constexpr bool STAGE = decltype(stage_c)::value, FETCH = decltype(fetch_c)::value;
    const S *sA = smem + (kt & 1) * STAGE_ELEMS;
    const S *sB = sA + A_ELEMS;
    S *nA = smem + ((kt + 1) & 1) * STAGE_ELEMS;
    S *nB = nA + A_ELEMS;
    const S *pA = gA + (int64_t)(kt + 2) * stepA, *pB = gB + (int64_t)(kt + 2) * stepB;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) {
      const int cur = ks & 1, nxt = cur ^ 1;
      if constexpr (STAGE) stage_step(ks, nA, nB);
      if constexpr (FETCH) fetch_step(ks, pA, pB);
      if (ks + 1 < KSTEPS) {
#pragma unroll
        for (int t = 0; t < TM; t++) fa[nxt][t] = frag_load<EL, A_KC, BM>(sA, wm + t * 32, ks + 1, lane);
#pragma unroll
        for (int u = 0; u < TN; u++) fb[nxt][u] = frag_load<EL, B_KC, BN>(sB, wn + u * 32, ks + 1, lane);
      } else if constexpr (STAGE) {
        __syncthreads();  // slab kt+1 is complete in LDS; nobody reads slab kt's buffer any more
#pragma unroll
        for (int t = 0; t < TM; t++) fa[nxt][t] = frag_load<EL, A_KC, BM>(nA, wm + t * 32, 0, lane);
#pragma unroll
        for (int u = 0; u < TN; u++) fb[nxt][u] = frag_load<EL, B_KC, BN>(nB, wn + u * 32, 0, lane);
      }
#pragma unroll
      for (int t = 0; t < TM; t++)
#pragma unroll
        for (int u = 0; u < TN; u++) mfma_step<EL>(acc[t][u], fa[cur][t], fb[cur][u]);
      // The memory instructions of this k-step are issued among its MFMAs, one LDS read, one
      // LDS write and one global load behind each (LDS returns in order, so the wait before the
      // first MFMA only covers the current fragments): queueing them all in front of the step
      // left the matrix pipe cold while they issued.
#pragma unroll
      for (int x = 0; x < TM * TN * (EL::F32 ? 4 : 1); x++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);  // LDS reads
        __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);  // LDS write
        __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // global load
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  using yes = std::integral_constant<bool, true>;
  using no = std::integral_constant<bool, false>;
  int kt = 0;
  for (; kt + 2 < nk; kt++) slab(kt, yes{}, yes{});
  if (kt + 1 < nk) slab(kt++, yes{}, no{});
  slab(kt, no{}, no{});

  // accumulator element e of lane l is C[(e/4)*8 + (l/32)*4 + e%4][l%32]
  S *C = (S *)a.C + co;
  const int r32 = lane & 31, kg = lane >> 5;
  auto narrow = [](float x) -> S {
    if constexpr (EL::F32) return x;
    else return EL::BF16 ? f32_to_bf16(x) : f32_to_f16(x);
  };
  auto widen = [](S x) -> float {
    if constexpr (EL::F32) return x;
    else return EL::BF16 ? bf16_to_f32(x) : f16_to_f32(x);
  };
  if constexpr (OUT32 && !EL::F32) {
    float *Cf = (float *)a.C + co;
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
          Cf[(m0 + rl) * a.ldc + n0 + cl] = acc[t][u][e];
        }
      }
    return;
  }
  if constexpr (!EL::F32) {
    // 16-bit outputs go through LDS: in accumulator order a lane would store
    // (and, with a residual, load) two bytes at a time. Each wave parks its
    // rounded TM*32 x TN*32 patch in a private piece of the (now idle) stage
    // buffers and sends it out as whole 16-byte row segments.
    constexpr int WC = TN * 32, WP = WC + 8;  // patch width and its LDS pitch (elements)
    static_assert((size_t)SH::WM * SH::WN * TM * 32 * WP * sizeof(S) <= SH::template lds_bytes<EL>(), "epilogue patch");
    const bool wide = ((uintptr_t)C % 16) == 0 && a.ldc % 8 == 0 &&
                      (!EPI || ((!a.bias || (uintptr_t)a.bias % 16 == 0) &&
                                (!a.R || (((uintptr_t)((const S *)a.R + ro)) % 16 == 0 && a.ldr % 8 == 0))));
    if (wide) {
      __syncthreads();  // every wave has read its last fragments
      S *patch = smem + wave * (TM * 32 * WP);
#pragma unroll
      for (int t = 0; t < TM; t++)
#pragma unroll
        for (int u = 0; u < TN; u++)
#pragma unroll
          for (int e = 0; e < 16; e++)
            patch[(t * 32 + (e >> 2) * 8 + kg * 4 + (e & 3)) * WP + u * 32 + r32] = narrow(acc[t][u][e]);
      // the patch is read back by other lanes of the same wave only: LDS serves a wave in order
      constexpr int CPR = WC / 8;  // 16-byte chunks per patch row
      if constexpr (EPI && !EDGE) {
        // Whole tiles of the fused linear: a lane keeps one column chunk for all its rows,
        // so the bias is read once, and every residual chunk is requested before the
        // first one is used. (Written as one loop with the loads where they are
        // consumed, each row waited for its own global load: 67 us against the plain
        // product's 51 at [8192,768] x [768,3072].)
        static_assert(64 % CPR == 0, "a lane's chunk column is the same in every pass");
        constexpr int NIT = TM * 32 * CPR / 64, RSTEP = 64 / CPR;
        const int col = (lane % CPR) * 8, row0 = lane / CPR;
        auto add2 = [](uint32_t x, uint32_t y) -> uint32_t { return epi_add2<EL>(x, y); };
        auto gelu2 = [&](uint32_t x) -> uint32_t { return epi_gelu2<EL>(x, a.gc[0], a.gc[1], a.gc[2], a.gc[3]); };
        S *c = C + (m0 + wm + row0) * a.ldc + n0 + wn + col;
        const S *p = patch + row0 * WP + col;
        V16 bq = {0, 0, 0, 0};
        if (a.bias) bq = *reinterpret_cast<const V16 *>((const S *)a.bias + n0 + wn + col);
        if (a.R) {
          const S *rp = (const S *)a.R + ro + (m0 + wm + row0) * a.ldr + n0 + wn + col;
          V16 rq[NIT];
#pragma unroll
          for (int i = 0; i < NIT; i++) rq[i] = *reinterpret_cast<const V16 *>(rp + (int64_t)i * RSTEP * a.ldr);
#pragma unroll
          for (int i = 0; i < NIT; i++) {
            V16 q = *reinterpret_cast<const V16 *>(p + i * RSTEP * WP);
#pragma unroll
            for (int w = 0; w < 4; w++) {
              if (a.bias) q[w] = add2(q[w], bq[w]);
              q[w] = add2(q[w], rq[i][w]);
            }
            *reinterpret_cast<V16 *>(c + (int64_t)i * RSTEP * a.ldc) = q;
          }
        } else {
#pragma unroll
          for (int i = 0; i < NIT; i++) {
            V16 q = *reinterpret_cast<const V16 *>(p + i * RSTEP * WP);
            if (a.bias) {
#pragma unroll
              for (int w = 0; w < 4; w++) q[w] = add2(q[w], bq[w]);
            }
            if (a.gelu) {
#pragma unroll
              for (int w = 0; w < 4; w++) q[w] = gelu2(q[w]);
            }
            *reinterpret_cast<V16 *>(c + (int64_t)i * RSTEP * a.ldc) = q;
          }
        }
        return;
      }
#pragma unroll
      for (int i = 0; i < TM * 32 * CPR / 64; i++) {
        const int ch = i * 64 + lane, row = ch / CPR, col = (ch % CPR) * 8;
        const int rl = wm + row, cl = wn + col;
        if (EDGE && (rl >= edge_m || cl >= edge_n)) continue;
        union {
          V16 q;
          S s[8];
        } v, bb, rr;
        v.q = *reinterpret_cast<const V16 *>(patch + row * WP + col);
        S *c = C + (m0 + rl) * a.ldc + n0 + cl;
        const bool whole = !EDGE || cl + 8 <= edge_n;
        if constexpr (EPI) {
          const S *bp = (const S *)a.bias + n0 + cl;
          const S *rp = (const S *)a.R + ro + (m0 + rl) * a.ldr + n0 + cl;
          if (whole) {
            if (a.bias) bb.q = *reinterpret_cast<const V16 *>(bp);
            if (a.R) rr.q = *reinterpret_cast<const V16 *>(rp);
          } else {
#pragma unroll
            for (int j = 0; j < 8; j++)
              if (cl + j < edge_n) {
                if (a.bias) bb.s[j] = bp[j];
                if (a.R) rr.s[j] = rp[j];
              }
          }
          // the bias add and the residual add of the op-by-op sequence, each rounded to the dtype
          if constexpr (EL::BF16) {
            // two neighbours per register: widened by a shift and a mask, narrowed by one conversion
            auto add2 = [](uint32_t x, uint32_t y) {
              const float lo = __builtin_bit_cast(float, x << 16) + __builtin_bit_cast(float, y << 16);
              const float hi = __builtin_bit_cast(float, x & 0xffff0000u) + __builtin_bit_cast(float, y & 0xffff0000u);
              return f32x2_to_bf16x2(lo, hi);
            };
#pragma unroll
            for (int w = 0; w < 4; w++) {
              if (a.bias) v.q[w] = add2(v.q[w], bb.q[w]);
              if (a.R) v.q[w] = add2(v.q[w], rr.q[w]);
            }
          } else {
#pragma unroll
            for (int j = 0; j < 8; j++) {
              if (a.bias) v.s[j] = narrow(widen(v.s[j]) + widen(bb.s[j]));
              if (a.R) v.s[j] = narrow(widen(v.s[j]) + widen(rr.s[j]));
            }
          }
        }
        if (whole) *reinterpret_cast<V16 *>(c) = v.q;
        else
#pragma unroll
          for (int j = 0; j < 8; j++)
            if (cl + j < edge_n) c[j] = v.s[j];
      }
      return;
    }
  }
#pragma unroll
  for (int t = 0; t < TM; t++)
#pragma unroll
    for (int u = 0; u < TN; u++) {
      const int cl = wn + u * 32 + r32;
      if (EDGE && cl >= edge_n) continue;
      float bias = 0.0f;
      if constexpr (EPI)
        if (a.bias) bias = widen(((const S *)a.bias)[n0 + cl]);
#pragma unroll
      for (int e = 0; e < 16; e++) {
        const int rl = wm + t * 32 + (e >> 2) * 8 + kg * 4 + (e & 3);
        if (EDGE && rl >= edge_m) continue;
        S *c = C + (m0 + rl) * a.ldc + n0 + cl;
        S v = narrow(acc[t][u][e]);
        if constexpr (EPI) {
          // the bias add and the residual add of the op-by-op sequence, each rounded to the dtype
          if (a.bias) v = narrow(widen(v) + bias);
          if (a.R) v = narrow(widen(v) + widen(((const S *)a.R)[ro + (m0 + rl) * a.ldr + n0 + cl]));
        }
        *c = v;
      }
    }
}

}  // namespace gemm_tile
