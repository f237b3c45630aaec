// matmul.hip — batched matrix multiply.
//
// Contract restated from packages/nx/lib/backend_c/nx_c_matmul.c:874-1108:
// [.., m, k] x [.., k, n] with batch dims broadcast by stride 0, arbitrary
// element strides on both inputs, products accumulated in the dtype's compute
// type (f32 for bf16/f16/f32/fp8, f64, int64/uint64 modular, complex) and
// rounded to storage ONCE per output element (nx_c_matmul.c:347-361, 424-440);
// k == 0 stores zeros.
//
// Kernels
//   gemm_mfma   bf16 / f16 (v_mfma_f32_32x32x16) and f32 (v_mfma_f32_32x32x2,
//               true f32, no xf32): 128x128 block tile, four wave64s each
//               owning 64x64 (2x2 MFMA tiles), K-contiguous LDS tiles with a
//               16-byte pad per row, global->register prefetch of the next
//               K-slab while the current one is multiplied. Either operand may
//               be K-contiguous or M/N-contiguous in memory; the turn happens
//               on the way into LDS.
//   gemm_tiny   batches of products of a few elements each: a lane per output.
//   gemm_rowdot n <= 4 with A's rows along K (matrix x vector): a wave per row of A,
//               16-byte pieces, float32 sums met through the cross-lane network.
//   gemm_skinny m <= 16 (decode-like GEMV): HBM-bound on B, which is streamed
//               once; K is split across blocks only as far as it takes to fill
//               the chip and the f32 partials are summed by a second pass. f32
//               runs lane-per-column FMAs, bf16 / f16 run v_mfma_f32_16x16x32
//               behind a wave-private transposing LDS tile.
//   gemm_block  (gemm_block.hip) integers, float8, complex: register-blocked through LDS.
//   gemm_any    what is left (thin products of those dtypes): one lane per output element.
// Summation order differs from the reference's k-sequential loop, so float
// results agree within the reference's GEMM tolerances; integer results are
// exact (modular arithmetic is order-free).

#include <algorithm>
#include <cstdlib>

#include "gemm_args.hpp"
#include "gemm_tile.hpp"
#include "gemm_dl.hpp"
#include "nxh_common.hpp"

typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
// A native vector, not a struct: arrays of these stay in registers.
typedef __attribute__((ext_vector_type(4))) uint32_t U4;

// Per-dtype MFMA traits. VL = elements per 16-byte vector; one "k-chunk" is
// 2*VL values of k: lanes 0-31 multiply the first VL of them, lanes 32-63 the
// second (any fixed assignment of k to lanes is valid as long as A and B agree).
struct MMbf16 {
  static constexpr int DT = NXH_BF16;
  using S = uint16_t;
  static constexpr int VL = 8;
  __device__ __forceinline__ static void mac(f32x16 &acc, const U4 &a, const U4 &b) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b),
                                                  acc, 0, 0, 0);
  }
};
struct MMf16 {
  static constexpr int DT = NXH_F16;
  using S = uint16_t;
  static constexpr int VL = 8;
  __device__ __forceinline__ static void mac(f32x16 &acc, const U4 &a, const U4 &b) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b),
                                                 acc, 0, 0, 0);
  }
};
struct MMf32 {
  static constexpr int DT = NXH_F32;
  using S = float;
  static constexpr int VL = 4;
  __device__ __forceinline__ static void mac(f32x16 &acc, const U4 &a, const U4 &b) {
    f32x4 x = __builtin_bit_cast(f32x4, a), y = __builtin_bit_cast(f32x4, b);
#pragma unroll
    for (int s = 0; s < 4; s++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(x[s], y[s], acc, 0, 0, 0);
  }
};

constexpr int GM = 128, GN = 128;  // block tile
constexpr int GT = 256;            // threads

// Loads this lane's two 16-byte pieces of one operand's K-slab into registers.
// ROWS = 128 rows (m or n) by BK k-values. `kc` says the operand is contiguous
// along k (then a vector runs along k), otherwise along its row index.
template <class MM, int BK>
__device__ __forceinline__ void slab_load(U4 (&r)[2], const typename MM::S *p, int64_t rs, int64_t ks,
                                          int64_t row0, int64_t k0, int64_t nrows, int64_t K, bool kc,
                                          bool vec) {
  using S = typename MM::S;
  constexpr int VL = MM::VL;
#pragma unroll
  for (int i = 0; i < 2; i++) {
    const int v = threadIdx.x + i * GT;
    int64_t row, k;
    if (kc) {
      row = row0 + v / (BK / VL);
      k = k0 + (v % (BK / VL)) * VL;
    } else {
      k = k0 + v / (GM / VL);
      row = row0 + (v % (GM / VL)) * VL;
    }
    const S *q = p + row * rs + k * ks;
    const bool full = kc ? (row < nrows && k + VL <= K) : (k < K && row + VL <= nrows);
    if (vec && full) {
      r[i] = *reinterpret_cast<const U4 *>(q);
    } else {
      union {
        S t[VL];
        U4 v;
      } u;
#pragma unroll
      for (int j = 0; j < VL; j++) {
        int64_t rr = kc ? row : row + j, kk = kc ? k + j : k;
        u.t[j] = (rr < nrows && kk < K) ? q[kc ? j * ks : j * rs] : (S)0;
      }
      r[i] = u.v;
    }
  }
}

// Writes the prefetched pieces into the K-contiguous LDS tile [128][LDP].
template <class MM, int BK, int LDP>
__device__ __forceinline__ void slab_store(const U4 (&r)[2], typename MM::S *lds, bool kc) {
  using S = typename MM::S;
  constexpr int VL = MM::VL;
#pragma unroll
  for (int i = 0; i < 2; i++) {
    const int v = threadIdx.x + i * GT;
    if (kc) {
      const int row = v / (BK / VL), k = (v % (BK / VL)) * VL;
      *reinterpret_cast<U4 *>(&lds[row * LDP + k]) = r[i];
    } else {
      const int k = v / (GM / VL), row = (v % (GM / VL)) * VL;
      union {
        U4 v;
        S t[VL];
      } u;
      u.v = r[i];
#pragma unroll
      for (int j = 0; j < VL; j++) lds[(row + j) * LDP + k] = u.t[j];
    }
  }
}

template <class MM>
__global__ __launch_bounds__(GT) void gemm_mfma_kernel(GemmArgs a) {
  using S = typename MM::S;
  constexpr int VL = MM::VL;
  constexpr int BK = 4 * VL;   // two k-chunks per slab
  constexpr int LDP = BK + VL; // 16-byte pad: rows land on distinct bank groups
  __shared__ alignas(16) S sA[GM * LDP];
  __shared__ alignas(16) S sB[GN * LDP];

  int64_t ao, bo, co;
  batch_decode(a.batch, a.batch0 + blockIdx.z, ao, bo, co);
  const S *A = (const S *)a.A + ao;
  const S *B = (const S *)a.B + bo;
  const int64_t m0 = (int64_t)blockIdx.y * GM, n0 = (int64_t)blockIdx.x * GN;
  const bool a_kc = a.acs == 1, b_kc = a.brs == 1;

  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;
  const int r32 = lane & 31, kg = lane >> 5;

  f32x16 acc[2][2];
#pragma unroll
  for (int t = 0; t < 2; t++)
#pragma unroll
    for (int u = 0; u < 2; u++)
#pragma unroll
      for (int e = 0; e < 16; e++) acc[t][u][e] = 0.0f;

  U4 ra[2], rb[2];
  const int64_t nk = (a.K + BK - 1) / BK;
  if (nk > 0) {
    slab_load<MM, BK>(ra, A, a.ars, a.acs, m0, 0, a.M, a.K, a_kc, a.a_vec);
    // B is addressed as rows = n, so its "row stride" is bcs and k stride brs
    slab_load<MM, BK>(rb, B, a.bcs, a.brs, n0, 0, a.N, a.K, b_kc, a.b_vec);
  }
  for (int64_t kt = 0; kt < nk; kt++) {
    slab_store<MM, BK, LDP>(ra, sA, a_kc);
    slab_store<MM, BK, LDP>(rb, sB, b_kc);
    __syncthreads();
    if (kt + 1 < nk) {
      slab_load<MM, BK>(ra, A, a.ars, a.acs, m0, (kt + 1) * BK, a.M, a.K, a_kc, a.a_vec);
      slab_load<MM, BK>(rb, B, a.bcs, a.brs, n0, (kt + 1) * BK, a.N, a.K, b_kc, a.b_vec);
    }
#pragma unroll
    for (int ch = 0; ch < 2; ch++) {
      U4 fa[2], fb[2];
#pragma unroll
      for (int t = 0; t < 2; t++) {
        fa[t] = *reinterpret_cast<const U4 *>(&sA[(wm + t * 32 + r32) * LDP + ch * 2 * VL + kg * VL]);
        fb[t] = *reinterpret_cast<const U4 *>(&sB[(wn + t * 32 + r32) * LDP + ch * 2 * VL + kg * VL]);
      }
#pragma unroll
      for (int t = 0; t < 2; t++)
#pragma unroll
        for (int u = 0; u < 2; u++) MM::mac(acc[t][u], fa[t], fb[u]);
    }
    __syncthreads();
  }

  // accumulator element e of lane l is C[(e/4)*8 + (l/32)*4 + e%4][l%32]
  S *C = (S *)a.C + co;
#pragma unroll
  for (int t = 0; t < 2; t++)
#pragma unroll
    for (int u = 0; u < 2; u++) {
      const int64_t col = n0 + wn + u * 32 + r32;
#pragma unroll
      for (int e = 0; e < 16; e++) {
        const int64_t row = m0 + wm + t * 32 + (e >> 2) * 8 + kg * 4 + (e & 3);
        if (row < a.M && col < a.N) C[row * a.crs + col * a.ccs] = Tr<MM::DT>::st(acc[t][u][e]);
      }
    }
}

// ── gemm_skinny: m <= 16, B streamed once ───────────────────────────────────
// HBM-bound on B. A block is 64 column lanes (VN adjacent columns each: one
// 16-byte load per row of B) by 4 row groups; row group g walks rows g, g + 4,
// ... of the block's K-chunk with SK_U loads in flight, multiplying against the
// chunk of A held in LDS as f32 [k][m]. The four partial tiles meet in LDS
// (two folding steps). K is split across blocks only as far as it takes to fill
// the chip; the [split][m][n] f32 partials are summed by skinny_finish.
constexpr int SK_LANES = 64, SK_RG = 4, SK_U = 4;
struct SkinnyArgs {
  const void *A, *B;
  void *C;       // storage-typed result (nsplit == 1) or f32 partials
  int64_t M, N, K;
  int64_t ars, acs, brs, crs, ccs;  // B has bcs == 1
  int64_t kchunk;
  int nsplit;
};
template <int DT, int MMAX, int VN>
__global__ __launch_bounds__(SK_LANES *SK_RG) void gemm_skinny_kernel(SkinnyArgs a) {
  using TR = Tr<DT>;
  using S = typename TR::S;
  struct alignas(sizeof(S) * VN) BV {
    S v[VN];
  };
  extern __shared__ __attribute__((aligned(16))) float sk_lds[];  // A chunk, then the fold buffer
  const int ln = threadIdx.x % SK_LANES, rg = threadIdx.x / SK_LANES;
  const int64_t n = ((int64_t)blockIdx.x * SK_LANES + ln) * VN;
  const int64_t k0 = (int64_t)blockIdx.y * a.kchunk;
  const int64_t k1 = k0 + a.kchunk < a.K ? k0 + a.kchunk : a.K;
  const int kn = (int)(k1 - k0);
  const S *A = (const S *)a.A;
  const S *B = (const S *)a.B;
  for (int idx = threadIdx.x; idx < kn * MMAX; idx += SK_LANES * SK_RG) {
    const int i = idx / kn, kk = idx - i * kn;  // lanes run along k
    sk_lds[kk * MMAX + i] = i < a.M ? TR::ld(A[i * a.ars + (k0 + kk) * a.acs]) : 0.0f;
  }
  __syncthreads();
  float acc[MMAX][VN];
#pragma unroll
  for (int i = 0; i < MMAX; i++)
#pragma unroll
    for (int j = 0; j < VN; j++) acc[i][j] = 0.0f;
  const bool col_ok = n + VN <= a.N;
  auto row_fma = [&](int kk, const BV &t) {
    float bv[VN];
#pragma unroll
    for (int j = 0; j < VN; j++) bv[j] = TR::ld(t.v[j]);
    const float *ar = sk_lds + kk * MMAX;
#pragma unroll
    for (int i = 0; i < MMAX; i++) {
      const float av = ar[i];
#pragma unroll
      for (int j = 0; j < VN; j++) acc[i][j] = __builtin_fmaf(av, bv[j], acc[i][j]);
    }
  };
  if (col_ok) {
    const S *bp = B + k0 * a.brs + n;
    int kk = rg;
    for (; kk + (SK_U - 1) * SK_RG < kn; kk += SK_U * SK_RG) {
      BV t[SK_U];
#pragma unroll
      for (int u = 0; u < SK_U; u++) t[u] = *reinterpret_cast<const BV *>(bp + (int64_t)(kk + u * SK_RG) * a.brs);
#pragma unroll
      for (int u = 0; u < SK_U; u++) row_fma(kk + u * SK_RG, t[u]);
    }
    for (; kk < kn; kk += SK_RG) row_fma(kk, *reinterpret_cast<const BV *>(bp + (int64_t)kk * a.brs));
  } else if (n < a.N) {  // the ragged last lane of a row: element loads
    for (int kk = rg; kk < kn; kk += SK_RG) {
      BV t;
#pragma unroll
      for (int j = 0; j < VN; j++) t.v[j] = n + j < a.N ? B[(k0 + kk) * a.brs + n + j] : S{};
      row_fma(kk, t);
    }
  }
  // fold the row groups into group 0, one at a time (the A chunk is dead now)
#pragma unroll 1
  for (int g = 1; g < SK_RG; g++) {
    __syncthreads();
    float *q = sk_lds + ln;
    if (rg == g) {
#pragma unroll
      for (int i = 0; i < MMAX; i++)
#pragma unroll
        for (int j = 0; j < VN; j++) q[(i * VN + j) * SK_LANES] = acc[i][j];
    }
    __syncthreads();
    if (rg == 0) {
#pragma unroll
      for (int i = 0; i < MMAX; i++)
#pragma unroll
        for (int j = 0; j < VN; j++) acc[i][j] += q[(i * VN + j) * SK_LANES];
    }
  }
  if (rg != 0 || n >= a.N) return;
  if (a.nsplit > 1) {
    float *P = (float *)a.C + (int64_t)blockIdx.y * a.M * a.N;
#pragma unroll
    for (int i = 0; i < MMAX; i++)
      if (i < a.M) {
#pragma unroll
        for (int j = 0; j < VN; j++)
          if (n + j < a.N) P[i * a.N + n + j] = acc[i][j];
      }
  } else {
    S *C = (S *)a.C;
#pragma unroll
    for (int i = 0; i < MMAX; i++)
      if (i < a.M) {
#pragma unroll
        for (int j = 0; j < VN; j++)
          if (n + j < a.N) C[i * a.crs + (n + j) * a.ccs] = TR::st(acc[i][j]);
      }
  }
}
// ── gemm_skinny_mfma: the same shape for bf16 / f16 on the matrix pipe ──────
// The lane-per-column kernel above spends 8 FMAs per 2-byte element of B and is
// VALU-bound for 16-bit types. Here every wave streams its own 64 columns of B:
// 32 k-rows x 64 columns per step go global -> registers -> a wave-private LDS
// tile in memory order ([k][n], no block barrier: LDS serves one wave's accesses
// in order), come back k-contiguous through the transposing LDS read, and feed
// four v_mfma_f32_16x16x32 against the A chunk held in LDS as [16][k] (rows
// >= m are zero). Loads run three steps ahead of the multiply.
constexpr int SM_KS = 32, SM_WN = 64, SM_PITCH = SM_WN + 8, SM_TILE = SM_KS * SM_PITCH;
template <bool BF16>
__global__ __launch_bounds__(256) void gemm_skinny_mfma_kernel(SkinnyArgs a) {
  using gemm_tile::lds_s16x4;
  using gemm_tile::s16x4;
  typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
  extern __shared__ __attribute__((aligned(16))) uint16_t sm_lds[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t n0 = ((int64_t)blockIdx.x * 4 + wave) * SM_WN;
  const int64_t k0 = (int64_t)blockIdx.y * a.kchunk;
  const int64_t k1 = k0 + a.kchunk < a.K ? k0 + a.kchunk : a.K;
  const int kn = (int)(k1 - k0), kc = (int)a.kchunk, kpitch = kc + 8;
  const uint16_t *A = (const uint16_t *)a.A;
  const uint16_t *B = (const uint16_t *)a.B;
  uint16_t *sA = sm_lds;
  uint16_t *sB = sm_lds + 16 * kpitch + wave * (2 * SM_TILE);
  for (int idx = threadIdx.x; idx < 16 * kc; idx += 256) {
    const int i = idx / kc, kk = idx - i * kc;
    sA[i * kpitch + kk] = (i < a.M && kk < kn) ? A[i * a.ars + (k0 + kk) * a.acs] : (uint16_t)0;
  }
  __syncthreads();
  // this lane's four 16-byte vectors of a step: vector v covers row v / 8,
  // columns (v % 8) * 8 .. + 7 of the wave's tile
  const int c8 = (lane & 7) * 8, rbase = lane >> 3;
  const bool col_ok = n0 + c8 < a.N;  // N is a multiple of 8: vectors are whole or absent
  const uint16_t *bp = B + k0 * a.brs + n0 + c8;
  // three register sets rotate through the steps: while step s multiplies, the
  // loads of steps s+2 .. s+4 are in flight (12 x 16 bytes per lane)
  U4 rb[3][4];
  auto load = [&](U4 (&r)[4], int step) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int kk = step * SM_KS + rbase + i * 8;
      r[i] = (col_ok && kk < kn) ? *reinterpret_cast<const U4 *>(bp + (int64_t)kk * a.brs) : U4{0, 0, 0, 0};
    }
  };
  auto store = [&](const U4 (&r)[4], int buf) {
#pragma unroll
    for (int i = 0; i < 4; i++)
      *reinterpret_cast<U4 *>(sB + buf * SM_TILE + (rbase + i * 8) * SM_PITCH + c8) = r[i];
  };
  f32x4 acc[4];
#pragma unroll
  for (int t = 0; t < 4; t++) acc[t] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  const int nsteps = (kn + SM_KS - 1) / SM_KS;
  const int g = lane >> 4, L = lane & 15;
  // step s: its tile is in LDS buffer s & 1; the registers of slot (s + 1) % 3
  // hold step s + 1 and are refilled with step s + 4 once stored
  auto step = [&](int s, auto slot_c) {
    constexpr int SL = decltype(slot_c)::value;
    if (s + 1 < nsteps) store(rb[SL], (s + 1) & 1);
    if (s + 4 < nsteps) load(rb[SL], s + 4);
    const U4 xa = *reinterpret_cast<const U4 *>(sA + L * kpitch + s * SM_KS + g * 8);
    const uint16_t *tile = sB + (s & 1) * SM_TILE + (g * 8 + (L >> 2)) * SM_PITCH + (L & 3) * 4;
#pragma unroll
    for (int t = 0; t < 4; t++) {
      const u32x2 lo = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(tile + t * 16)));
      const u32x2 hi = __builtin_bit_cast(
          u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(tile + t * 16 + 4 * SM_PITCH)));
      const U4 yb = U4{lo[0], lo[1], hi[0], hi[1]};
      if constexpr (BF16)
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, xa), __builtin_bit_cast(bf16x8, yb),
                                                         acc[t], 0, 0, 0);
      else
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, xa), __builtin_bit_cast(f16x8, yb),
                                                        acc[t], 0, 0, 0);
    }
  };
  load(rb[0], 0);
  if (nsteps > 1) load(rb[1], 1);
  if (nsteps > 2) load(rb[2], 2);
  store(rb[0], 0);
  if (nsteps > 3) load(rb[0], 3);
  for (int s = 0; s < nsteps; s += 3) {
    step(s, std::integral_constant<int, 1>{});
    if (s + 1 < nsteps) step(s + 1, std::integral_constant<int, 2>{});
    if (s + 2 < nsteps) step(s + 2, std::integral_constant<int, 0>{});
  }
  // accumulator element e of lane l is C[4 * (l / 16) + e][l % 16] of its tile
#pragma unroll
  for (int t = 0; t < 4; t++) {
    const int64_t n = n0 + t * 16 + L;
    if (n >= a.N) continue;
#pragma unroll
    for (int e = 0; e < 4; e++) {
      const int m = g * 4 + e;
      if (m >= a.M) continue;
      if (a.nsplit > 1) ((float *)a.C)[((int64_t)blockIdx.y * a.M + m) * a.N + n] = acc[t][e];
      else ((uint16_t *)a.C)[m * a.crs + n * a.ccs] = BF16 ? f32_to_bf16(acc[t][e]) : f32_to_f16(acc[t][e]);
    }
  }
}

// ── gemm_skinny_mfma_k8: the same stream when N alone fills the chip ────────
// One block of eight waves owns 64 columns; the waves split K eight ways and fold their
// accumulators through LDS in wave order at the end, so there are no f32 partials in memory
// and no second launch. A (at most 16 x K, a few dozen KiB, resident in L2) is not staged:
// each lane reads its 16-byte fragment of the step straight from memory, three steps ahead
// like the B vectors, so a block starts streaming with its first instruction.
constexpr int SM8_WAVES = 8;
template <bool BF16>
__global__ __launch_bounds__(64 * SM8_WAVES) void gemm_skinny_mfma_k8_kernel(SkinnyArgs a) {
  using gemm_tile::lds_s16x4;
  using gemm_tile::s16x4;
  typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
  extern __shared__ __attribute__((aligned(16))) uint16_t sm_lds[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t n0 = (int64_t)blockIdx.x * SM_WN;
  const int64_t k0 = (int64_t)wave * a.kchunk;
  const int64_t k1 = k0 + a.kchunk < a.K ? k0 + a.kchunk : a.K;
  const int kn = k1 > k0 ? (int)(k1 - k0) : 0;  // a multiple of 8 (K is)
  const uint16_t *A = (const uint16_t *)a.A;
  const uint16_t *B = (const uint16_t *)a.B;
  uint16_t *sB = sm_lds + wave * (2 * SM_TILE);
  const int c8 = (lane & 7) * 8, rbase = lane >> 3;
  const bool col_ok = n0 + c8 < a.N;
  const uint16_t *bp = B + k0 * a.brs + n0 + c8;
  const int g = lane >> 4, L = lane & 15;
  const uint16_t *ap = A + (int64_t)L * a.ars + k0 + g * 8;  // rows >= M read as zero
  const bool row_ok = L < a.M;
  U4 rb[3][4], ra[3];
  auto load = [&](U4 (&r)[4], U4 &x, int step) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int kk = step * SM_KS + rbase + i * 8;
      r[i] = (col_ok && kk < kn) ? *reinterpret_cast<const U4 *>(bp + (int64_t)kk * a.brs) : U4{0, 0, 0, 0};
    }
    const int ka = step * SM_KS + g * 8;
    x = (row_ok && ka < kn) ? *reinterpret_cast<const U4 *>(ap + step * SM_KS) : U4{0, 0, 0, 0};
  };
  auto store = [&](const U4 (&r)[4], int buf) {
#pragma unroll
    for (int i = 0; i < 4; i++)
      *reinterpret_cast<U4 *>(sB + buf * SM_TILE + (rbase + i * 8) * SM_PITCH + c8) = r[i];
  };
  f32x4 acc[4];
#pragma unroll
  for (int t = 0; t < 4; t++) acc[t] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  const int nsteps = (kn + SM_KS - 1) / SM_KS;
  // step s multiplies the tile in LDS buffer s & 1 by the A fragment of slot s % 3; slot (s + 1) % 3
  // is stored for step s + 1 and refilled with step s + 4
  auto step = [&](int s, auto slot_c) {
    constexpr int SL = decltype(slot_c)::value;       // slot of step s + 1
    constexpr int CUR = (SL + 2) % 3;                 // slot of step s
    const U4 xa = ra[CUR];
    if (s + 1 < nsteps) store(rb[SL], (s + 1) & 1);
    const uint16_t *tile = sB + (s & 1) * SM_TILE + (g * 8 + (L >> 2)) * SM_PITCH + (L & 3) * 4;
    U4 yb[4];
#pragma unroll
    for (int t = 0; t < 4; t++) {
      const u32x2 lo = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(tile + t * 16)));
      const u32x2 hi = __builtin_bit_cast(
          u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(tile + t * 16 + 4 * SM_PITCH)));
      yb[t] = U4{lo[0], lo[1], hi[0], hi[1]};
    }
#pragma unroll
    for (int t = 0; t < 4; t++) {
      if constexpr (BF16)
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, xa), __builtin_bit_cast(bf16x8, yb[t]),
                                                         acc[t], 0, 0, 0);
      else
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, xa), __builtin_bit_cast(f16x8, yb[t]),
                                                        acc[t], 0, 0, 0);
    }
    // the slot of step s is free once its fragment has been multiplied: refill it with step s + 3
    if (s + 3 < nsteps) load(rb[CUR], ra[CUR], s + 3);
  };
  // slots: step s lives in slot s % 3
  if (nsteps > 0) load(rb[0], ra[0], 0);
  if (nsteps > 1) load(rb[1], ra[1], 1);
  if (nsteps > 2) load(rb[2], ra[2], 2);
  if (nsteps > 0) store(rb[0], 0);
  for (int s = 0; s < nsteps; s += 3) {
    step(s, std::integral_constant<int, 1>{});
    if (s + 1 < nsteps) step(s + 1, std::integral_constant<int, 2>{});
    if (s + 2 < nsteps) step(s + 2, std::integral_constant<int, 0>{});
  }
  // fold the eight waves' [16][64] tiles in wave order
  __syncthreads();  // every wave is done with its tiles: the buffer becomes [wave][16][64] floats
  float *red = reinterpret_cast<float *>(sm_lds);
#pragma unroll
  for (int t = 0; t < 4; t++)
#pragma unroll
    for (int e = 0; e < 4; e++) red[(wave * 16 + g * 4 + e) * SM_WN + t * 16 + L] = acc[t][e];
  __syncthreads();
  for (int o = threadIdx.x; o < 16 * SM_WN; o += 64 * SM8_WAVES) {
    const int m = o / SM_WN, c = o - m * SM_WN;
    const int64_t n = n0 + c;
    if (m >= a.M || n >= a.N) continue;
    float sum = red[o];
#pragma unroll
    for (int w = 1; w < SM8_WAVES; w++) sum += red[w * 16 * SM_WN + o];
    ((uint16_t *)a.C)[m * a.crs + n * a.ccs] = BF16 ? f32_to_bf16(sum) : f32_to_f16(sum);
  }
}

// ── gemm_skinny_f32_k8: float32, N alone fills the chip ──────────────────────
// The matrix pipe straight from registers, no LDS on the way: a lane loads 16 bytes of one row
// of B (k = k0 + lane / 16, columns 4 (lane % 16) .. + 3) and feeds the four values to four
// v_mfma_f32_16x16x4_f32 (true float32), whose B operand wants exactly one value of row
// lane / 16 per lane; that MFMA j then holds columns 4 l + j instead of l is undone at the
// store. The A operand of the same instructions is A[lane % 16][k], one 4-byte load from L2
// (rows >= M read as zero). A wave so covers 64 columns by 4 k-rows per load instruction,
// 256 contiguous bytes per row; the eight waves of a block split K and fold through LDS.
constexpr int SF_U = 8;  // steps (of 4 k-rows) in flight per wave
__global__ __launch_bounds__(64 * SM8_WAVES) void gemm_skinny_f32_k8_kernel(SkinnyArgs a) {
  typedef __attribute__((ext_vector_type(4))) float f32x4_t;
  __shared__ float red[SM8_WAVES * 16 * 64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int kg = lane >> 4, l = lane & 15;
  const int64_t n0 = (int64_t)blockIdx.x * 64;
  const int64_t k0 = (int64_t)wave * a.kchunk;
  const int64_t k1 = k0 + a.kchunk < a.K ? k0 + a.kchunk : a.K;
  const float *A = (const float *)a.A;
  const float *B = (const float *)a.B;
  const bool col_ok = n0 + 4 * l < a.N;  // N is a multiple of 4: vectors are whole or absent
  const bool row_ok = l < a.M;
  const float *bp = B + n0 + 4 * l;
  const float *ap = A + (int64_t)l * a.ars;
  f32x4_t acc[4];
#pragma unroll
  for (int j = 0; j < 4; j++) acc[j] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
  for (int64_t kb = k0; kb < k1; kb += 4 * SF_U) {
    f32x4_t b[SF_U];
    float av[SF_U];
#pragma unroll
    for (int u = 0; u < SF_U; u++) {
      const int64_t k = kb + 4 * u + kg;
      const bool in = k < k1;
      b[u] = (in && col_ok) ? *reinterpret_cast<const f32x4_t *>(bp + k * a.brs) : f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
      av[u] = (in && row_ok) ? ap[k * a.acs] : 0.0f;
    }
#pragma unroll
    for (int u = 0; u < SF_U; u++)
#pragma unroll
      for (int j = 0; j < 4; j++) acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[u], b[u][j], acc[j], 0, 0, 0);
  }
  // accumulator element e of MFMA j is C[4 kg + e][column 4 l + j] of the wave's partial tile
#pragma unroll
  for (int j = 0; j < 4; j++)
#pragma unroll
    for (int e = 0; e < 4; e++) red[(wave * 16 + 4 * kg + e) * 64 + 4 * l + j] = acc[j][e];
  __syncthreads();
  for (int o = threadIdx.x; o < 16 * 64; o += 64 * SM8_WAVES) {
    const int m = o >> 6, c = o & 63;
    const int64_t n = n0 + c;
    if (m >= a.M || n >= a.N) continue;
    float sum = red[o];
#pragma unroll
    for (int w = 1; w < SM8_WAVES; w++) sum += red[w * 16 * 64 + o];  // wave order: the bits repeat
    ((float *)a.C)[m * a.crs + n * a.ccs] = sum;
  }
}

// Sums the [nsplit][m * n] partials in split order, four outputs per lane.
template <int DT>
__global__ __launch_bounds__(256) void skinny_finish_kernel(const float *P, void *Cv, int64_t M, int64_t N,
                                                            int nsplit, int64_t crs, int64_t ccs) {
  using TR = Tr<DT>;
  typedef __attribute__((ext_vector_type(4))) float f32x4;
  const int64_t total = M * N;
  const int64_t e = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (e >= total) return;
  typename TR::S *C = (typename TR::S *)Cv;
  if (e + 4 <= total && (total & 3) == 0) {
    f32x4 s = {0.0f, 0.0f, 0.0f, 0.0f};
    int c = 0;
    for (; c + 8 <= nsplit; c += 8) {
      f32x4 t[8];
#pragma unroll
      for (int u = 0; u < 8; u++) t[u] = *reinterpret_cast<const f32x4 *>(P + (int64_t)(c + u) * total + e);
#pragma unroll
      for (int u = 0; u < 8; u++) s += t[u];
    }
    for (; c < nsplit; c++) s += *reinterpret_cast<const f32x4 *>(P + (int64_t)c * total + e);
#pragma unroll
    for (int j = 0; j < 4; j++) C[((e + j) / N) * crs + ((e + j) % N) * ccs] = TR::st(s[j]);
  } else {
    for (int64_t x = e; x < total && x < e + 4; x++) {
      float s = 0.0f;
      for (int c = 0; c < nsplit; c++) s += P[(int64_t)c * total + x];
      C[(x / N) * crs + (x % N) * ccs] = TR::st(s);
    }
  }
}

// ── gemm_any: one lane per output, any dtype, any strides ───────────────────
template <int DT>
__global__ __launch_bounds__(256) void gemm_any_kernel(GemmArgs a) {
  using TR = Tr<DT>;
  using S = typename TR::S;
  using C = typename TR::C;
  int64_t ao, bo, co;
  batch_decode(a.batch, a.batch0 + blockIdx.z, ao, bo, co);
  const int64_t col = (int64_t)blockIdx.x * 16 + (threadIdx.x & 15);
  const int64_t row = (int64_t)blockIdx.y * 16 + (threadIdx.x >> 4);
  if (row >= a.M || col >= a.N) return;
  const S *A = (const S *)a.A + ao + row * a.ars;
  const S *B = (const S *)a.B + bo + col * a.bcs;
  C acc;
  if constexpr (TR::cat == CAT_COMPLEX) acc = C{0, 0};
  else acc = (C)0;
  for (int64_t k = 0; k < a.K; k++) {
    C x = TR::ld(A[k * a.acs]), y = TR::ld(B[k * a.brs]);
    if constexpr (TR::cat == CAT_SINT) acc = (C)((uint64_t)acc + (uint64_t)x * (uint64_t)y);
    else acc = acc + x * y;
  }
  ((S *)a.C)[co + row * a.crs + col * a.ccs] = TR::st(acc);
}

typedef int (*mm_fn)(nxh_context *, GemmArgs &, uint32_t nbatch);

template <int DT>
static int launch_any(nxh_context *ctx, GemmArgs &a, uint32_t nbatch) {
  nxh_set_path("gemm_any");
  const uint32_t gx = (uint32_t)((a.N + 15) / 16), gy = (uint32_t)((a.M + 15) / 16);
  if (gy > 65535) return nxh_fail(NXH_FAILURE, "matmul", "m too large for this dtype's kernel");
  for (uint32_t b0 = 0; b0 < nbatch; b0 += 65535) {
    a.batch0 = b0;
    hipLaunchKernelGGL((gemm_any_kernel<DT>), dim3(gx, gy, std::min<uint32_t>(65535, nbatch - b0)), dim3(256), 0,
                       ctx->stream, a);
    NXH_HIP("matmul", hipGetLastError());
  }
  return NXH_OK;
}

// ── gemm_f64: float64 on the f64 matrix instruction ─────────────────────────
// v_mfma_f64_16x16x4: lane l supplies A[l % 16][l / 16] and B[l / 16][l % 16]; register v of
// lane l of the result is D[4 v + l / 16][l % 16]. A block is WM x WN waves of TM x TN result
// tiles each (128 x 128 as 2 x 2 waves of 4 x 4 tiles or 4 x 2 waves of 2 x 4; 64 x 64 as 4 x 2 of
// 1 x 2; 32 x 32 as 2 x 2 of 1 x 1), K-slabs of BK: global -> registers (the
// next slab, while this one is multiplied) -> K-contiguous LDS tiles [row][BK + 2] (the pad puts
// the 16 rows and 2 k-columns a half-wave reads on distinct banks). Operands are read
// element by element with bounds checks (zeros outside), lanes running along whichever of the
// operand's two dims is contiguous: any strides (negative too), any edge, no alignment condition. One
// instruction is 64 cycles on this chip, so a k-step's T^2 instructions hide its 2 T LDS
// reads with room to spare; several blocks per unit hide the slab barrier.
typedef __attribute__((ext_vector_type(4))) double f64x4;
__device__ double gemm_f64_zero[2] = {0.0, 0.0};  // (not const: a load through it stays a global load)
template <int WM, int WN, int TM, int TN, int BK>
__global__ __launch_bounds__(64 * WM * WN) __attribute__((amdgpu_waves_per_eu(2))) void gemm_f64_kernel(GemmArgs a) {
  constexpr int BM = 16 * TM * WM, BN = 16 * TN * WN, THREADS = 64 * WM * WN, LDP = BK + 2;
  constexpr int NLA = BM * BK / THREADS, NLB = BN * BK / THREADS;
  static_assert(NLA >= 1 && NLB >= 1 && NLA * THREADS == BM * BK && NLB * THREADS == BN * BK, "slab loads");
  static_assert(THREADS % BK == 0 && THREADS % BM == 0 && THREADS % BN == 0, "lanes along k or along rows");
  __shared__ double sA[BM * LDP];
  __shared__ double sB[BN * LDP];
  int64_t ao, bo, co;
  batch_decode(a.batch, a.batch0 + blockIdx.z, ao, bo, co);
  const double *A = (const double *)a.A + ao;
  const double *B = (const double *)a.B + bo;
  const int64_t m0 = (int64_t)blockIdx.y * BM, n0 = (int64_t)blockIdx.x * BN;
  const bool a_kc = a.acs == 1, b_kc = a.brs == 1;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wm = (wave / WN) * (16 * TM), wn = (wave % WN) * (16 * TN);
  const int r16 = lane & 15, kq = lane >> 4;

  // Element e = thread + THREADS i of an operand's slab: lanes run along k (kc) or along the row
  // index; element e + THREADS then lies a fixed number of rows or k-values further on, one uniform
  // pointer step. No branch around a load and nothing to do to its result (the wait counters
  // stay exact, so a slab's stores wait only for their own loads): an element outside the
  // operand is read from a zero in memory instead.
  struct Lane {
    const double *p;  // this lane's element of slab 0
    int64_t step;     // to element e + THREADS
    int row, k, drow, dk;
  };
  auto lane_of = [&](const double *P, bool kc, int64_t rs, int64_t ks, int rows) {
    Lane l;
    l.row = kc ? threadIdx.x / BK : threadIdx.x % rows;
    l.k = kc ? threadIdx.x % BK : threadIdx.x / rows;
    l.drow = kc ? THREADS / BK : 0;
    l.dk = kc ? 0 : THREADS / rows;
    l.p = P + l.row * rs + l.k * ks;
    l.step = l.drow * rs + l.dk * ks;
    return l;
  };
  const Lane la = lane_of(A + m0 * a.ars, a_kc, a.ars, a.acs, BM);
  const Lane lb = lane_of(B + n0 * a.bcs, b_kc, a.bcs, a.brs, BN);  // B by rows = n
  const int64_t a_left = a.M - m0, b_left = a.N - n0;
  auto load = [&](auto &r, const Lane &l, int64_t ks, int64_t rows_left, int rows, int64_t k0) {
    constexpr int NL = sizeof(r) / sizeof(double);
    const double *p = l.p + k0 * ks;
    if (rows_left >= rows && k0 + BK <= a.K) {  // (uniform) a whole slab: nothing to check
#pragma unroll
      for (int i = 0; i < NL; i++) r[i] = p[i * l.step];
      return;
    }
#pragma unroll
    for (int i = 0; i < NL; i++) {
      const bool ok = l.row + i * l.drow < rows_left && k0 + l.k + i * l.dk < a.K;
      r[i] = *(ok ? p : gemm_f64_zero);
      p += l.step;
    }
  };
  auto store = [&](const auto &r, const Lane &l, double *s) {
    constexpr int NL = sizeof(r) / sizeof(double);
#pragma unroll
    for (int i = 0; i < NL; i++) s[(l.row + i * l.drow) * LDP + l.k + i * l.dk] = r[i];
  };

  f64x4 acc[TM][TN];
#pragma unroll
  for (int t = 0; t < TM; t++)
#pragma unroll
    for (int u = 0; u < TN; u++) acc[t][u] = f64x4{0.0, 0.0, 0.0, 0.0};
  const int64_t nk = (a.K + BK - 1) / BK;
  // one slab: registers -> LDS, the loads of slab kt + 1 into the registers just freed, multiply
  auto slab = [&](int64_t kt, double(&ra)[NLA], double(&rb)[NLB]) {
    store(ra, la, sA);
    store(rb, lb, sB);
    __syncthreads();
    load(ra, la, a.acs, a_left, BM, (kt + 1) * BK);  // (past K: zeros nobody uses)
    load(rb, lb, a.brs, b_left, BN, (kt + 1) * BK);
    // the fragments of k-step ks + 1 are read behind the first instructions of k-step ks
    double fa[2][TM], fb[2][TN];
    auto frags = [&](int ks, double(&fa_)[TM], double(&fb_)[TN]) {
#pragma unroll
      for (int t = 0; t < TM; t++) fa_[t] = sA[(wm + t * 16 + r16) * LDP + ks * 4 + kq];
#pragma unroll
      for (int u = 0; u < TN; u++) fb_[u] = sB[(wn + u * 16 + r16) * LDP + ks * 4 + kq];
    };
    frags(0, fa[0], fb[0]);
#pragma unroll
    for (int ks = 0; ks < BK / 4; ks++) {
      const int cur = ks & 1;
      if (ks + 1 < BK / 4) frags(ks + 1, fa[cur ^ 1], fb[cur ^ 1]);
#pragma unroll
      for (int t = 0; t < TM; t++)
#pragma unroll
        for (int u = 0; u < TN; u++)
          acc[t][u] = __builtin_amdgcn_mfma_f64_16x16x4f64(fa[cur][t], fb[cur][u], acc[t][u], 0, 0, 0);
      // behind each matrix instruction (64 cycles): an LDS read, and the address arithmetic and
      // issue of one or two of the next slab's loads
#pragma unroll
      for (int x = 0; x < TM * TN; x++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // matrix instruction
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // LDS read
        __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);  // VALU
        __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // global load
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
  };
  double ra0[NLA], rb0[NLB];
  if (nk > 0) {
    load(ra0, la, a.acs, a_left, BM, 0);
    load(rb0, lb, a.brs, b_left, BN, 0);
  }
  for (int64_t kt = 0; kt < nk; kt++) slab(kt, ra0, rb0);
  double *C = (double *)a.C + co;
#pragma unroll
  for (int t = 0; t < TM; t++)
#pragma unroll
    for (int u = 0; u < TN; u++) {
      const int64_t col = n0 + wn + u * 16 + r16;
#pragma unroll
      for (int v = 0; v < 4; v++) {
        const int64_t row = m0 + wm + t * 16 + 4 * v + kq;
        if (row < a.M && col < a.N) C[row * a.crs + col * a.ccs] = acc[t][u][v];
      }
    }
}
static int launch_f64(nxh_context *ctx, GemmArgs &a, uint32_t nbatch) {
  // Block shape: rounds of one block per unit x block area x the shape's measured cost per flop
  // against the 128 x 128 block (4096^3: 57-63 TFLOP/s there; one wave per SIMD leaves about
  // half of a small block's time to its loads and barriers).
  const int cus = ctx->compute_units > 0 ? ctx->compute_units : 256;
  auto cost = [&](int b, double pen) {
    const int64_t tiles = ((a.M + b - 1) / b) * ((a.N + b - 1) / b) * (int64_t)nbatch;
    return (double)((tiles + cus - 1) / cus) * b * b * pen;
  };
  int bmn = 128;
  double best = cost(128, 1.0);
  if (cost(64, 1.3) < best) bmn = 64, best = cost(64, 1.3);
  if (cost(32, 1.6) < best) bmn = 32;
  const uint32_t gx = (uint32_t)((a.N + bmn - 1) / bmn), gy = (uint32_t)((a.M + bmn - 1) / bmn);
  if (gy > 65535) return launch_any<NXH_F64>(ctx, a, nbatch);
  nxh_set_path(bmn == 128 ? "gemm_f64_128x128" : bmn == 64 ? "gemm_f64_64x64" : "gemm_f64_32x32");
  for (uint32_t b0 = 0; b0 < nbatch; b0 += 65535) {
    a.batch0 = b0;
    const dim3 grid(gx, gy, std::min<uint32_t>(65535, nbatch - b0));
    // eight waves (two per SIMD from the one block) where a unit holds a single block: a wave's
    // waits are then covered by its neighbour's matrix instructions (2048^3: 372 -> 342 us)
    const bool one_round = (int64_t)gx * gy * nbatch <= cus;
    if (bmn == 128 && one_round) hipLaunchKernelGGL((gemm_f64_kernel<4, 2, 2, 4, 16>), grid, dim3(512), 0, ctx->stream, a);
    else if (bmn == 128) hipLaunchKernelGGL((gemm_f64_kernel<2, 2, 4, 4, 16>), grid, dim3(256), 0, ctx->stream, a);
    else if (bmn == 64) hipLaunchKernelGGL((gemm_f64_kernel<4, 2, 1, 2, 32>), grid, dim3(512), 0, ctx->stream, a);
    else hipLaunchKernelGGL((gemm_f64_kernel<2, 2, 1, 1, 32>), grid, dim3(256), 0, ctx->stream, a);
    NXH_HIP("matmul", hipGetLastError());
  }
  return NXH_OK;
}

template <class MM>
static int launch_mfma(nxh_context *ctx, GemmArgs &a, uint32_t nbatch) {
  nxh_set_path("gemm_mfma");
  const uint32_t gx = (uint32_t)((a.N + GN - 1) / GN), gy = (uint32_t)((a.M + GM - 1) / GM);
  if (gy > 65535) return launch_any<MM::DT>(ctx, a, nbatch);
  for (uint32_t b0 = 0; b0 < nbatch; b0 += 65535) {
    a.batch0 = b0;
    hipLaunchKernelGGL((gemm_mfma_kernel<MM>), dim3(gx, gy, std::min<uint32_t>(65535, nbatch - b0)), dim3(GT), 0,
                       ctx->stream, a);
    NXH_HIP("matmul", hipGetLastError());
  }
  return NXH_OK;
}

template <int DT, int VN>
static int launch_skinny(nxh_context *ctx, GemmArgs &g) {
  using S = typename Tr<DT>::S;
  SkinnyArgs a;
  a.A = g.A;
  a.B = g.B;
  a.M = g.M;
  a.N = g.N;
  a.K = g.K;
  a.ars = g.ars;
  a.acs = g.acs;
  a.brs = g.brs;
  a.crs = g.crs;
  a.ccs = g.ccs;
  const int cus = ctx->compute_units > 0 ? ctx->compute_units : 256;
  if constexpr (DT == NXH_F32) {
    // N alone fills the chip with 64-column blocks: K is split inside the block, one launch
    const int64_t strips = (g.N + 63) / 64;
    if (strips >= cus && strips <= 0x7fffffffLL && g.N % 4 == 0 && g.brs % 4 == 0 && ((uintptr_t)g.B % 16) == 0 &&
        g.K >= 4 * SF_U * SM8_WAVES) {
      a.kchunk = ((g.K + SM8_WAVES - 1) / SM8_WAVES + 3) / 4 * 4;
      a.nsplit = 1;
      a.C = g.C;
      nxh_set_path("gemm_skinny_f32_k8");
      hipLaunchKernelGGL(gemm_skinny_f32_k8_kernel, dim3((unsigned)strips), dim3(64 * SM8_WAVES), 0, ctx->stream, a);
      NXH_HIP("matmul", hipGetLastError());
      return NXH_OK;
    }
  }
  const int mmax = g.M <= 8 ? 8 : 16;
  const int64_t col_blocks = (g.N + SK_LANES * VN - 1) / (SK_LANES * VN);
  // two blocks per CU keep enough loads in flight; more splits only add partials
  int64_t want = std::max<int64_t>(1, ((int64_t)cus * 2 + col_blocks - 1) / col_blocks);
  int64_t nsplit = std::min<int64_t>(want, std::max<int64_t>(1, g.K / 64));
  int64_t kchunk = (g.K + nsplit - 1) / nsplit;
  kchunk = std::min<int64_t>((kchunk + 7) / 8 * 8, 1024);  // the A chunk must fit in LDS
  if (kchunk < g.K) kchunk = chunk_off_channel_stride(kchunk, g.brs * (int64_t)sizeof(S));
  nsplit = std::max<int64_t>(1, (g.K + kchunk - 1) / kchunk);
  a.kchunk = kchunk;
  a.nsplit = (int)nsplit;
  const size_t lds = sizeof(float) * (size_t)std::max<int64_t>(kchunk * mmax, (int64_t)mmax * VN * SK_LANES);
  void *part = nullptr;
  if (nsplit > 1) {
    int rc = nxh_alloc_locked(ctx, (size_t)nsplit * g.M * g.N * sizeof(float), &part);
    if (rc) return rc;
    a.C = part;
  } else {
    a.C = g.C;
  }
  nxh_set_path(nsplit > 1 ? "gemm_skinny_split" : "gemm_skinny");
  dim3 grid((unsigned)col_blocks, (unsigned)nsplit);
  if (mmax == 8) hipLaunchKernelGGL((gemm_skinny_kernel<DT, 8, VN>), grid, dim3(SK_LANES * SK_RG), lds, ctx->stream, a);
  else hipLaunchKernelGGL((gemm_skinny_kernel<DT, 16, VN>), grid, dim3(SK_LANES * SK_RG), lds, ctx->stream, a);
  hipError_t e = hipGetLastError();
  if (e == hipSuccess && nsplit > 1) {
    const int64_t total = g.M * g.N;
    hipLaunchKernelGGL((skinny_finish_kernel<DT>), dim3((unsigned)((total + 1023) / 1024)), dim3(256), 0, ctx->stream,
                       (const float *)part, g.C, g.M, g.N, (int)nsplit, g.crs, g.ccs);
    e = hipGetLastError();
  }
  if (part) nxh_free_locked(ctx, part);
  if (e != hipSuccess) return nxh_hip_fail("matmul", e);
  return NXH_OK;
}

// bf16 / f16, whole 8-column vectors: the MFMA form of the skinny product.
template <int DT>
static int launch_skinny_mfma(nxh_context *ctx, GemmArgs &g) {
  SkinnyArgs a;
  a.A = g.A;
  a.B = g.B;
  a.M = g.M;
  a.N = g.N;
  a.K = g.K;
  a.ars = g.ars;
  a.acs = g.acs;
  a.brs = g.brs;
  a.crs = g.crs;
  a.ccs = g.ccs;
  const int cus = ctx->compute_units > 0 ? ctx->compute_units : 256;
  // N alone fills the chip with 64-column blocks: K is split inside the block, one launch
  const int64_t strips = (g.N + SM_WN - 1) / SM_WN;
  if (strips >= cus && g.K % 8 == 0 && g.K >= SM8_WAVES * 2 * SM_KS && (g.M == 1 || (g.acs == 1 && g.ars % 8 == 0)) &&
      (g.M > 1 || g.acs == 1) && ((uintptr_t)g.A % 16) == 0 && strips <= 0x7fffffffLL) {
    auto kern = gemm_skinny_mfma_k8_kernel<DT == NXH_BF16>;
    constexpr size_t LDS = sizeof(uint16_t) * (size_t)(SM8_WAVES * 2 * SM_TILE);
    static_assert(LDS >= sizeof(float) * SM8_WAVES * 16 * SM_WN, "the fold buffer reuses the tiles");
    static std::once_flag once;
    static hipError_t attr_status = hipSuccess;
    std::call_once(once, [&] {
      attr_status = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS);
    });
    NXH_HIP("matmul", attr_status);
    a.kchunk = ((g.K + SM8_WAVES - 1) / SM8_WAVES + SM_KS - 1) / SM_KS * SM_KS;
    a.nsplit = 1;
    a.C = g.C;
    nxh_set_path("gemm_skinny_mfma_k8");
    hipLaunchKernelGGL(kern, dim3((unsigned)strips), dim3(64 * SM8_WAVES), LDS, ctx->stream, a);
    NXH_HIP("matmul", hipGetLastError());
    return NXH_OK;
  }
  const int64_t col_blocks = (g.N + 4 * SM_WN - 1) / (4 * SM_WN);
  int64_t want = std::max<int64_t>(1, ((int64_t)cus * 2 + col_blocks - 1) / col_blocks);
  int64_t nsplit = std::min<int64_t>(want, std::max<int64_t>(1, g.K / 128));
  int64_t kchunk = (g.K + nsplit - 1) / nsplit;
  kchunk = std::min<int64_t>((kchunk + SM_KS - 1) / SM_KS * SM_KS, 1024);  // the A chunk must fit in LDS
  if (kchunk < g.K) {
    kchunk = chunk_off_channel_stride(kchunk, g.brs * 2);
    kchunk = (kchunk + SM_KS - 1) / SM_KS * SM_KS;
  }
  nsplit = std::max<int64_t>(1, (g.K + kchunk - 1) / kchunk);
  a.kchunk = kchunk;
  a.nsplit = (int)nsplit;
  const size_t lds = sizeof(uint16_t) * (size_t)(16 * (kchunk + 8) + 4 * 2 * SM_TILE);
  void *part = nullptr;
  if (nsplit > 1) {
    int rc = nxh_alloc_locked(ctx, (size_t)nsplit * g.M * g.N * sizeof(float), &part);
    if (rc) return rc;
    a.C = part;
  } else {
    a.C = g.C;
  }
  nxh_set_path(nsplit > 1 ? "gemm_skinny_mfma_split" : "gemm_skinny_mfma");
  dim3 grid((unsigned)col_blocks, (unsigned)nsplit);
  hipLaunchKernelGGL((gemm_skinny_mfma_kernel<DT == NXH_BF16>), grid, dim3(256), lds, ctx->stream, a);
  hipError_t e = hipGetLastError();
  if (e == hipSuccess && nsplit > 1) {
    const int64_t total = g.M * g.N;
    hipLaunchKernelGGL((skinny_finish_kernel<DT>), dim3((unsigned)((total + 1023) / 1024)), dim3(256), 0, ctx->stream,
                       (const float *)part, g.C, g.M, g.N, (int)nsplit, g.crs, g.ccs);
    e = hipGetLastError();
  }
  if (part) nxh_free_locked(ctx, part);
  if (e != hipSuccess) return nxh_hip_fail("matmul", e);
  return NXH_OK;
}

static bool al16(const void *p) { return ((uintptr_t)p & 15) == 0; }

// The LDS-tiled family of gemm_tile.hpp: K a multiple of one slab (64 two-byte or
// 32 four-byte elements), 16-byte aligned rows, unit-stride C. Returns -1 when the call does not qualify.
template <class EL, bool A_KC, bool B_KC, class SH, bool EDGE, bool EPI, bool OUT32 = false>
static int launch_tile(nxh_context *ctx, gemm_tile::Args &g, const char *path) {
  auto kern = gemm_tile::kernel<EL, A_KC, B_KC, SH, EDGE, EPI, OUT32>;
  constexpr size_t LDS = SH::template lds_bytes<EL>();
  // once per process and kernel (contexts have separate mutexes): allow > 64 KiB of dynamic LDS
  static std::once_flag once;
  static hipError_t attr_status = hipSuccess;
  std::call_once(once, [&] {
    attr_status = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS);
  });
  NXH_HIP("matmul", attr_status);
  g.tiles_m = (uint32_t)((g.M + SH::BM - 1) / SH::BM);
  g.tiles_n = (uint32_t)((g.N + SH::BN - 1) / SH::BN);
  if (EPI && g.ngroup > 1) {
    g.gtn = g.tiles_n;
    g.tiles_n *= g.ngroup;  // the members side by side, as one product of ngroup x N columns would be walked
  }
  nxh_set_path(path);
  hipLaunchKernelGGL(kern, dim3(g.tiles_m * g.tiles_n * g.nbatch), dim3(SH::THREADS), LDS, ctx->stream, g);
  NXH_HIP("matmul", hipGetLastError());
  return NXH_OK;
}
template <class EL, class SH, bool EPI, bool OUT32 = false>
static int launch_tile_oriented(nxh_context *ctx, gemm_tile::Args &g, bool a_kc, bool b_kc, const char *path) {
  const bool edge = g.M % SH::BM != 0 || g.N % SH::BN != 0;
#define NXH_TILE(AK, BK_)                                                                  \
  (edge ? launch_tile<EL, AK, BK_, SH, true, EPI, OUT32>(ctx, g, path) : launch_tile<EL, AK, BK_, SH, false, EPI, OUT32>(ctx, g, path))
  if (a_kc) return b_kc ? NXH_TILE(true, true) : NXH_TILE(true, false);
  return b_kc ? NXH_TILE(false, true) : NXH_TILE(false, false);
#undef NXH_TILE
}
// The direct-to-LDS kernels (gemm_dl.hpp): whole tiles of 16-bit operands.
template <class EL, bool A_KC, bool B_KC, class SH, bool EPI>
static int launch_dl(nxh_context *ctx, gemm_tile::Args &g, const char *path) {
  auto kern = gemm_dl::kernel<EL, A_KC, B_KC, SH, EPI>;
  static std::once_flag once;
  static hipError_t attr_status = hipSuccess;
  std::call_once(once, [&] {
    attr_status = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)SH::LDS_BYTES);
  });
  NXH_HIP("matmul", attr_status);
  g.tiles_m = (uint32_t)(g.M / SH::BM);
  g.tiles_n = (uint32_t)(g.N / SH::BN);
  if (EPI && g.ngroup > 1) {
    g.gtn = g.tiles_n;
    g.tiles_n *= g.ngroup;  // the members side by side, as in launch_tile
  }
  nxh_set_path(path);
  hipLaunchKernelGGL(kern, dim3(g.tiles_m * g.tiles_n * g.nbatch), dim3(SH::THREADS), SH::LDS_BYTES, ctx->stream, g);
  NXH_HIP("matmul", hipGetLastError());
  return NXH_OK;
}
// Returns -1 for an orientation that has no instance: a transposed A (contiguous along M)
// is only built for the plain 256 x 256 product.
template <class EL, class SH, bool EPI>
static int launch_dl_oriented(nxh_context *ctx, gemm_tile::Args &g, bool a_kc, bool b_kc, const char *path) {
  if constexpr (EL::F32) {
    return -1;
  } else {
    if (a_kc) return b_kc ? launch_dl<EL, true, true, SH, EPI>(ctx, g, path) : launch_dl<EL, true, false, SH, EPI>(ctx, g, path);
    if constexpr (!EPI && SH::BM == 256)
      return b_kc ? launch_dl<EL, false, true, SH, EPI>(ctx, g, path) : launch_dl<EL, false, false, SH, EPI>(ctx, g, path);
    return -1;
  }
}
// 0: pick by shape; 256 / 192 / 128 / 64 / 1264 / 6464: force that block shape (192: 128 x 192, direct to
// LDS; 128: the register-staged 128 x 128; 1264: 128 x 64; 6464: 64 x 64, f32); 257: the 256 shape in its
// register-staged form (tuning aid, read once from NXH_GEMM_TILE)
static int forced_tile() {
  static const int v = [] {
    const char *e = getenv("NXH_GEMM_TILE");
    return e ? atoi(e) : 0;
  }();
  return v;
}
// The epilogue operands of nxh_linear (null members: that step is left out).
struct Epilogue {
  const void *bias = nullptr, *R = nullptr;
  int64_t ldr = 0, br[MM_MAXB] = {};
  const double *gelu = nullptr;  // c0..c3 of the tanh GELU, applied to the biased product
  // further members of a grouped launch: byte distances of their B, C and bias from the first's
  int ngroup = 1;
  int64_t goff_b[2] = {}, goff_c[2] = {}, goff_bias[2] = {};
};
template <class EL, bool EPI = false>
static int try_tile(nxh_context *ctx, const GemmArgs &a, uint32_t nbatch, bool al_a, bool al_b,
                    const Epilogue *epi = nullptr) {
  constexpr int VE = EL::VE, BK = gemm_tile::Geo<EL>::BK;
  if (a.K % BK || a.K < BK || a.M < VE || a.N < VE) return -1;
  if (a.ccs != 1 || a.batch.n > 4 || !al_a || !al_b) return -1;
  const bool a_kc = a.acs == 1, b_kc = a.brs == 1;
  // A wide 16-bit product whose N is no whole number of 256-column blocks (GPT-2's tied head,
  // [8192,768] x [768,50257]): the whole blocks take the direct-to-LDS kernel, which has no
  // ragged form, and the last columns a launch of their own. Every output element is still
  // one k-ordered f32 sum rounded once, so the split changes no bit of the result.
  if constexpr (!EL::F32 && !EPI) {
    const int64_t n0 = a.N / 256 * 256;
    if (a.N % 256 && n0 >= 8 * 256 && a.M % 256 == 0 && a.M >= 1024 && !forced_tile() && a.n_ld == a.N) {
      GemmArgs left = a, right = a;
      left.N = left.n_ld = n0;
      right.N = right.n_ld = a.N - n0;
      right.B = (const char *)a.B + n0 * a.bcs * (int64_t)sizeof(typename EL::S);
      right.C = (char *)a.C + n0 * (int64_t)sizeof(typename EL::S);
      int rc = try_tile<EL, false>(ctx, left, nbatch, al_a, al_b, nullptr);
      if (rc == NXH_OK) {
        const char *path = nxh_last_path(ctx);
        // (the right part's B starts n0 columns in: 16-byte aligned, since n0 is a multiple of 256)
        rc = try_tile<EL, false>(ctx, right, nbatch, al_a, al_b, nullptr);
        nxh_set_path(path);
      }
      if (rc != -1) return rc;  // (-1: the whole product takes the ordinary path below; what the left part wrote is rewritten)
    }
  }
  gemm_tile::Args g{};
  g.A = a.A;
  g.B = a.B;
  g.C = a.C;
  g.lda = a_kc ? a.ars : a.acs;
  g.ldb = b_kc ? a.bcs : a.brs;
  g.ldc = a.crs;
  if (!al16(g.A) || !al16(g.B) || g.lda % VE || g.ldb % VE) return -1;
  // an operand contiguous along M / N is read in whole 16-byte vectors
  if ((!a_kc && a.m_ld % VE) || (!b_kc && a.n_ld % VE)) return -1;
  g.M = a.M;
  g.N = a.N;
  g.K = a.K;
  g.Mld = a.m_ld;
  g.Nld = a.n_ld;
  g.nbatch = nbatch;
  g.nbd = a.batch.n;
  for (int i = 0; i < a.batch.n; i++) {
    g.bshape[i] = a.batch.shape[i];
    g.ba[i] = a.batch.a[i];
    g.bb[i] = a.batch.b[i];
    g.bc[i] = a.batch.c[i];
    if (EPI) g.br[i] = epi->br[i];
  }
  if (EPI) {
    g.bias = epi->bias;
    g.R = epi->R;
    g.ldr = epi->ldr;
    if (epi->ngroup > 1) {
      constexpr int64_t es = (int64_t)sizeof(typename EL::S);
      g.ngroup = (uint32_t)epi->ngroup;
      for (int i = 0; i + 1 < epi->ngroup; i++) {
        // the members' rows must be as aligned as the first's: whole 16-byte steps apart
        if (epi->goff_b[i] % 16 || epi->goff_c[i] % 16 || epi->goff_bias[i] % 16) return -1;
        g.goff_b[i] = epi->goff_b[i] / es;
        g.goff_c[i] = epi->goff_c[i] / es;
        g.goff_bias[i] = epi->goff_bias[i] / es;
      }
    }
    if (epi->gelu) {
      // only the paths that send whole 16-byte row segments of whole tiles apply it
      const bool whole = (a.M % 128 == 0 && a.N % 128 == 0) || (a_kc && a.M % 128 == 0 && a.N % 192 == 0);
      if (EL::F32 || epi->R || !whole || !al16(g.C) || g.ldc % 8 || (g.bias && !al16(g.bias))) return -1;
      for (int i = 0; i < a.batch.n; i++)
        if (g.bc[i] % 8) return -1;
      g.gelu = 1;
      for (int i = 0; i < 4; i++) g.gc[i] = (float)epi->gelu[i];
      if constexpr (EL::BF16) {
        const void *lut = nullptr;
        uint32_t lo = 0, n = 0;
        if (nxh_gelu_epilogue_table(ctx, epi->gelu, &lut, &lo, &n)) {
          g.gelu_lut = lut;
          g.lut_lo = lo;
          g.lut_n = n;
        }
      }
    }
  }
  // tiles of one member: a grouped launch picks the block shape its members would pick alone,
  // so that each member's bits are those of its own call
  const int members = EPI && epi ? epi->ngroup : 1;
  auto tiles = [&](int bm, int bn) { return ((a.M + bm - 1) / bm) * ((a.N + bn - 1) / bn) * (int64_t)nbatch; };
  if (tiles(128, 64) * members > 0x7fffffffLL) return -1;
  const int cus = ctx->compute_units > 0 ? ctx->compute_units : 256;
  // Block shape: rounds of resident blocks x relative cost of one block. One
  // 256x256 block (8 waves, 144 KiB of LDS) fills a CU; two 128x128 blocks fit,
  // each a quarter of the work at about 0.8 of the big tile's efficiency.
  int pick = forced_tile();
  if (!pick && EL::F32) {
    // f32: a compute unit's f32 matrix rate is a sixteenth of its 16-bit rate, so a block's time
    // is all arithmetic and the shapes differ only in what they leave idle: rounds of one block
    // per unit x the block's area (ragged edges count as whole blocks) x the shape's measured cost
    // per flop against the 256 x 256 block (4096^3: 138 TFLOP/s there, 123 with half blocks;
    // 1024^3 on quarter blocks about 100 inside the K loop).
    struct Cand {
      int pick, bm, bn;
      double pen;
    };
    const Cand cands[] = {{256, 256, 256, 1.0}, {128, 128, 128, 1.12}, {64, 256, 64, 1.12},
                          {1264, 128, 64, 1.15}, {6464, 64, 64, 1.3}};
    double best = 0.0;
    for (const Cand &c : cands) {
      if (c.pick == 64 && a.N > 64) continue;
      if (EPI && epi->gelu && c.pick != 256 && c.pick != 128) continue;
      const double cost = (double)((tiles(c.bm, c.bn) * members + cus - 1) / cus) * c.bm * c.bn * c.pen;
      if (!pick || cost < best) {
        pick = c.pick;
        best = cost;
      }
    }
  } else if (!pick) {
    if (a.N <= 64) pick = 64;
    else {
      const double c256 = (double)((tiles(256, 256) + cus - 1) / cus);
      const double c128 = (double)((tiles(128, 128) + 2 * cus - 1) / (2 * cus)) * 0.6;
      pick = c256 <= c128 ? 256 : 128;
    }
    // Fewer blocks than half the compute units: half blocks (128 x 64, four waves of 64 x 32)
    // put twice as many of them to work (bf16 [1024,768] x [768,768]: 9.5 -> 7.9 us).
    if (pick != 256 && !(EPI && epi->gelu) && (pick == 64 ? tiles(256, 64) : tiles(128, 128)) * members <= cus / 2)
      pick = 1264;
  }
  // Whole tiles of 16-bit operands go straight into LDS (gemm_dl.hpp; load offsets are 32-bit:
  // 256 rows of a k-contiguous operand must stay below 4 GiB, and every row segment the
  // epilogue touches must be 16-byte aligned).
  // A 16-bit product larger than the memory-side cache, rows of C whole 16-byte pieces: the
  // direct-to-LDS kernels store C past the cache, which then keeps the operand panels that the
  // other row and column blocks read again (bf16 [16,4096,4096]^2: 1 199-1 202 -> 1 205-1 224
  // TFLOP/s). Not for rows at odd offsets (GPT-2's tied head, pitch 50 257): partial lines
  // written past the cache cost that product 0.34 of its 0.72 ms.
  if constexpr (!EPI && !EL::F32)
    g.stream_c = (ctx->cache_hints & 2) && al16(g.C) && g.ldc % 8 == 0 && (uint64_t)nbatch * a.M * a.N * 2 > ((uint64_t)256 << 20);
  if constexpr (!EL::F32) {
    const int forced = forced_tile();
    // (without an epilogue C's rows may start at any element: the stores are unaligned-capable)
    bool dl_ok = (pick == 256 || pick == 128 || pick == 192) && forced != 257 && forced != 128 &&
                 (!EPI || (al16(g.C) && g.ldc % 8 == 0)) && g.lda < ((int64_t)1 << 22) && g.ldb < ((int64_t)1 << 22);
    for (int i = 0; i < a.batch.n; i++)
      if (EPI && (g.bc[i] % 8 || (g.R && g.br[i] % 8))) dl_ok = false;
    if (EPI && ((g.bias && !al16(g.bias)) || (g.R && (!al16(g.R) || g.ldr % 8)))) dl_ok = false;
    if (dl_ok) {
      // (the f16 conversions make the large shape's epilogue spill: f16 linears keep to the others)
      const bool can256 = a.M % 256 == 0 && a.N % 256 == 0 && forced != 192 && !(EPI && !EL::BF16);
      const bool can192 = a_kc && a.M % 128 == 0 && a.N % 192 == 0 && forced != 256;
      // rounds of one block per compute unit x the block's share of a 256 x 256 tile's work,
      // the smaller shape at about 0.8 of the large one's rate
      const double d256 = (double)((tiles(256, 256) + cus - 1) / cus);
      const double d192 = (double)((tiles(128, 192) + cus - 1) / cus) * (128.0 * 192.0 / 65536.0 / 0.8);
      int rc = -1;
      if (can192 && (!can256 || pick != 256 || d192 < d256)) {
        // one block per compute unit at most: nothing shares the unit, so the ring goes deeper
        if (tiles(128, 192) * members <= cus)
          rc = launch_dl_oriented<EL, gemm_dl::Shape128x192Deep, EPI>(ctx, g, a_kc, b_kc, EPI ? "linear_dl_128x192" : "gemm_dl_128x192");
        else
          rc = launch_dl_oriented<EL, gemm_dl::Shape128x192, EPI>(ctx, g, a_kc, b_kc, EPI ? "linear_dl_128x192" : "gemm_dl_128x192");
      }
      else if (can256 && pick == 256) {
        if constexpr (!EPI || EL::BF16)
          rc = launch_dl_oriented<EL, gemm_dl::Shape256x256, EPI>(ctx, g, a_kc, b_kc, EPI ? "linear_dl_256x256" : "gemm_dl_256x256");
      }
      if (rc != -1) return rc;
    }
  }
  if (g.gelu && (a.M % 128 || a.N % 128)) return -1;
  if (pick == 192) pick = 128;
  if constexpr (!EPI) {
    // One product (no batch) cut along K: `split` equal runs of whole slabs are walked as a batch
    // dim that writes [split][M][N] f32 partial sums (the 16-bit kernels in their f32-output
    // form), which a second kernel adds in run order (a fixed order: the same bits on every
    // call) and rounds to the dtype once. shape: 0 = 64 x 64 (f32), 1 = 128 x 64, 2 = 128 x 128 (16-bit).
    auto cut_along_k = [&](int64_t split, int shape) -> int {
      constexpr int DT = EL::F32 ? NXH_F32 : EL::BF16 ? NXH_BF16 : NXH_F16;
      void *part = nullptr;
      int rc = nxh_alloc_locked(ctx, (size_t)split * a.M * a.N * sizeof(float), &part);
      if (rc) return rc;
      gemm_tile::Args gs = g;
      gs.K = a.K / split;
      gs.nbatch = (uint32_t)split;
      gs.nbd = 1;
      gs.bshape[0] = (uint32_t)split;
      gs.ba[0] = gs.K * (a_kc ? 1 : g.lda);
      gs.bb[0] = gs.K * (b_kc ? 1 : g.ldb);
      gs.bc[0] = a.M * a.N;
      gs.C = part;
      gs.ldc = a.N;
      if constexpr (EL::F32) {
        rc = shape == 0 ? launch_tile_oriented<EL, gemm_tile::Shape64x64, false>(ctx, gs, a_kc, b_kc, "gemm_tile_64x64_splitk")
                        : launch_tile_oriented<EL, gemm_tile::Shape128x64, false>(ctx, gs, a_kc, b_kc, "gemm_tile_128x64_splitk");
      } else {
        rc = shape == 2 ? launch_tile_oriented<EL, gemm_tile::Shape128x128, false, true>(ctx, gs, a_kc, b_kc, "gemm_tile_128x128_splitk")
                        : launch_tile_oriented<EL, gemm_tile::Shape128x64, false, true>(ctx, gs, a_kc, b_kc, "gemm_tile_128x64_splitk");
      }
      if (rc == NXH_OK) {
        const int64_t total = a.M * a.N;
        hipLaunchKernelGGL((skinny_finish_kernel<DT>), dim3((unsigned)((total + 1023) / 1024)), dim3(256), 0, ctx->stream,
                           (const float *)part, g.C, a.M, a.N, (int)split, g.ldc, (int64_t)1);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) rc = nxh_hip_fail("matmul", e);
      }
      nxh_free_locked(ctx, part);
      return rc;
    };
    const int64_t slabs = a.K / BK;
    // A 16-bit weight matrix of 16 MiB or more streamed once past at most 128 rows (a decode step
    // of 17 to 128 sequences): memory-bound on B. 128-column blocks keep 256-byte row segments and
    // two slabs of 16 KiB in flight each ([32,4096] x [4096,32000], 250 such blocks, streams B
    // at 6 TB/s); with fewer column blocks than units K is cut until the blocks fill the chip.
    if constexpr (!EL::F32) {
      if (nbatch == 1 && a.batch.n == 0 && a.M <= 128 && !forced_tile() &&
          (double)a.K * (double)a.N * 2.0 >= (double)(16 << 20) && tiles(128, 128) < cus) {
        int64_t split = std::min<int64_t>(cus / tiles(128, 128), slabs / 8);
        while (split > 1 && slabs % split) split--;
        if (split >= 2) return cut_along_k(split, 2);
      }
    }
    // A product whose blocks leave half of the units idle and whose K is long (a weight gradient:
    // [768, 8192] x [8192, 768]).
    if (nbatch == 1 && a.batch.n == 0 && (pick == 1264 || pick == 6464)) {
      const int64_t blocks = pick == 6464 ? tiles(64, 64) : tiles(128, 64);
      // Worth it when the slabs a block no longer walks (about 0.3 us each for a 16-bit block that
      // has its unit to itself, 0.7 us for f32) outweigh the second launch and the partial sums'
      // trip through memory (bf16 [1000,8192] x [8192,1000]: 57 -> 39 us with two runs; [1024,1024]^2
      // would go from 9.5 to 15 us and stays whole).
      int64_t split = 1;
      double best_gain = 0.0;
      for (int64_t sp = std::min<int64_t>(cus / blocks, slabs / 4); sp >= 2; sp--) {
        if (slabs % sp) continue;
        const double saved = (double)slabs * (1.0 - 1.0 / (double)sp) * (EL::F32 ? 0.7 : 0.3);
        const double cost = 4.0 + (double)sp * (double)a.M * (double)a.N * 8.0 / 4e6;
        if (saved - 1.2 * cost > best_gain) {
          best_gain = saved - 1.2 * cost;
          split = sp;
        }
      }
      if (split >= 2) return cut_along_k(split, pick == 6464 ? 0 : 1);
    }
  }
  if constexpr (EL::F32) {
    if (pick == 6464)
      return launch_tile_oriented<EL, gemm_tile::Shape64x64, EPI>(ctx, g, a_kc, b_kc, EPI ? "linear_tile_64x64" : "gemm_tile_64x64");
  }
  if constexpr (EPI) {
    // Two block shapes are enough for the epilogue family; f16 keeps to the small one (its
    // conversions make the 256x256 epilogue too large to stay in registers).
    constexpr bool big_ok = EL::F32 || EL::BF16;
    if (pick == 1264)
      return launch_tile_oriented<EL, gemm_tile::Shape128x64, true>(ctx, g, a_kc, b_kc, "linear_tile_128x64");
    if (pick == 64 || !big_ok || (g.gelu && (a.M % 256 || a.N % 256))) pick = 128;
    if (pick == 128)
      return launch_tile_oriented<EL, gemm_tile::Shape128x128, true>(ctx, g, a_kc, b_kc, "linear_tile_128x128");
    if constexpr (big_ok)
      return launch_tile_oriented<EL, gemm_tile::Shape256x256, true>(ctx, g, a_kc, b_kc, "linear_tile_256x256");
  }
  if (pick == 1264) return launch_tile_oriented<EL, gemm_tile::Shape128x64, false>(ctx, g, a_kc, b_kc, "gemm_tile_128x64");
  if (pick == 64) return launch_tile_oriented<EL, gemm_tile::Shape256x64, false>(ctx, g, a_kc, b_kc, "gemm_tile_256x64");
  if (pick == 128)
    return launch_tile_oriented<EL, gemm_tile::Shape128x128, false>(ctx, g, a_kc, b_kc, "gemm_tile_128x128");
  return launch_tile_oriented<EL, gemm_tile::Shape256x256, false>(ctx, g, a_kc, b_kc, "gemm_tile_256x256");
}

// ── padded copies for the tiled kernels ─────────────────────────────────────
// The tiled kernels read whole 16-byte vectors of whole K-slabs. An operand whose rows are not
// that (a [.., K, 196] matrix of unfolded 14 x 14 windows, a K of 196) is copied once into a
// buffer whose contiguous dim is rounded up to whole vectors and whose K is rounded up to
// whole slabs, the new positions filled with zeros (0 x 0 adds nothing to any sum; both operands
// are padded along K). A broadcast batch dim stays a zero stride of the copy.
struct RepackArgs {
  const void *src;
  void *dst;
  int64_t rows, cols;    // logical extents: `cols` is the dim that becomes contiguous
  int64_t prows, pcols;  // padded extents (pcols a multiple of the vector)
  int64_t srs, scs;      // source strides of (row, col), elements
  int nbd;
  uint32_t bshape[MM_MAXB];
  int64_t bsrc[MM_MAXB];  // source strides of the batch dims that are not broadcast
  int64_t total;          // vectors to write
};
template <class S>
__global__ __launch_bounds__(256) void gemm_repack_kernel(RepackArgs a) {
  constexpr int VE = 16 / (int)sizeof(S);
  const int64_t v = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (v >= a.total) return;
  const int64_t vpr = a.pcols / VE;
  const int64_t t = v / vpr, c0 = (v - t * vpr) * VE;
  int64_t bidx = t / a.prows;
  const int64_t r = t - bidx * a.prows;
  int64_t so = 0;
  for (int i = a.nbd - 1; i >= 0; i--) {
    const int64_t q = bidx / a.bshape[i];
    so += (bidx - q * a.bshape[i]) * a.bsrc[i];
    bidx = q;
  }
  const S *src = (const S *)a.src + so + r * a.srs;
  union {
    U4 v4;
    uint32_t w[4];
    S s[VE];
  } o;
  o.v4 = U4{0, 0, 0, 0};
  if (r < a.rows) {
    if constexpr (sizeof(S) == 2) {
      if (a.scs == 1) {
        // 16-bit elements of a contiguous row: whole 4-byte words from the word-aligned address
        // at or below the first element, shifted by one element where the row starts on an odd
        // one (eight 2-byte loads per lane held this copy at half the memory rate). A word is
        // read only if its first element belongs to the row; elements past the row's end are
        // cleared afterwards.
        const uintptr_t first = (uintptr_t)(src + c0);
        const uint32_t *wp = (const uint32_t *)(first & ~(uintptr_t)3);
        const int odd = (int)((first >> 1) & 1);
        const int64_t left = a.cols - c0 + odd;  // elements from wp's first to the row's end
        uint32_t w[5];
#pragma unroll
        for (int j = 0; j < 5; j++) w[j] = (2 * j < left && (j < 4 || odd)) ? wp[j] : 0u;
#pragma unroll
        for (int j = 0; j < 4; j++) o.w[j] = odd ? __builtin_amdgcn_alignbit(w[j + 1], w[j], 16) : w[j];
#pragma unroll
        for (int j = 0; j < VE; j++)
          if (c0 + j >= a.cols) o.s[j] = (S)0;
        ((U4 *)a.dst)[v] = o.v4;
        return;
      }
    }
#pragma unroll
    for (int j = 0; j < VE; j++)
      if (c0 + j < a.cols) o.s[j] = src[(c0 + j) * a.scs];
  }
  ((U4 *)a.dst)[v] = o.v4;
}

// Copies one operand (kc: contiguous along K in the copy, else along its M / N dim) and
// rewrites its strides in place. `bstr` are the operand's batch strides.
template <class S>
static int repack_operand(nxh_context *ctx, const GemmArgs &g, const void *src, bool kc, int64_t rows_mn, int64_t Kp,
                          int64_t &stride_mn, int64_t &stride_k, int64_t *bstr, int64_t &ld_mn, void **block) {
  constexpr int VE = 16 / (int)sizeof(S);
  RepackArgs r{};
  r.src = src;
  if (kc) {
    r.rows = r.prows = rows_mn;
    r.cols = g.K;
    r.pcols = Kp;
    r.srs = stride_mn;
    r.scs = stride_k;
  } else {
    r.rows = g.K;
    r.prows = Kp;
    r.cols = rows_mn;
    r.pcols = (rows_mn + VE - 1) / VE * VE;
    r.srs = stride_k;
    r.scs = stride_mn;
  }
  // the copy's batch layout: dense over the dims the operand really has
  int64_t run = r.prows * r.pcols, nstr[MM_MAXB] = {};
  for (int i = g.batch.n - 1; i >= 0; i--) {
    if (bstr[i] == 0) continue;
    nstr[i] = run;
    run *= g.batch.shape[i];
  }
  for (int i = 0; i < g.batch.n; i++) {
    if (bstr[i] == 0) continue;
    r.bshape[r.nbd] = g.batch.shape[i];
    r.bsrc[r.nbd] = bstr[i];
    r.nbd++;
  }
  if (run > ((int64_t)1 << 32)) return -1;  // more than the fast path is worth
  int rc = nxh_alloc_locked(ctx, (size_t)run * sizeof(S), block);
  if (rc) return rc;
  r.dst = *block;
  r.total = run / VE;
  hipLaunchKernelGGL((gemm_repack_kernel<S>), dim3((unsigned)((r.total + 255) / 256)), dim3(256), 0, ctx->stream, r);
  NXH_HIP("matmul", hipGetLastError());
  if (kc) {
    stride_mn = Kp;
    stride_k = 1;
  } else {
    stride_mn = 1;
    stride_k = r.pcols;
    ld_mn = r.pcols;
  }
  for (int i = 0; i < g.batch.n; i++) bstr[i] = nstr[i];
  return NXH_OK;
}

// The tiled path over padded copies of the operands that do not fit it as they are. -1: not
// worth it or not possible (the caller falls back to the general kernel).
template <class EL>
static int try_tile_repacked(nxh_context *ctx, const GemmArgs &a0, uint32_t nbatch, bool al_a, bool al_b) {
  using S = typename EL::S;
  constexpr int VE = EL::VE, BK = gemm_tile::Geo<EL>::BK;
  if (a0.ccs != 1 || a0.batch.n > 4 || a0.M < 32 || a0.N < 32 || a0.K < 32) return -1;
  // two more launches and a pass over the copied operand: only for products that outweigh them
  if ((double)a0.M * (double)a0.N * (double)a0.K * (double)nbatch < (double)(1 << 27)) return -1;
  GemmArgs a = a0;
  const int64_t Kp = (a.K + BK - 1) / BK * BK;
  const bool a_kc = a.acs == 1, b_kc = a.brs == 1;
  const bool fit_a = Kp == a.K && al_a && al16(a.A) && (a_kc ? a.ars % VE == 0 : (a.acs % VE == 0 && a.M % VE == 0));
  const bool fit_b = Kp == a.K && al_b && al16(a.B) && (b_kc ? a.bcs % VE == 0 : (a.brs % VE == 0 && a.N % VE == 0));
  if (fit_a && fit_b) return -1;  // the tiled path refused for another reason
  void *blk_a = nullptr, *blk_b = nullptr;
  int rc = NXH_OK;
  if (!fit_a) rc = repack_operand<S>(ctx, a, a.A, a_kc, a.M, Kp, a.ars, a.acs, a.batch.a, a.m_ld, &blk_a);
  if (rc == NXH_OK && !fit_b) rc = repack_operand<S>(ctx, a, a.B, b_kc, a.N, Kp, a.bcs, a.brs, a.batch.b, a.n_ld, &blk_b);
  if (rc == NXH_OK) {
    if (blk_a) a.A = blk_a;
    if (blk_b) a.B = blk_b;
    a.K = Kp;
    rc = try_tile<EL>(ctx, a, nbatch, true, true);
    if (rc == NXH_OK) nxh_set_path("gemm_tile_padded");
  }
  if (blk_a) nxh_free_locked(ctx, blk_a);
  if (blk_b) nxh_free_locked(ctx, blk_b);
  return rc;
}

// ── gemm_tiny: many products of matrices of a few elements each ─────────────
// ([65536, 4, 4] x [65536, 4, 4]: transforms, small covariance blocks.) One lane per output over
// the whole batch, so a wave holds the outputs of several products and neighbouring lanes share
// their operands' cache lines; a tiled block per product left all but a few of its lanes on
// padding (that shape: 798 us).
template <int DT>
__global__ __launch_bounds__(256) void gemm_tiny_kernel(GemmArgs a, uint32_t total) {
  using TR = Tr<DT>;
  using S = typename TR::S;
  const uint32_t o = blockIdx.x * 256u + threadIdx.x;
  if (o >= total) return;
  const uint32_t per = (uint32_t)(a.M * a.N);
  const uint32_t b = o / per, r = o - b * per;
  const uint32_t m = r / (uint32_t)a.N, n = r - m * (uint32_t)a.N;
  int64_t ao, bo, co;
  batch_decode(a.batch, a.batch0 + b, ao, bo, co);
  const S *A = (const S *)a.A + ao + (int64_t)m * a.ars;
  const S *B = (const S *)a.B + bo + (int64_t)n * a.bcs;
  float acc = 0.0f;
  for (int64_t k = 0; k < a.K; k++) acc = acc + (float)TR::ld(A[k * a.acs]) * (float)TR::ld(B[k * a.brs]);
  ((S *)a.C)[co + (int64_t)m * a.crs + (int64_t)n * a.ccs] = TR::st((typename TR::C)acc);
}
template <int DT>
static int launch_tiny(nxh_context *ctx, GemmArgs &a, uint32_t nbatch) {
  nxh_set_path("gemm_tiny");
  const uint32_t per = (uint32_t)(a.M * a.N), step = 0x7fffff00u / per;  // products per launch
  for (uint32_t b0 = 0; b0 < nbatch; b0 += step) {
    a.batch0 = b0;
    const uint32_t total = std::min<uint32_t>(step, nbatch - b0) * per;
    hipLaunchKernelGGL((gemm_tiny_kernel<DT>), dim3((total + 255) / 256), dim3(256), 0, ctx->stream, a, total);
    NXH_HIP("matmul", hipGetLastError());
  }
  return NXH_OK;
}

// ── gemm_rowdot: a matrix whose rows run along K, times one to four columns ──
// (matrix x vector: C[m][n] = sum over k of A[m][k] B[k][n], N <= 4.) A wave per row of A: its
// lanes take the row in 16-byte pieces, four in flight, multiply by the matching pieces of the
// columns (a few KB, served by the caches), add in float32 and meet through the cross-lane
// network. A is read once at the rate of a reduction over its rows; the tiled kernels spent a whole
// 128-column block on the one column ([4096,4096] x [4096,1] f32: 444 us).
template <int DT, int NC>
__global__ __launch_bounds__(256) void gemm_rowdot_kernel(GemmArgs a) {
  using TR = Tr<DT>;
  using S = typename TR::S;
  constexpr int V = 16 / (int)sizeof(S);
  struct alignas(16) Piece {
    S v[V];
  };
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t m = (int64_t)blockIdx.x * 4 + wave;
  if (m >= a.M) return;
  int64_t ao, bo, co;
  batch_decode(a.batch, a.batch0 + blockIdx.y, ao, bo, co);
  const S *A = (const S *)a.A + ao + m * a.ars;
  const S *B = (const S *)a.B + bo;
  float acc[NC];
#pragma unroll
  for (int n = 0; n < NC; n++) acc[n] = 0.0f;
  const int64_t nv = a.a_vec ? a.K / V : 0;
  const bool b_pieces = NC == 1 && a.b_vec;  // the one column is a contiguous, aligned run
  auto piece = [&](int64_t i, const Piece &x) {
    if (b_pieces) {
      const Piece y = *reinterpret_cast<const Piece *>(B + i * V);
#pragma unroll
      for (int j = 0; j < V; j++) acc[0] = acc[0] + (float)TR::ld(x.v[j]) * (float)TR::ld(y.v[j]);
    } else {
#pragma unroll
      for (int j = 0; j < V; j++) {
        const float av = (float)TR::ld(x.v[j]);
        const S *b = B + (i * V + j) * a.brs;
#pragma unroll
        for (int n = 0; n < NC; n++)
          if (n < a.N) acc[n] = acc[n] + av * (float)TR::ld(b[n * a.bcs]);
      }
    }
  };
  int64_t i = lane;
  for (; i + 192 < nv; i += 256) {
    Piece x[4];
#pragma unroll
    for (int u = 0; u < 4; u++) x[u] = *reinterpret_cast<const Piece *>(A + (i + 64 * u) * V);
#pragma unroll
    for (int u = 0; u < 4; u++) piece(i + 64 * u, x[u]);
  }
  for (; i < nv; i += 64) piece(i, *reinterpret_cast<const Piece *>(A + i * V));
  for (int64_t k = nv * V + lane; k < a.K; k += 64) {
    const float av = (float)TR::ld(A[k]);
#pragma unroll
    for (int n = 0; n < NC; n++)
      if (n < a.N) acc[n] = acc[n] + av * (float)TR::ld(B[k * a.brs + n * a.bcs]);
  }
#pragma unroll
  for (int n = 0; n < NC; n++)
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) acc[n] = acc[n] + __shfl_down(acc[n], d, 64);
  if (lane == 0) {
    S *C = (S *)a.C + co + m * a.crs;
#pragma unroll
    for (int n = 0; n < NC; n++)
      if (n < a.N) C[n * a.ccs] = TR::st((typename TR::C)acc[n]);
  }
}

template <int DT>
static int launch_rowdot(nxh_context *ctx, GemmArgs &a, uint32_t nbatch, bool batch_aligned_a, bool batch_aligned_b) {
  using S = typename Tr<DT>::S;
  constexpr int V = 16 / (int)sizeof(S);
  a.a_vec = al16(a.A) && batch_aligned_a && a.ars % V == 0;
  a.b_vec = a.N == 1 && a.brs == 1 && al16(a.B) && batch_aligned_b;
  nxh_set_path("gemm_rowdot");
  const dim3 block(256);
  for (uint32_t b0 = 0; b0 < nbatch; b0 += 65535) {
    a.batch0 = b0;
    const dim3 grid((unsigned)((a.M + 3) / 4), std::min<uint32_t>(65535, nbatch - b0));
    if (a.N == 1) hipLaunchKernelGGL((gemm_rowdot_kernel<DT, 1>), grid, block, 0, ctx->stream, a);
    else if (a.N == 2) hipLaunchKernelGGL((gemm_rowdot_kernel<DT, 2>), grid, block, 0, ctx->stream, a);
    else hipLaunchKernelGGL((gemm_rowdot_kernel<DT, 4>), grid, block, 0, ctx->stream, a);
    NXH_HIP("matmul", hipGetLastError());
  }
  return NXH_OK;
}

template <class MM>
static int run_mfma_dtype(nxh_context *ctx, GemmArgs &a, uint32_t nbatch, bool batch_aligned_a,
                          bool batch_aligned_b) {
  using S = typename MM::S;
  constexpr int VL = MM::VL;
  // many products of a few elements each: a lane per output over the whole batch
  if (a.M * a.N <= 256 && a.K <= 64 && nbatch >= 256) return launch_tiny<MM::DT>(ctx, a, nbatch);
  // matrix x vector (up to four columns), the matrix's rows along K: a wave per row
  if (a.N <= 4 && a.acs == 1 && a.K >= 64 && (double)a.M * (double)nbatch >= 256.0 && a.M <= 0x7fffffffLL)
    return launch_rowdot<MM::DT>(ctx, a, nbatch, batch_aligned_a, batch_aligned_b);
  // decode-like shape: one batch, few rows, B row-major: stream B once
  if (nbatch == 1 && a.M <= 16 && a.bcs == 1 && a.N >= 1024 && a.K >= 256 && a.batch.n == 0) {
    constexpr int VN = 16 / (int)sizeof(S);  // one 16-byte load per lane and row of B
    if (a.brs % VN == 0 && ((uintptr_t)a.B % (sizeof(S) * VN)) == 0) {
      if constexpr (sizeof(S) == 2) {
        // fewer 64-column strips than units: the 128-column blocks cut along K (try_tile) stream
        // B faster than the strips with K split across blocks ([16,4096] x [4096,8192]: 24.5 us there)
        const int cus = ctx->compute_units > 0 ? ctx->compute_units : 256;
        // (only when the cut will be taken: try_tile's own rule, 128-column blocks and runs of
        // at least eight 64-wide slabs of K; a whole-K tile kernel on 8-16 rows would lose to the strips)
        const int64_t col_blocks = (a.N + 127) / 128, slabs = a.K / 64;
        int64_t split = a.K % 64 ? 0 : std::min<int64_t>(cus / std::max<int64_t>(col_blocks, 1), slabs / 8);
        while (split > 1 && slabs % split) split--;
        if (a.M >= 8 && split >= 2 && a.N < (int64_t)64 * cus && (double)a.K * (double)a.N * 2.0 >= (double)(16 << 20)) {
          using EL = std::conditional_t<MM::DT == NXH_BF16, gemm_tile::ElBF16, gemm_tile::ElF16>;
          const int rc = try_tile<EL>(ctx, a, nbatch, batch_aligned_a, batch_aligned_b);
          if (rc != -1) return rc;
        }
        if (a.N % 8 == 0) return launch_skinny_mfma<MM::DT>(ctx, a);
      }
      return launch_skinny<MM::DT, VN>(ctx, a);
    }
  }
  const bool a_ok = a.acs == 1 || a.ars == 1, b_ok = a.brs == 1 || a.bcs == 1;
  if (!a_ok || !b_ok) return launch_any<MM::DT>(ctx, a, nbatch);
  {
    using EL = std::conditional_t<MM::DT == NXH_F32, gemm_tile::ElF32,
                                  std::conditional_t<MM::DT == NXH_BF16, gemm_tile::ElBF16, gemm_tile::ElF16>>;
    int rc = try_tile<EL>(ctx, a, nbatch, batch_aligned_a, batch_aligned_b);
    if (rc == -1) rc = try_tile_repacked<EL>(ctx, a, nbatch, batch_aligned_a, batch_aligned_b);
    if (rc != -1) return rc;
  }
  // 16-byte loads need an aligned base and every other stride a multiple of VL
  a.a_vec = al16(a.A) && batch_aligned_a && ((a.acs == 1 ? a.ars : a.acs) % VL == 0);
  a.b_vec = al16(a.B) && batch_aligned_b && ((a.brs == 1 ? a.bcs : a.brs) % VL == 0);
  return launch_mfma<MM>(ctx, a, nbatch);
}

// matmul, and with `bias` / `R` the fused linear: C = A B, then + bias[col], then
// + R, each rounded to the dtype (tiled MFMA path only).
struct GroupRest {  // members 1.. of a grouped linear, checked against member 0 by the caller
  int n = 0;
  const nxh_tensor *B[2] = {}, *bias[2] = {}, *C[2] = {};
};
static int matmul_entry(nxh_context *ctx, const char *op, const nxh_tensor *C, const nxh_tensor *A,
                        const nxh_tensor *B, const nxh_tensor *bias, const nxh_tensor *R, const double *gelu = nullptr,
                        const GroupRest *rest = nullptr) {
  if (!ctx || !C || !A || !B) return nxh_fail(NXH_INVALID_ARGUMENT, op, "null argument");
  int rc = nxh_check_tensor(op, C);
  if (!rc) rc = nxh_check_tensor(op, A);
  if (!rc) rc = nxh_check_tensor(op, B);
  if (!rc && bias) rc = nxh_check_tensor(op, bias);
  if (!rc && R) rc = nxh_check_tensor(op, R);
  if (rc) return rc;
  if (A->dtype != B->dtype || A->dtype != C->dtype) return nxh_fail(NXH_FAILURE, op, NXH_ERR_MM_DTYPE);
  const int dt = A->dtype;
  if (nxh_is_packed(dt)) return nxh_fail(NXH_FAILURE, op, NXH_ERR_PACKED);
  if (dt == NXH_BOOL) return nxh_fail(NXH_FAILURE, op, NXH_ERR_UNSUPPORTED);
  if (A->ndim < 2 || B->ndim < 2) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
  const int nd = std::max(A->ndim, B->ndim);
  if (C->ndim != nd) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
  const int64_t m = A->shape[A->ndim - 2], k = A->shape[A->ndim - 1];
  const int64_t kk = B->shape[B->ndim - 2], n = B->shape[B->ndim - 1];
  if (k != kk || C->shape[nd - 2] != m || C->shape[nd - 1] != n)
    return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
  const bool fused = bias || R || gelu;
  if (bias && (bias->dtype != dt || bias->ndim != 1 || bias->shape[0] != n))
    return nxh_fail(bias->dtype != dt ? NXH_FAILURE : NXH_INVALID_ARGUMENT, op, bias->dtype != dt ? NXH_ERR_MM_DTYPE : NXH_ERR_SHAPE);
  if (R) {
    if (R->dtype != dt) return nxh_fail(NXH_FAILURE, op, NXH_ERR_MM_DTYPE);
    if (R->ndim != nd) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
    for (int i = 0; i < nd; i++)
      if (R->shape[i] != C->shape[i]) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
  }
  if (fused && dt != NXH_BF16 && dt != NXH_F16 && dt != NXH_F32) return nxh_fail(NXH_FAILURE, op, NXH_ERR_UNSUPPORTED);
  if (fused && ((bias && n > 1 && bias->strides[0] != 1) || (R && n > 1 && R->strides[nd - 1] != 1)))
    return nxh_fail(NXH_FAILURE, op, "bias and residual must be contiguous along the columns");

  GemmArgs g;
  // batch broadcast strides (nx_c_matmul.c:895-926), then drop size-1 dims and
  // merge neighbours that compose on all three operands
  const int bnd = nd - 2, abo = nd - A->ndim, bbo = nd - B->ndim;
  int64_t bs[NXH_MAX_NDIM], as_[NXH_MAX_NDIM], bs_[NXH_MAX_NDIM], cs_[NXH_MAX_NDIM], rs_[NXH_MAX_NDIM];
  int nb = 0;
  int64_t nbatch = 1;
  for (int i = 0; i < bnd; i++) {
    int64_t sa = 1, sb = 1, sta = 0, stb = 0;
    if (i >= abo) {
      sa = A->shape[i - abo];
      sta = A->strides[i - abo];
    }
    if (i >= bbo) {
      sb = B->shape[i - bbo];
      stb = B->strides[i - bbo];
    }
    if (sa != sb && sa != 1 && sb != 1) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
    const int64_t s = std::max(sa, sb);
    if (C->shape[i] != s) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
    if (s > 1 && C->strides[i] == 0) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_OUT_ALIASED);
    nbatch *= s;
    if (s == 1) continue;
    const int64_t xa = sa == 1 ? 0 : sta, xb = sb == 1 ? 0 : stb, xc = C->strides[i];
    const int64_t xr = R ? R->strides[i] : 0;
    if (nb > 0 && as_[nb - 1] == xa * s && bs_[nb - 1] == xb * s && cs_[nb - 1] == xc * s &&
        rs_[nb - 1] == xr * s) {
      bs[nb - 1] *= s;
      as_[nb - 1] = xa;
      bs_[nb - 1] = xb;
      cs_[nb - 1] = xc;
      rs_[nb - 1] = xr;
    } else {
      bs[nb] = s;
      as_[nb] = xa;
      bs_[nb] = xb;
      cs_[nb] = xc;
      rs_[nb] = xr;
      nb++;
    }
  }
  if (m == 0 || n == 0 || nbatch == 0) return NXH_OK;
  g.ars = A->strides[A->ndim - 2];
  g.acs = A->strides[A->ndim - 1];
  g.brs = B->strides[B->ndim - 2];
  g.bcs = B->strides[B->ndim - 1];
  g.crs = C->strides[nd - 2];
  g.ccs = C->strides[nd - 1];
  if ((m > 1 && g.crs == 0) || (n > 1 && g.ccs == 0)) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_OUT_ALIASED);
  if (nb > MM_MAXB || nbatch > 0xffffffffLL) return nxh_fail(NXH_FAILURE, op, "too many batch dimensions");
  // a size-1 matrix dim carries no meaningful stride: pick the value that lets
  // the operand count as contiguous along its other dim
  if (m == 1) g.ars = g.acs == 1 ? 0 : 1;
  if (n == 1) g.bcs = g.brs == 1 ? 0 : 1;
  if (k == 1) {
    if (g.ars != 1) g.acs = 1;
    if (g.bcs != 1) g.brs = 1;
  }
  const int64_t es = nxh_elem_size(dt);
  g.A = (const char *)A->data + A->offset * es;
  g.B = (const char *)B->data + B->offset * es;
  g.C = (char *)C->data + C->offset * es;
  g.M = g.m_ld = m;
  g.N = g.n_ld = n;
  g.K = k;
  g.batch.n = nb;
  bool al_a = true, al_b = true;
  for (int i = 0; i < nb; i++) {
    if (bs[i] > 0xffffffffLL) return nxh_fail(NXH_FAILURE, op, "batch dimension too large");
    g.batch.shape[i] = (uint32_t)bs[i];
    g.batch.a[i] = as_[i];
    g.batch.b[i] = bs_[i];
    g.batch.c[i] = cs_[i];
    if ((as_[i] * es) % 16) al_a = false;
    if ((bs_[i] * es) % 16) al_b = false;
  }
  g.batch0 = 0;
  g.a_vec = g.b_vec = 0;

  std::lock_guard<std::mutex> guard(ctx->mu);
  NXH_HIP(op, hipSetDevice(ctx->device));
  if (fused) {
    Epilogue epi;
    epi.bias = bias ? (const char *)bias->data + bias->offset * es : nullptr;
    epi.R = R ? (const char *)R->data + R->offset * es : nullptr;
    epi.ldr = R ? R->strides[nd - 2] : 0;
    epi.gelu = gelu;
    if (rest && rest->n > 0) {
      epi.ngroup = 1 + rest->n;
      for (int i = 0; i < rest->n; i++) {
        epi.goff_b[i] = ((const char *)rest->B[i]->data + rest->B[i]->offset * es) - (const char *)g.B;
        epi.goff_c[i] = ((const char *)rest->C[i]->data + rest->C[i]->offset * es) - (const char *)g.C;
        epi.goff_bias[i] = ((const char *)rest->bias[i]->data + rest->bias[i]->offset * es) - (const char *)epi.bias;
      }
    }
    for (int i = 0; i < nb && i < MM_MAXB; i++) epi.br[i] = rs_[i];
    const bool a_ok = g.acs == 1 || g.ars == 1, b_ok = g.brs == 1 || g.bcs == 1;
    rc = -1;
    if (a_ok && b_ok) {
      if (dt == NXH_BF16) rc = try_tile<gemm_tile::ElBF16, true>(ctx, g, (uint32_t)nbatch, al_a, al_b, &epi);
      else if (dt == NXH_F16) rc = try_tile<gemm_tile::ElF16, true>(ctx, g, (uint32_t)nbatch, al_a, al_b, &epi);
      else rc = try_tile<gemm_tile::ElF32, true>(ctx, g, (uint32_t)nbatch, al_a, al_b, &epi);
    }
    if (rc == -1) return nxh_fail(NXH_FAILURE, op, "operands do not fit the tiled GEMM (K a multiple of 64 bytes-of-k slabs, aligned rows)");
    return rc;
  }
  switch (dt) {
    case NXH_BF16: return run_mfma_dtype<MMbf16>(ctx, g, (uint32_t)nbatch, al_a, al_b);
    case NXH_F16: return run_mfma_dtype<MMf16>(ctx, g, (uint32_t)nbatch, al_a, al_b);
    case NXH_F32: return run_mfma_dtype<MMf32>(ctx, g, (uint32_t)nbatch, al_a, al_b);
#define NXH_CASE(DT)                                         \
  case DT: {                                                 \
    const int rc = nxh_gemm_block(ctx, DT, g, (uint32_t)nbatch); \
    return rc != -1 ? rc : launch_any<DT>(ctx, g, (uint32_t)nbatch); \
  }
    case NXH_F64: return launch_f64(ctx, g, (uint32_t)nbatch);
      NXH_CASE(NXH_F8E4M3)
      NXH_CASE(NXH_F8E5M2)
      NXH_CASE(NXH_I8)
      NXH_CASE(NXH_U8)
      NXH_CASE(NXH_I16)
      NXH_CASE(NXH_U16)
      NXH_CASE(NXH_I32)
      NXH_CASE(NXH_U32)
      NXH_CASE(NXH_I64)
      NXH_CASE(NXH_U64)
      NXH_CASE(NXH_C32)
      NXH_CASE(NXH_C64)
#undef NXH_CASE
    default: return nxh_fail(NXH_FAILURE, op, NXH_ERR_UNSUPPORTED);
  }
}

NXH_EXPORT int nxh_matmul(nxh_context *ctx, const nxh_tensor *C, const nxh_tensor *A, const nxh_tensor *B) {
  NXH_DEFER_RECORD(ctx, NXH_D_MATMUL, 0, C, 2, nullptr, 0, nullptr, A, B);
  if (ctx) {
    const nxh_tensor *touched[] = {C, A, B};
    nxh_cache_touch(ctx, touched, 3, 1);
  }
  return matmul_entry(ctx, "matmul", C, A, B, nullptr, nullptr);
}

NXH_EXPORT int nxh_linear(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x, const nxh_tensor *w,
                          const nxh_tensor *bias, const nxh_tensor *residual) {
  NXH_DEFER_TOUCH(ctx, 1, out, x, w, bias, residual);
  if (!bias && !residual) return matmul_entry(ctx, "matmul", out, x, w, nullptr, nullptr);
  return matmul_entry(ctx, "linear", out, x, w, bias, residual);
}

// linear.ml:50-52 followed by the tanh GELU of fn.ml:31-38 (the first half of gpt2.ml's MLP) in
// the GEMM's epilogue; anything the epilogue cannot take is Failure and runs as two calls.
NXH_EXPORT int nxh_linear_gelu_tanh(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x, const nxh_tensor *w,
                                    const nxh_tensor *bias, const void *constants) {
  NXH_DEFER_TOUCH(ctx, 1, out, x, w, bias);
  if (!constants) return nxh_fail(NXH_INVALID_ARGUMENT, "linear_gelu", "null argument");
  if (!out || (out->dtype != NXH_BF16 && out->dtype != NXH_F16))
    return nxh_fail(NXH_FAILURE, "linear_gelu", "the fused form takes bfloat16 / float16 operands");
  double c[4];
  for (int i = 0; i < 4; i++) {
    const uint16_t h = ((const uint16_t *)constants)[i];
    if (out->dtype == NXH_BF16) {
      c[i] = (double)bf16_to_f32(h);
    } else {  // float16, exact
      const int e = (h >> 10) & 31, m = h & 1023;
      const double v = e == 0 ? std::ldexp((double)m, -24) : (e == 31 ? (m ? std::nan("") : HUGE_VAL) : std::ldexp((double)(m | 1024), e - 25));
      c[i] = (h & 0x8000) ? -v : v;
    }
  }
  return matmul_entry(ctx, "linear_gelu", out, x, w, bias, nullptr, c);
}

// out[i] = matmul x w[i] + bias[i] for two or three (w, bias, out) of one dtype, shape and layout
// as ONE launch (the q / k / v projections of attention.ml:218-265 all read the same x). Failure
// when the members differ in anything but their addresses, or the tiled GEMM does not take them;
// the caller then runs them one by one.
int nxh_linear_group(nxh_context *ctx, int n, const nxh_tensor *const *outs, const nxh_tensor *x,
                     const nxh_tensor *const *ws, const nxh_tensor *const *biases) {
  if (n < 2 || n > 3) return nxh_fail(NXH_FAILURE, "linear", "a group has two or three members");
  nxh_cache_opaque(ctx);  // several outputs and weights, not named one by one to the cache policy
  auto same_layout = [](const nxh_tensor *a, const nxh_tensor *b) {
    if (!a || !b || a->dtype != b->dtype || a->ndim != b->ndim) return false;
    for (int d = 0; d < a->ndim; d++)
      if (a->shape[d] != b->shape[d] || (a->shape[d] > 1 && a->strides[d] != b->strides[d])) return false;
    return true;
  };
  GroupRest rest;
  for (int i = 1; i < n; i++) {
    if (!same_layout(outs[0], outs[i]) || !same_layout(ws[0], ws[i]) || !same_layout(biases[0], biases[i]))
      return nxh_fail(NXH_FAILURE, "linear", "the members of a group differ in shape or layout");
    if (int rc = nxh_check_tensor("linear", outs[i])) return rc;
    if (int rc = nxh_check_tensor("linear", ws[i])) return rc;
    if (int rc = nxh_check_tensor("linear", biases[i])) return rc;
    rest.B[i - 1] = ws[i], rest.bias[i - 1] = biases[i], rest.C[i - 1] = outs[i];
  }
  rest.n = n - 1;
  return matmul_entry(ctx, "linear", outs[0], x, ws[0], biases[0], nullptr, nullptr, &rest);
}
