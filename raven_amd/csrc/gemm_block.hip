// gemm_block: the register-blocked GEMM of the dtypes that have no matrix instruction here — the
// integers, the two float8 formats and the complex pair — in place of one lane per output.
//
// Reference contract: packages/nx/lib/backend_c/nx_c_matmul.c:128-605 (one blocked microkernel
// per dtype family, accumulation in the compute type, one store per output) behind
// nx_c_matmul_run (:874-1108).
//
// A block of 256 lanes owns a (16 T) x (16 T) tile of C; a lane owns T x T of it in registers
// (T = 4: with 8 x 8 a lane reads half the LDS bytes per multiply-add, but a unit then holds one
// or two blocks and nothing covers their waits — measured slower at every size from 1024^3 to
// 4096^3, int8 28.6 against 38.6 Top/s, float8 24.1 against 34.7 at 2048^3).
// K is walked in slabs of 16: global -> registers (the next slab, while this one is multiplied)
// -> two LDS tiles [k][row] widened to the compute type, from which a lane reads its T
// values of A and T of B per k as whole vectors. Every output is therefore still the k-ordered
// sum of its products, exactly the one-lane kernel's arithmetic, at 2 T LDS elements per T^2
// multiply-adds instead of 2 global loads per multiply-add.
//
// Integers up to 32 bits are multiplied and summed modulo 2^32: narrowing to the stored width
// is a ring homomorphism, so the result equals the reference's 64-bit accumulation narrowed
// once (nx_c_matmul.c:197-209) at a quarter of its multiplier work. 64-bit integers wrap modulo
// 2^64 as the reference's do.
//
// Operands are read element by element, lanes along whichever of the two dims is contiguous,
// with bounds checks (an element outside the operand is read from a zero in memory): any
// strides, any edge, no alignment condition.

#include <algorithm>
#include <type_traits>

#include "gemm_args.hpp"

namespace {

template <int DT>
struct Blk {
  using TR = Tr<DT>;
  using S = typename TR::S;
  static constexpr bool narrow_int =
      (TR::cat == CAT_SINT || TR::cat == CAT_UINT) && sizeof(S) <= 4;
  static constexpr bool wide_int = (TR::cat == CAT_SINT || TR::cat == CAT_UINT) && sizeof(S) == 8;
  using CT = std::conditional_t<narrow_int, uint32_t, std::conditional_t<wide_int, uint64_t, typename TR::C>>;
  __device__ __forceinline__ static CT ld(S s) {
    if constexpr (narrow_int) {
      if constexpr (std::is_signed<S>::value) return (uint32_t)(int32_t)s;
      else return (uint32_t)s;
    } else if constexpr (wide_int) {
      return (uint64_t)s;
    } else {
      return TR::ld(s);
    }
  }
  __device__ __forceinline__ static S st(CT c) {
    if constexpr (narrow_int || wide_int) return (S)c;
    else return TR::st(c);
  }
  __device__ __forceinline__ static CT zero() {
    if constexpr (TR::cat == CAT_COMPLEX) return CT{0, 0};
    else return (CT)0;
  }
  __device__ __forceinline__ static void mac(CT &acc, CT x, CT y) { acc = acc + x * y; }
};

__device__ uint64_t gemm_block_zero[2] = {0, 0};  // (not const: a load through it stays a global load)

constexpr int GB_THREADS = 256, GB_BK = 16;

template <int DT, int T>
__global__ __launch_bounds__(GB_THREADS) void gemm_block_kernel(GemmArgs a) {
  using E = Blk<DT>;
  using S = typename E::S;
  using CT = typename E::CT;
  constexpr int BM = 16 * T, BN = 16 * T, BK = GB_BK, THREADS = GB_THREADS;
  constexpr int PAD = sizeof(CT) >= 16 ? 1 : 16 / (int)sizeof(CT);  // the row pitch stays a multiple of 16 bytes
  constexpr int LDA = BM + PAD, LDB = BN + PAD;
  constexpr int NL = BM * BK / THREADS;
  static_assert(NL * THREADS == BM * BK && THREADS % BK == 0 && THREADS % BM == 0, "slab loads");
  struct alignas(16) Vec {
    CT v[T];
  };
  static_assert((T * sizeof(CT)) % 16 == 0 && (LDA * sizeof(CT)) % 16 == 0, "vector reads of the LDS tiles");
  __shared__ __align__(16) CT sA[BK * LDA];
  __shared__ __align__(16) CT sB[BK * LDB];

  int64_t ao, bo, co;
  batch_decode(a.batch, a.batch0 + blockIdx.z, ao, bo, co);
  const S *A = (const S *)a.A + ao;
  const S *B = (const S *)a.B + bo;
  const int64_t m0 = (int64_t)blockIdx.y * BM, n0 = (int64_t)blockIdx.x * BN;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;

  // Element e = thread + THREADS i of an operand's slab: lanes run along k (when k is the
  // contiguous dim) or along the row index; element e + THREADS lies a fixed number of rows or
  // k-values further on, one uniform pointer step.
  struct Lane {
    const S *p;
    int64_t step;
    int row, k, drow, dk;
  };
  auto lane_of = [&](const S *P, bool kc, int64_t rs, int64_t ks) {
    Lane l;
    l.row = kc ? threadIdx.x / BK : threadIdx.x % BM;
    l.k = kc ? threadIdx.x % BK : threadIdx.x / BM;
    l.drow = kc ? THREADS / BK : 0;
    l.dk = kc ? 0 : THREADS / BM;
    l.p = P + l.row * rs + l.k * ks;
    l.step = l.drow * rs + l.dk * ks;
    return l;
  };
  const Lane la = lane_of(A + m0 * a.ars, a.acs == 1 && a.ars != 1, a.ars, a.acs);
  const Lane lb = lane_of(B + n0 * a.bcs, a.brs == 1 && a.bcs != 1, a.bcs, a.brs);  // B by rows = n
  const int64_t a_left = a.M - m0, b_left = a.N - n0;
  // A slab waits in registers as stored values and is widened on its way into LDS, after the
  // multiply-adds of the slab before it: a conversion at the load would make the loads' wait
  // precede those multiply-adds instead of hiding behind them.
  auto load = [&](S(&r)[NL], const Lane &l, int64_t ks, int64_t rows_left, int64_t k0) {
    const S *p = l.p + k0 * ks;
    if (rows_left >= BM && k0 + BK <= a.K) {  // (uniform) a whole slab: nothing to check
#pragma unroll
      for (int i = 0; i < NL; i++) r[i] = p[i * l.step];
      return;
    }
#pragma unroll
    for (int i = 0; i < NL; i++) {
      const bool ok = l.row + i * l.drow < rows_left && k0 + l.k + i * l.dk < a.K;
      r[i] = *(ok ? p : (const S *)gemm_block_zero);
      p += l.step;
    }
  };
  auto store = [&](const S(&r)[NL], const Lane &l, CT *s, int ld) {
#pragma unroll
    for (int i = 0; i < NL; i++) s[(l.k + i * l.dk) * ld + l.row + i * l.drow] = E::ld(r[i]);
  };

  CT acc[T][T];
#pragma unroll
  for (int i = 0; i < T; i++)
#pragma unroll
    for (int j = 0; j < T; j++) acc[i][j] = E::zero();

  const int64_t nk = (a.K + BK - 1) / BK;
  S ra[NL], rb[NL];
  if (nk > 0) {
    load(ra, la, a.acs, a_left, 0);
    load(rb, lb, a.brs, b_left, 0);
  }
  for (int64_t kt = 0; kt < nk; kt++) {
    store(ra, la, sA, LDA);
    store(rb, lb, sB, LDB);
    __syncthreads();
    if (kt + 1 < nk) {
      load(ra, la, a.acs, a_left, (kt + 1) * BK);
      load(rb, lb, a.brs, b_left, (kt + 1) * BK);
    }
#pragma unroll
    for (int kk = 0; kk < BK; kk++) {
      const Vec fa = *reinterpret_cast<const Vec *>(&sA[kk * LDA + ty * T]);
      const Vec fb = *reinterpret_cast<const Vec *>(&sB[kk * LDB + tx * T]);
#pragma unroll
      for (int i = 0; i < T; i++)
#pragma unroll
        for (int j = 0; j < T; j++) E::mac(acc[i][j], fa.v[i], fb.v[j]);
    }
    __syncthreads();
  }

  S *C = (S *)a.C + co;
#pragma unroll
  for (int i = 0; i < T; i++) {
    const int64_t row = m0 + ty * T + i;
    if (row >= a.M) break;
#pragma unroll
    for (int j = 0; j < T; j++) {
      const int64_t col = n0 + tx * T + j;
      if (col < a.N) C[row * a.crs + col * a.ccs] = E::st(acc[i][j]);
    }
  }
}

template <int DT, int T>
static int launch(nxh_context *ctx, GemmArgs &a, uint32_t nbatch) {
  constexpr int B = 16 * T;
  const uint32_t gx = (uint32_t)((a.N + B - 1) / B), gy = (uint32_t)((a.M + B - 1) / B);
  if (gy > 65535) return -1;
  nxh_set_path("gemm_block_64x64");
  for (uint32_t b0 = 0; b0 < nbatch; b0 += 65535) {
    a.batch0 = b0;
    hipLaunchKernelGGL((gemm_block_kernel<DT, T>), dim3(gx, gy, std::min<uint32_t>(65535, nbatch - b0)),
                       dim3(GB_THREADS), 0, ctx->stream, a);
    NXH_HIP("matmul", hipGetLastError());
  }
  return NXH_OK;
}

}  // namespace

int nxh_gemm_block(nxh_context *ctx, int dtype, GemmArgs &a, uint32_t nbatch) {
  // a thin product leaves most of a block's tile empty: one lane per output serves it better
  if (a.M < 16 || a.N < 16 || a.K < 8) return -1;
  switch (dtype) {
#define NXH_CASE(DT) \
  case DT: return launch<DT, 4>(ctx, a, nbatch);
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
    default: return -1;
  }
}
