// rowfuse.hip — three sequences of backend operations that the frontend and
// Kaun issue one primitive at a time, each as ONE kernel that reads its input
// once and writes its result once:
//
//   nxh_softmax_rows     frontend.ml:4242-4252 (max, sub, exp, sum, div over the
//                        last axis), optionally behind the scale and mask of
//                        kaun/lib/attention.ml:67-110 (mul by a scalar, where
//                        against a scalar) and in front of a cast;
//   nxh_layer_norm_rows  kaun/lib/layer_norm.ml:43-68 (mean, centre, biased
//                        variance, divide by sqrt(var + eps); statistics in
//                        float32 for 16-bit inputs; then * gamma + beta);
//   nxh_gelu_tanh        kaun/lib/fn.ml:31-38.
//
// Every elementwise step is the expression of the corresponding primitive
// (map_ops.hpp) and is rounded to the dtype that primitive would have stored,
// so a fused result differs from the op-by-op one only through the order in
// which a row's sum is added up.
//
// Rows live in registers: one wave64 per row up to 2048 elements, one block of
// four waves up to 8192. A longer row (a softmax over 50 257 logits) is walked
// three times by its block — the statistics first, then the results — out of
// the caches the first walk filled (softmax_long_kernel, layer_norm_long_kernel).

#include <cmath>
#include <cstring>
#include <type_traits>
#include <vector>

#include "fold_common.hpp"
#include "softmax_math.hpp"
#include "stream_access.hpp"
#include "map_ops.hpp"

namespace {

constexpr int ROW_MAXD = 8;
constexpr int EPL = 32;  // elements per lane at most (rows held in registers)
constexpr int ROW_REGS = 64 * 4 * EPL;  // the longest row a block holds in registers
constexpr int LONG_THREADS = 1024, LONG_WAVES = LONG_THREADS / 64;  // a block of the long-row kernels
constexpr int64_t ROW_MAX = (int64_t)1 << 24;  // the longest row at all (float32 counts it exactly)

struct RowGeom {
  int64_t rows;
  int n, nouter;
  uint32_t oshape[ROW_MAXD];
};
struct RowOperand {
  const char *base;
  int64_t stride[ROW_MAXD];  // per outer dim, elements
};

template <int DT>
__device__ __forceinline__ typename Tr<DT>::C rnd(typename Tr<DT>::C v) {
  return Tr<DT>::ld(Tr<DT>::st(v));
}

template <class S, int V>
struct alignas(sizeof(S) * V) Pk {
  S v[V];
};

// Sum / max of one value per lane over the row's lanes; every lane gets the
// result (the butterfly adds the same two operands on both sides of a pair).
template <int OP, class C, int RW>
__device__ __forceinline__ C row_combine(C v, C *lds) {
  using CB = Combine<OP, C, CAT_FLOAT>;
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) {
    C o;
    if constexpr (sizeof(C) == 8) {
      const uint64_t u = __builtin_bit_cast(uint64_t, v);
      const uint32_t lo = __shfl_xor((uint32_t)u, d, 64), hi = __shfl_xor((uint32_t)(u >> 32), d, 64);
      o = __builtin_bit_cast(C, ((uint64_t)hi << 32) | lo);
    } else {
      o = __builtin_bit_cast(C, __shfl_xor(__builtin_bit_cast(uint32_t, v), d, 64));
    }
    // operands in lane order on both sides, so a pair computes identical bits
    const bool low = (threadIdx.x & d) == 0;
    v = low ? CB::apply(v, o) : CB::apply(o, v);
  }
  if constexpr (RW > 1) {
    const int w = threadIdx.x >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) lds[w] = v;
    __syncthreads();
    v = lds[0];
#pragma unroll
    for (int i = 1; i < RW; i++) v = CB::apply(v, lds[i]);
  }
  return v;
}

__device__ __forceinline__ int64_t row_offsets(const RowGeom &g, int64_t row, const RowOperand &a,
                                               const RowOperand &b, const RowOperand &c, int64_t &ob,
                                               int64_t &oc) {
  int64_t oa = 0;
  ob = 0;
  oc = 0;
  // rows fit 32 bits (checked on the host) and the host has merged the outer dims that compose, so
  // the usual case is one dim and no division; the rest are 32-bit divisions, not 64-bit ones
  uint32_t r = (uint32_t)row;
  for (int d = g.nouter - 1; d >= 0; d--) {
    uint32_t i = r;
    if (d > 0) {
      const uint32_t q = r / g.oshape[d];
      i = r - q * g.oshape[d];
      r = q;
    }
    oa += (int64_t)i * a.stride[d];
    ob += (int64_t)i * b.stride[d];
    oc += (int64_t)i * c.stride[d];
  }
  return oa;
}

// ── softmax ─────────────────────────────────────────────────────────────────
struct SoftmaxArgs {
  RowGeom g;
  RowOperand x, out, mask;
  int has_scale, has_mask;
  int64_t mask_last;  // 0 or 1
  double scale, masked;  // exact images of the encoded scalars
  // NXH_STREAM_IN / _OUT: the scores are read, the probabilities written past the memory-side
  // cache (decided per call on the host, runtime.hip nxh_cache_hints)
  uint32_t stream;
};
// EP: elements a lane holds at most (a row of up to 64 * RW * EP elements). The short forms
// exist for their register count: 87 registers for EP = 32 leave five waves per SIMD, and
// a launch of 2048 blocks then runs as two rounds of blocks instead of one.
template <int DTX, int DTO, int V, int RW, int EP = EPL>
__global__ __launch_bounds__(256) void softmax_rows_kernel(SoftmaxArgs a) {
  using TX = Tr<DTX>;
  using TO = Tr<DTO>;
  using C = typename TX::C;
  using SX = typename TX::S;
  using SO = typename TO::S;
  constexpr int NV = EP / V, T = 64 * RW;
  __shared__ C lds[4];
  const int tid = RW == 1 ? (threadIdx.x & 63) : threadIdx.x;
  const int64_t row = RW == 1 ? (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6) : (int64_t)blockIdx.x;
  if (row >= a.g.rows) return;  // whole waves (RW == 1) or whole blocks leave together
  int64_t oo, mo;
  const int64_t xo = row_offsets(a.g, row, a.x, a.out, a.mask, oo, mo);
  const SX *x = reinterpret_cast<const SX *>(a.x.base) + xo;
  SO *out = reinterpret_cast<SO *>(const_cast<char *>(a.out.base)) + oo;
  const uint8_t *mask = reinterpret_cast<const uint8_t *>(a.mask.base) + mo;
  const int nvec = a.g.n / V;
  C t[NV][V];
  Pk<SX, V> raw[NV];
  Pk<uint8_t, V> mk[NV];
#pragma unroll
  for (int v = 0; v < NV; v++) {
    const int c = v * T + tid;
    if (c < nvec) {
      const Pk<SX, V> *src = reinterpret_cast<const Pk<SX, V> *>(x + (int64_t)c * V);
      raw[v] = (a.stream & NXH_STREAM_IN) ? load_stream(src) : *src;
      if (a.has_mask) {
        if (a.mask_last) mk[v] = *reinterpret_cast<const Pk<uint8_t, V> *>(mask + (int64_t)c * V);
        else
#pragma unroll
          for (int j = 0; j < V; j++) mk[v].v[j] = mask[0];
      }
    }
  }
  const C scale = (C)a.scale, masked = (C)a.masked;
  // float32 scores narrowed to 16 bits on the way out (the probabilities of an
  // attention): the exponential, the quotient and the maximum take the short forms
  // of softmax_math.hpp, whose differences from the primitives' disappear under
  // the narrowing in all but rare elements. The hardware maximum skips NaNs; a
  // NaN element still turns the whole row into NaNs through the sum.
  constexpr bool SHORT = DTX == NXH_F32 && (DTO == NXH_BF16 || DTO == NXH_F16);
  C m = Combine<NXH_RMAX, C, CAT_FLOAT>::init();
#pragma unroll
  for (int v = 0; v < NV; v++) {
    if (v * T + tid < nvec) {
#pragma unroll
      for (int j = 0; j < V; j++) {
        C e = TX::ld(raw[v].v[j]);
        if (a.has_scale) e = rnd<DTX>(OpMul::eval<CAT_FLOAT, C>(e, scale));
        if (a.has_mask) e = mk[v].v[j] != 0 ? e : masked;
        t[v][j] = e;
        if constexpr (SHORT) m = __builtin_fmaxf(m, e);
        else m = Combine<NXH_RMAX, C, CAT_FLOAT>::apply(m, e);
      }
    }
  }
  m = row_combine<NXH_RMAX, C, RW>(m, lds);
  C s = 0;
#pragma unroll
  for (int v = 0; v < NV; v++) {
    if (v * T + tid < nvec) {
#pragma unroll
      for (int j = 0; j < V; j++) {
        const C d = rnd<DTX>(OpSub::eval<CAT_FLOAT, C>(t[v][j], m));
        C e;
        if constexpr (SHORT) e = exp_nonpositive(d);
        else e = rnd<DTX>(OpExp::eval<CAT_FLOAT, C>(d));
        t[v][j] = e;
        s = s + e;
      }
    }
  }
  s = rnd<DTX>(row_combine<NXH_SUM, C, RW>(s, lds));
  C s_recip = 0;
  if constexpr (SHORT) s_recip = 1.0f / s;
#pragma unroll
  for (int v = 0; v < NV; v++) {
    const int c = v * T + tid;
    if (c < nvec) {
      Pk<SO, V> o;
#pragma unroll
      for (int j = 0; j < V; j++) {
        C y;
        if constexpr (SHORT) y = div_by_reciprocal(t[v][j], s, s_recip);
        else y = rnd<DTX>(OpFdiv::eval<CAT_FLOAT, C>(t[v][j], s));
        o.v[j] = TO::st((typename TO::C)y);
      }
      Pk<SO, V> *dst = reinterpret_cast<Pk<SO, V> *>(out + (int64_t)c * V);
      if (a.stream & NXH_STREAM_OUT) store_stream(dst, o);
      else *dst = o;
    }
  }
}

// ── layer norm ──────────────────────────────────────────────────────────────
struct LayerNormArgs {
  RowGeom g;
  RowOperand x, out, unused;
  const char *gamma, *beta;  // null: that step is left out
  double eps, count;         // exact images of the float scalars the chain would have filled
};
template <int DT, int V, int RW, int EP = EPL>
__global__ __launch_bounds__(256) void layer_norm_rows_kernel(LayerNormArgs a) {
  using TX = Tr<DT>;
  using C = typename TX::C;  // float for the 16-bit dtypes: their float32 island
  using S = typename TX::S;
  constexpr int NV = EP / V, T = 64 * RW;
  __shared__ C lds[4];
  const int tid = RW == 1 ? (threadIdx.x & 63) : threadIdx.x;
  const int64_t row = RW == 1 ? (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6) : (int64_t)blockIdx.x;
  if (row >= a.g.rows) return;
  int64_t oo, uo;
  const int64_t xo = row_offsets(a.g, row, a.x, a.out, a.unused, oo, uo);
  const S *x = reinterpret_cast<const S *>(a.x.base) + xo;
  S *out = reinterpret_cast<S *>(const_cast<char *>(a.out.base)) + oo;
  const S *gamma = reinterpret_cast<const S *>(a.gamma), *beta = reinterpret_cast<const S *>(a.beta);
  const int nvec = a.g.n / V;
  C t[NV][V];
  Pk<S, V> raw[NV];
#pragma unroll
  for (int v = 0; v < NV; v++) {
    const int c = v * T + tid;
    if (c < nvec) raw[v] = *reinterpret_cast<const Pk<S, V> *>(x + (int64_t)c * V);
  }
  // gamma and beta do not depend on the row: their loads go out with the row's, ahead of the
  // two reductions, instead of starting a second trip to memory after them
  Pk<S, V> gv[NV], bv[NV];
#pragma unroll
  for (int v = 0; v < NV; v++) {
    const int c = v * T + tid;
    if (c < nvec) {
      if (gamma) gv[v] = *reinterpret_cast<const Pk<S, V> *>(gamma + (int64_t)c * V);
      if (beta) bv[v] = *reinterpret_cast<const Pk<S, V> *>(beta + (int64_t)c * V);
    }
  }
  const C count = (C)a.count, eps = (C)a.eps;
  C s = 0;
#pragma unroll
  for (int v = 0; v < NV; v++)
    if (v * T + tid < nvec)
#pragma unroll
      for (int j = 0; j < V; j++) {
        t[v][j] = TX::ld(raw[v].v[j]);
        s = s + t[v][j];
      }
  const C mu = row_combine<NXH_SUM, C, RW>(s, lds) / count;
  s = 0;
#pragma unroll
  for (int v = 0; v < NV; v++)
    if (v * T + tid < nvec)
#pragma unroll
      for (int j = 0; j < V; j++) {
        t[v][j] = t[v][j] - mu;
        s = s + t[v][j] * t[v][j];
      }
  const C var = row_combine<NXH_SUM, C, RW>(s, lds) / count;
  const C r = m_sqrt(var + eps);
#pragma unroll
  for (int v = 0; v < NV; v++) {
    const int c = v * T + tid;
    if (c < nvec) {
      Pk<S, V> o;
#pragma unroll
      for (int j = 0; j < V; j++) {
        C y = rnd<DT>(t[v][j] / r);  // leaves the float32 island here
        if (gamma) y = rnd<DT>(y * TX::ld(gv[v].v[j]));
        if (beta) y = rnd<DT>(y + TX::ld(bv[v].v[j]));
        o.v[j] = TX::st(y);
      }
      *reinterpret_cast<Pk<S, V> *>(out + (int64_t)c * V) = o;
    }
  }
}

// ── rows longer than a block holds in registers ─────────────────────────────
// A block of sixteen waves per row, as many blocks as the chip has units (each takes every
// gridDim.x-th row): the rows in flight then fit the caches, and the second and third walk do not
// go back to memory (one block of four waves per row, all rows at once: 380 us for [2048, 50257]
// float32, the working set of 2048 rows being larger than the memory-side cache). Three walks: the maximum, the sum of the exponentials, the
// quotients (softmax); the sum, the sum of squared differences, the results (layer norm). Every
// elementwise step is the expression of the short kernels, so a result differs from theirs (and
// from the primitives') only through the order of a row's sum; the second and third walk find
// the row in the caches.
template <int DTX, int DTO, int V>
__global__ __launch_bounds__(LONG_THREADS) void softmax_long_kernel(SoftmaxArgs a) {
  using TX = Tr<DTX>;
  using TO = Tr<DTO>;
  using C = typename TX::C;
  using SX = typename TX::S;
  using SO = typename TO::S;
  __shared__ C lds[LONG_WAVES];
  for (int64_t row = blockIdx.x; row < a.g.rows; row += gridDim.x) {
    int64_t oo, mo;
    const int64_t xo = row_offsets(a.g, row, a.x, a.out, a.mask, oo, mo);
    const SX *x = reinterpret_cast<const SX *>(a.x.base) + xo;
    SO *out = reinterpret_cast<SO *>(const_cast<char *>(a.out.base)) + oo;
    const uint8_t *mask = reinterpret_cast<const uint8_t *>(a.mask.base) + mo;
    // A row that starts off a vector boundary, or ends off one: `head` single elements, whole
    // vectors, then the rest as single elements (the host has checked that out and mask are
    // off their boundaries by as much as x). The single elements go one to a lane.
    const int off = V > 1 ? (V - (int)(((uintptr_t)x / sizeof(SX)) % V)) % V : 0;
    const int head = off < a.g.n ? off : a.g.n;
    const int nvec = (a.g.n - head) / V;
    const int nedge = a.g.n - nvec * V;
    const C scale = (C)a.scale, masked = (C)a.masked;
    constexpr bool SHORT = DTX == NXH_F32 && (DTO == NXH_BF16 || DTO == NXH_F16);
    // the scaled, masked scores of the W elements from i on
    auto scores = [&](int64_t i, auto w, C *e) {
      constexpr int W = decltype(w)::value;
      const Pk<SX, W> raw = *reinterpret_cast<const Pk<SX, W> *>(x + i);
      Pk<uint8_t, W> mk;
      if (a.has_mask) {
        if (a.mask_last) mk = *reinterpret_cast<const Pk<uint8_t, W> *>(mask + i);
        else
#pragma unroll
          for (int j = 0; j < W; j++) mk.v[j] = mask[0];
      }
#pragma unroll
      for (int j = 0; j < W; j++) {
        C v = TX::ld(raw.v[j]);
        if (a.has_scale) v = rnd<DTX>(OpMul::eval<CAT_FLOAT, C>(v, scale));
        if (a.has_mask) v = mk.v[j] != 0 ? v : masked;
        e[j] = v;
      }
    };
    // body(i, W): once for every vector of the row and once for every single element
    auto walk = [&](auto &&body) {
#pragma unroll 8
      for (int c = threadIdx.x; c < nvec; c += LONG_THREADS) body(head + (int64_t)c * V, std::integral_constant<int, V>{});
      if (V > 1 && (int)threadIdx.x < nedge)
        body((int)threadIdx.x < head ? (int64_t)threadIdx.x : (int64_t)nvec * V + threadIdx.x, std::integral_constant<int, 1>{});
    };
    C m = Combine<NXH_RMAX, C, CAT_FLOAT>::init();
    walk([&](int64_t i, auto w) {
      constexpr int W = decltype(w)::value;
      C e[W];
      scores(i, w, e);
#pragma unroll
      for (int j = 0; j < W; j++) {
        if constexpr (SHORT) m = __builtin_fmaxf(m, e[j]);
        else m = Combine<NXH_RMAX, C, CAT_FLOAT>::apply(m, e[j]);
      }
    });
    m = row_combine<NXH_RMAX, C, LONG_WAVES>(m, lds);
    auto exponential = [&](C v) -> C {
      const C d = rnd<DTX>(OpSub::eval<CAT_FLOAT, C>(v, m));
      if constexpr (SHORT) return exp_nonpositive(d);
      else return rnd<DTX>(OpExp::eval<CAT_FLOAT, C>(d));
    };
    C s = 0;
    walk([&](int64_t i, auto w) {
      constexpr int W = decltype(w)::value;
      C e[W];
      scores(i, w, e);
#pragma unroll
      for (int j = 0; j < W; j++) s = s + exponential(e[j]);
    });
    s = rnd<DTX>(row_combine<NXH_SUM, C, LONG_WAVES>(s, lds));
    C s_recip = 0;
    if constexpr (SHORT) s_recip = 1.0f / s;
    walk([&](int64_t i, auto w) {
      constexpr int W = decltype(w)::value;
      C e[W];
      scores(i, w, e);
      Pk<SO, W> o;
#pragma unroll
      for (int j = 0; j < W; j++) {
        const C t = exponential(e[j]);
        C y;
        if constexpr (SHORT) y = div_by_reciprocal(t, s, s_recip);
        else y = rnd<DTX>(OpFdiv::eval<CAT_FLOAT, C>(t, s));
        o.v[j] = TO::st((typename TO::C)y);
      }
      *reinterpret_cast<Pk<SO, W> *>(out + i) = o;
    });
  }
}

template <int DT, int V>
__global__ __launch_bounds__(LONG_THREADS) void layer_norm_long_kernel(LayerNormArgs a) {
  using TX = Tr<DT>;
  using C = typename TX::C;
  using S = typename TX::S;
  __shared__ C lds[LONG_WAVES];
  for (int64_t row = blockIdx.x; row < a.g.rows; row += gridDim.x) {
    int64_t oo, uo;
    const int64_t xo = row_offsets(a.g, row, a.x, a.out, a.unused, oo, uo);
    const S *x = reinterpret_cast<const S *>(a.x.base) + xo;
    S *out = reinterpret_cast<S *>(const_cast<char *>(a.out.base)) + oo;
    const S *gamma = reinterpret_cast<const S *>(a.gamma), *beta = reinterpret_cast<const S *>(a.beta);
    // head, vectors, rest: as in softmax_long_kernel; gamma and beta, which every row shares, are
    // read by vectors only from a row that is off its boundary by as much as they are
    const int off = V > 1 ? (V - (int)(((uintptr_t)x / sizeof(S)) % V)) % V : 0;
    const int head = off < a.g.n ? off : a.g.n;
    const int nvec = (a.g.n - head) / V;
    const int nedge = a.g.n - nvec * V;
    const bool gvec = !gamma || ((uintptr_t)(gamma + head) / sizeof(S)) % V == 0;
    const bool bvec = !beta || ((uintptr_t)(beta + head) / sizeof(S)) % V == 0;
    const C count = (C)a.count, eps = (C)a.eps;
    auto walk = [&](auto &&body) {
#pragma unroll 8
      for (int c = threadIdx.x; c < nvec; c += LONG_THREADS) body(head + (int64_t)c * V, std::integral_constant<int, V>{});
      if (V > 1 && (int)threadIdx.x < nedge)
        body((int)threadIdx.x < head ? (int64_t)threadIdx.x : (int64_t)nvec * V + threadIdx.x, std::integral_constant<int, 1>{});
    };
    C s = 0;
    walk([&](int64_t i, auto w) {
      constexpr int W = decltype(w)::value;
      const Pk<S, W> raw = *reinterpret_cast<const Pk<S, W> *>(x + i);
#pragma unroll
      for (int j = 0; j < W; j++) s = s + TX::ld(raw.v[j]);
    });
    const C mu = row_combine<NXH_SUM, C, LONG_WAVES>(s, lds) / count;
    s = 0;
    walk([&](int64_t i, auto w) {
      constexpr int W = decltype(w)::value;
      const Pk<S, W> raw = *reinterpret_cast<const Pk<S, W> *>(x + i);
#pragma unroll
      for (int j = 0; j < W; j++) {
        const C t = TX::ld(raw.v[j]) - mu;
        s = s + t * t;
      }
    });
    const C var = row_combine<NXH_SUM, C, LONG_WAVES>(s, lds) / count;
    const C r = m_sqrt(var + eps);
    walk([&](int64_t i, auto w) {
      constexpr int W = decltype(w)::value;
      const Pk<S, W> raw = *reinterpret_cast<const Pk<S, W> *>(x + i);
      Pk<S, W> gv, bv, o;
      if (gamma) {
        if (W == 1 || gvec) gv = *reinterpret_cast<const Pk<S, W> *>(gamma + i);
        else
#pragma unroll
          for (int j = 0; j < W; j++) gv.v[j] = gamma[i + j];
      }
      if (beta) {
        if (W == 1 || bvec) bv = *reinterpret_cast<const Pk<S, W> *>(beta + i);
        else
#pragma unroll
          for (int j = 0; j < W; j++) bv.v[j] = beta[i + j];
      }
#pragma unroll
      for (int j = 0; j < W; j++) {
        C y = rnd<DT>((TX::ld(raw.v[j]) - mu) / r);  // leaves the float32 island here
        if (gamma) y = rnd<DT>(y * TX::ld(gv.v[j]));
        if (beta) y = rnd<DT>(y + TX::ld(bv.v[j]));
        o.v[j] = TX::st(y);
      }
      *reinterpret_cast<Pk<S, W> *>(out + i) = o;
    });
  }
}

// ── gelu (tanh form) ────────────────────────────────────────────────────────
struct GeluArgs {
  const char *x;
  char *out;
  int64_t n;
  double c[4];
};
// One element through the nine primitives of the sequence, each result rounded to the dtype.
template <int DT>
__device__ __forceinline__ typename Tr<DT>::S gelu_one(typename Tr<DT>::S in, typename Tr<DT>::C c0, typename Tr<DT>::C c1,
                                                       typename Tr<DT>::C c2, typename Tr<DT>::C c3) {
  using TX = Tr<DT>;
  using C = typename TX::C;
  const C v = TX::ld(in);
  const C x2 = rnd<DT>(v * v);
  const C x3 = rnd<DT>(v * x2);
  const C p = rnd<DT>(x3 * c0);
  const C q = rnd<DT>(v + p);
  const C inner = rnd<DT>(q * c1);
  C th;
  if constexpr (DT == NXH_BF16 || DT == NXH_F16) th = rnd<DT>(tanh_for_16bit(inner));  // as the tanh primitive of these dtypes
  else th = rnd<DT>(m_tanh(inner));
  const C u = rnd<DT>(th + c2);
  const C w = rnd<DT>(v * u);
  return TX::st(w * c3);
}
template <int DT, int V>
__global__ __launch_bounds__(256) void gelu_tanh_kernel(GeluArgs a) {
  using TX = Tr<DT>;
  using C = typename TX::C;
  using S = typename TX::S;
  const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * V;
  if (i >= a.n) return;
  const S *x = reinterpret_cast<const S *>(a.x);
  S *out = reinterpret_cast<S *>(a.out);
  Pk<S, V> in, o;
  if (V > 1 && i + V <= a.n) in = *reinterpret_cast<const Pk<S, V> *>(x + i);
  else
#pragma unroll
    for (int j = 0; j < V; j++) in.v[j] = i + j < a.n ? x[i + j] : S{};
  const C c0 = (C)a.c[0], c1 = (C)a.c[1], c2 = (C)a.c[2], c3 = (C)a.c[3];
#pragma unroll
  for (int j = 0; j < V; j++) o.v[j] = gelu_one<DT>(in.v[j], c0, c1, c2, c3);
  if (V > 1 && i + V <= a.n) *reinterpret_cast<Pk<S, V> *>(out + i) = o;
  else
#pragma unroll
    for (int j = 0; j < V; j++)
      if (i + j < a.n) out[i + j] = o.v[j];
}

// The same function by table. A 16-bit dtype has 65 536 inputs: their results, computed once by
// gelu_one (so every entry holds the bits the arithmetic gives), are 128 KiB, which a block of
// sixteen waves keeps in LDS; an element then costs one LDS read instead of some forty vector
// instructions, and a large tensor goes through at the rate of memory ([8192,3072] bf16, 100 MB
// of traffic: 32.2 us of arithmetic, 17.3 us by table). One block per compute unit walks its
// share of the tensor, two 16-byte vectors per lane and turn, the next turn's requested before
// this turn's are looked up.
template <int DT>
__global__ __launch_bounds__(256) void gelu_table_kernel(uint16_t *table, GeluArgs a) {
  using C = typename Tr<DT>::C;
  const uint32_t i = blockIdx.x * 256 + threadIdx.x;
  table[i] = gelu_one<DT>((uint16_t)i, (C)a.c[0], (C)a.c[1], (C)a.c[2], (C)a.c[3]);
}
constexpr int LUT_THREADS = 1024, LUT_BYTES = 65536 * 2;
__global__ __launch_bounds__(LUT_THREADS) void gelu_lut_kernel(const uint16_t *table, const uint4 *x, uint4 *out, int64_t nvec,
                                                               int64_t per_block) {
  extern __shared__ uint16_t lut[];
  for (int i = threadIdx.x; i < LUT_BYTES / 16; i += LUT_THREADS) reinterpret_cast<uint4 *>(lut)[i] = reinterpret_cast<const uint4 *>(table)[i];
  __syncthreads();
  const int64_t v0 = (int64_t)blockIdx.x * per_block, v1 = v0 + per_block < nvec ? v0 + per_block : nvec;
  auto through = [&](uint32_t w) -> uint32_t { return (uint32_t)lut[w & 0xffffu] | ((uint32_t)lut[w >> 16] << 16); };
  // the vectors of the next turn are requested before this turn's are looked up
  constexpr int U = 2;
  uint4 cur[U], nxt[U];
  int64_t v = v0 + threadIdx.x;
#pragma unroll
  for (int u = 0; u < U; u++)
    if (v + u * LUT_THREADS < v1) cur[u] = x[v + u * LUT_THREADS];
  for (; v < v1; v += U * LUT_THREADS) {
    const int64_t vn = v + U * LUT_THREADS;
#pragma unroll
    for (int u = 0; u < U; u++)
      if (vn + u * LUT_THREADS < v1) nxt[u] = x[vn + u * LUT_THREADS];
#pragma unroll
    for (int u = 0; u < U; u++)
      if (v + u * LUT_THREADS < v1) {
        const uint4 p = cur[u];
        out[v + u * LUT_THREADS] = uint4{through(p.x), through(p.y), through(p.z), through(p.w)};
      }
#pragma unroll
    for (int u = 0; u < U; u++) cur[u] = nxt[u];
  }
}

// ── host side ───────────────────────────────────────────────────────────────
bool float_dtype_ok(int dt) { return dt == NXH_F32 || dt == NXH_F64 || dt == NXH_BF16 || dt == NXH_F16; }

double decode_scalar(int dt, const void *p) {
  switch (dt) {
    case NXH_F32: return (double)*(const float *)p;
    case NXH_F64: return *(const double *)p;
    case NXH_BF16: return (double)bf16_to_f32(*(const uint16_t *)p);
    default: {  // NXH_F16, exact by construction
      const uint16_t h = *(const uint16_t *)p;
      const int e = (h >> 10) & 31, m = h & 1023;
      double v = e == 0 ? std::ldexp((double)m, -24)
                        : (e == 31 ? (m ? std::nan("") : HUGE_VAL) : std::ldexp((double)(m | 1024), e - 25));
      return (h & 0x8000) ? -v : v;
    }
  }
}

// Fills the row geometry from `x` (rows = product of the outer extents).
int row_geometry(const char *op, const nxh_tensor *x, RowGeom &g) {
  if (x->ndim < 1) return nxh_fail(NXH_INVALID_ARGUMENT, op, "input must not be a scalar");
  if (x->ndim - 1 > ROW_MAXD) return nxh_fail(NXH_FAILURE, op, "more than 8 outer dimensions");
  if (x->shape[x->ndim - 1] > ROW_MAX) return nxh_fail(NXH_FAILURE, op, "rows longer than 2^24 elements");
  g.n = (int)x->shape[x->ndim - 1];
  g.nouter = x->ndim - 1;
  g.rows = 1;
  for (int d = 0; d < g.nouter; d++) {
    if (x->shape[d] > 0xffffffffLL) return nxh_fail(NXH_FAILURE, op, "extent exceeds 32 bits");
    g.oshape[d] = (uint32_t)x->shape[d];
    g.rows *= x->shape[d];
  }
  return NXH_OK;
}
void row_operand(const nxh_tensor *t, RowOperand &o) {
  o.base = t ? (const char *)t->data + t->offset * (int64_t)nxh_elem_size(t->dtype) : nullptr;
  for (int d = 0; d < ROW_MAXD; d++) o.stride[d] = (t && d < t->ndim - 1) ? t->strides[d] : 0;
}
// Outer dims that compose on every operand (stride[d - 1] == stride[d] * extent[d], a broadcast
// with both strides 0 included) become one: contiguous rows end up with a single outer dim.
void merge_outer_dims(RowGeom &g, std::initializer_list<RowOperand *> ops) {
  int n = g.nouter;
  for (int d = n - 1; d > 0; d--) {
    bool composes = true;
    for (RowOperand *o : ops) composes = composes && o->stride[d - 1] == o->stride[d] * (int64_t)g.oshape[d];
    if (!composes || (uint64_t)g.oshape[d - 1] * g.oshape[d] > 0xffffffffULL) continue;
    g.oshape[d - 1] *= g.oshape[d];
    for (RowOperand *o : ops) o->stride[d - 1] = o->stride[d];
    for (int e = d; e + 1 < n; e++) {
      g.oshape[e] = g.oshape[e + 1];
      for (RowOperand *o : ops) o->stride[e] = o->stride[e + 1];
    }
    n--;
  }
  g.nouter = n;
}
// A row operand can be moved V elements at a time when its rows are contiguous
// and every row starts on a V-element boundary.
bool rows_vector_ok(const nxh_tensor *t, int v) {
  const int es = (int)nxh_elem_size(t->dtype);
  if ((((uintptr_t)t->data + t->offset * es) % (uintptr_t)(es * v)) != 0) return false;
  for (int d = 0; d < t->ndim - 1; d++)
    if (t->shape[d] > 1 && t->strides[d] % v != 0) return false;
  return true;
}
// Rows of a and b are off their V-element boundaries by the same amount, row by row: the
// long-row kernels then peel the same head and tail from both.
bool rows_congruent(const nxh_tensor *a, const nxh_tensor *b, int v) {
  const uintptr_t ea = (uintptr_t)a->data / nxh_elem_size(a->dtype) + (uintptr_t)a->offset;
  const uintptr_t eb = (uintptr_t)b->data / nxh_elem_size(b->dtype) + (uintptr_t)b->offset;
  if ((uintptr_t)a->data % nxh_elem_size(a->dtype) || (uintptr_t)b->data % nxh_elem_size(b->dtype)) return false;
  if (ea % v != eb % v) return false;
  for (int d = 0; d < a->ndim - 1; d++)
    if (a->shape[d] > 1 && ((a->strides[d] - b->strides[d]) % v) != 0) return false;
  return true;
}
int same_shape(const char *op, const nxh_tensor *a, const nxh_tensor *b) {
  if (a->ndim != b->ndim) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
  for (int d = 0; d < a->ndim; d++)
    if (a->shape[d] != b->shape[d]) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
  return NXH_OK;
}
int out_rows_ok(const char *op, const nxh_tensor *out) {
  for (int d = 0; d < out->ndim; d++)
    if (out->shape[d] > 1 && out->strides[d] == 0) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_OUT_ALIASED);
  return NXH_OK;
}

// Elements per lane of the vector forms: the smallest of 8 / 16 / 32 that holds the row.
inline int lane_share(int n, bool wave) {
  const int need = (n + (wave ? 64 : 256) - 1) / (wave ? 64 : 256);
  return need <= 8 ? 8 : need <= 16 ? 16 : 32;
}
template <int DTX, int DTO>
void softmax_launch(nxh_context *ctx, const SoftmaxArgs &a, bool vec) {
  if (a.g.n > ROW_REGS) {
    const dim3 grid((unsigned)std::min<int64_t>(a.g.rows, ctx->compute_units > 0 ? ctx->compute_units : 256));
    if (vec) hipLaunchKernelGGL((softmax_long_kernel<DTX, DTO, 4>), grid, dim3(LONG_THREADS), 0, ctx->stream, a);
    else hipLaunchKernelGGL((softmax_long_kernel<DTX, DTO, 1>), grid, dim3(LONG_THREADS), 0, ctx->stream, a);
    return;
  }
  const bool wave = a.g.n <= 64 * EPL;
  const dim3 grid((unsigned)(wave ? (a.g.rows + 3) / 4 : a.g.rows));
  const int ep = lane_share(a.g.n, wave);
  if (wave && vec) {
    if (ep == 8) hipLaunchKernelGGL((softmax_rows_kernel<DTX, DTO, 4, 1, 8>), grid, dim3(256), 0, ctx->stream, a);
    else if (ep == 16) hipLaunchKernelGGL((softmax_rows_kernel<DTX, DTO, 4, 1, 16>), grid, dim3(256), 0, ctx->stream, a);
    else hipLaunchKernelGGL((softmax_rows_kernel<DTX, DTO, 4, 1>), grid, dim3(256), 0, ctx->stream, a);
  } else if (wave) hipLaunchKernelGGL((softmax_rows_kernel<DTX, DTO, 1, 1>), grid, dim3(256), 0, ctx->stream, a);
  else if (vec) {
    if (ep == 16) hipLaunchKernelGGL((softmax_rows_kernel<DTX, DTO, 4, 4, 16>), grid, dim3(256), 0, ctx->stream, a);
    else hipLaunchKernelGGL((softmax_rows_kernel<DTX, DTO, 4, 4>), grid, dim3(256), 0, ctx->stream, a);
  } else hipLaunchKernelGGL((softmax_rows_kernel<DTX, DTO, 1, 4>), grid, dim3(256), 0, ctx->stream, a);
}
template <int DT>
void layer_norm_launch(nxh_context *ctx, const LayerNormArgs &a, bool vec) {
  if (a.g.n > ROW_REGS) {
    const dim3 grid((unsigned)std::min<int64_t>(a.g.rows, ctx->compute_units > 0 ? ctx->compute_units : 256));
    if (vec) hipLaunchKernelGGL((layer_norm_long_kernel<DT, 4>), grid, dim3(LONG_THREADS), 0, ctx->stream, a);
    else hipLaunchKernelGGL((layer_norm_long_kernel<DT, 1>), grid, dim3(LONG_THREADS), 0, ctx->stream, a);
    return;
  }
  const bool wave = a.g.n <= 64 * EPL;
  const dim3 grid((unsigned)(wave ? (a.g.rows + 3) / 4 : a.g.rows));
  const int ep = lane_share(a.g.n, wave);
  if (wave && vec) {
    if (ep == 8) hipLaunchKernelGGL((layer_norm_rows_kernel<DT, 4, 1, 8>), grid, dim3(256), 0, ctx->stream, a);
    else if (ep == 16) hipLaunchKernelGGL((layer_norm_rows_kernel<DT, 4, 1, 16>), grid, dim3(256), 0, ctx->stream, a);
    else hipLaunchKernelGGL((layer_norm_rows_kernel<DT, 4, 1>), grid, dim3(256), 0, ctx->stream, a);
  } else if (wave) hipLaunchKernelGGL((layer_norm_rows_kernel<DT, 1, 1>), grid, dim3(256), 0, ctx->stream, a);
  else if (vec) {
    if (ep == 16) hipLaunchKernelGGL((layer_norm_rows_kernel<DT, 4, 4, 16>), grid, dim3(256), 0, ctx->stream, a);
    else hipLaunchKernelGGL((layer_norm_rows_kernel<DT, 4, 4>), grid, dim3(256), 0, ctx->stream, a);
  } else hipLaunchKernelGGL((layer_norm_rows_kernel<DT, 1, 4>), grid, dim3(256), 0, ctx->stream, a);
}
template <int DT>
void gelu_launch(nxh_context *ctx, const GeluArgs &a, bool vec) {
  constexpr int V = 16 / (int)sizeof(typename Tr<DT>::S);
  if (vec) hipLaunchKernelGGL((gelu_tanh_kernel<DT, V>), dim3((unsigned)(((a.n + V - 1) / V + 255) / 256)), dim3(256), 0, ctx->stream, a);
  else hipLaunchKernelGGL((gelu_tanh_kernel<DT, 1>), dim3((unsigned)((a.n + 255) / 256)), dim3(256), 0, ctx->stream, a);
}

}  // namespace

NXH_EXPORT int nxh_softmax_rows(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x, const void *scale,
                                const nxh_tensor *mask, const void *masked_value) {
  NXH_DEFER_SETTLE(ctx, 1, out, x, mask);  // (the cache policy is asked below, once the call is known to launch)
  const char *op = "softmax_rows";
  if (!ctx || !out || !x || (mask && !masked_value)) return nxh_fail(NXH_INVALID_ARGUMENT, op, "null argument");
  int rc = nxh_check_tensor(op, out);
  if (!rc) rc = nxh_check_tensor(op, x);
  if (!rc && mask) rc = nxh_check_tensor(op, mask);
  if (!rc) rc = same_shape(op, out, x);
  if (!rc && mask) rc = same_shape(op, mask, x);
  if (!rc) rc = out_rows_ok(op, out);
  if (rc) return rc;
  const int dx = x->dtype, dout = out->dtype;
  if (!float_dtype_ok(dx) || (mask && mask->dtype != NXH_BOOL) ||
      !(dout == dx || (dx == NXH_F32 && (dout == NXH_BF16 || dout == NXH_F16))))
    return nxh_fail(NXH_FAILURE, op, NXH_ERR_UNSUPPORTED);
  SoftmaxArgs a;
  if ((rc = row_geometry(op, x, a.g))) return rc;
  if (a.g.rows == 0) return NXH_OK;
  if (a.g.n == 0) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_EMPTY_REDUCE);
  const int nd = x->ndim;
  if (x->strides[nd - 1] != 1 || out->strides[nd - 1] != 1 ||
      (mask && mask->strides[nd - 1] != 1 && mask->strides[nd - 1] != 0))
    return nxh_fail(NXH_FAILURE, op, "rows must be contiguous");
  if (a.g.rows > 0x7fffffffLL) return nxh_fail(NXH_FAILURE, op, "too many rows for one launch");
  row_operand(x, a.x);
  row_operand(out, a.out);
  row_operand(mask, a.mask);
  merge_outer_dims(a.g, {&a.x, &a.out, &a.mask});
  a.has_scale = scale != nullptr;
  a.has_mask = mask != nullptr;
  a.mask_last = mask ? mask->strides[nd - 1] : 0;
  a.scale = scale ? decode_scalar(dx, scale) : 1.0;
  a.masked = mask ? decode_scalar(dx, masked_value) : 0.0;
  const bool vec = a.g.n > ROW_REGS
                       ? rows_congruent(x, out, 4) && (!mask || a.mask_last == 0 || rows_congruent(x, mask, 4))
                       : a.g.n % 4 == 0 && rows_vector_ok(x, 4) && rows_vector_ok(out, 4) &&
                             (!mask || a.mask_last == 0 || rows_vector_ok(mask, 4));
  std::lock_guard<std::mutex> guard(ctx->mu);
  NXH_HIP(op, hipSetDevice(ctx->device));
  nxh_set_path(a.g.n > ROW_REGS ? "softmax_rows_long" : "softmax_rows");
  {
    const nxh_tensor *ts[3] = {out, x, mask};
    const void *base[3];
    uint64_t bytes[3];
    int nop = 0;
    for (int k = 0; k < 3; k++) {
      if (!ts[k]) continue;
      uint64_t n = 1;
      for (int d = 0; d < ts[k]->ndim; d++)
        if (ts[k]->strides[d] != 0) n *= (uint64_t)ts[k]->shape[d];
      base[nop] = ts[k]->data;
      bytes[nop++] = n * (uint64_t)nxh_elem_size(ts[k]->dtype);
    }
    a.stream = nxh_cache_hints(ctx, nop, base, bytes);
  }
  if (dx == NXH_F32 && dout == NXH_F32) softmax_launch<NXH_F32, NXH_F32>(ctx, a, vec);
  else if (dx == NXH_F32 && dout == NXH_BF16) softmax_launch<NXH_F32, NXH_BF16>(ctx, a, vec);
  else if (dx == NXH_F32) softmax_launch<NXH_F32, NXH_F16>(ctx, a, vec);
  else if (dx == NXH_BF16) softmax_launch<NXH_BF16, NXH_BF16>(ctx, a, vec);
  else if (dx == NXH_F16) softmax_launch<NXH_F16, NXH_F16>(ctx, a, vec);
  else softmax_launch<NXH_F64, NXH_F64>(ctx, a, vec);
  NXH_HIP(op, hipGetLastError());
  return NXH_OK;
}

NXH_EXPORT int nxh_layer_norm_rows(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x,
                                   const nxh_tensor *gamma, const nxh_tensor *beta, double eps) {
  NXH_DEFER_TOUCH(ctx, 1, out, x, gamma, beta);
  const char *op = "layer_norm_rows";
  if (!ctx || !out || !x) return nxh_fail(NXH_INVALID_ARGUMENT, op, "null argument");
  int rc = nxh_check_tensor(op, out);
  if (!rc) rc = nxh_check_tensor(op, x);
  if (!rc && gamma) rc = nxh_check_tensor(op, gamma);
  if (!rc && beta) rc = nxh_check_tensor(op, beta);
  if (!rc) rc = same_shape(op, out, x);
  if (!rc) rc = out_rows_ok(op, out);
  if (rc) return rc;
  if (!(eps >= 0.0)) return nxh_fail(NXH_INVALID_ARGUMENT, op, "eps must be >= 0");
  const int dx = x->dtype;
  if (!float_dtype_ok(dx) || out->dtype != dx || (gamma && gamma->dtype != dx) || (beta && beta->dtype != dx))
    return nxh_fail(NXH_FAILURE, op, NXH_ERR_UNSUPPORTED);
  LayerNormArgs a;
  if ((rc = row_geometry(op, x, a.g))) return rc;
  for (const nxh_tensor *p : {gamma, beta})
    if (p && (p->ndim != 1 || p->shape[0] != a.g.n)) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
  if (a.g.rows == 0) return NXH_OK;
  if (a.g.n == 0) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_EMPTY_REDUCE);
  const int nd = x->ndim;
  if (x->strides[nd - 1] != 1 || out->strides[nd - 1] != 1 || (gamma && a.g.n > 1 && gamma->strides[0] != 1) ||
      (beta && a.g.n > 1 && beta->strides[0] != 1))
    return nxh_fail(NXH_FAILURE, op, "rows must be contiguous");
  if (a.g.rows > 0x7fffffffLL) return nxh_fail(NXH_FAILURE, op, "too many rows for one launch");
  row_operand(x, a.x);
  row_operand(out, a.out);
  row_operand(nullptr, a.unused);
  merge_outer_dims(a.g, {&a.x, &a.out, &a.unused});
  const int es = (int)nxh_elem_size(dx);
  a.gamma = gamma ? (const char *)gamma->data + gamma->offset * es : nullptr;
  a.beta = beta ? (const char *)beta->data + beta->offset * es : nullptr;
  // the scalars the primitives would have been given: eps and the row length
  // filled into the statistics dtype (float32 for 16-bit inputs)
  a.eps = dx == NXH_F64 ? eps : (double)(float)eps;
  a.count = dx == NXH_F64 ? (double)a.g.n : (double)(float)a.g.n;
  const bool vec = a.g.n > ROW_REGS
                       ? rows_congruent(x, out, 4)
                       : a.g.n % 4 == 0 && rows_vector_ok(x, 4) && rows_vector_ok(out, 4) &&
                             (!gamma || ((uintptr_t)a.gamma % (es * 4)) == 0) && (!beta || ((uintptr_t)a.beta % (es * 4)) == 0);
  std::lock_guard<std::mutex> guard(ctx->mu);
  NXH_HIP(op, hipSetDevice(ctx->device));
  nxh_set_path(a.g.n > ROW_REGS ? "layer_norm_rows_long" : "layer_norm_rows");
  if (dx == NXH_F32) layer_norm_launch<NXH_F32>(ctx, a, vec);
  else if (dx == NXH_BF16) layer_norm_launch<NXH_BF16>(ctx, a, vec);
  else if (dx == NXH_F16) layer_norm_launch<NXH_F16>(ctx, a, vec);
  else layer_norm_launch<NXH_F64>(ctx, a, vec);
  NXH_HIP(op, hipGetLastError());
  return NXH_OK;
}

// The table of a 16-bit dtype's 65 536 results (slot 0 bfloat16, 1 float16) for the constants c,
// made on first use and again when the constants differ. *have is false when there is none for
// these constants and none can be made now (a capture can neither allocate nor refill it).
static int gelu_full_table(nxh_context *ctx, const char *op, int slot, const double *c, bool *have) {
  *have = ctx->gelu_lut[slot] != nullptr;
  if (!*have && !ctx->capture) {
    void *t = nullptr;
    NXH_HIP(op, hipMalloc(&t, LUT_BYTES));
    ctx->gelu_lut[slot] = t;
    ctx->gelu_lut_c[slot][0] = std::nan("");
    *have = true;
  }
  if (*have && memcmp(ctx->gelu_lut_c[slot], c, 4 * sizeof(double)) != 0) {
    // a captured refill would run at every replay, behind the back of this record; a refill
    // outside a capture would change what an earlier record's launches read at their next replay
    if (ctx->capture || ctx->gelu_lut_recorded[slot]) {
      *have = false;
      return NXH_OK;
    }
    GeluArgs a{};
    for (int i = 0; i < 4; i++) a.c[i] = c[i];
    if (slot == 0) hipLaunchKernelGGL((gelu_table_kernel<NXH_BF16>), dim3(256), dim3(256), 0, ctx->stream, (uint16_t *)ctx->gelu_lut[slot], a);
    else hipLaunchKernelGGL((gelu_table_kernel<NXH_F16>), dim3(256), dim3(256), 0, ctx->stream, (uint16_t *)ctx->gelu_lut[slot], a);
    NXH_HIP(op, hipGetLastError());
    memcpy(ctx->gelu_lut_c[slot], c, 4 * sizeof(double));
  }
  if (*have && ctx->capture) ctx->gelu_lut_recorded[slot] = true;
  return NXH_OK;
}

// narrow(x * c3) for every bfloat16 x, computed where the epilogue computes it
__global__ __launch_bounds__(256) void gelu_small_kernel(uint16_t *out, float c3) {
  const uint32_t i = blockIdx.x * 256 + threadIdx.x;
  out[i] = f32_to_bf16(bf16_to_f32((uint16_t)i) * c3);
}

int nxh_gelu_epilogue_table(nxh_context *ctx, const double *c, const void **table, uint32_t *lo, uint32_t *n) {
  const char *op = "linear_gelu_tanh";
  auto &e = ctx->gelu_epi;
  auto give = [&]() -> int {
    if (e.state <= 0) return 0;
    if (ctx->capture) e.recorded = true;
    *table = e.dev;
    *lo = e.lo;
    *n = e.n;
    return 1;
  };
  if (e.state != 0 && memcmp(e.c, c, sizeof e.c) == 0) return give();
  if (ctx->capture) return 0;  // making it waits for the stream
  if (e.recorded) return 0;    // a recorded graph reads the table made for other constants
  // The whole table and the closed form of its low end, read back once. The part kept in LDS is
  // [lo, hi): below lo every result must equal narrow(x * c3), from hi to the last finite binade
  // x itself (positive) or -0 (negative); both bounds fall on binades (multiples of 128).
  bool have = false;
  if (gelu_full_table(ctx, op, 0, c, &have) != NXH_OK || !have) return 0;
  void *small_dev = nullptr;
  if (hipMalloc(&small_dev, LUT_BYTES) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  hipLaunchKernelGGL(gelu_small_kernel, dim3(256), dim3(256), 0, ctx->stream, (uint16_t *)small_dev, (float)c[3]);
  std::vector<uint16_t> full(65536), small(65536);
  hipError_t err = hipMemcpyAsync(full.data(), ctx->gelu_lut[0], LUT_BYTES, hipMemcpyDeviceToHost, ctx->stream);
  if (err == hipSuccess) err = hipMemcpyAsync(small.data(), small_dev, LUT_BYTES, hipMemcpyDeviceToHost, ctx->stream);
  if (err == hipSuccess) err = hipStreamSynchronize(ctx->stream);
  (void)hipFree(small_dev);
  memcpy(e.c, c, sizeof e.c);
  e.state = -1;
  if (err != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  constexpr uint32_t TOP = 0x7f00u, MAXN = 2048;
  uint32_t low = 0, high = TOP;
  while (low < TOP) {  // extend [0, low) binade by binade
    bool ok = true;
    for (uint32_t m = low; m < low + 128 && ok; m++) ok = full[m] == small[m] && full[0x8000u | m] == small[0x8000u | m];
    if (!ok) break;
    low += 128;
  }
  while (high > 0) {  // extend [high, TOP) downwards
    bool ok = true;
    for (uint32_t m = high - 128; m < high && ok; m++) ok = full[m] == m && full[0x8000u | m] == 0x8000u;
    if (!ok) break;
    high -= 128;
  }
  if (low >= high) low = high >= 128 ? high - 128 : 0;  // (the two forms overlap: keep one binade)
  if (high <= low || high - low > MAXN) return 0;
  const uint32_t cnt = high - low;
  std::vector<uint16_t> compact(2 * cnt);
  for (uint32_t i = 0; i < cnt; i++) {
    compact[i] = full[low + i];
    compact[cnt + i] = full[0x8000u | (low + i)];
  }
  if (!e.dev && hipMalloc(&e.dev, 2 * MAXN * sizeof(uint16_t)) != hipSuccess) {
    (void)hipGetLastError();
    e.dev = nullptr;
    return 0;
  }
  err = hipMemcpyAsync(e.dev, compact.data(), compact.size() * sizeof(uint16_t), hipMemcpyHostToDevice, ctx->stream);
  if (err == hipSuccess) err = hipStreamSynchronize(ctx->stream);  // (the host copy dies with this call)
  if (err != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  e.lo = low;
  e.n = cnt;
  e.state = 1;
  return give();
}

NXH_EXPORT int nxh_gelu_tanh(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x, const void *constants) {
  NXH_DEFER_TOUCH(ctx, 1, out, x);
  const char *op = "gelu_tanh";
  if (!ctx || !out || !x || !constants) return nxh_fail(NXH_INVALID_ARGUMENT, op, "null argument");
  int rc = nxh_check_tensor(op, out);
  if (!rc) rc = nxh_check_tensor(op, x);
  if (!rc) rc = same_shape(op, out, x);
  if (rc) return rc;
  const int dx = x->dtype;
  if (!float_dtype_ok(dx) || out->dtype != dx) return nxh_fail(NXH_FAILURE, op, NXH_ERR_UNSUPPORTED);
  int64_t n = 1, expect = 1;
  bool dense = x->offset >= 0;
  for (int d = x->ndim - 1; d >= 0; d--) {
    if (x->shape[d] > 1 && (x->strides[d] != expect || out->strides[d] != expect)) dense = false;
    expect *= x->shape[d];
    n *= x->shape[d];
  }
  if (!dense) return nxh_fail(NXH_FAILURE, op, "operands must be C-contiguous");
  if (n == 0) return NXH_OK;
  const int es = (int)nxh_elem_size(dx);
  GeluArgs a;
  a.x = (const char *)x->data + x->offset * es;
  a.out = (char *)out->data + out->offset * es;
  a.n = n;
  for (int i = 0; i < 4; i++) a.c[i] = decode_scalar(dx, (const char *)constants + i * es);
  if (n / 256 > 0x7ffffff0LL) return nxh_fail(NXH_FAILURE, op, "too many elements for one launch");
  const bool vec = ((uintptr_t)a.x % 16) == 0 && ((uintptr_t)a.out % 16) == 0;
  std::lock_guard<std::mutex> guard(ctx->mu);
  NXH_HIP(op, hipSetDevice(ctx->device));
  // 16-bit dtypes, four million elements or more, whole aligned vectors: by table (the table of a
  // dtype is made on first use and again when the constants differ; not while a graph is being
  // captured unless it already exists, since a capture cannot allocate it)
  if ((dx == NXH_BF16 || dx == NXH_F16) && vec && n % 8 == 0 && n >= ((int64_t)1 << 22)) {
    const int slot = dx == NXH_BF16 ? 0 : 1;
    bool have = false;
    if (int trc = gelu_full_table(ctx, op, slot, a.c, &have)) return trc;
    if (have) {
      static std::once_flag once;
      static hipError_t attr_status = hipSuccess;
      std::call_once(once, [] {
        attr_status = hipFuncSetAttribute((const void *)gelu_lut_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, LUT_BYTES);
      });
      NXH_HIP(op, attr_status);
      const int64_t nvec = n / 8;
      const int blocks = ctx->compute_units > 0 ? ctx->compute_units : 256;
      const int64_t per_block = (nvec + blocks - 1) / blocks;
      nxh_set_path("gelu_tanh_table");
      hipLaunchKernelGGL(gelu_lut_kernel, dim3(blocks), dim3(LUT_THREADS), LUT_BYTES, ctx->stream,
                         (const uint16_t *)ctx->gelu_lut[slot], (const uint4 *)a.x, (uint4 *)a.out, nvec, per_block);
      NXH_HIP(op, hipGetLastError());
      return NXH_OK;
    }
  }
  nxh_set_path("gelu_tanh");
  if (dx == NXH_F32) gelu_launch<NXH_F32>(ctx, a, vec);
  else if (dx == NXH_BF16) gelu_launch<NXH_BF16>(ctx, a, vec);
  else if (dx == NXH_F16) gelu_launch<NXH_F16>(ctx, a, vec);
  else gelu_launch<NXH_F64>(ctx, a, vec);
  NXH_HIP(op, hipGetLastError());
  return NXH_OK;
}
