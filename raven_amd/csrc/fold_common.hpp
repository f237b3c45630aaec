// fold_common.hpp — what the reduction (fold.hip), argmax/argmin (arg.hip) and
// scan (scan.hip) translation units share: combine rules, storage/compute
// adapters, lane exchange and index decoding on the device; reduction
// geometry, output squeezing, scratch blocks and split sizing on the host.
#pragma once

#include <algorithm>
#include <type_traits>

#include "nxh_common.hpp"

constexpr int FOLD_MAXD = NXH_MAX_NDIM;  // any view the ABI can describe: kept and reduced dims together never exceed it
constexpr int FOLD_THREADS = 256;

static inline bool aligned_to16(const void *p) { return ((uintptr_t)p & 15) == 0; }

// ── combine rules ───────────────────────────────────────────────────────────
template <int OP, class C, Cat cat>
struct Combine {
  __device__ __forceinline__ static C init() {
    if constexpr (OP == NXH_SUM) {
      if constexpr (cat == CAT_COMPLEX) return C{0, 0};
      else return (C)0;
    } else if constexpr (OP == NXH_PROD) {
      if constexpr (cat == CAT_COMPLEX) return C{1, 0};
      else return (C)1;
    } else if constexpr (OP == NXH_RMAX) {
      if constexpr (cat == CAT_FLOAT) return (C)(-__builtin_inff());
      else if constexpr (cat == CAT_SINT || (cat == CAT_UINT && std::is_signed<C>::value)) return (C)INT64_MIN;
      else return (C)0;
    } else {
      if constexpr (cat == CAT_FLOAT) return (C)__builtin_inff();
      else if constexpr (cat == CAT_BOOL) return (C)1;
      else if constexpr (std::is_signed<C>::value) return (C)INT64_MAX;
      else return (C)UINT64_MAX;
    }
  }
  __device__ __forceinline__ static C apply(C m, C v) {
    if constexpr (OP == NXH_SUM) {
      if constexpr (cat == CAT_SINT) return (C)((uint64_t)m + (uint64_t)v);
      else return m + v;
    } else if constexpr (OP == NXH_PROD) {
      if constexpr (cat == CAT_SINT) return (C)((uint64_t)m * (uint64_t)v);
      else return m * v;
    } else if constexpr (OP == NXH_RMAX) {
      if constexpr (cat == CAT_FLOAT) return (v > m) ? v : ((v != v) ? v : m);
      else if constexpr (cat == CAT_BOOL) return (C)(m | v);
      else return v > m ? v : m;
    } else {
      if constexpr (cat == CAT_FLOAT) return (v < m) ? v : ((v != v) ? v : m);
      else if constexpr (cat == CAT_BOOL) return (C)(m & v);
      else return v < m ? v : m;
    }
  }
};
constexpr bool fold_ok(int op, Cat c) {
  return (op == NXH_SUM || op == NXH_PROD) ? (c != CAT_BOOL) : (c != CAT_COMPLEX);
}

// ── lane exchange for any trivially copyable accumulator ───────────────────
template <class T>
__device__ __forceinline__ T shfl_down_any(T v, int delta) {
  constexpr int W = (sizeof(T) + 3) / 4;
  union {
    T t;
    uint32_t w[W];
  } u;
  u.w[W - 1] = 0;
  u.t = v;
#pragma unroll
  for (int i = 0; i < W; i++) u.w[i] = __shfl_down(u.w[i], delta, 64);
  return u.t;
}


// Input / output adaptors: storage-typed (through the dtype converters) or raw
// compute-typed partials between the two passes.
template <int DT>
struct InS {
  using T = typename Tr<DT>::S;
  using C = typename Tr<DT>::C;
  __device__ __forceinline__ static C ld(T s) { return Tr<DT>::ld(s); }
};
template <class C_>
struct InC {
  using T = C_;
  using C = C_;
  __device__ __forceinline__ static C ld(T s) { return s; }
};
template <int DT>
struct OutS {
  using T = typename Tr<DT>::S;
  __device__ __forceinline__ static T st(typename Tr<DT>::C c) { return Tr<DT>::st(c); }
};
template <class C_>
struct OutC {
  using T = C_;
  __device__ __forceinline__ static T st(C_ c) { return c; }
};

template <class T, int N>
struct alignas(sizeof(T) * N >= 16 ? 16 : sizeof(T) * N) FVec {
  T v[N];
};

struct FoldDims {
  int n;
  uint32_t shape[FOLD_MAXD];
  int64_t in_stride[FOLD_MAXD];
  int64_t out_stride[FOLD_MAXD];
};
__device__ __forceinline__ void fold_decode(const FoldDims &d, uint64_t idx, int64_t &in_off,
                                            int64_t &out_off) {
  in_off = 0;
  out_off = 0;
  if (idx <= 0xffffffffull) {  // the common case: 32-bit divisions are an order cheaper
    uint32_t x = (uint32_t)idx;
    for (int i = d.n - 1; i >= 0; i--) {
      const uint32_t q = x / d.shape[i], c = x - q * d.shape[i];
      x = q;
      in_off += (int64_t)c * d.in_stride[i];
      out_off += (int64_t)c * d.out_stride[i];
    }
    return;
  }
  for (int i = d.n - 1; i >= 0; i--) {
    uint64_t q = idx / d.shape[i];
    uint32_t c = (uint32_t)(idx - q * d.shape[i]);
    idx = q;
    in_off += (int64_t)c * d.in_stride[i];
    out_off += (int64_t)c * d.out_stride[i];
  }
}

// ── host: geometry ──────────────────────────────────────────────────────────
struct Geom {
  int nk = 0, nr = 0;
  int64_t kshape[NXH_MAX_NDIM], kin[NXH_MAX_NDIM], kout[NXH_MAX_NDIM];
  int64_t rshape[NXH_MAX_NDIM], rin[NXH_MAX_NDIM];
  int64_t n_out = 1, R = 1;
  bool fixed_scratch = false;  // partial results go to the static workspace (no allocation)
};

// Splits dims into kept / reduced (strides in elements), drops size-1 dims and
// merges neighbours of the same class that compose.
static void geom_build(const nxh_tensor *in, const nxh_tensor *out_sq, const bool *reduced, Geom *g) {
  int oj = 0;
  int last_class = -1;  // 0 kept, 1 reduced: merging needs ADJACENT dims of one class
  for (int a = 0; a < in->ndim; a++) {
    int64_t s = in->shape[a], st = in->strides[a];
    if (reduced[a]) {
      g->R *= s;
      if (s != 1) {
        if (last_class == 1 && g->rin[g->nr - 1] == st * s) {
          g->rshape[g->nr - 1] *= s;
          g->rin[g->nr - 1] = st;
        } else {
          g->rshape[g->nr] = s;
          g->rin[g->nr++] = st;
        }
        last_class = 1;
      }
    } else {
      int64_t so = out_sq->strides[oj++];
      g->n_out *= s;
      if (s != 1) {
        if (last_class == 0 && g->kin[g->nk - 1] == st * s && g->kout[g->nk - 1] == so * s) {
          g->kshape[g->nk - 1] *= s;
          g->kin[g->nk - 1] = st;
          g->kout[g->nk - 1] = so;
        } else {
          g->kshape[g->nk] = s;
          g->kin[g->nk] = st;
          g->kout[g->nk++] = so;
        }
        last_class = 0;
      }
    }
  }
}

static bool dims_fill(FoldDims *d, int n, const int64_t *shape, const int64_t *in_s, const int64_t *out_s,
                      int skip = -1) {
  d->n = 0;
  for (int i = 0; i < n; i++) {
    if (i == skip) continue;
    if (d->n >= FOLD_MAXD || shape[i] > 0xffffffffLL) return false;
    d->shape[d->n] = (uint32_t)shape[i];
    d->in_stride[d->n] = in_s[i];
    d->out_stride[d->n] = out_s ? out_s[i] : 0;
    d->n++;
  }
  return true;
}
// Contiguous (row-major) input strides over the same kept shape, scaled.
static void dims_contig_in(FoldDims *d, int64_t inner) {
  int64_t acc = inner;
  for (int i = d->n - 1; i >= 0; i--) {
    d->in_stride[i] = acc;
    acc *= d->shape[i];
  }
}

// Scratch blocks of one call. Normally they come from the context's allocator.
// With `fixed` the single block is the device's static workspace instead:
// nothing is allocated or freed, and a request beyond its size fails.
struct Scratch {
  nxh_context *ctx;
  bool fixed;
  void *p[2] = {nullptr, nullptr};
  explicit Scratch(nxh_context *c, bool fixed_ = false) : ctx(c), fixed(fixed_) {}
  int get(int i, size_t bytes) {
    if (!fixed) return nxh_alloc_locked(ctx, bytes, &p[i]);
    if (i != 0 || bytes > NXH_STATIC_WS_BYTES || !ctx->static_ws)
      return nxh_fail(NXH_FAILURE, "reduce_noalloc",
                      "the partial results of this reduction exceed the static workspace "
                      "(NXH_STATIC_WORKSPACE_BYTES); use nxh_reduce");
    p[0] = ctx->static_ws;
    return NXH_OK;
  }
  ~Scratch() {  // stream-ordered: queued kernels keep using the blocks safely
    if (fixed) return;
    for (void *q : p)
      if (q) nxh_free_locked(ctx, q);
  }
};

static int pick_split(int64_t blocks, int64_t R, int64_t min_chunk, int cus) {
  // aim for ~8 blocks per CU when a single pass would leave the chip idle
  const int64_t target = (int64_t)cus * 8;
  if (blocks >= target / 2 || R < 2 * min_chunk) return 1;
  int64_t want = (target + blocks - 1) / blocks;
  int64_t cap = R / min_chunk;
  int64_t s = std::min<int64_t>(std::min(want, cap), 1024);
  return (int)std::max<int64_t>(s, 1);
}

typedef int (*fold_fn)(nxh_context *, const char *, const nxh_tensor *, const nxh_tensor *, const Geom &);

// nx_c_engine.c:1392-1420: accept a squeezed or a keepdims-shaped output.
static int squeeze_out(const char *op, const nxh_tensor *in, const nxh_tensor *out, const int32_t *axes,
                       int nred, bool *reduced, nxh_tensor *sq) {
  if (nred < 0 || nred > in->ndim) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_AXES);
  for (int a = 0; a < in->ndim; a++) reduced[a] = false;
  for (int i = 0; i < nred; i++) {
    int a = axes[i];
    if (a < 0 || a >= in->ndim || reduced[a]) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_AXES);
    if (i > 0 && axes[i] <= axes[i - 1]) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_AXES);
    reduced[a] = true;
  }
  const int kept = in->ndim - nred;
  *sq = *out;
  if (out->ndim != kept) {
    if (out->ndim != in->ndim) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_OUT_RANK);
    sq->ndim = kept;
    int j = 0;
    for (int a = 0; a < in->ndim; a++)
      if (!reduced[a]) {
        sq->shape[j] = out->shape[a];
        sq->strides[j] = out->strides[a];
        j++;
      }
  }
  int j = 0;
  for (int a = 0; a < in->ndim; a++)
    if (!reduced[a]) {
      if (sq->shape[j] != in->shape[a]) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
      j++;
    }
  return NXH_OK;
}


// Tells the cache policy (runtime.hip) what a reduction or argreduce reads and writes.
// Its kernels take no hints: a reduction's input measured slower through non-temporal
// loads both alone ([8192,8192] f32 sum along rows in a loop: 6.6 against 6.8 TB/s) and
// behind its producer, where it is still cached.
static inline void fold_note_access(nxh_context *ctx, const nxh_tensor *in, const nxh_tensor *out, int64_t n_out, int64_t R) {
  const void *base[2] = {out->data, in->data};
  const uint64_t bytes[2] = {(uint64_t)n_out * (uint64_t)nxh_elem_size(out->dtype),
                             (uint64_t)n_out * (uint64_t)R * (uint64_t)nxh_elem_size(in->dtype)};
  (void)nxh_cache_hints(ctx, 2, base, bytes, 0);
}
