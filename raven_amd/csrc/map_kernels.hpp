// map_kernels.hpp — the elementwise ("map") kernel family and its planner.
//
// Host side: descriptor lowering. K operands sharing one shape are stripped of
// size-1 dims, reordered so the output's strides descend, and merged wherever
// adjacent dims compose on EVERY operand (the reference's rule,
// nx_c_engine.c:542-590). The plan then picks one of three kernels:
//   map_contig   every operand is one contiguous run or a broadcast scalar:
//                16-byte vector loads/stores, 2 vectors in flight per lane.
//   map_tiled    some input's unit-stride dim differs from the output's: patches of
//                8 KiB (64 x 32 four-byte elements), that input is read along ITS
//                contiguous dim and turned through LDS, so both sides of HBM see
//                coalesced rows.
//   map_generic  anything else: per-lane index decomposition with precomputed
//                multiply-shift divisors; vectorised along the inner dim when
//                every operand is contiguous or broadcast there.
// Kernels are HBM-bound byte movers: no MFMA, LDS only for the turn.
#pragma once

#include <algorithm>
#include <type_traits>

#include "nxh_common.hpp"
#include "stream_access.hpp"

constexpr int MAP_MAXOP = 4;
constexpr int MAP_MAXD = 8;
constexpr int MAP_THREADS = 256;
constexpr int MAP_UNROLL = 4;     // vectors in flight per lane, map_generic
#ifndef MAP_CONTIG_UNROLL_X
#define MAP_CONTIG_UNROLL_X 2
#endif
constexpr int MAP_CONTIG_UNROLL = MAP_CONTIG_UNROLL_X;  // the same for map_contig

struct MapPlan {
  int nop = 0, ndim = 0;
  int64_t total = 0;
  int64_t shape[NXH_MAX_NDIM];
  int64_t stride[MAP_MAXOP][NXH_MAX_NDIM];  // element strides
  char *base[MAP_MAXOP];                    // byte address of logical element 0
  int esize[MAP_MAXOP];
  uint32_t stream = 0;  // NXH_STREAM_OUT / NXH_STREAM_IN: accesses that go past the memory-side cache
};

// Builds the coalesced plan. Returns NXH_OK or a status (aliased output).
static inline int map_plan_build(const char *op, const nxh_tensor *const *ops, int nop,
                                 const int *esize, MapPlan *p) {
  const int nd_in = ops[0]->ndim;
  p->nop = nop;
  p->total = 1;
  for (int i = 0; i < nd_in; i++) p->total *= ops[0]->shape[i];
  for (int k = 0; k < nop; k++) {
    p->esize[k] = esize[k];
    p->base[k] = (char *)ops[k]->data + ops[k]->offset * (int64_t)esize[k];
  }
  int order[NXH_MAX_NDIM], n = 0;
  for (int i = 0; i < nd_in; i++)
    if (ops[0]->shape[i] != 1) order[n++] = i;
  if (p->total != 0) {
    for (int j = 0; j < n; j++)
      if (ops[0]->strides[order[j]] == 0) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_OUT_ALIASED);
    // Elementwise work is order-free: walk the output in its own memory order.
    std::stable_sort(order, order + n, [&](int a, int b) {
      return std::llabs(ops[0]->strides[a]) > std::llabs(ops[0]->strides[b]);
    });
  }
  int nd = 0;
  for (int j = 0; j < n; j++) {
    int i = order[j];
    int64_t s = ops[0]->shape[i];
    bool merge = nd > 0;
    for (int k = 0; merge && k < nop; k++)
      if (p->stride[k][nd - 1] != ops[k]->strides[i] * s) merge = false;
    if (merge) {
      p->shape[nd - 1] *= s;
      for (int k = 0; k < nop; k++) p->stride[k][nd - 1] = ops[k]->strides[i];
    } else {
      p->shape[nd] = s;
      for (int k = 0; k < nop; k++) p->stride[k][nd] = ops[k]->strides[i];
      nd++;
    }
  }
  if (nd == 0) {
    p->shape[0] = 1;
    for (int k = 0; k < nop; k++) p->stride[k][0] = 0;
    nd = 1;
  }
  p->ndim = nd;
  return NXH_OK;
}

// ── device helpers ──────────────────────────────────────────────────────────

template <class T, int N>
struct alignas(sizeof(T) * N) Vec {
  T v[N];
};

struct Unused {};  // placeholder input type

// n / d for n < 2^31 by multiply-high and shift (d >= 1).
struct FastDiv {
  uint32_t d, m, s;
};
static inline FastDiv fastdiv_make(uint32_t d) {
  FastDiv f;
  f.d = d;
  uint32_t s = 0;
  while (s < 32 && ((uint64_t)1 << s) < d) s++;
  f.s = s;
  f.m = (uint32_t)((((uint64_t)1 << 32) * (((uint64_t)1 << s) - d)) / d + 1);
  return f;
}
__device__ __forceinline__ uint32_t fastdiv(uint32_t n, const FastDiv &f) {
  return (__umulhi(n, f.m) + n) >> f.s;
}

template <class F>
struct MapTypes {
  using Out = typename F::Out;
  using In0 = typename F::In0;
  using In1 = typename F::In1;
  using In2 = typename F::In2;
  static constexpr int s0 = sizeof(In0);
  static constexpr int s1 = F::NIN > 1 ? sizeof(In1) : 1;
  static constexpr int s2 = F::NIN > 2 ? sizeof(In2) : 1;
  static constexpr int smax = std::max(std::max((int)sizeof(Out), s0), std::max(s1, s2));
  static constexpr int VEC = 16 / smax > 0 ? 16 / smax : 1;
};

template <class F>
__device__ __forceinline__ typename F::Out map_apply(typename F::In0 a, typename F::In1 b,
                                                     typename F::In2 c) {
  if constexpr (F::NIN == 1) return F::apply(a);
  else if constexpr (F::NIN == 2) return F::apply(a, b);
  else return F::apply(a, b, c);
}

// Loads V elements of operand type T starting at element index e.
template <bool STREAM, class T, int V>
__device__ __forceinline__ Vec<T, V> load_vec(const T *p, int64_t e) {
  if constexpr (STREAM) return load_stream(reinterpret_cast<const Vec<T, V> *>(p + e));
  else return *reinterpret_cast<const Vec<T, V> *>(p + e);
}
// The same, or a broadcast of the single element at e.
template <class T, int V>
__device__ __forceinline__ Vec<T, V> load_vec_or_splat(const T *p, int64_t e, bool bc) {
  Vec<T, V> r;
  if (bc) {
    T x = p[e];
#pragma unroll
    for (int i = 0; i < V; i++) r.v[i] = x;
  } else {
    r = *reinterpret_cast<const Vec<T, V> *>(p + e);
  }
  return r;
}

// ── map_contig ──────────────────────────────────────────────────────────────
template <class F>
struct ContigArgs {
  typename F::Out *out;
  const typename F::In0 *in0;
  const typename F::In1 *in1;
  const typename F::In2 *in2;
  int64_t n;       // elements
  uint32_t bcast;   // bit k set: input k is a broadcast scalar
  uint32_t stream;  // NXH_STREAM_OUT / NXH_STREAM_IN
};

// The loads of one lane: UNR vectors of every input that is not a broadcast scalar, issued
// back to back. Nothing here uses a loaded value, so no load waits for another.
template <bool STREAM, class F, int V, int UNR>
__device__ __forceinline__ void contig_fetch(const ContigArgs<F> &a, int64_t base, int64_t nvec,
                                             Vec<typename F::In0, V> (&x0)[UNR], Vec<typename F::In1, V> (&x1)[UNR],
                                             Vec<typename F::In2, V> (&x2)[UNR]) {
  const bool b0 = a.bcast & 1u, b1 = a.bcast & 2u, b2 = a.bcast & 4u;
#pragma unroll
  for (int j = 0; j < UNR; j++) {
    const int64_t u = base + (int64_t)j * MAP_THREADS;
    if (u < nvec) {
      if (!b0) x0[j] = load_vec<STREAM, typename F::In0, V>(a.in0, u * V);
      if constexpr (F::NIN > 1)
        if (!b1) x1[j] = load_vec<STREAM, typename F::In1, V>(a.in1, u * V);
      if constexpr (F::NIN > 2)
        if (!b2) x2[j] = load_vec<STREAM, typename F::In2, V>(a.in2, u * V);
    }
  }
}

template <class F, int V, int UNR>
__global__ __launch_bounds__(MAP_THREADS) void map_contig_kernel(ContigArgs<F> a) {
  using MT = MapTypes<F>;
  const int64_t nvec = a.n / V;
  const int64_t base = (int64_t)blockIdx.x * (MAP_THREADS * UNR) + threadIdx.x;
  const bool b0 = a.bcast & 1u, b1 = a.bcast & 2u, b2 = a.bcast & 4u;
  // a broadcast scalar is read once, in front of the vector loads, and chosen per element
  // afterwards: filling a vector with it between the loads would make every later load
  // wait for the earlier ones
  typename MT::In0 s0{};
  typename MT::In1 s1{};
  typename MT::In2 s2{};
  if (b0) s0 = a.in0[0];
  if constexpr (F::NIN > 1)
    if (b1) s1 = a.in1[0];
  if constexpr (F::NIN > 2)
    if (b2) s2 = a.in2[0];
  Vec<typename MT::In0, V> x0[UNR];
  Vec<typename MT::In1, V> x1[UNR];
  Vec<typename MT::In2, V> x2[UNR];
  if (a.stream & NXH_STREAM_IN) contig_fetch<true, F, V, UNR>(a, base, nvec, x0, x1, x2);
  else contig_fetch<false, F, V, UNR>(a, base, nvec, x0, x1, x2);
  wait_for_loads();
  Vec<typename MT::Out, V> r[UNR];
#pragma unroll
  for (int j = 0; j < UNR; j++)
    if (base + (int64_t)j * MAP_THREADS < nvec) {
#pragma unroll
      for (int i = 0; i < V; i++) {
        typename MT::In0 v0 = b0 ? s0 : x0[j].v[i];
        typename MT::In1 v1{};
        typename MT::In2 v2{};
        if constexpr (F::NIN > 1) v1 = b1 ? s1 : x1[j].v[i];
        if constexpr (F::NIN > 2) v2 = b2 ? s2 : x2[j].v[i];
        r[j].v[i] = map_apply<F>(v0, v1, v2);
      }
    }
  if (a.stream & NXH_STREAM_OUT) {
#pragma unroll
    for (int j = 0; j < UNR; j++) {
      const int64_t u = base + (int64_t)j * MAP_THREADS;
      if (u < nvec) store_stream(reinterpret_cast<Vec<typename MT::Out, V> *>(a.out + u * V), r[j]);
    }
  } else {
#pragma unroll
    for (int j = 0; j < UNR; j++) {
      const int64_t u = base + (int64_t)j * MAP_THREADS;
      if (u < nvec) *reinterpret_cast<Vec<typename MT::Out, V> *>(a.out + u * V) = r[j];
    }
  }
  // ragged tail: fewer than V elements, one lane each
  if (blockIdx.x == 0 && threadIdx.x < (unsigned)(a.n - nvec * V)) {
    int64_t e = nvec * V + threadIdx.x;
    typename MT::In0 v0 = a.in0[b0 ? 0 : e];
    typename MT::In1 v1{};
    typename MT::In2 v2{};
    if constexpr (F::NIN > 1) v1 = a.in1[b1 ? 0 : e];
    if constexpr (F::NIN > 2) v2 = a.in2[b2 ? 0 : e];
    a.out[e] = map_apply<F>(v0, v1, v2);
  }
}

// ── map_generic ─────────────────────────────────────────────────────────────
template <class F>
struct GenericArgs {
  char *base[MAP_MAXOP];  // byte pointers: out, in0, in1, in2
  int ndim;
  uint32_t units;                 // total / V
  FastDiv div[MAP_MAXD];          // per dim, in units for the innermost
  int64_t stride[MAP_MAXOP][MAP_MAXD];  // element strides (innermost: per unit = stride * V)
  uint32_t inner_bcast;           // bit k: operand k has inner stride 0 (V > 1 only)
};

template <class F, int V>
__global__ __launch_bounds__(MAP_THREADS) void map_generic_kernel(GenericArgs<F> a) {
  using MT = MapTypes<F>;
  const uint32_t first = blockIdx.x * (MAP_THREADS * MAP_UNROLL) + threadIdx.x;
  Vec<typename MT::In0, V> x0[MAP_UNROLL];
  Vec<typename MT::In1, V> x1[MAP_UNROLL];
  Vec<typename MT::In2, V> x2[MAP_UNROLL];
  int64_t oo[MAP_UNROLL];
#pragma unroll
  for (int j = 0; j < MAP_UNROLL; j++) {
    uint32_t u = first + j * MAP_THREADS;
    if (u < a.units) {
      int64_t off[MAP_MAXOP] = {0, 0, 0, 0};
      uint32_t rem = u;
      for (int d = a.ndim - 1; d >= 0; d--) {
        uint32_t q = fastdiv(rem, a.div[d]);
        uint32_t c = rem - q * a.div[d].d;
        rem = q;
#pragma unroll
        for (int k = 0; k <= F::NIN; k++) off[k] += (int64_t)c * a.stride[k][d];
      }
      oo[j] = off[0];
      x0[j] = load_vec_or_splat<typename MT::In0, V>((const typename MT::In0 *)a.base[1], off[1],
                                            V > 1 && (a.inner_bcast & 2u));
      if constexpr (F::NIN > 1)
        x1[j] = load_vec_or_splat<typename MT::In1, V>((const typename MT::In1 *)a.base[2], off[2],
                                              V > 1 && (a.inner_bcast & 4u));
      if constexpr (F::NIN > 2)
        x2[j] = load_vec_or_splat<typename MT::In2, V>((const typename MT::In2 *)a.base[3], off[3],
                                              V > 1 && (a.inner_bcast & 8u));
    }
  }
#pragma unroll
  for (int j = 0; j < MAP_UNROLL; j++) {
    uint32_t u = first + j * MAP_THREADS;
    if (u < a.units) {
      Vec<typename MT::Out, V> r;
#pragma unroll
      for (int i = 0; i < V; i++) r.v[i] = map_apply<F>(x0[j].v[i], x1[j].v[i], x2[j].v[i]);
      *reinterpret_cast<Vec<typename MT::Out, V> *>((typename MT::Out *)a.base[0] + oo[j]) = r;
    }
  }
}

// ── map_tiled ───────────────────────────────────────────────────────────────
// Plane (y, x): x is the output's unit-stride dim, y the dim along which the
// turned inputs are contiguous. All other dims are batch dims decoded per
// block. A block of 256 lanes owns a TILE x TILE patch; every lane moves V
// consecutive elements per access (16 bytes of the widest operand type), so a
// wave touches whole 256-byte rows on both sides of the turn.
enum { TILE_ROW = 0, TILE_TURN = 1, TILE_BX = 2 };

template <class F>
struct TiledArgs {
  char *base[MAP_MAXOP];
  uint32_t nx, ny, tiles_x, tiles_y;
  int nbatch_dims;
  uint32_t bshape[MAP_MAXD];
  int64_t bstride[MAP_MAXOP][MAP_MAXD];
  int64_t sx[MAP_MAXOP], sy[MAP_MAXOP];  // element strides along x / y
  // per input: TILE_ROW unit stride along x, TILE_TURN unit stride along y (read
  // along y, turned through LDS), TILE_BX broadcast along x
  uint32_t mode[MAP_MAXOP];
  uint32_t any_turn;
  uint32_t stream;  // NXH_STREAM_OUT / NXH_STREAM_IN (the vector accesses of ROW / TURN operands)
};

// Tile geometry. The patch is TX (along x) by TY (along y) elements. Everything that is
// stored, and every input with a unit stride along x, moves in the OUTPUT arrangement: VX
// consecutive x per lane, GXO lanes across a row, RYO rows per pass of the block, NYO
// passes. A turned input is fetched in its own arrangement: VY consecutive y per lane, GYT
// lanes along y, RXT columns per pass, NXT passes. The kernel uses VX = VY, which makes
// NYO = NXT.
template <int TX, int TY, int VX, int VY>
struct TileGeom {
  static constexpr int GXO = TX / VX, RYO = MAP_THREADS / GXO, NYO = TY / RYO;
  static constexpr int GYT = TY / VY, RXT = MAP_THREADS / GYT, NXT = TX / RXT;
  static constexpr int PITCH = TX + 1;  // odd: element-wide LDS accesses of 4-byte types spread over the banks
  static_assert(GXO * VX == TX && GXO * RYO == MAP_THREADS && NYO * RYO == TY && NYO >= 1, "output arrangement");
  static_assert(GYT * VY == TY && GYT * RXT == MAP_THREADS && NXT * RXT == TX && NXT >= 1, "fetch arrangement");
};

// One input of the tile and this lane's share of it, in two steps. address() works out
// where the lane's NYO accesses go; fetch() only issues them. The kernel runs address() for
// every operand before the first fetch(), so that no vector instruction stands between the
// loads: the compiler reuses registers across the kernel's mutually exclusive paths and, at
// any instruction that writes a register some other path loads into, waits for all loads.
// An operand with a unit stride along x (ROW) or along y (TURN) is fetched as V-element
// vectors along that dim by one piece of code: the two arrangements differ only in which
// coordinate the lane's vector runs along, a choice that is uniform over the launch. A
// turned operand then goes through LDS to reach the output arrangement; an operand
// broadcast along x keeps one value per row in b and is chosen per element where the
// results are formed.
template <class T, class TG, int V>
struct TileOperand {
  static_assert(TG::NYO == TG::NXT, "both arrangements hold the same number of vectors per lane");
  Vec<T, V> r[TG::NYO];
  T b[TG::NYO];
  const NXH_GLOBAL char *at[TG::NYO];
  bool ok[TG::NYO];
  __device__ __forceinline__ void address(const T *p, int64_t sx, int64_t sy, uint32_t x0, uint32_t y0, uint32_t nx,
                                          uint32_t ny, uint32_t mode) {
    const bool turn = mode == TILE_TURN;
    // along: the coordinate the vector runs along (x, or y when turned); across: the other
    const uint32_t G = turn ? TG::GYT : TG::GXO, R = turn ? TG::RXT : TG::RYO;
    const uint32_t g = threadIdx.x % G, q = threadIdx.x / G;
    const uint32_t along = (turn ? y0 : x0) + g * V, n_along = turn ? ny : nx;
    const uint32_t across = (turn ? x0 : y0) + q, n_across = turn ? nx : ny;
    const int64_t pitch = turn ? sx : sy;
    const T *s = p + (int64_t)(mode == TILE_BX ? 0u : along) + (int64_t)across * pitch;
    const int64_t step = (int64_t)R * pitch;
#pragma unroll
    for (int i = 0; i < TG::NYO; i++) {
      at[i] = (const NXH_GLOBAL char *)s;
      ok[i] = along < n_along && across + i * R < n_across;
      s += step;
    }
  }
  // keeps the addresses computed where address() stands
  __device__ __forceinline__ void pin() {
#pragma unroll
    for (int i = 0; i < TG::NYO; i++) asm volatile("" : "+v"(at[i]));
  }
  template <bool STREAM>
  __device__ __forceinline__ void fetch(uint32_t mode) {
    if (mode == TILE_BX) {
#pragma unroll
      for (int i = 0; i < TG::NYO; i++)
        if (ok[i]) b[i] = load_global<false, T>(at[i]);
    } else {
#pragma unroll
      for (int i = 0; i < TG::NYO; i++)
        if (ok[i]) r[i] = load_global<STREAM, Vec<T, V>>(at[i]);
    }
  }
  // The turn: lds is [y][x] with a one-element pad, written from the fetch arrangement,
  // read in the output arrangement, one element per access.
  __device__ __forceinline__ void put(T *lds) const {
    const uint32_t g = threadIdx.x % TG::GYT, q = threadIdx.x / TG::GYT;
#pragma unroll
    for (int i = 0; i < TG::NXT; i++)
#pragma unroll
      for (int j = 0; j < V; j++) lds[(g * V + j) * TG::PITCH + q + i * TG::RXT] = r[i].v[j];
  }
  __device__ __forceinline__ void get(const T *lds) {
    const uint32_t g = threadIdx.x % TG::GXO, q = threadIdx.x / TG::GXO;
#pragma unroll
    for (int i = 0; i < TG::NYO; i++)
#pragma unroll
      for (int j = 0; j < V; j++) r[i].v[j] = lds[(q + i * TG::RYO) * TG::PITCH + g * V + j];
  }
  __device__ __forceinline__ T value(int i, int j, bool bx) const { return bx ? b[i] : r[i].v[j]; }
};

template <bool STREAM, class F, class R0, class R1, class R2>
__device__ __forceinline__ void tile_fetch_all(const TiledArgs<F> &a, R0 &r0, R1 &r1, R2 &r2) {
  r0.template fetch<STREAM>(a.mode[1]);
  if constexpr (F::NIN > 1) r1.template fetch<STREAM>(a.mode[2]);
  if constexpr (F::NIN > 2) r2.template fetch<STREAM>(a.mode[3]);
}

template <class F, int TX, int TY, int VX>
__global__ __launch_bounds__(MAP_THREADS) void map_tiled_kernel(TiledArgs<F> a) {
  using MT = MapTypes<F>;
  using TG = TileGeom<TX, TY, VX, VX>;
  using I0 = typename MT::In0;
  using I1 = typename MT::In1;
  using I2 = typename MT::In2;
  using O = typename MT::Out;
  __shared__ I0 l0[TY * TG::PITCH];
  __shared__ I1 l1[F::NIN > 1 ? TY * TG::PITCH : 1];
  __shared__ I2 l2[F::NIN > 2 ? TY * TG::PITCH : 1];
  // Blocks with equal id modulo 8 share an XCD (and its L2): hand each XCD a
  // contiguous run of tiles, so neighbouring tiles that split a cache line of a
  // narrow operand fetch it once.
  uint32_t b = blockIdx.x;
  if ((gridDim.x & 7u) == 0) b = (b & 7u) * (gridDim.x >> 3) + (b >> 3);
  const uint32_t tx = b % a.tiles_x;
  b /= a.tiles_x;
  const uint32_t ty = b % a.tiles_y;
  b /= a.tiles_y;
  int64_t off[MAP_MAXOP] = {0, 0, 0, 0};
  for (int d = a.nbatch_dims - 1; d >= 0; d--) {
    uint32_t c = b % a.bshape[d];
    b /= a.bshape[d];
#pragma unroll
    for (int k = 0; k <= F::NIN; k++) off[k] += (int64_t)c * a.bstride[k][d];
  }
  const uint32_t x0 = tx * TX, y0 = ty * TY;
  TileOperand<I0, TG, VX> r0;
  TileOperand<I1, TG, VX> r1;
  TileOperand<I2, TG, VX> r2;
  r0.address((const I0 *)a.base[1] + off[1], a.sx[1], a.sy[1], x0, y0, a.nx, a.ny, a.mode[1]);
  if constexpr (F::NIN > 1) r1.address((const I1 *)a.base[2] + off[2], a.sx[2], a.sy[2], x0, y0, a.nx, a.ny, a.mode[2]);
  if constexpr (F::NIN > 2) r2.address((const I2 *)a.base[3] + off[3], a.sx[3], a.sy[3], x0, y0, a.nx, a.ny, a.mode[3]);
  r0.pin();
  if constexpr (F::NIN > 1) r1.pin();
  if constexpr (F::NIN > 2) r2.pin();
  asm volatile("" ::: "memory");
  if (a.stream & NXH_STREAM_IN) tile_fetch_all<true, F>(a, r0, r1, r2);
  else tile_fetch_all<false, F>(a, r0, r1, r2);
  wait_for_loads();
  if (a.any_turn) {
    if (a.mode[1] == TILE_TURN) r0.put(l0);
    if constexpr (F::NIN > 1)
      if (a.mode[2] == TILE_TURN) r1.put(l1);
    if constexpr (F::NIN > 2)
      if (a.mode[3] == TILE_TURN) r2.put(l2);
    __syncthreads();
    if (a.mode[1] == TILE_TURN) r0.get(l0);
    if constexpr (F::NIN > 1)
      if (a.mode[2] == TILE_TURN) r1.get(l1);
    if constexpr (F::NIN > 2)
      if (a.mode[3] == TILE_TURN) r2.get(l2);
  }
  const uint32_t g = threadIdx.x % TG::GXO, q = threadIdx.x / TG::GXO;
  const uint32_t x = x0 + g * VX;
  O *o = (O *)a.base[0] + off[0] + (int64_t)(y0 + q) * a.sy[0] + x;
  const int64_t step = (int64_t)TG::RYO * a.sy[0];
  const bool bx0 = a.mode[1] == TILE_BX, bx1 = a.mode[2] == TILE_BX, bx2 = a.mode[3] == TILE_BX;
  Vec<O, VX> v[TG::NYO];
#pragma unroll
  for (int i = 0; i < TG::NYO; i++)
    if (x < a.nx && y0 + q + i * TG::RYO < a.ny) {
#pragma unroll
      for (int j = 0; j < VX; j++) {
        I1 v1{};
        I2 v2{};
        if constexpr (F::NIN > 1) v1 = r1.value(i, j, bx1);
        if constexpr (F::NIN > 2) v2 = r2.value(i, j, bx2);
        v[i].v[j] = map_apply<F>(r0.value(i, j, bx0), v1, v2);
      }
    }
  if (a.stream & NXH_STREAM_OUT) {
#pragma unroll
    for (int i = 0; i < TG::NYO; i++) {
      if (x < a.nx && y0 + q + i * TG::RYO < a.ny) store_stream(reinterpret_cast<Vec<O, VX> *>(o), v[i]);
      o += step;
    }
  } else {
#pragma unroll
    for (int i = 0; i < TG::NYO; i++) {
      if (x < a.nx && y0 + q + i * TG::RYO < a.ny) *reinterpret_cast<Vec<O, VX> *>(o) = v[i];
      o += step;
    }
  }
}

// ── host launcher ───────────────────────────────────────────────────────────

static inline bool aligned_to(const void *p, size_t a) { return ((uintptr_t)p % a) == 0; }

template <class F>
static int map_launch_generic(nxh_context *ctx, const char *op, const MapPlan &p) {
  using MT = MapTypes<F>;
  constexpr int V = MT::VEC;
  const int last = p.ndim - 1;
  const int esz[MAP_MAXOP] = {(int)sizeof(typename MT::Out), MT::s0, MT::s1, MT::s2};
  bool vec_ok = V > 1 && p.shape[last] % V == 0 && p.stride[0][last] == 1;
  uint32_t inner_bcast = 0;
  for (int k = 0; vec_ok && k < p.nop; k++) {
    int64_t s = p.stride[k][last];
    if (s == 0) inner_bcast |= 1u << k;
    else if (s != 1) vec_ok = false;
    if (s == 1) {
      if (!aligned_to(p.base[k], (size_t)esz[k] * V)) vec_ok = false;
      for (int d = 0; d < last; d++)
        if (p.stride[k][d] % V != 0) vec_ok = false;
    }
  }
  GenericArgs<F> a;
  for (int k = 0; k < MAP_MAXOP; k++) a.base[k] = k < p.nop ? p.base[k] : nullptr;
  a.ndim = p.ndim;
  const int v = vec_ok ? V : 1;
  a.units = (uint32_t)(p.total / v);
  a.inner_bcast = vec_ok ? inner_bcast : 0;
  for (int d = 0; d < p.ndim; d++) {
    uint32_t sh = (uint32_t)(d == last ? p.shape[d] / v : p.shape[d]);
    a.div[d] = fastdiv_make(sh);
    for (int k = 0; k < MAP_MAXOP; k++)
      a.stride[k][d] = k < p.nop ? p.stride[k][d] * (d == last ? v : 1) : 0;
  }
  const uint32_t per_block = MAP_THREADS * MAP_UNROLL;
  const uint32_t blocks = (a.units + per_block - 1) / per_block;
  if (vec_ok) {
    if constexpr (V > 1) {
      nxh_set_path("map_generic_vec");
      hipLaunchKernelGGL((map_generic_kernel<F, V>), dim3(blocks), dim3(MAP_THREADS), 0, ctx->stream, a);
    }
  } else {
    nxh_set_path("map_generic");
    hipLaunchKernelGGL((map_generic_kernel<F, 1>), dim3(blocks), dim3(MAP_THREADS), 0, ctx->stream, a);
  }
  NXH_HIP(op, hipGetLastError());
  return NXH_OK;
}

// One launch over a plan whose total is < 2^31 and whose rank is <= MAP_MAXD.
template <class F>
static int map_launch_one(nxh_context *ctx, const char *op, const MapPlan &p) {
  using MT = MapTypes<F>;
  constexpr int V = MT::VEC;
  const int esz[MAP_MAXOP] = {(int)sizeof(typename MT::Out), MT::s0, MT::s1, MT::s2};
  // 1. contiguous / scalar-broadcast
  if (p.ndim == 1 && (p.stride[0][0] == 1 || p.total == 1)) {
    bool ok = true;
    uint32_t bc = 0;
    for (int k = 1; k < p.nop; k++) {
      int64_t s = p.stride[k][0];
      if (s == 0 || p.total == 1) bc |= (p.total == 1 ? 0u : 1u << (k - 1));
      else if (s != 1) ok = false;
    }
    // A narrow output (compare, narrowing casts) widens the lane's vector until
    // it stores 16 bytes, with fewer vectors per lane so that the bytes in
    // flight stay the same; operands must then be aligned to the wider vector.
    constexpr int VW = (int)sizeof(typename MT::Out) < MT::smax
                           ? std::min(16 / (int)sizeof(typename MT::Out), V * MAP_CONTIG_UNROLL) : V;
    constexpr int UW = V * MAP_CONTIG_UNROLL / VW;
    bool wide = VW > V;
    for (int k = 0; ok && k < p.nop; k++) {
      bool is_bc = k > 0 && (bc & (1u << (k - 1)));
      if (is_bc) continue;
      if (!aligned_to(p.base[k], (size_t)esz[k] * V)) ok = false;
      if (!aligned_to(p.base[k], (size_t)esz[k] * VW)) wide = false;
    }
    if (ok) {
      ContigArgs<F> a;
      a.out = (typename MT::Out *)p.base[0];
      a.in0 = (const typename MT::In0 *)p.base[1];
      a.in1 = (const typename MT::In1 *)(p.nop > 2 ? p.base[2] : nullptr);
      a.in2 = (const typename MT::In2 *)(p.nop > 3 ? p.base[3] : nullptr);
      a.n = p.total;
      a.bcast = bc;
      a.stream = p.stream;
      nxh_set_path("map_contig");
      if (wide) {
        const int64_t nvec = (p.total + VW - 1) / VW, per_block = MAP_THREADS * UW;
        const uint32_t blocks = (uint32_t)((nvec + per_block - 1) / per_block);
        hipLaunchKernelGGL((map_contig_kernel<F, VW, UW>), dim3(blocks), dim3(MAP_THREADS), 0, ctx->stream, a);
      } else {
        const int64_t nvec = (p.total + V - 1) / V, per_block = MAP_THREADS * MAP_CONTIG_UNROLL;
        const uint32_t blocks = (uint32_t)((nvec + per_block - 1) / per_block);
        hipLaunchKernelGGL((map_contig_kernel<F, V, MAP_CONTIG_UNROLL>), dim3(blocks), dim3(MAP_THREADS), 0, ctx->stream, a);
      }
      NXH_HIP(op, hipGetLastError());
      return NXH_OK;
    }
  }
  // 2. an input whose unit-stride dim is not the output's: turn it through LDS
  const int last = p.ndim - 1;
  if (p.ndim >= 2 && p.stride[0][last] == 1 && p.shape[last] >= 16) {
    int ydim = -1;
    for (int k = 1; k < p.nop && ydim < 0; k++) {
      int64_t s = p.stride[k][last];
      if (s == 0 || s == 1) continue;
      for (int d = last - 1; d >= 0; d--)
        if (p.stride[k][d] == 1 && p.shape[d] >= 16) {
          ydim = d;
          break;
        }
    }
    if (ydim >= 0) {
      // A patch holds 8 KiB of the widest type (4 KiB for one-byte types): 64 x 32 elements of 4
      // bytes, 64 x 64 of 1 or 2, 32 x 32 of 8 or 16. Measured on [64,512,512] int32 / float32
      // with a permuted operand: 64 x 64 patches of 4-byte elements ran the config-2 step in
      // 172 us, 64 x 32 in 162 us (more blocks per compute unit, shorter dependent chains
      // through the barrier), 32 x 32 in 177 us, 128 x 64 with 16-byte stores of one-byte
      // results in 173 us; 128 x 32 patches for the one-byte results of a compare (whole
      // 128-byte rows per store) ran that call four times slower (15.8 -> 60.8 us; the cast of
      // a permuted int32 to int8 14.7 -> 46.6). The same compare on contiguous operands takes
      // 12.7-15.5 us, a permuted add with four-byte results 20.8 against 28.4 x 2/3 for a
      // contiguous one: the turn through LDS costs every tiled call about a tenth, and the
      // calls with narrow results show it most because they move the fewest bytes per element.
      constexpr int TX = MT::smax <= 4 ? 64 : 32;
      constexpr int TY = MT::smax == 4 ? 32 : (MT::smax < 4 ? 64 : 32);
      TiledArgs<F> a;
      a.any_turn = 0;
      a.stream = p.stream;
      bool every_mode = true;
      // 16-byte lanes need every vector of every operand aligned and whole
      bool vec = V > 1 && p.shape[last] % V == 0 && p.shape[ydim] % V == 0;
      for (int k = 0; k < MAP_MAXOP; k++) {
        a.base[k] = k < p.nop ? p.base[k] : nullptr;
        a.sx[k] = k < p.nop ? p.stride[k][last] : 0;
        a.sy[k] = k < p.nop ? p.stride[k][ydim] : 0;
        a.mode[k] = TILE_ROW;
        if (k >= p.nop) continue;
        if (a.sx[k] == 1) a.mode[k] = TILE_ROW;
        else if (a.sx[k] == 0) a.mode[k] = TILE_BX;
        else if (a.sy[k] == 1) a.mode[k] = TILE_TURN, a.any_turn = 1;
        else every_mode = false;  // strided along both: the per-lane index kernel takes it
        if (a.mode[k] == TILE_ROW || a.mode[k] == TILE_TURN) {
          if (!aligned_to(p.base[k], (size_t)esz[k] * V)) vec = false;
          for (int d = 0; d < p.ndim; d++)
            if (p.stride[k][d] != 1 && p.stride[k][d] % V != 0) vec = false;
        }
      }
      a.nx = (uint32_t)p.shape[last];
      a.ny = (uint32_t)p.shape[ydim];
      a.tiles_x = (a.nx + TX - 1) / TX;
      a.tiles_y = (a.ny + TY - 1) / TY;
      a.nbatch_dims = 0;
      int64_t nb = 1;
      for (int d = 0; d < last; d++) {
        if (d == ydim) continue;
        a.bshape[a.nbatch_dims] = (uint32_t)p.shape[d];
        for (int k = 0; k < MAP_MAXOP; k++)
          a.bstride[k][a.nbatch_dims] = k < p.nop ? p.stride[k][d] : 0;
        a.nbatch_dims++;
        nb *= p.shape[d];
      }
      int64_t blocks = nb * a.tiles_x * a.tiles_y;
      if (blocks < ((int64_t)1 << 31) && every_mode) {
        nxh_set_path("map_tiled");
        if (vec)
          hipLaunchKernelGGL((map_tiled_kernel<F, TX, TY, V>), dim3((uint32_t)blocks), dim3(MAP_THREADS), 0,
                             ctx->stream, a);
        else
          hipLaunchKernelGGL((map_tiled_kernel<F, TX, TY, 1>), dim3((uint32_t)blocks), dim3(MAP_THREADS), 0,
                             ctx->stream, a);
        NXH_HIP(op, hipGetLastError());
        return NXH_OK;
      }
    }
  }
  return map_launch_generic<F>(ctx, op, p);
}

// Splits plans that exceed one launch (rank > MAP_MAXD or >= 2^31 elements)
// along their outer dims.
template <class F>
static int map_launch(nxh_context *ctx, const char *op, const MapPlan &p) {
  if (p.total == 0) return NXH_OK;
  const int64_t LIM = ((int64_t)1 << 31) - 1;
  if (p.ndim <= MAP_MAXD && p.total <= LIM) return map_launch_one<F>(ctx, op, p);
  int64_t rest = p.total / p.shape[0];
  MapPlan q = p;
  if (p.ndim > 1 && (p.ndim > MAP_MAXD || rest > LIM)) {
    // peel dim 0 entirely
    q.ndim = p.ndim - 1;
    q.total = rest;
    for (int d = 0; d < q.ndim; d++) {
      q.shape[d] = p.shape[d + 1];
      for (int k = 0; k < p.nop; k++) q.stride[k][d] = p.stride[k][d + 1];
    }
    for (int64_t i = 0; i < p.shape[0]; i++) {
      for (int k = 0; k < p.nop; k++) q.base[k] = p.base[k] + i * p.stride[k][0] * p.esize[k];
      int rc = map_launch<F>(ctx, op, q);
      if (rc) return rc;
    }
    return NXH_OK;
  }
  // chunk dim 0
  int64_t chunk = std::max<int64_t>(1, LIM / std::max<int64_t>(rest, 1));
  if (p.ndim == 1) chunk = (int64_t)1 << 30;
  for (int64_t i = 0; i < p.shape[0]; i += chunk) {
    q.shape[0] = std::min(chunk, p.shape[0] - i);
    q.total = q.shape[0] * rest;
    for (int k = 0; k < p.nop; k++) q.base[k] = p.base[k] + i * p.stride[k][0] * p.esize[k];
    int rc = map_launch_one<F>(ctx, op, q);
    if (rc) return rc;
  }
  return NXH_OK;
}

typedef int (*map_launch_fn)(nxh_context *, const char *, const MapPlan &);
