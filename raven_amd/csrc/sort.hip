// sort.hip — sort and argsort along one axis (packages/nx/lib/backend_c/
// nx_c_sort.c).
//
// Order (nx_c_sort.c:46-112): each slice is compared in the dtype's compute
// type; NaN-class elements (either part of a complex) go last in both
// directions; complex is lexicographic (real, then imaginary). argsort breaks
// ties by the original index in both directions, so it is stable. The value
// sort of the reference is an unstable introsort whose descending result is the
// ascending finite prefix reversed (:283-289); elements that compare equal are
// indistinguishable except IEEE +-0, whose order it leaves open. Here every
// comparison is a TOTAL order on (class, value, index) — ties by ascending
// index, by descending index for the descending value sort (what reversing a
// stable ascending sort gives), NaN-class elements in index order — so the
// result is unique and a sorting network reproduces it whatever its exchange
// pattern.
//
// Algorithm: bitonic sorting network, the slice padded to a power of two with
// elements that sort last. Elements are (key, index) pairs for 64-bit and
// complex keys and one packed 64-bit word otherwise (see "packed keys").
//   sort_registers  packed slices of up to 4096 elements: the whole network in
//                registers, eight or sixteen elements a lane;
//   sort_lds     (key, index) slices of up to 4096 elements (2048 for 16-byte keys):
//                whole network in LDS, several short slices per block;
//   sort_global  longer slices of (key, index) pairs: staged in scratch memory;
//                chunks are sorted in LDS, then each merge level runs its
//                long-distance exchanges as passes over global memory and
//                finishes the short-distance ones in LDS;
//   sort_radix   longer slices of packed words: a stable radix sort over the key
//                half (see "a radix sort" below).

#include "fold_common.hpp"

namespace {

constexpr int SORT_MAXD = 12;
constexpr int32_t PAD_INDEX = 0x7fffffff;

enum SortMode { VALUE_ASC = 0, VALUE_DESC = 1, ARG_ASC = 2, ARG_DESC = 3 };

template <int DT>
struct Key {
  using TR = Tr<DT>;
  using C = typename TR::C;
  __device__ __forceinline__ static bool is_nan(C x) {
    if constexpr (TR::cat == CAT_FLOAT) return x != x;
    else if constexpr (TR::cat == CAT_COMPLEX) return x.re != x.re || x.im != x.im;
    else return false;
  }
  __device__ __forceinline__ static bool lt(C a, C b) {
    if constexpr (TR::cat == CAT_COMPLEX) return a.re < b.re || (a.re == b.re && a.im < b.im);
    else return a < b;
  }
  // (ka, ia) sorts strictly before (kb, ib)
  template <int MODE>
  __device__ __forceinline__ static bool before(C ka, int32_t ia, C kb, int32_t ib) {
    const int ca = ia == PAD_INDEX ? 2 : (is_nan(ka) ? 1 : 0);
    const int cb = ib == PAD_INDEX ? 2 : (is_nan(kb) ? 1 : 0);
    if (ca != cb) return ca < cb;
    if (ca == 2) return false;
    if (ca == 1) return ia < ib;
    const bool l = lt(ka, kb), g = lt(kb, ka);
    constexpr bool desc = MODE == VALUE_DESC || MODE == ARG_DESC;
    if (l != g) return desc ? g : l;
    return MODE == VALUE_DESC ? ia > ib : ia < ib;
  }
};

struct SortArgs {
  const char *in;
  char *out;
  void *keys;      // scratch (sort_global): slices * n_pad keys
  int32_t *index;  // scratch (sort_global): slices * n_pad indices
  int64_t slices, n, n_pad;
  int64_t in_axis, out_axis;  // strides along the sorted axis, elements
  int nk;
  int64_t kshape[SORT_MAXD], k_in[SORT_MAXD], k_out[SORT_MAXD];
};

__device__ __forceinline__ void slice_offsets(const SortArgs &a, int64_t s, int64_t &io, int64_t &oo) {
  io = 0;
  oo = 0;
  for (int d = a.nk - 1; d >= 0; d--) {
    const int64_t c = s % a.kshape[d];
    s /= a.kshape[d];
    io += c * a.k_in[d];
    oo += c * a.k_out[d];
  }
}

template <int DT>
constexpr int lds_elems() {
  return sizeof(typename Tr<DT>::C) > 8 ? 2048 : 4096;
}

// One compare-exchange step of distance j inside LDS over `count` elements;
// `up` tells the direction of element i's subsequence. `base` is added to a
// local position to get the position inside its slice (direction bits).
template <int DT, int MODE>
__device__ __forceinline__ void lds_step(typename Tr<DT>::C *k, int32_t *ix, int count, int j, int64_t kk,
                                         int64_t base, int64_t mask) {
  using K = Key<DT>;
  for (int p = threadIdx.x; p < count / 2; p += 256) {
    const int i = ((p & ~(j - 1)) << 1) | (p & (j - 1));
    const int l = i | j;
    const bool up = (((base + i) & mask) & kk) == 0;
    const auto ka = k[i], kb = k[l];
    const int32_t ia = ix[i], ib = ix[l];
    const bool swap = up ? K::template before<MODE>(kb, ib, ka, ia) : K::template before<MODE>(ka, ia, kb, ib);
    if (swap) {
      k[i] = kb;
      k[l] = ka;
      ix[i] = ib;
      ix[l] = ia;
    }
  }
  __syncthreads();
}

// Whole slices in LDS: a block holds `spb` slices of n_pad elements each.
template <int DT, int MODE>
__global__ __launch_bounds__(256) void sort_lds_kernel(SortArgs a, int spb) {
  using TR = Tr<DT>;
  using C = typename TR::C;
  using S = typename TR::S;
  constexpr int NL = lds_elems<DT>();
  __shared__ C k[NL];
  __shared__ int32_t ix[NL];
  const int np = (int)a.n_pad, count = spb * np;
  const int64_t first = (int64_t)blockIdx.x * spb;
  for (int e = threadIdx.x; e < count; e += 256) {
    const int64_t s = first + e / np;
    const int i = e % np;
    C key{};
    int32_t id = PAD_INDEX;
    if (s < a.slices && i < a.n) {
      int64_t io, oo;
      slice_offsets(a, s, io, oo);
      key = TR::ld(reinterpret_cast<const S *>(a.in)[io + i * a.in_axis]);
      id = i;
    }
    k[e] = key;
    ix[e] = id;
  }
  __syncthreads();
  for (int kk = 2; kk <= np; kk <<= 1)
    for (int j = kk >> 1; j >= 1; j >>= 1) lds_step<DT, MODE>(k, ix, count, j, kk, 0, np - 1);
  for (int e = threadIdx.x; e < count; e += 256) {
    const int64_t s = first + e / np;
    const int i = e % np;
    if (s < a.slices && i < a.n) {
      int64_t io, oo;
      slice_offsets(a, s, io, oo);
      if constexpr (MODE >= ARG_ASC) reinterpret_cast<int32_t *>(a.out)[oo + i * a.out_axis] = ix[e];
      else reinterpret_cast<S *>(a.out)[oo + i * a.out_axis] = TR::st(k[e]);
    }
  }
}

// sort_global, phase 0: gather the slices into scratch and sort each chunk of
// NL elements (all levels kk <= NL).
template <int DT, int MODE>
__global__ __launch_bounds__(256) void sort_chunks_kernel(SortArgs a) {
  using TR = Tr<DT>;
  using C = typename TR::C;
  using S = typename TR::S;
  constexpr int NL = lds_elems<DT>();
  __shared__ C k[NL];
  __shared__ int32_t ix[NL];
  const int64_t chunks = a.n_pad / NL;
  const int64_t s = blockIdx.x / chunks, base = (blockIdx.x % chunks) * NL;
  int64_t io, oo;
  slice_offsets(a, s, io, oo);
  for (int e = threadIdx.x; e < NL; e += 256) {
    const int64_t i = base + e;
    C key{};
    int32_t id = PAD_INDEX;
    if (i < a.n) {
      key = TR::ld(reinterpret_cast<const S *>(a.in)[io + i * a.in_axis]);
      id = (int32_t)i;
    }
    k[e] = key;
    ix[e] = id;
  }
  __syncthreads();
  for (int kk = 2; kk <= NL; kk <<= 1)
    for (int j = kk >> 1; j >= 1; j >>= 1) lds_step<DT, MODE>(k, ix, NL, j, kk, base, a.n_pad - 1);
  C *gk = reinterpret_cast<C *>(a.keys) + s * a.n_pad + base;
  int32_t *gi = a.index + s * a.n_pad + base;
  for (int e = threadIdx.x; e < NL; e += 256) {
    gk[e] = k[e];
    gi[e] = ix[e];
  }
}

// One long-distance exchange pass of level kk, distance j >= NL, over scratch.
template <int DT, int MODE>
__global__ __launch_bounds__(256) void sort_exchange_kernel(SortArgs a, int64_t kk, int64_t j) {
  using C = typename Tr<DT>::C;
  using K = Key<DT>;
  const int64_t half = a.n_pad / 2;
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= a.slices * half) return;
  const int64_t s = t / half, p = t % half;
  const int64_t i = ((p & ~(j - 1)) << 1) | (p & (j - 1)), l = i | j;
  C *gk = reinterpret_cast<C *>(a.keys) + s * a.n_pad;
  int32_t *gi = a.index + s * a.n_pad;
  const bool up = (i & kk) == 0;
  const C ka = gk[i], kb = gk[l];
  const int32_t ia = gi[i], ib = gi[l];
  const bool swap = up ? K::template before<MODE>(kb, ib, ka, ia) : K::template before<MODE>(ka, ia, kb, ib);
  if (swap) {
    gk[i] = kb;
    gk[l] = ka;
    gi[i] = ib;
    gi[l] = ia;
  }
}

// The short-distance steps (j < NL) of level kk, chunk by chunk in LDS. After
// the last level (`final`), the chunk goes to the output instead of scratch.
template <int DT, int MODE>
__global__ __launch_bounds__(256) void sort_merge_kernel(SortArgs a, int64_t kk, int final) {
  using TR = Tr<DT>;
  using C = typename TR::C;
  using S = typename TR::S;
  constexpr int NL = lds_elems<DT>();
  __shared__ C k[NL];
  __shared__ int32_t ix[NL];
  const int64_t chunks = a.n_pad / NL;
  const int64_t s = blockIdx.x / chunks, base = (blockIdx.x % chunks) * NL;
  C *gk = reinterpret_cast<C *>(a.keys) + s * a.n_pad + base;
  int32_t *gi = a.index + s * a.n_pad + base;
  for (int e = threadIdx.x; e < NL; e += 256) {
    k[e] = gk[e];
    ix[e] = gi[e];
  }
  __syncthreads();
  for (int j = NL >> 1; j >= 1; j >>= 1) lds_step<DT, MODE>(k, ix, NL, j, kk, base, a.n_pad - 1);
  if (!final) {
    for (int e = threadIdx.x; e < NL; e += 256) {
      gk[e] = k[e];
      gi[e] = ix[e];
    }
    return;
  }
  int64_t io, oo;
  slice_offsets(a, s, io, oo);
  for (int e = threadIdx.x; e < NL; e += 256) {
    const int64_t i = base + e;
    if (i < a.n) {
      if constexpr (MODE >= ARG_ASC) reinterpret_cast<int32_t *>(a.out)[oo + i * a.out_axis] = ix[e];
      else reinterpret_cast<S *>(a.out)[oo + i * a.out_axis] = TR::st(k[e]);
    }
  }
}

// ── packed keys ─────────────────────────────────────────────────────────────
// Dtypes whose compute-type value fits 32 bits (every float but f64, every
// integer up to 32 bits, bool) are sorted as ONE 64-bit word per element:
//   high half  the value mapped to an unsigned that ascends in sort order
//              (floats: sign-flipped bits with -0 folded onto +0; ints offset by
//              2^31; the whole half inverted for descending); 0xFFFFFFFE for a
//              NaN; 0xFFFFFFFF for padding;
//   low half   the original index (2^31 - 1 - index for the descending value
//              sort, whose ties go by descending index; NaNs always keep index
//              order). Indices stay below 2^30, so no element equals the padding.
// Unsigned order of the words is then exactly the total order above, one
// compare-exchange is a 64-bit min / max, and both halves of a pair are always
// written, so the network has no data-dependent branch.
template <int DT>
struct Packed {
  using TR = Tr<DT>;
  using C = typename TR::C;
  static constexpr bool ok = DT == NXH_F16 || DT == NXH_F32 || DT == NXH_BF16 || DT == NXH_F8E4M3 ||
                             DT == NXH_F8E5M2 || DT == NXH_I8 || DT == NXH_U8 || DT == NXH_I16 || DT == NXH_U16 ||
                             DT == NXH_I32 || DT == NXH_U32 || DT == NXH_BOOL;
  static constexpr uint32_t K_NAN = 0xFFFFFFFEu;
  template <int MODE>
  __device__ __forceinline__ static uint64_t pack(C x, uint32_t index) {
    constexpr bool desc = MODE == VALUE_DESC || MODE == ARG_DESC;
    uint32_t m;
    if constexpr (TR::cat == CAT_FLOAT) {
      if (x != x) return ((uint64_t)K_NAN << 32) | index;
      uint32_t u = __builtin_bit_cast(uint32_t, (float)x);
      if ((u << 1) == 0) u = 0;  // -0 and +0 compare equal
      m = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
    } else if constexpr (TR::cat == CAT_SINT) {
      m = (uint32_t)(int32_t)x ^ 0x80000000u;
    } else {
      m = (uint32_t)x;
    }
    if (desc) m = ~m;
    return ((uint64_t)m << 32) | (MODE == VALUE_DESC ? 0x7FFFFFFFu - index : index);
  }
  template <int MODE>
  __device__ __forceinline__ static uint32_t index_of(uint64_t w) {
    const uint32_t lo = (uint32_t)w;
    if constexpr (MODE == VALUE_DESC) {
      if (TR::cat != CAT_FLOAT || (uint32_t)(w >> 32) != K_NAN) return 0x7FFFFFFFu - lo;
    }
    return lo;
  }
};
constexpr uint64_t PACKED_PAD = ~(uint64_t)0;
template <int DT, int MODE>
__device__ __forceinline__ void packed_store(const SortArgs &a, int64_t oo, int64_t io, int64_t i, uint64_t word) {
  using TR = Tr<DT>;
  using S = typename TR::S;
  const uint32_t src = Packed<DT>::template index_of<MODE>(word);
  if constexpr (MODE >= ARG_ASC) reinterpret_cast<int32_t *>(a.out)[oo + i * a.out_axis] = (int32_t)src;
  else  // through the compute type, as the reference's gather-sort-scatter does (nx_c_sort.c:270-291)
    reinterpret_cast<S *>(a.out)[oo + i * a.out_axis] =
        TR::st(TR::ld(reinterpret_cast<const S *>(a.in)[io + (int64_t)src * a.in_axis]));
}

// Slices of up to 4096 padded elements: the whole network in registers. A lane holds E = 8
// consecutive elements of its slice (16 for slices of 4096), NP / E lanes a slice, 256 E / NP
// slices a block; slices shorter than 64 are padded to 64. Exchanges at distances below E stay
// inside the lane; distances E .. 32 E meet the lane 1 .. 32 places away through the cross-lane
// network, the lane keeping the smaller or the larger word of each pair; only distances of 64 E
// and more (the last one or three steps of the largest slices) go through LDS. No barrier and no LDS traffic in any other step, and the slice's offsets are worked out
// once per lane: [16384,1024] f32 along axis 1, 398 us with the network in LDS.
// The word of the lane m places away (lane ^ m). Distances 1, 2 and 8 are data-parallel moves
// inside the vector unit (the pairs of a quad swapped, a row of sixteen turned by eight); the others
// go through the cross-lane network of the LDS, which this kernel keeps busier than anything
// else (eight clocks a 32-bit move: with every distance there, [16384,1024] f32 took 168 us).
__device__ __forceinline__ uint64_t lane_xor64(uint64_t x, int m) {
  int lo = (int)(uint32_t)x, hi = (int)(uint32_t)(x >> 32);
  switch (m) {
    case 1:  // quad_perm:[1,0,3,2]
      lo = __builtin_amdgcn_update_dpp(0, lo, 0xB1, 0xF, 0xF, false);
      hi = __builtin_amdgcn_update_dpp(0, hi, 0xB1, 0xF, 0xF, false);
      break;
    case 2:  // quad_perm:[2,3,0,1]
      lo = __builtin_amdgcn_update_dpp(0, lo, 0x4E, 0xF, 0xF, false);
      hi = __builtin_amdgcn_update_dpp(0, hi, 0x4E, 0xF, 0xF, false);
      break;
    case 8:  // row_ror:8
      lo = __builtin_amdgcn_update_dpp(0, lo, 0x128, 0xF, 0xF, false);
      hi = __builtin_amdgcn_update_dpp(0, hi, 0x128, 0xF, 0xF, false);
      break;
    default:
      lo = __shfl_xor(lo, m, 64);
      hi = __shfl_xor(hi, m, 64);
  }
  return ((uint64_t)(uint32_t)hi << 32) | (uint32_t)lo;
}

template <int DT, int MODE, int LOGNP>
__global__ __launch_bounds__(256) void psort_reg_kernel(SortArgs a) {
  using TR = Tr<DT>;
  using S = typename TR::S;
  constexpr int NP = 1 << LOGNP, E = LOGNP >= 12 ? 16 : 8, TPS = NP / E, SPB = 256 / TPS;
  static_assert(TPS >= 1 && TPS <= 256, "a slice is held by one block");
  constexpr bool CROSS_WAVE = TPS > 64;
  __shared__ uint64_t xch[CROSS_WAVE ? 256 * E : 1];
  const int t = threadIdx.x % TPS;
  const int64_t s = (int64_t)blockIdx.x * SPB + threadIdx.x / TPS;
  const bool live = s < a.slices;
  int64_t io = 0, oo = 0;
  if (live) slice_offsets(a, s, io, oo);
  const S *in = reinterpret_cast<const S *>(a.in) + io;
  const int i0 = t * E;
  uint64_t e[E];
  if (live && a.in_axis == 1 && i0 + E <= a.n && ((uintptr_t)(in + i0) % alignof(FVec<S, E>)) == 0) {
    const FVec<S, E> x = *reinterpret_cast<const FVec<S, E> *>(in + i0);
#pragma unroll
    for (int r = 0; r < E; r++) e[r] = Packed<DT>::template pack<MODE>(TR::ld(x.v[r]), (uint32_t)(i0 + r));
  } else {
#pragma unroll
    for (int r = 0; r < E; r++)
      e[r] = live && i0 + r < a.n
                 ? Packed<DT>::template pack<MODE>(TR::ld(in[(int64_t)(i0 + r) * a.in_axis]), (uint32_t)(i0 + r))
                 : PACKED_PAD;
  }
#pragma unroll
  for (int lk = 1; lk <= LOGNP; lk++) {
    const int kk = 1 << lk;
#pragma unroll
    for (int lj = lk - 1; lj >= 0; lj--) {
      const int j = 1 << lj;
      if (j < E) {
#pragma unroll
        for (int r = 0; r < E; r++) {
          if (r & j) continue;
          // ascending run: the pair changes places when the second is smaller; descending: when
          // the first is (one comparison, the direction folded into its lane mask; equal words
          // are padding and may go either way)
          const bool down = ((i0 + r) & kk) != 0;
          const uint64_t x = e[r], y = e[r | j];
          const bool change = (y < x) != down;
          e[r] = change ? y : x;
          e[r | j] = change ? x : y;
        }
      } else {
        const int m = j / E;  // the partner lane's distance
        const bool keep_max = ((i0 & kk) == 0) != ((t & m) == 0);
        if (m >= 64) {
          if constexpr (CROSS_WAVE) {
            __syncthreads();
#pragma unroll
            for (int r = 0; r < E; r++) xch[r * 256 + threadIdx.x] = e[r];
            __syncthreads();
#pragma unroll
            for (int r = 0; r < E; r++) {
              const uint64_t y = xch[r * 256 + (threadIdx.x ^ m)];
              e[r] = ((y < e[r]) != keep_max) ? y : e[r];
            }
          }
        } else {
#pragma unroll
          for (int r = 0; r < E; r++) {
            const uint64_t y = lane_xor64(e[r], m);
            e[r] = ((y < e[r]) != keep_max) ? y : e[r];
          }
        }
      }
    }
  }
  // Values are fetched from the input by index, through the compute type (nx_c_sort.c:270-291);
  // every lane of the block has fetched before any stores, so a result may overwrite its input.
  uint32_t src[E];
  S val[E];
#pragma unroll
  for (int r = 0; r < E; r++) {
    src[r] = Packed<DT>::template index_of<MODE>(e[r]);
    if constexpr (MODE < ARG_ASC)
      if (live && i0 + r < a.n) val[r] = TR::st(TR::ld(in[(int64_t)src[r] * a.in_axis]));
  }
  __syncthreads();
  if (!live) return;
  if constexpr (MODE >= ARG_ASC) {
    int32_t *out = reinterpret_cast<int32_t *>(a.out) + oo;
    if (a.out_axis == 1 && i0 + E <= a.n && ((uintptr_t)(out + i0) % alignof(FVec<int32_t, E>)) == 0) {
      FVec<int32_t, E> o;
#pragma unroll
      for (int r = 0; r < E; r++) o.v[r] = (int32_t)src[r];
      *reinterpret_cast<FVec<int32_t, E> *>(out + i0) = o;
    } else {
#pragma unroll
      for (int r = 0; r < E; r++)
        if (i0 + r < a.n) out[(int64_t)(i0 + r) * a.out_axis] = (int32_t)src[r];
    }
  } else {
    S *out = reinterpret_cast<S *>(a.out) + oo;
    if (a.out_axis == 1 && i0 + E <= a.n && ((uintptr_t)(out + i0) % alignof(FVec<S, E>)) == 0) {
      FVec<S, E> o;
#pragma unroll
      for (int r = 0; r < E; r++) o.v[r] = val[r];
      *reinterpret_cast<FVec<S, E> *>(out + i0) = o;
    } else {
#pragma unroll
      for (int r = 0; r < E; r++)
        if (i0 + r < a.n) out[(int64_t)(i0 + r) * a.out_axis] = val[r];
    }
  }
}

// ── long slices of packed words: a radix sort ──────────────────────────────
// The network costs log^2 n passes over a slice that does not fit LDS; the packed words of
// such a slice are sorted least significant digit first instead, eight bits at a time, over
// the HIGH half only: the low half (the index) ascends with the position the words start at
// and every pass is stable, so words with equal high halves stay in index order. The
// descending value sort wants its ties in descending index order and its NaNs in ascending:
// it sorts ascending and writes the non-NaN prefix out reversed, which is how the reference
// defines it (nx_c_sort.c:283-289).
// One pass is four launches: a histogram of the digit per 4096-word tile, laid out bin by
// bin ([256][tiles], so that its exclusive scan is a tile's first output position for each
// digit), the scan in two levels (segments of 4096 entries, then the segment totals), and the
// scatter, in which every tile ranks its words stably: a wave owns 1024 consecutive words,
// takes them 64 at a time in order, finds for each lane the lanes with the same digit by
// eight ballots, and keeps a running count per digit; the waves' counts are then offset
// against each other. No inter-block waiting anywhere.
// Digits that cannot change the order are skipped: the low bits of a widened 16- or 8-bit
// float, and the sign-extension bytes of a narrow integer, are functions of higher bits.
constexpr int RX_TILE = 4096;
constexpr int RX_ROWS = RX_TILE / 256;
constexpr int RX_SEG = 4096;

template <int DT>
constexpr int rx_pass_mask() {  // bit p: the pass over bits 8p .. 8p+7 of the mapped value is needed
  switch (DT) {
    case NXH_BF16: case NXH_F8E4M3: case NXH_F8E5M2: return 0b1100;
    case NXH_F16: return 0b1110;
    case NXH_U8: case NXH_BOOL: return 0b0001;
    case NXH_I8: return 0b1001;
    case NXH_U16: return 0b0011;
    case NXH_I16: return 0b1011;
    default: return 0b1111;
  }
}

struct RadixArgs {
  const uint64_t *src;
  uint64_t *dst;
  uint32_t *hist;  // [slices][256 * nblk], bin-major; after the scans: exclusive inside its segment
  uint32_t *seg;   // [slices][nseg]: segment totals, then their exclusive scan
  int64_t slices, n;
  int nblk, nseg, shift;
};

__global__ __launch_bounds__(256) void rx_zero_kernel(uint32_t *p, int64_t count) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < count) p[i] = 0;
}

// Packs the slices into words (position = index); counts the NaN words of each slice.
template <int DT, int PM, bool COUNT_NAN>
__global__ __launch_bounds__(256) void rx_pack_kernel(SortArgs a, uint64_t *w, uint32_t *nan_count, int nblk) {
  using TR = Tr<DT>;
  using S = typename TR::S;
  const int64_t s = blockIdx.x / nblk, base = (int64_t)(blockIdx.x % nblk) * RX_TILE;
  int64_t io, oo;
  slice_offsets(a, s, io, oo);
  uint32_t nans = 0;
  for (int e = threadIdx.x; e < RX_TILE; e += 256) {
    const int64_t i = base + e;
    if (i >= a.n) break;
    const uint64_t word = Packed<DT>::template pack<PM>(TR::ld(reinterpret_cast<const S *>(a.in)[io + i * a.in_axis]), (uint32_t)i);
    w[s * a.n + i] = word;
    nans += (uint32_t)(word >> 32) == Packed<DT>::K_NAN && TR::cat == CAT_FLOAT;
  }
  if constexpr (COUNT_NAN) {
    if (TR::cat == CAT_FLOAT && nans) atomicAdd(nan_count + s, nans);
  }
}

__global__ __launch_bounds__(256) void rx_hist_kernel(RadixArgs r) {
  __shared__ uint32_t h[256];
  const int64_t s = blockIdx.x / r.nblk;
  const int blk = (int)(blockIdx.x % r.nblk);
  h[threadIdx.x] = 0;
  __syncthreads();
  const uint64_t *src = r.src + s * r.n;
  for (int e = threadIdx.x; e < RX_TILE; e += 256) {
    const int64_t i = (int64_t)blk * RX_TILE + e;
    if (i < r.n) atomicAdd(&h[(uint32_t)(src[i] >> r.shift) & 255u], 1u);
  }
  __syncthreads();
  r.hist[s * 256 * r.nblk + (int64_t)threadIdx.x * r.nblk + blk] = h[threadIdx.x];
}

// Exclusive scan of 256 per-thread values across the block; returns this thread's offset and
// the block total. `tmp` holds 4 words.
__device__ __forceinline__ uint32_t rx_block_scan(uint32_t v, uint32_t *tmp, uint32_t &total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  uint32_t inc = v;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const uint32_t o = (uint32_t)__shfl_up((int)inc, d, 64);
    if (lane >= d) inc += o;
  }
  if (lane == 63) tmp[wave] = inc;
  __syncthreads();
  uint32_t before = 0;
  for (int w = 0; w < wave; w++) before += tmp[w];
  total = tmp[0] + tmp[1] + tmp[2] + tmp[3];
  __syncthreads();
  return before + inc - v;
}

// Level one of the scan: every segment of RX_SEG histogram entries in place, its total to `seg`.
__global__ __launch_bounds__(256) void rx_scan_segments_kernel(RadixArgs r) {
  __shared__ uint32_t tmp[4];
  const int64_t s = blockIdx.x / r.nseg;
  const int g = (int)(blockIdx.x % r.nseg);
  const int64_t len = (int64_t)256 * r.nblk;
  uint32_t *h = r.hist + s * len;
  constexpr int PER = RX_SEG / 256;
  const int64_t first = (int64_t)g * RX_SEG + (int64_t)threadIdx.x * PER;
  uint32_t v[PER], sum = 0;
#pragma unroll
  for (int k = 0; k < PER; k++) {
    v[k] = first + k < len ? h[first + k] : 0;
    sum += v[k];
  }
  uint32_t total;
  uint32_t run = rx_block_scan(sum, tmp, total);
#pragma unroll
  for (int k = 0; k < PER; k++) {
    if (first + k < len) h[first + k] = run;
    run += v[k];
  }
  if (threadIdx.x == 0) r.seg[s * r.nseg + g] = total;
}

// Level two: the segment totals of a slice, one block per slice.
__global__ __launch_bounds__(256) void rx_scan_totals_kernel(RadixArgs r) {
  __shared__ uint32_t tmp[4];
  uint32_t *t = r.seg + (int64_t)blockIdx.x * r.nseg;
  uint32_t carry = 0;
  for (int base = 0; base < r.nseg; base += 256) {
    const int i = base + threadIdx.x;
    const uint32_t v = i < r.nseg ? t[i] : 0;
    uint32_t total;
    const uint32_t off = rx_block_scan(v, tmp, total);
    if (i < r.nseg) t[i] = carry + off;
    carry += total;
  }
}

__global__ __launch_bounds__(256) void rx_scatter_kernel(RadixArgs r) {
  __shared__ uint64_t sorted[RX_TILE];  // the tile in digit order, so that lanes next to each other write next to each other
  __shared__ uint32_t cnt[4][256];
  __shared__ uint32_t base[256];   // first output position of this tile's words with digit d
  __shared__ uint32_t first[256];  // first position inside the tile of those words
  __shared__ uint32_t tmp[4];
  const int64_t s = blockIdx.x / r.nblk;
  const int blk = (int)(blockIdx.x % r.nblk);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int w = 0; w < 4; w++) cnt[w][threadIdx.x] = 0;
  {
    const int64_t at = (int64_t)threadIdx.x * r.nblk + blk;  // this tile's entry for digit threadIdx.x
    base[threadIdx.x] = r.hist[s * 256 * r.nblk + at] + r.seg[s * r.nseg + at / RX_SEG];
  }
  __syncthreads();
  const uint64_t *src = r.src + s * r.n;
  uint64_t *dst = r.dst + s * r.n;
  const int64_t tile0 = (int64_t)blk * RX_TILE;
  const int64_t i0 = tile0 + wave * (RX_ROWS * 64) + lane;
  uint64_t w[RX_ROWS];
  uint32_t rk[RX_ROWS];
#pragma unroll
  for (int q = 0; q < RX_ROWS; q++) {
    const int64_t i = i0 + q * 64;
    w[q] = i < r.n ? src[i] : ~(uint64_t)0;
  }
  const uint64_t lower = ((uint64_t)1 << lane) - 1;
#pragma unroll
  for (int q = 0; q < RX_ROWS; q++) {
    const bool valid = i0 + q * 64 < r.n;
    const uint32_t d = (uint32_t)(w[q] >> r.shift) & 255u;
    uint64_t same = __builtin_amdgcn_ballot_w64(valid);
#pragma unroll
    for (int b = 0; b < 8; b++) {
      const bool bit = (d >> b) & 1u;
      const uint64_t bal = __builtin_amdgcn_ballot_w64(bit);
      same &= bit ? bal : ~bal;
    }
    const uint32_t below = (uint32_t)__builtin_popcountll(same & lower);
    const uint32_t prev = cnt[wave][d];
    rk[q] = prev + below;
    // the first lane of each group of equal digits moves the wave's count on (LDS serves a wave in order)
    if (valid && below == 0) cnt[wave][d] = prev + (uint32_t)__builtin_popcountll(same);
  }
  __syncthreads();
  uint32_t mine;
  {
    const uint32_t c0 = cnt[0][threadIdx.x], c1 = cnt[1][threadIdx.x], c2 = cnt[2][threadIdx.x], c3 = cnt[3][threadIdx.x];
    cnt[0][threadIdx.x] = 0;
    cnt[1][threadIdx.x] = c0;
    cnt[2][threadIdx.x] = c0 + c1;
    cnt[3][threadIdx.x] = c0 + c1 + c2;
    mine = c0 + c1 + c2 + c3;
  }
  uint32_t total;
  first[threadIdx.x] = rx_block_scan(mine, tmp, total);  // (its barriers also publish cnt)
  __syncthreads();
#pragma unroll
  for (int q = 0; q < RX_ROWS; q++) {
    if (i0 + q * 64 < r.n) {
      const uint32_t d = (uint32_t)(w[q] >> r.shift) & 255u;
      sorted[first[d] + cnt[wave][d] + rk[q]] = w[q];
    }
  }
  __syncthreads();
  const int count = (int)(r.n - tile0 < RX_TILE ? r.n - tile0 : RX_TILE);
#pragma unroll
  for (int q = 0; q < RX_ROWS; q++) {
    const int p = q * 256 + threadIdx.x;
    if (p < count) {
      const uint64_t word = sorted[p];
      const uint32_t d = (uint32_t)(word >> r.shift) & 255u;
      dst[base[d] + ((uint32_t)p - first[d])] = word;
    }
  }
}

// Writes the sorted words out: indices, or the values they point at. DESC_VALUES: the
// non-NaN prefix reversed.
template <int DT, int PM, bool DESC_VALUES>
__global__ __launch_bounds__(256) void rx_unpack_kernel(SortArgs a, const uint64_t *w, const uint32_t *nan_count, int nblk) {
  const int64_t s = blockIdx.x / nblk, base = (int64_t)(blockIdx.x % nblk) * RX_TILE;
  int64_t io, oo;
  slice_offsets(a, s, io, oo);
  const int64_t reals = DESC_VALUES ? a.n - (int64_t)nan_count[s] : 0;
  for (int e = threadIdx.x; e < RX_TILE; e += 256) {
    const int64_t i = base + e;
    if (i >= a.n) break;
    const int64_t from = DESC_VALUES && i < reals ? reals - 1 - i : i;
    const uint64_t word = w[s * a.n + from];
    if constexpr (PM == VALUE_ASC) {
      // The value is the mapped key read backwards; only a zero (both signs share a key) and a
      // NaN (its payload is not in the key) are fetched from the input through the index. A
      // gather for every element cost a third of the whole sort.
      using TR = Tr<DT>;
      using C = typename TR::C;
      using S = typename TR::S;
      const uint32_t m = (uint32_t)(word >> 32);
      bool direct = true;
      C x;
      if constexpr (TR::cat == CAT_FLOAT) {
        direct = m != Packed<DT>::K_NAN && m != 0x80000000u;
        const uint32_t u = (m & 0x80000000u) ? m ^ 0x80000000u : ~m;
        x = (C)__builtin_bit_cast(float, u);
      } else if constexpr (TR::cat == CAT_SINT) {
        x = (C)(int32_t)(m ^ 0x80000000u);
      } else {
        x = (C)m;
      }
      if (direct) {
        reinterpret_cast<S *>(a.out)[oo + i * a.out_axis] = TR::st(x);
        continue;
      }
    }
    packed_store<DT, PM>(a, oo, io, i, word);
  }
}

template <int DT, int MODE>
int radix_run(nxh_context *ctx, const char *op, SortArgs &a) {
  constexpr int PM = MODE == VALUE_DESC ? VALUE_ASC : MODE;
  constexpr bool DESC_VALUES = MODE == VALUE_DESC;
  const int64_t nblk = (a.n + RX_TILE - 1) / RX_TILE, len = 256 * nblk, nseg = (len + RX_SEG - 1) / RX_SEG;
  if (a.slices * nblk > 0x7fffffffLL || a.slices * nseg > 0x7fffffffLL || nblk > 0x7fffffffLL / 256)
    return nxh_fail(NXH_FAILURE, op, "too many elements for one launch");
  auto up = [](size_t b) { return (b + 255) / 256 * 256; };
  const size_t words = up((size_t)(a.slices * a.n) * sizeof(uint64_t));
  const size_t hist = up((size_t)(a.slices * len) * sizeof(uint32_t)), seg = up((size_t)(a.slices * nseg) * sizeof(uint32_t));
  const size_t nans = up((size_t)a.slices * sizeof(uint32_t));
  Scratch scratch(ctx);
  if (scratch.get(0, 2 * words + hist + seg + nans)) return nxh_fail(NXH_FAILURE, op, NXH_ERR_ALLOC);
  char *p = (char *)scratch.p[0];
  uint64_t *w0 = (uint64_t *)p, *w1 = (uint64_t *)(p + words);
  RadixArgs r{};
  r.hist = (uint32_t *)(p + 2 * words);
  r.seg = (uint32_t *)(p + 2 * words + hist);
  uint32_t *nan_count = (uint32_t *)(p + 2 * words + hist + seg);
  r.slices = a.slices;
  r.n = a.n;
  r.nblk = (int)nblk;
  r.nseg = (int)nseg;
  const dim3 tiles((unsigned)(a.slices * nblk)), block(256);
  nxh_set_path("sort_radix");
  if (DESC_VALUES)
    hipLaunchKernelGGL(rx_zero_kernel, dim3((unsigned)((a.slices + 255) / 256)), block, 0, ctx->stream, nan_count, a.slices);
  hipLaunchKernelGGL((rx_pack_kernel<DT, PM, DESC_VALUES>), tiles, block, 0, ctx->stream, a, w0, nan_count, (int)nblk);
  uint64_t *src = w0, *dst = w1;
  for (int pass = 0; pass < 4; pass++) {
    if (!(rx_pass_mask<DT>() >> pass & 1)) continue;
    r.src = src;
    r.dst = dst;
    r.shift = 32 + 8 * pass;
    hipLaunchKernelGGL(rx_hist_kernel, tiles, block, 0, ctx->stream, r);
    hipLaunchKernelGGL(rx_scan_segments_kernel, dim3((unsigned)(a.slices * nseg)), block, 0, ctx->stream, r);
    hipLaunchKernelGGL(rx_scan_totals_kernel, dim3((unsigned)a.slices), block, 0, ctx->stream, r);
    hipLaunchKernelGGL(rx_scatter_kernel, tiles, block, 0, ctx->stream, r);
    std::swap(src, dst);
  }
  hipLaunchKernelGGL((rx_unpack_kernel<DT, PM, DESC_VALUES>), tiles, block, 0, ctx->stream, a, src, nan_count, (int)nblk);
  NXH_HIP(op, hipGetLastError());
  return NXH_OK;
}

template <int DT, int MODE>
int psort_run(nxh_context *ctx, const char *op, SortArgs &a) {
  if (a.n_pad <= 4096) {
    const int64_t np = std::max<int64_t>(a.n_pad, 64);
    const int64_t spb = np == 4096 ? 1 : 2048 / np, blocks = (a.slices + spb - 1) / spb;
    if (blocks > 0x7fffffffLL) return nxh_fail(NXH_FAILURE, op, "too many slices for one launch");
    nxh_set_path("sort_registers");
    const dim3 grid((unsigned)blocks), block(256);
    switch (np) {
      case 64: hipLaunchKernelGGL((psort_reg_kernel<DT, MODE, 6>), grid, block, 0, ctx->stream, a); break;
      case 128: hipLaunchKernelGGL((psort_reg_kernel<DT, MODE, 7>), grid, block, 0, ctx->stream, a); break;
      case 256: hipLaunchKernelGGL((psort_reg_kernel<DT, MODE, 8>), grid, block, 0, ctx->stream, a); break;
      case 512: hipLaunchKernelGGL((psort_reg_kernel<DT, MODE, 9>), grid, block, 0, ctx->stream, a); break;
      case 1024: hipLaunchKernelGGL((psort_reg_kernel<DT, MODE, 10>), grid, block, 0, ctx->stream, a); break;
      case 2048: hipLaunchKernelGGL((psort_reg_kernel<DT, MODE, 11>), grid, block, 0, ctx->stream, a); break;
      default: hipLaunchKernelGGL((psort_reg_kernel<DT, MODE, 12>), grid, block, 0, ctx->stream, a); break;
    }
    NXH_HIP(op, hipGetLastError());
    return NXH_OK;
  }
  return radix_run<DT, MODE>(ctx, op, a);
}

template <int DT, int MODE>
int sort_run(nxh_context *ctx, const char *op, SortArgs &a) {
  using C = typename Tr<DT>::C;
  constexpr int NL = lds_elems<DT>();
  if constexpr (Packed<DT>::ok) return psort_run<DT, MODE>(ctx, op, a);
  if (a.n_pad <= NL) {
    // several short slices per block, at least 1024 elements of work
    int spb = (int)std::max<int64_t>(1, std::min<int64_t>(NL, 1024) / a.n_pad);
    if (spb > a.slices) spb = (int)a.slices;
    const int64_t blocks = (a.slices + spb - 1) / spb;
    if (blocks > 0x7fffffffLL) return nxh_fail(NXH_FAILURE, op, "too many slices for one launch");
    nxh_set_path("sort_lds");
    hipLaunchKernelGGL((sort_lds_kernel<DT, MODE>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, a, spb);
    NXH_HIP(op, hipGetLastError());
    return NXH_OK;
  }
  const int64_t chunks = a.n_pad / NL, blocks = a.slices * chunks;
  const int64_t pairs = a.slices * (a.n_pad / 2);
  if (blocks > 0x7fffffffLL || (pairs + 255) / 256 > 0x7fffffffLL)
    return nxh_fail(NXH_FAILURE, op, "too many elements for one launch");
  Scratch scratch(ctx);
  int rc = scratch.get(0, (size_t)(a.slices * a.n_pad) * sizeof(C));
  if (!rc) rc = scratch.get(1, (size_t)(a.slices * a.n_pad) * sizeof(int32_t));
  if (rc) return nxh_fail(NXH_FAILURE, op, NXH_ERR_ALLOC);
  a.keys = scratch.p[0];
  a.index = (int32_t *)scratch.p[1];
  nxh_set_path("sort_global");
  hipLaunchKernelGGL((sort_chunks_kernel<DT, MODE>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, a);
  for (int64_t kk = 2 * (int64_t)NL; kk <= a.n_pad; kk <<= 1) {
    for (int64_t j = kk >> 1; j >= NL; j >>= 1)
      hipLaunchKernelGGL((sort_exchange_kernel<DT, MODE>), dim3((unsigned)((pairs + 255) / 256)), dim3(256), 0,
                         ctx->stream, a, kk, j);
    hipLaunchKernelGGL((sort_merge_kernel<DT, MODE>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, a, kk,
                       kk == a.n_pad ? 1 : 0);
  }
  NXH_HIP(op, hipGetLastError());
  return NXH_OK;
}

typedef int (*sort_fn)(nxh_context *, const char *, SortArgs &);
struct SortTable {
  sort_fn fn[NXH_DTYPE_COUNT][4] = {};
  template <int DT>
  void set() {
    fn[DT][VALUE_ASC] = &sort_run<DT, VALUE_ASC>;
    fn[DT][VALUE_DESC] = &sort_run<DT, VALUE_DESC>;
    fn[DT][ARG_ASC] = &sort_run<DT, ARG_ASC>;
    fn[DT][ARG_DESC] = &sort_run<DT, ARG_DESC>;
  }
  SortTable() {
#define NXH_ST(DT) set<DT>();
    NXH_FOR_COMPUTE_DTYPES(NXH_ST)
#undef NXH_ST
  }
};

int sort_entry(nxh_context *ctx, const char *op, const nxh_tensor *out, const nxh_tensor *x, int axis,
               int descending, bool is_arg) {
  if (!ctx || !out || !x) return nxh_fail(NXH_INVALID_ARGUMENT, op, "null argument");
  int rc = nxh_check_tensor(op, out);
  if (!rc) rc = nxh_check_tensor(op, x);
  if (rc) return rc;
  const int dt = x->dtype;
  if (nxh_is_packed(dt)) return nxh_fail(NXH_FAILURE, op, NXH_ERR_PACKED);
  if (out->dtype != (is_arg ? NXH_I32 : dt)) return nxh_fail(NXH_FAILURE, op, NXH_ERR_UNSUPPORTED);
  if (axis < 0 || axis >= x->ndim) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_AXIS);
  if (out->ndim != x->ndim) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_OUT_RANK);
  for (int d = 0; d < x->ndim; d++)
    if (out->shape[d] != x->shape[d]) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
  SortArgs a;
  a.n = x->shape[axis];
  // indices are int32 (nx_c_sort.c:41-43); the value sort carries them too
  if (a.n > ((int64_t)1 << 30))
    return nxh_fail(NXH_FAILURE, op, is_arg ? "argsort axis length exceeds INT32_MAX" : "sort axis longer than 2^30 elements");
  a.slices = 1;
  a.nk = 0;
  for (int d = 0; d < x->ndim; d++) {
    if (d == axis) continue;
    a.slices *= x->shape[d];
    if (x->shape[d] == 1) continue;
    if (a.nk == SORT_MAXD) return nxh_fail(NXH_FAILURE, op, "more than 12 dimensions beside the sorted axis");
    a.kshape[a.nk] = x->shape[d];
    a.k_in[a.nk] = x->strides[d];
    a.k_out[a.nk] = out->strides[d];
    a.nk++;
  }
  if (a.slices == 0 || a.n == 0) return NXH_OK;
  for (int d = 0; d < x->ndim; d++)
    if (x->shape[d] > 1 && out->strides[d] == 0) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_OUT_ALIASED);
  a.n_pad = 2;
  while (a.n_pad < a.n) a.n_pad <<= 1;
  a.in_axis = x->strides[axis];
  a.out_axis = out->strides[axis];
  a.in = (const char *)x->data + x->offset * (int64_t)nxh_elem_size(dt);
  a.out = (char *)out->data + out->offset * (int64_t)nxh_elem_size(out->dtype);
  a.keys = nullptr;
  a.index = nullptr;
  static const SortTable table;
  const int mode = (is_arg ? 2 : 0) + (descending ? 1 : 0);
  if (!table.fn[dt][mode]) return nxh_fail(NXH_FAILURE, op, NXH_ERR_UNSUPPORTED);
  std::lock_guard<std::mutex> guard(ctx->mu);
  NXH_HIP(op, hipSetDevice(ctx->device));
  return table.fn[dt][mode](ctx, op, a);
}

}  // namespace

NXH_EXPORT int nxh_sort(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x, int axis, int descending) {
  NXH_DEFER_BARRIER(ctx, out);
  return sort_entry(ctx, "sort", out, x, axis, descending, false);
}
NXH_EXPORT int nxh_argsort(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x, int axis, int descending) {
  NXH_DEFER_BARRIER(ctx, out);
  return sort_entry(ctx, "argsort", out, x, axis, descending, true);
}
