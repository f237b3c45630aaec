// arg.hip — argmax / argmin along one axis, int32 indices.
//
// Semantics restate packages/nx/lib/backend_c/nx_c_fold.c:93-101, 180-198: a
// strictly better value displaces the running best, a NaN displaces a non-NaN,
// and among equal candidates the smallest index wins. Two launch forms:
//   arg_row   the axis is walked by a group of lanes per output (a wave for short
//             rows, a 256-lane block for long ones; 16-byte loads when the axis has
//             unit stride); long rows with few outputs are split into chunks and
//             finished by a second pass over (value, index) partials.
//   arg_col   a kept dim is the unit-stride one: lanes own adjacent columns and
//             row groups of a block walk interleaved rows; splits as above.

#include "fold_common.hpp"

// ── argmax / argmin (nx_c_fold.c:93-101, 180-198) ──────────────────────────
// `beats(v, b)`: v displaces the running best b. Strict, and a NaN displaces a
// non-NaN, so among equal candidates the smaller index is kept explicitly.
template <bool IS_MIN, class C, Cat cat>
struct ArgCmp {
  __device__ __forceinline__ static bool beats(C v, C b) {
    if constexpr (cat == CAT_FLOAT) {
      if constexpr (IS_MIN) return (v < b) || ((v != v) && !(b != b));
      else return (v > b) || ((v != v) && !(b != b));
    } else {
      if constexpr (IS_MIN) return v < b;
      else return v > b;
    }
  }
  static constexpr Cat category = cat;
  // strictly better, no NaN rule (a NaN on either side: false)
  __device__ __forceinline__ static bool better(C v, C b) {
    if constexpr (IS_MIN) return v < b;
    else return v > b;
  }
  // the value nothing is worse than
  __device__ __forceinline__ static C worst() {
    if constexpr (cat == CAT_FLOAT) return IS_MIN ? (C)__builtin_inff() : (C)(-__builtin_inff());
    else if constexpr (std::is_signed<C>::value) return IS_MIN ? (C)INT64_MAX : (C)INT64_MIN;
    else return IS_MIN ? (C)UINT64_MAX : (C)0;
  }
  // merge two (value, index) candidates; index < 0 means "none yet". Written as
  // selects on one predicate: an if-statement form of this function compiled
  // (hipcc 7.2, gfx950, several candidates per lane) to code that never took
  // the update for float candidates.
  template <class I>
  __device__ __forceinline__ static void merge(C &bv, I &bi, C v, I i) {
    const bool take = (int)(i >= 0) & ((int)(bi < 0) | (int)beats(v, bv) | ((int)!beats(bv, v) & (int)(i < bi)));
    bv = take ? v : bv;
    bi = take ? i : bi;
  }
};

struct ArgArgs {
  const void *in;         // values (storage-typed first pass, compute-typed second)
  const int32_t *in_idx;  // second pass only: index carried by each partial
  void *out_val;          // first pass with nsplit > 1: partial values (compute-typed)
  int32_t *out_idx;       // int32 result, or partial indices
  FoldDims kept;          // row form: all kept dims; col form: kept dims other than the lane
  uint64_t n_out;
  int64_t R, r_stride;
  int64_t chunk;
  int nsplit;
  uint32_t L, lane_blocks;  // col form
  int64_t out_lane_stride;
};

// A lane meets its candidates in ascending index order, so only a strictly
// better one (or the first) replaces its running best.
template <class CMP, class C, class I>
__device__ __forceinline__ void arg_take(C &bv, I &bi, C v, I i) {
  const bool take = (bi < 0) | CMP::beats(v, bv);
  bv = take ? v : bv;
  bi = take ? i : bi;
}

// Row form: a group of G lanes per output walks the axis. V > 1 (unit axis
// stride, aligned rows, no carried indices): 16-byte loads, four in flight.
template <class IN, class CMP, int G, int V, bool HAS_IDX>
__global__ __launch_bounds__(FOLD_THREADS) void arg_row_kernel(ArgArgs a) {
  using T = typename IN::T;
  using C = typename IN::C;
  static_assert(V == 1 || !HAS_IDX, "carried indices are read one at a time");
  __shared__ C lv[4];
  __shared__ int64_t li[4];
  constexpr int GROUPS = FOLD_THREADS / G;
  const int lane = threadIdx.x % G;
  // blocks walk the input from its end: the tail of a tensor that was just
  // written front to back is still in the memory-side cache
  const uint64_t o = (uint64_t)(gridDim.x - 1 - blockIdx.x) * GROUPS + threadIdx.x / G;
  const bool live = o < a.n_out;
  const int c = gridDim.y - 1 - blockIdx.y;
  int64_t in_off = 0, out_off = 0;
  if (live) fold_decode(a.kept, o, in_off, out_off);
  const int64_t r0 = (int64_t)c * a.chunk;
  const int64_t r1 = live ? (r0 + a.chunk < a.R ? r0 + a.chunk : a.R) : r0;
  const T *p = (const T *)a.in + in_off;
  C bv{};
  int64_t bi = -1;
  if constexpr (V > 1) {
    const int64_t nv = (r1 - r0) / V;
    const FVec<T, V> *pv = reinterpret_cast<const FVec<T, V> *>(p + r0);
    int64_t i = lane;
    for (; i + 3 * G < nv; i += 4 * G) {
      FVec<T, V> x[4];
#pragma unroll
      for (int j = 0; j < 4; j++) x[j] = pv[i + j * G];
#pragma unroll
      for (int j = 0; j < 4; j++)
#pragma unroll
        for (int k = 0; k < V; k++) arg_take<CMP, C>(bv, bi, IN::ld(x[j].v[k]), r0 + (i + j * G) * V + k);
    }
    for (; i < nv; i += G) {
      FVec<T, V> x = pv[i];
#pragma unroll
      for (int k = 0; k < V; k++) arg_take<CMP, C>(bv, bi, IN::ld(x.v[k]), r0 + i * V + k);
    }
    for (int64_t r = r0 + nv * V + lane; r < r1; r += G) arg_take<CMP, C>(bv, bi, IN::ld(p[r]), r);
  } else {
    for (int64_t r = r0 + lane; r < r1; r += G) {
      C v = IN::ld(p[r * a.r_stride]);
      int64_t idx = HAS_IDX ? (int64_t)a.in_idx[in_off + r * a.r_stride] : r;
      CMP::merge(bv, bi, v, idx);
    }
  }
#pragma unroll
  for (int d = G < 64 ? G / 2 : 32; d >= 1; d >>= 1) {
    C ov = shfl_down_any(bv, d);
    int64_t oi = shfl_down_any(bi, d);
    CMP::merge(bv, bi, ov, oi);
  }
  if constexpr (G == 256) {
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) {
      lv[wave] = bv;
      li[wave] = bi;
    }
    __syncthreads();
    if (threadIdx.x == 0)
      for (int w = 1; w < 4; w++) CMP::merge(bv, bi, lv[w], li[w]);
  }
  if (live && lane == 0) {
    if (a.nsplit > 1) {
      ((C *)a.out_val)[o * a.nsplit + c] = bv;
      a.out_idx[o * a.nsplit + c] = (int32_t)bi;
    } else {
      a.out_idx[out_off] = (int32_t)bi;
    }
  }
}

// Column form: LANES = 256 / RG column lanes (V adjacent columns each) by RG row
// groups, as in fold_col; every column keeps its own (value, index) candidate.
template <class IN, class CMP, int V, int RG, bool HAS_IDX>
__global__ __launch_bounds__(FOLD_THREADS) void arg_col_kernel(ArgArgs a) {
  using T = typename IN::T;
  using C = typename IN::C;
  static_assert(V == 1 || !HAS_IDX, "carried indices are read one at a time");
  constexpr int LANES = FOLD_THREADS / RG;
  constexpr int U = HAS_IDX ? 4 : 8;  // loads in flight per lane
  using I = int32_t;               // row indices fit the int32 result
  __shared__ C lv[RG > 1 ? (RG - 1) * LANES * V : 1];
  __shared__ int32_t li[RG > 1 ? (RG - 1) * LANES * V : 1];
  const uint32_t bx = gridDim.x - 1 - blockIdx.x;  // from the end, as in arg_row_kernel
  const uint32_t lb = bx % a.lane_blocks;
  const uint64_t ob = bx / a.lane_blocks;
  const int c = gridDim.y - 1 - blockIdx.y;
  const uint32_t ln = threadIdx.x % LANES, rg = threadIdx.x / LANES;
  const uint32_t l = (lb * LANES + ln) * V;
  const bool live = l < a.L;
  int64_t in_off, out_off;
  fold_decode(a.kept, ob, in_off, out_off);
  const int64_t r0 = (int64_t)c * a.chunk;
  const int64_t r1 = live ? (r0 + a.chunk < a.R ? r0 + a.chunk : a.R) : r0;
  const T *p = (const T *)a.in + in_off + l;
  C bv[V];
  I bi[V];
  int64_t r = r0 + rg;
  if constexpr (!HAS_IDX && (CMP::category == CAT_FLOAT || CMP::category == CAT_SINT || CMP::category == CAT_UINT)) {
    // The first pass over plain values, three instructions per element: the running best
    // starts at the worst value there is with the lane's first row as its index, so "strictly
    // better" alone decides (equal values keep the earlier row). A NaN never compares better
    // and is only noted; a lane that met one (rare) walks its rows again by the full rule below.
    const I first = r < r1 ? (I)r : (I)-1;
#pragma unroll
    for (int k = 0; k < V; k++) bv[k] = CMP::worst(), bi[k] = first;
    bool odd = false;
    for (; r + (U - 1) * RG < r1; r += U * RG) {
      FVec<T, V> x[U];
#pragma unroll
      for (int j = 0; j < U; j++) x[j] = *reinterpret_cast<const FVec<T, V> *>(p + (r + j * RG) * a.r_stride);
#pragma unroll
      for (int j = 0; j < U; j++)
#pragma unroll
        for (int k = 0; k < V; k++) {
          const C v = IN::ld(x[j].v[k]);
          const bool take = CMP::better(v, bv[k]);
          bv[k] = take ? v : bv[k];
          bi[k] = take ? (I)(r + j * RG) : bi[k];
          if constexpr (CMP::category == CAT_FLOAT) odd |= v != v;
        }
    }
    if (r < r1) {  // the rest, fewer than U rows of this group: requested together, taken in row order
      FVec<T, V> x[U - 1];
#pragma unroll
      for (int j = 0; j < U - 1; j++)
        if (r + j * RG < r1) x[j] = *reinterpret_cast<const FVec<T, V> *>(p + (r + j * RG) * a.r_stride);
#pragma unroll
      for (int j = 0; j < U - 1; j++)
        if (r + j * RG < r1)
#pragma unroll
          for (int k = 0; k < V; k++) {
            const C v = IN::ld(x[j].v[k]);
            const bool take = CMP::better(v, bv[k]);
            bv[k] = take ? v : bv[k];
            bi[k] = take ? (I)(r + j * RG) : bi[k];
            if constexpr (CMP::category == CAT_FLOAT) odd |= v != v;
          }
    }
    if (!odd) goto combine;
    r = r0 + rg;
  }
#pragma unroll
  for (int k = 0; k < V; k++) bv[k] = C{}, bi[k] = -1;
  for (; r + (U - 1) * RG < r1; r += U * RG) {
    FVec<T, V> x[U];
    int32_t xi[U];
#pragma unroll
    for (int j = 0; j < U; j++) {
      x[j] = *reinterpret_cast<const FVec<T, V> *>(p + (r + j * RG) * a.r_stride);
      if (HAS_IDX) xi[j] = a.in_idx[in_off + l + (r + j * RG) * a.r_stride];
    }
#pragma unroll
    for (int j = 0; j < U; j++)
#pragma unroll
      for (int k = 0; k < V; k++) {
        if (HAS_IDX) CMP::merge(bv[k], bi[k], IN::ld(x[j].v[k]), (I)xi[j]);
        else arg_take<CMP, C>(bv[k], bi[k], IN::ld(x[j].v[k]), (I)(r + j * RG));
      }
  }
  if (r < r1) {  // the rest of this group, requested together
    FVec<T, V> x[U - 1];
    int32_t xi[U - 1];
#pragma unroll
    for (int j = 0; j < U - 1; j++)
      if (r + j * RG < r1) {
        x[j] = *reinterpret_cast<const FVec<T, V> *>(p + (r + j * RG) * a.r_stride);
        if (HAS_IDX) xi[j] = a.in_idx[in_off + l + (r + j * RG) * a.r_stride];
      }
#pragma unroll
    for (int j = 0; j < U - 1; j++)
      if (r + j * RG < r1)
#pragma unroll
        for (int k = 0; k < V; k++) {
          if (HAS_IDX) CMP::merge(bv[k], bi[k], IN::ld(x[j].v[k]), (I)xi[j]);
          else arg_take<CMP, C>(bv[k], bi[k], IN::ld(x[j].v[k]), (I)(r + j * RG));
        }
  }
combine:
  if constexpr (RG > 1) {
    if (rg > 0) {
#pragma unroll
      for (int k = 0; k < V; k++) {
        lv[((rg - 1) * V + k) * LANES + ln] = bv[k];
        li[((rg - 1) * V + k) * LANES + ln] = (int32_t)bi[k];
      }
    }
    __syncthreads();
    if (rg > 0) return;
#pragma unroll
    for (int g = 1; g < RG; g++)
#pragma unroll
      for (int k = 0; k < V; k++)
        CMP::merge(bv[k], bi[k], lv[((g - 1) * V + k) * LANES + ln], (I)li[((g - 1) * V + k) * LANES + ln]);
  }
  if (!live) return;
  if (a.nsplit > 1) {
    uint64_t po = ((uint64_t)c * a.n_out + ob) * a.L + l;
#pragma unroll
    for (int k = 0; k < V; k++) {
      ((C *)a.out_val)[po + k] = bv[k];
      a.out_idx[po + k] = (int32_t)bi[k];
    }
  } else {
    int32_t *o = a.out_idx + out_off + (int64_t)l * a.out_lane_stride;
#pragma unroll
    for (int k = 0; k < V; k++) o[(int64_t)k * a.out_lane_stride] = (int32_t)bi[k];
  }
}

// ── argreduce host ──────────────────────────────────────────────────────────
template <bool IS_MIN, int DT>
static int arg_launch(nxh_context *ctx, const char *op, const nxh_tensor *in, const nxh_tensor *out,
                      const Geom &g) {
  using TR = Tr<DT>;
  using C = typename TR::C;
  using S = typename TR::S;
  using CMP = ArgCmp<IS_MIN, C, TR::cat>;
  const S *ibase = (const S *)in->data + in->offset;
  int32_t *obase = (int32_t *)out->data + out->offset;
  const int cus = ctx->compute_units > 0 ? ctx->compute_units : 256;
  Scratch scratch(ctx);
  ArgArgs a;
  a.in = ibase;
  a.in_idx = nullptr;
  a.R = g.R;
  a.r_stride = g.nr ? g.rin[0] : 0;
  a.n_out = (uint64_t)g.n_out;
  a.L = 0;
  a.lane_blocks = 0;
  a.out_lane_stride = 0;

  // column form: some kept dim is the unit-stride one and the axis is strided
  int lane = -1;
  for (int j = 0; j < g.nk; j++)
    if (g.kin[j] == 1 && g.kshape[j] >= 16 && g.kshape[j] <= 0x7fffffffLL) lane = j;
  if (lane >= 0 && std::llabs(a.r_stride) > 1 && dims_fill(&a.kept, g.nk, g.kshape, g.kin, g.kout, lane)) {
    const int64_t L = g.kshape[lane], n_outer = g.n_out / L;
    constexpr int V = 16 / (int)sizeof(S) > 0 ? 16 / (int)sizeof(S) : 1;
    bool vec = V > 1 && aligned_to16(ibase) && L % V == 0 && a.r_stride % V == 0;
    for (int i = 0; vec && i < g.nk; i++)
      if (i != lane && g.kin[i] % V != 0) vec = false;
    const int v = vec ? V : 1;
    const bool rg4 = g.R >= 64;
    const int64_t lanes = rg4 ? FOLD_THREADS / 4 : FOLD_THREADS;
    const int64_t lane_blocks = (L + lanes * v - 1) / (lanes * v);
    const int64_t blocks = lane_blocks * n_outer;
    if (blocks <= 0x7fffffffLL) {
      // four blocks per unit, not eight: fewer partial rows for the second pass ([8192,8192] f32: 48.0 -> 45.6 us)
      int nsplit = pick_split(blocks, g.R, rg4 ? 64 : 16, (cus + 1) / 2);
      int64_t chunk = (g.R + nsplit - 1) / nsplit;
      if (nsplit > 1) chunk = chunk_off_channel_stride(chunk, a.r_stride * (int64_t)sizeof(S));
      nsplit = (int)((g.R + chunk - 1) / chunk);
      a.n_out = (uint64_t)n_outer;  // col form: number of outer slices
      a.L = (uint32_t)L;
      a.lane_blocks = (uint32_t)lane_blocks;
      a.out_lane_stride = g.kout[lane];
      a.chunk = chunk;
      a.nsplit = nsplit;
      a.out_idx = obase;
      a.out_val = nullptr;
      if (nsplit > 1) {
        int rc = scratch.get(0, (size_t)nsplit * g.n_out * sizeof(C));
        if (!rc) rc = scratch.get(1, (size_t)nsplit * g.n_out * sizeof(int32_t));
        if (rc) return rc;
        a.out_val = scratch.p[0];
        a.out_idx = (int32_t *)scratch.p[1];
      }
      nxh_set_path(nsplit > 1 ? "arg_col_split" : "arg_col");
      dim3 grid((unsigned)blocks, (unsigned)nsplit);
      if (rg4) {
        if (vec) hipLaunchKernelGGL((arg_col_kernel<InS<DT>, CMP, V, 4, false>), grid, dim3(FOLD_THREADS), 0, ctx->stream, a);
        else hipLaunchKernelGGL((arg_col_kernel<InS<DT>, CMP, 1, 4, false>), grid, dim3(FOLD_THREADS), 0, ctx->stream, a);
      } else {
        if (vec) hipLaunchKernelGGL((arg_col_kernel<InS<DT>, CMP, V, 1, false>), grid, dim3(FOLD_THREADS), 0, ctx->stream, a);
        else hipLaunchKernelGGL((arg_col_kernel<InS<DT>, CMP, 1, 1, false>), grid, dim3(FOLD_THREADS), 0, ctx->stream, a);
      }
      NXH_HIP(op, hipGetLastError());
      if (nsplit > 1) {
        ArgArgs b = a;
        b.in = scratch.p[0];
        b.in_idx = (const int32_t *)scratch.p[1];
        b.out_idx = obase;
        b.out_val = nullptr;
        dims_contig_in(&b.kept, L);
        b.R = nsplit;
        b.r_stride = g.n_out;
        b.chunk = nsplit;
        b.nsplit = 1;
        // 48 partial rows or more: sixteen row groups, a lane's four (value, index) pairs in
        // flight at once (the second pass is all latency)
        const bool rg16b = nsplit >= 48;
        const bool rg4b = nsplit >= 16;
        const int64_t lanes2 = rg16b ? FOLD_THREADS / 16 : rg4b ? FOLD_THREADS / 4 : FOLD_THREADS;
        b.lane_blocks = (uint32_t)((L + lanes2 - 1) / lanes2);
        dim3 grid2((unsigned)(b.lane_blocks * n_outer), 1);
        if (rg16b) hipLaunchKernelGGL((arg_col_kernel<InC<C>, CMP, 1, 16, true>), grid2, dim3(FOLD_THREADS), 0, ctx->stream, b);
        else if (rg4b) hipLaunchKernelGGL((arg_col_kernel<InC<C>, CMP, 1, 4, true>), grid2, dim3(FOLD_THREADS), 0, ctx->stream, b);
        else hipLaunchKernelGGL((arg_col_kernel<InC<C>, CMP, 1, 1, true>), grid2, dim3(FOLD_THREADS), 0, ctx->stream, b);
        NXH_HIP(op, hipGetLastError());
      }
      return NXH_OK;
    }
  }

  // row form: a group of lanes per output walks the axis at its own stride
  if (!dims_fill(&a.kept, g.nk, g.kshape, g.kin, g.kout))
    return nxh_fail(NXH_FAILURE, op, "view has too many non-mergeable dimensions for one launch");
  // Rows of fewer than 32 elements, plenty of them (the class of each of a million samples): a lane
  // per row; a wave per row left most of its lanes idle ([2^20, 10] f32: 350 us).
  if (g.R < 32 && g.n_out >= (int64_t)cus * 256 && g.n_out <= 0x7fffffffLL * 64) {
    a.chunk = g.R;
    a.nsplit = 1;
    a.out_idx = obase;
    a.out_val = nullptr;
    nxh_set_path("arg_row_lane");
    hipLaunchKernelGGL((arg_row_kernel<InS<DT>, CMP, 1, 1, false>), dim3((unsigned)((g.n_out + FOLD_THREADS - 1) / FOLD_THREADS), 1),
                       dim3(FOLD_THREADS), 0, ctx->stream, a);
    NXH_HIP(op, hipGetLastError());
    return NXH_OK;
  }
  // a wave per row while rows are short, or of medium length but plentiful
  const bool wave_rows = g.R < 1024 || (g.R <= 4096 && g.n_out >= (int64_t)cus * 16);
  const int64_t blocks = wave_rows ? (g.n_out + 3) / 4 : g.n_out;
  if (blocks > 0x7fffffffLL) return nxh_fail(NXH_FAILURE, op, "too many outputs for one launch");
  int nsplit = wave_rows ? 1 : pick_split(blocks, g.R, 8192, cus);
  int64_t chunk = (g.R + nsplit - 1) / nsplit;
  if (nsplit > 1) chunk = (chunk + 63) / 64 * 64;  // keeps every chunk start 16-byte aligned
  nsplit = (int)((g.R + chunk - 1) / chunk);
  a.chunk = chunk;
  a.nsplit = nsplit;
  a.out_idx = obase;
  a.out_val = nullptr;
  if (nsplit > 1) {
    int rc = scratch.get(0, (size_t)nsplit * g.n_out * sizeof(C));
    if (!rc) rc = scratch.get(1, (size_t)nsplit * g.n_out * sizeof(int32_t));
    if (rc) return rc;
    a.out_val = scratch.p[0];
    a.out_idx = (int32_t *)scratch.p[1];
  }
  dim3 grid((unsigned)blocks, (unsigned)nsplit);
  nxh_set_path(nsplit > 1 ? "arg_row_split" : (wave_rows ? "arg_row_wave" : "arg_row"));
  {
    constexpr int V = 16 / (int)sizeof(S) > 0 ? 16 / (int)sizeof(S) : 1;
    bool vec = V > 1 && a.r_stride == 1 && aligned_to16(ibase) && (nsplit == 1 || chunk % V == 0);
    for (int i = 0; vec && i < g.nk; i++)
      if (g.kin[i] % V != 0) vec = false;
    if (wave_rows) {
      if (vec) hipLaunchKernelGGL((arg_row_kernel<InS<DT>, CMP, 64, V, false>), grid, dim3(FOLD_THREADS), 0, ctx->stream, a);
      else hipLaunchKernelGGL((arg_row_kernel<InS<DT>, CMP, 64, 1, false>), grid, dim3(FOLD_THREADS), 0, ctx->stream, a);
    } else {
      if (vec) hipLaunchKernelGGL((arg_row_kernel<InS<DT>, CMP, 256, V, false>), grid, dim3(FOLD_THREADS), 0, ctx->stream, a);
      else hipLaunchKernelGGL((arg_row_kernel<InS<DT>, CMP, 256, 1, false>), grid, dim3(FOLD_THREADS), 0, ctx->stream, a);
    }
  }
  NXH_HIP(op, hipGetLastError());
  if (nsplit > 1) {
    ArgArgs b = a;
    b.in = scratch.p[0];
    b.in_idx = (const int32_t *)scratch.p[1];
    b.out_idx = obase;
    b.out_val = nullptr;
    dims_contig_in(&b.kept, nsplit);
    b.R = nsplit;
    b.r_stride = 1;
    b.chunk = nsplit;
    b.nsplit = 1;
    hipLaunchKernelGGL((arg_row_kernel<InC<C>, CMP, 64, 1, true>), dim3((unsigned)((g.n_out + 3) / 4), 1),
                       dim3(FOLD_THREADS), 0, ctx->stream, b);
    NXH_HIP(op, hipGetLastError());
  }
  return NXH_OK;
}

template <bool IS_MIN>
struct ArgRow {
  fold_fn fn[NXH_DTYPE_COUNT] = {};
  template <int DT>
  void set() {
    if constexpr (Tr<DT>::cat != CAT_COMPLEX) fn[DT] = &arg_launch<IS_MIN, DT>;
  }
  ArgRow() {
#define NXH_SET(DT) set<DT>();
    NXH_FOR_COMPUTE_DTYPES(NXH_SET)
#undef NXH_SET
  }
};

NXH_EXPORT int nxh_argreduce(nxh_context *ctx, int is_min, const nxh_tensor *out, const nxh_tensor *x,
                             int axis) {
  NXH_DEFER_TOUCH(ctx, 1, out, x);
  const char *name = is_min ? "argmin" : "argmax";
  if (!ctx || !out || !x) return nxh_fail(NXH_INVALID_ARGUMENT, name, "null argument");
  int rc = nxh_check_tensor(name, out);
  if (!rc) rc = nxh_check_tensor(name, x);
  if (rc) return rc;
  static const ArgRow<false> row_max;
  static const ArgRow<true> row_min;
  const int dt = x->dtype;
  fold_fn fn = (is_min ? row_min.fn : row_max.fn)[dt];
  if (axis < 0 || axis >= x->ndim) return nxh_fail(NXH_INVALID_ARGUMENT, name, NXH_ERR_AXIS);
  bool reduced[NXH_MAX_NDIM];
  nxh_tensor sq;
  int32_t ax = axis;
  rc = squeeze_out(name, x, out, &ax, 1, reduced, &sq);
  if (rc) return rc;
  if (!fn) return nxh_fail(NXH_FAILURE, name, nxh_is_packed(dt) ? NXH_ERR_PACKED : NXH_ERR_UNSUPPORTED);
  if (out->dtype != NXH_I32) return nxh_fail(NXH_FAILURE, name, NXH_ERR_UNSUPPORTED);
  const int64_t alen = x->shape[axis];
  if (alen == 0) return nxh_fail(NXH_INVALID_ARGUMENT, name, NXH_ERR_EMPTY_REDUCE);
  if (alen > INT32_MAX) return nxh_fail(NXH_FAILURE, name, NXH_ERR_ARGCAP);
  Geom g;
  geom_build(x, &sq, reduced, &g);
  if (g.n_out == 0) return NXH_OK;
  if (g.nr == 0) {  // axis of length 1: every index is 0
    g.nr = 1;
    g.rshape[0] = 1;
    g.rin[0] = 0;
  }
  std::lock_guard<std::mutex> guard(ctx->mu);
  NXH_HIP(name, hipSetDevice(ctx->device));
  return fn(ctx, name, x, &sq, g);
}
