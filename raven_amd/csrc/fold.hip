// fold.hip — reductions (sum, prod, max, min) and argmax/argmin.
//
// Semantics restate packages/nx/lib/backend_c/nx_c_fold.c:63-101 (combine
// rules, NaN propagation, first-index ties) with the reference's accumulator
// widths (nx_c.h:109-116: f16/bf16/fp8 -> f32, small ints -> int64, u32/u64 ->
// uint64, wrap on store). The driver (nx_c_engine.c:1052-1254) is replaced by a
// planner that picks, per call:
//   fold_row   the reduced extent is one unit-stride run: a wave (short rows) or
//              a 256-lane block (long rows) per output, 16-byte loads, wave64
//              shuffle + LDS combine; long rows with few outputs are split into
//              chunks and finished by a second pass over the partials.
//   fold_col   a kept dim is the unit-stride one (axis-0 style): each lane owns
//              up to four adjacent output columns and walks the reduced rows;
//              rows are split across blocks with a second pass over partials.
//   fold_any   everything else: one lane per output, odometer over the reduced
//              dims.
// Float sums are reassociated (tree order); results agree with the reference
// within its own tolerance, integer results are exact (modular).

#include "fold_common.hpp"

// Reduces `acc` over a group of G lanes (64: one wave; 256: the block). The
// result is valid in the group's first lane.
template <class CB, class C, int G>
__device__ __forceinline__ C group_reduce(C acc, C *lds) {
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) acc = CB::apply(acc, shfl_down_any(acc, d));
  if constexpr (G == 256) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) lds[wave] = acc;
    __syncthreads();
    if (threadIdx.x == 0) acc = CB::apply(CB::apply(lds[0], lds[1]), CB::apply(lds[2], lds[3]));
  }
  return acc;
}

// ── fold_row ────────────────────────────────────────────────────────────────
struct RowArgs {
  const void *in;
  void *out;
  FoldDims kept;      // output index -> offsets
  uint64_t n_out;     // number of outputs
  int64_t R;          // reduced run length (unit stride)
  int64_t chunk;      // elements per split (== R when unsplit)
  int64_t split_stride;  // elements from one split's first element to the next one's (== chunk for a cut run;
                         // the outer reduced dim's stride when every index of that dim is a split)
  int nsplit;         // > 1: out is partial[o * nsplit + c], compute-typed
};

template <class IN, class CB, class OUT, int G, int V>
__global__ __launch_bounds__(FOLD_THREADS) void fold_row_kernel(RowArgs a) {
  using T = typename IN::T;
  using C = typename IN::C;
  __shared__ C lds[4];
  constexpr int GROUPS = FOLD_THREADS / G;
  const int lane = threadIdx.x % G;
  // Blocks walk the input from its end: a tensor that the previous kernel has
  // just written front to back still has its tail in the memory-side cache, and
  // a reader that starts there finds it (measured on a 402 MB row max right
  // after its producer: 77 us against 105 us front to back).
  const uint64_t o = (uint64_t)(gridDim.x - 1 - blockIdx.x) * GROUPS + threadIdx.x / G;
  const bool live = o < a.n_out;
  const int c = gridDim.y - 1 - blockIdx.y;
  int64_t in_off = 0, out_off = 0;
  if (live) fold_decode(a.kept, o, in_off, out_off);
  const int64_t r0 = 0, before = (int64_t)c * a.chunk;
  const int64_t r1 = live ? (before + a.chunk < a.R ? a.chunk : a.R - before) : 0;
  const T *p = (const T *)a.in + in_off + (int64_t)c * a.split_stride;
  C acc0 = CB::init(), acc1 = CB::init(), acc2 = CB::init(), acc3 = CB::init();
  const int64_t nv = (r1 - r0) / V;
  const FVec<T, V> *pv = reinterpret_cast<const FVec<T, V> *>(p + r0);
  int64_t i = lane;
  for (; i + 3 * G < nv; i += 4 * G) {
    FVec<T, V> x0 = pv[i], x1 = pv[i + G], x2 = pv[i + 2 * G], x3 = pv[i + 3 * G];
#pragma unroll
    for (int k = 0; k < V; k++) {
      acc0 = CB::apply(acc0, IN::ld(x0.v[k]));
      acc1 = CB::apply(acc1, IN::ld(x1.v[k]));
      acc2 = CB::apply(acc2, IN::ld(x2.v[k]));
      acc3 = CB::apply(acc3, IN::ld(x3.v[k]));
    }
  }
  for (; i < nv; i += G) {
    FVec<T, V> x0 = pv[i];
#pragma unroll
    for (int k = 0; k < V; k++) acc0 = CB::apply(acc0, IN::ld(x0.v[k]));
  }
  for (int64_t e = r0 + nv * V + lane; e < r1; e += G) acc1 = CB::apply(acc1, IN::ld(p[e]));
  C acc = CB::apply(CB::apply(acc0, acc1), CB::apply(acc2, acc3));
  acc = group_reduce<CB, C, G>(acc, lds);
  if (live && lane == 0) {
    if (a.nsplit > 1) ((C *)a.out)[o * a.nsplit + c] = acc;
    else ((typename OUT::T *)a.out)[out_off] = OUT::st(acc);
  }
}

// ── fold_col ────────────────────────────────────────────────────────────────
struct ColArgs {
  const void *in;
  void *out;
  FoldDims outer;       // kept dims other than the lane dim
  uint64_t n_outer;
  uint32_t L;           // lane extent (unit input stride)
  uint32_t lane_blocks; // blocks along the lane dim
  int64_t out_lane_stride;
  int64_t R, r_stride;  // reduced extent and its input stride
  int64_t chunk;
  int64_t split_stride; // elements from one split's first row to the next one's (chunk * r_stride for a cut
                        // run; the outer reduced dim's stride when every index of that dim is a split)
  int nsplit;           // > 1: out is partial[(c * n_outer + ob) * L + l]
};

// A block is LANES = 256 / RG column lanes (V adjacent columns each, one
// 16-byte load per row) by RG row groups: row group g walks rows g, g + RG, ...
// of the block's chunk with 8 loads in flight, and the RG partial results meet
// in LDS. RG > 1 keeps the number of partial rows a split leaves for the
// second pass small while the grid still fills the chip.
template <class IN, class CB, class OUT, int V, int RG, int U = 8>
__global__ __launch_bounds__(FOLD_THREADS) void fold_col_kernel(ColArgs a) {
  using T = typename IN::T;
  using C = typename IN::C;
  constexpr int LANES = FOLD_THREADS / RG;
  __shared__ C lds[RG > 1 ? (RG - 1) * LANES * V : 1];
  // blocks walk the input from its end (see fold_row_kernel)
  const uint32_t bx = gridDim.x - 1 - blockIdx.x;
  const uint32_t lb = bx % a.lane_blocks;
  const uint64_t ob = bx / a.lane_blocks;
  const int c = gridDim.y - 1 - blockIdx.y;
  const uint32_t ln = threadIdx.x % LANES, rg = threadIdx.x / LANES;
  const uint32_t l = (lb * LANES + ln) * V;
  const bool live = l < a.L;
  int64_t in_off, out_off;
  fold_decode(a.outer, ob, in_off, out_off);
  const int64_t r0 = 0, before = (int64_t)c * a.chunk;
  const int64_t r1 = live ? (before + a.chunk < a.R ? a.chunk : a.R - before) : 0;
  const T *p = (const T *)a.in + in_off + l + (int64_t)c * a.split_stride;
  C acc[V];
#pragma unroll
  for (int k = 0; k < V; k++) acc[k] = CB::init();
  int64_t r = r0 + rg;
  for (; r + (U - 1) * RG < r1; r += U * RG) {
    FVec<T, V> x[U];
#pragma unroll
    for (int j = 0; j < U; j++) x[j] = *reinterpret_cast<const FVec<T, V> *>(p + (r + j * RG) * a.r_stride);
#pragma unroll
    for (int j = 0; j < U; j++)
#pragma unroll
      for (int k = 0; k < V; k++) acc[k] = CB::apply(acc[k], IN::ld(x[j].v[k]));
  }
  if (r < r1) {  // the rest, fewer than U rows of this group: requested together, added in row order
    FVec<T, V> x[U - 1];
#pragma unroll
    for (int j = 0; j < U - 1; j++)
      if (r + j * RG < r1) x[j] = *reinterpret_cast<const FVec<T, V> *>(p + (r + j * RG) * a.r_stride);
#pragma unroll
    for (int j = 0; j < U - 1; j++)
      if (r + j * RG < r1)
#pragma unroll
        for (int k = 0; k < V; k++) acc[k] = CB::apply(acc[k], IN::ld(x[j].v[k]));
  }
  if constexpr (RG > 1) {
    if (rg > 0) {
#pragma unroll
      for (int k = 0; k < V; k++) lds[((rg - 1) * V + k) * LANES + ln] = acc[k];
    }
    __syncthreads();
    if (rg > 0) return;
#pragma unroll
    for (int g = 1; g < RG; g++)
#pragma unroll
      for (int k = 0; k < V; k++) acc[k] = CB::apply(acc[k], lds[((g - 1) * V + k) * LANES + ln]);
  }
  if (!live) return;
  if (a.nsplit > 1) {
    C *o = (C *)a.out + ((uint64_t)c * a.n_outer + ob) * a.L + l;
#pragma unroll
    for (int k = 0; k < V; k++) o[k] = acc[k];
  } else {
    typename OUT::T *o = (typename OUT::T *)a.out + out_off + (int64_t)l * a.out_lane_stride;
#pragma unroll
    for (int k = 0; k < V; k++) o[(int64_t)k * a.out_lane_stride] = OUT::st(acc[k]);
  }
}

// ── fold_narrow ─────────────────────────────────────────────────────────────
// A contiguous [rows][L] matrix with fewer than 16 columns, reduced down its rows (class counts,
// the bias gradient of a small output layer): too narrow for fold_col's column lanes. The matrix
// is read as the flat run it is: the block's first (256 / L) * L lanes step through it that many
// elements at a time, so a lane always meets the same column and neighbouring lanes neighbouring
// addresses; the lanes of a column then meet in LDS. Blocks take runs of rows and leave partial
// results [block][L], which one more block of the same kernel folds.
struct NarrowArgs {
  const void *in;
  void *out;
  int64_t R, rows_per_block;
  int L, final_;
};
template <class IN, class CB, class OUT>
__global__ __launch_bounds__(FOLD_THREADS) void fold_narrow_kernel(NarrowArgs a) {
  using T = typename IN::T;
  using C = typename IN::C;
  __shared__ C lds[FOLD_THREADS];
  const int per_pass = FOLD_THREADS / a.L, active = per_pass * a.L;
  const int t = threadIdx.x;
  const int64_t r_begin = (int64_t)blockIdx.x * a.rows_per_block;
  const int64_t rows = (r_begin + a.rows_per_block < a.R ? r_begin + a.rows_per_block : a.R) - r_begin;
  C acc = CB::init();
  if (t < active) {
    const T *q = (const T *)a.in + r_begin * a.L + t;
    const int row0 = t / a.L;
    const int64_t mine = rows > row0 ? (rows - row0 + per_pass - 1) / per_pass : 0;  // this lane's elements
    int64_t i = 0;
    for (; i + 8 <= mine; i += 8) {
      T x[8];
#pragma unroll
      for (int j = 0; j < 8; j++) x[j] = q[(i + j) * active];
#pragma unroll
      for (int j = 0; j < 8; j++) acc = CB::apply(acc, IN::ld(x[j]));
    }
    for (; i < mine; i++) acc = CB::apply(acc, IN::ld(q[i * active]));
  }
  lds[t] = acc;
  __syncthreads();
  if (t < a.L) {
    C r = lds[t];
    for (int i = 1; i < per_pass; i++) r = CB::apply(r, lds[t + i * a.L]);
    if (a.final_) ((typename OUT::T *)a.out)[t] = OUT::st(r);
    else ((C *)a.out)[(int64_t)blockIdx.x * a.L + t] = r;
  }
}

// ── fold_short_rows ─────────────────────────────────────────────────────────
// Many contiguous rows of 2 .. 32 elements each (the classes of a batch of logits), reduced along
// the row: too short for a wave per row. A block brings 256 rows into LDS with neighbouring lanes
// on neighbouring addresses (row pitch odd, so that the lanes' walks along their rows meet
// different banks), then a lane folds its own row in row order.
struct ShortRowsArgs {
  const void *in;
  void *out;
  int64_t rows;
  int R;
};
template <class IN, class CB, class OUT>
__global__ __launch_bounds__(FOLD_THREADS) void fold_short_rows_kernel(ShortRowsArgs a) {
  using T = typename IN::T;
  using C = typename IN::C;
  static_assert(sizeof(T) <= 4, "the tile is sized for storage types of up to four bytes");
  __shared__ T tile[FOLD_THREADS * 33];
  const int R = a.R, pitch = R | 1;
  const int64_t row_base = (int64_t)blockIdx.x * FOLD_THREADS;
  const int64_t left = a.rows - row_base;
  const int nrows = (int)(left < FOLD_THREADS ? left : FOLD_THREADS);
  const int count = nrows * R;
  const T *src = (const T *)a.in + row_base * R;
  int row = (int)threadIdx.x / R, col = (int)threadIdx.x - row * R;
  const int drow = FOLD_THREADS / R, dcol = FOLD_THREADS - drow * R;
  for (int i = threadIdx.x; i < count; i += FOLD_THREADS) {
    tile[row * pitch + col] = src[i];
    row += drow;
    col += dcol;
    if (col >= R) {
      col -= R;
      row++;
    }
  }
  __syncthreads();
  if ((int)threadIdx.x >= nrows) return;
  const T *mine = tile + threadIdx.x * pitch;
  C acc = CB::init();
  for (int j = 0; j < R; j++) acc = CB::apply(acc, IN::ld(mine[j]));
  ((typename OUT::T *)a.out)[row_base + threadIdx.x] = OUT::st(acc);
}

// ── fold_any ────────────────────────────────────────────────────────────────
struct AnyArgs {
  const void *in;
  void *out;
  FoldDims kept;
  uint64_t n_out;
  int nr;
  uint32_t rshape[FOLD_MAXD];
  int64_t rstride[FOLD_MAXD];
  uint64_t R;
};
template <class IN, class CB, class OUT>
__global__ __launch_bounds__(FOLD_THREADS) void fold_any_kernel(AnyArgs a) {
  using T = typename IN::T;
  using C = typename IN::C;
  const uint64_t o = (uint64_t)blockIdx.x * FOLD_THREADS + threadIdx.x;
  if (o >= a.n_out) return;
  int64_t in_off, out_off;
  fold_decode(a.kept, o, in_off, out_off);
  const T *p = (const T *)a.in + in_off;
  uint32_t coord[FOLD_MAXD];
  for (int d = 0; d < a.nr; d++) coord[d] = 0;
  C acc = CB::init();
  int64_t off = 0;
  for (uint64_t r = 0; r < a.R; r++) {
    acc = CB::apply(acc, IN::ld(p[off]));
    for (int d = a.nr - 1; d >= 0; d--) {
      if (++coord[d] < a.rshape[d]) {
        off += a.rstride[d];
        break;
      }
      coord[d] = 0;
      off -= (int64_t)(a.rshape[d] - 1) * a.rstride[d];
    }
  }
  ((typename OUT::T *)a.out)[out_off] = OUT::st(acc);
}

template <int OP, int DT>
static int fold_launch(nxh_context *ctx, const char *op, const nxh_tensor *in, const nxh_tensor *out,
                       const Geom &g) {
  using TR = Tr<DT>;
  using C = typename TR::C;
  using S = typename TR::S;
  using CB = Combine<OP, C, TR::cat>;
  constexpr int V = 16 / (int)sizeof(S) > 0 ? 16 / (int)sizeof(S) : 1;
  constexpr int VC = 16 / (int)sizeof(C) > 0 ? 16 / (int)sizeof(C) : 1;
  const S *ibase = (const S *)in->data + in->offset;
  S *obase = (S *)out->data + out->offset;
  const int cus = ctx->compute_units > 0 ? ctx->compute_units : 256;
  Scratch scratch(ctx, g.fixed_scratch);

  // Two reduced dims that do not merge (the batch and the positions of [N, C, H, W] with the
  // channels kept; axes 0 and 2 of a rank-3 tensor): the longer or the unit-stride one is walked
  // as the single-dim forms walk theirs, and every index of the other one is a "split": its
  // partial results go to the block of partials and the second pass folds them, exactly as for
  // a run cut into chunks. (One lane per output, which such reductions took before, walked all
  // of a [64,512,512] tensor with 512 lanes: 7.0 ms for sums over axes 0 and 2.)
  auto outer_fits = [&](int64_t outer_extent) {
    if (outer_extent > 65535 || g.n_out > ((int64_t)1 << 30) / outer_extent) return false;
    const size_t bytes = (size_t)g.n_out * (size_t)outer_extent * sizeof(C);  // the partial results
    return bytes <= ((size_t)1 << 30) && (!g.fixed_scratch || bytes <= NXH_STATIC_WS_BYTES);
  };

  // ---- fold_row: a unit-stride reduced run, alone or under one outer reduced dim ----
  const int row_dim = g.nr == 1 ? 0 : (g.nr == 2 ? (g.rin[1] == 1 ? 1 : (g.rin[0] == 1 ? 0 : -1)) : -1);
  const bool row_two = g.nr == 2 && row_dim >= 0;
  if (row_dim >= 0 && g.rin[row_dim] == 1 && g.n_out <= 0x7fffffffLL * 4 &&
      (row_two ? g.rshape[row_dim] >= 8 && outer_fits(g.rshape[1 - row_dim]) : g.R >= 64)) {
    RowArgs a;
    if (dims_fill(&a.kept, g.nk, g.kshape, g.kin, g.kout)) {
      const int64_t run = g.rshape[row_dim], outer = row_two ? g.rshape[1 - row_dim] : 1;
      a.in = ibase;
      a.n_out = (uint64_t)g.n_out;
      a.R = g.R;
      // a wave per row while rows are short, or of medium length but plentiful
      const bool wave_rows = run < 1024 || (run <= 4096 && g.n_out * outer >= (int64_t)cus * 16);
      const int64_t blocks = wave_rows ? (g.n_out + 3) / 4 : g.n_out;
      int nsplit = row_two ? (int)outer : (wave_rows ? 1 : pick_split(blocks, g.R, 8192, cus));
      int64_t chunk = run;
      if (!row_two && nsplit > 1) {
        chunk = (g.R + nsplit - 1) / nsplit;
        chunk = (chunk + 63) / 64 * 64;  // keeps every chunk start 16-byte aligned
        nsplit = (int)((g.R + chunk - 1) / chunk);
      }
      a.chunk = chunk;
      a.split_stride = row_two ? g.rin[1 - row_dim] : chunk;
      a.nsplit = nsplit;
      bool vec = aligned_to16(ibase) && (!row_two || a.split_stride % V == 0);
      for (int i = 0; vec && i < g.nk; i++)
        if (g.kin[i] % V != 0) vec = false;
      if (nsplit > 1) {
        int rc = scratch.get(0, (size_t)g.n_out * nsplit * sizeof(C));
        if (rc) return rc;
        a.out = scratch.p[0];
      } else {
        a.out = obase;
      }
      dim3 grid((unsigned)blocks, (unsigned)nsplit);
      nxh_set_path(row_two ? "fold_row_outer" : nsplit > 1 ? "fold_row_split" : (wave_rows ? "fold_row_wave" : "fold_row"));
      if (wave_rows) {
        if (vec) hipLaunchKernelGGL((fold_row_kernel<InS<DT>, CB, OutS<DT>, 64, V>), grid, dim3(FOLD_THREADS), 0, ctx->stream, a);
        else hipLaunchKernelGGL((fold_row_kernel<InS<DT>, CB, OutS<DT>, 64, 1>), grid, dim3(FOLD_THREADS), 0, ctx->stream, a);
      } else {
        if (vec) hipLaunchKernelGGL((fold_row_kernel<InS<DT>, CB, OutS<DT>, 256, V>), grid, dim3(FOLD_THREADS), 0, ctx->stream, a);
        else hipLaunchKernelGGL((fold_row_kernel<InS<DT>, CB, OutS<DT>, 256, 1>), grid, dim3(FOLD_THREADS), 0, ctx->stream, a);
      }
      NXH_HIP(op, hipGetLastError());
      if (nsplit > 1) {
        RowArgs b = a;
        b.in = scratch.p[0];
        b.out = obase;
        dims_contig_in(&b.kept, nsplit);
        b.R = nsplit;
        b.chunk = nsplit;
        b.split_stride = nsplit;
        b.nsplit = 1;
        dim3 grid2((unsigned)((g.n_out + 3) / 4), 1);
        hipLaunchKernelGGL((fold_row_kernel<InC<C>, CB, OutS<DT>, 64, 1>), grid2, dim3(FOLD_THREADS), 0, ctx->stream, b);
        NXH_HIP(op, hipGetLastError());
      }
      return NXH_OK;
    }
  }

  // ---- fold_short_rows: many contiguous rows of 2 .. 32 elements, reduced along the row ----
  if constexpr (sizeof(S) <= 4) {
    if (g.nr == 1 && g.nk == 1 && g.rin[0] == 1 && g.R >= 2 && g.R <= 32 && g.kin[0] == g.R && g.kout[0] == 1 &&
        g.n_out >= 4096 && g.n_out <= 0x7fffffffLL * 128) {
      ShortRowsArgs a;
      a.in = ibase;
      a.out = obase;
      a.rows = g.n_out;
      a.R = (int)g.R;
      nxh_set_path("fold_short_rows");
      hipLaunchKernelGGL((fold_short_rows_kernel<InS<DT>, CB, OutS<DT>>), dim3((unsigned)((g.n_out + FOLD_THREADS - 1) / FOLD_THREADS)),
                         dim3(FOLD_THREADS), 0, ctx->stream, a);
      NXH_HIP(op, hipGetLastError());
      return NXH_OK;
    }
  }

  // ---- fold_narrow: a contiguous [rows][L] matrix, L < 16, reduced down its rows ----
  if (g.nr == 1 && g.nk == 1 && g.kin[0] == 1 && g.kout[0] == 1 && g.kshape[0] < 16 && g.rin[0] == g.kshape[0] &&
      g.R >= 512) {
    NarrowArgs a;
    a.L = (int)g.kshape[0];
    a.R = g.R;
    const int64_t nblocks = std::min<int64_t>((int64_t)cus * 8, (g.R + 1023) / 1024);
    a.rows_per_block = (g.R + nblocks - 1) / nblocks;
    const int64_t used = (g.R + a.rows_per_block - 1) / a.rows_per_block;
    const size_t bytes = (size_t)used * a.L * sizeof(C);
    if (!g.fixed_scratch || bytes <= NXH_STATIC_WS_BYTES) {
      a.in = ibase;
      a.final_ = used == 1;
      a.out = obase;
      if (used > 1) {
        int rc = scratch.get(0, bytes);
        if (rc) return rc;
        a.out = scratch.p[0];
      }
      nxh_set_path("fold_narrow");
      hipLaunchKernelGGL((fold_narrow_kernel<InS<DT>, CB, OutS<DT>>), dim3((unsigned)used), dim3(FOLD_THREADS), 0, ctx->stream, a);
      NXH_HIP(op, hipGetLastError());
      if (used > 1) {
        NarrowArgs b = a;
        b.in = scratch.p[0];
        b.out = obase;
        b.R = used;
        b.rows_per_block = used;
        b.final_ = 1;
        hipLaunchKernelGGL((fold_narrow_kernel<InC<C>, CB, OutS<DT>>), dim3(1), dim3(FOLD_THREADS), 0, ctx->stream, b);
        NXH_HIP(op, hipGetLastError());
      }
      return NXH_OK;
    }
  }

  // ---- fold_col: a kept dim is the unit-stride one ----
  if ((g.nr == 1 || g.nr == 2) && g.nk >= 1) {
    int lane = -1;
    for (int j = 0; j < g.nk; j++)
      if (g.kin[j] == 1 && g.kshape[j] >= 16 && g.kshape[j] <= 0x7fffffffLL) lane = j;
    ColArgs a;
    // two reduced dims: the longer one is walked, every index of the other is a split
    const bool col_two = g.nr == 2;
    const int walk = col_two && g.rshape[1] > g.rshape[0] ? 1 : 0;
    const int64_t run = g.rshape[walk], run_stride = g.rin[walk];
    if (lane >= 0 && std::llabs(run_stride) > 1 && (!col_two || (run >= 8 && outer_fits(g.rshape[1 - walk]))) &&
        dims_fill(&a.outer, g.nk, g.kshape, g.kin, g.kout, lane)) {
      const int64_t L = g.kshape[lane];
      const int64_t n_outer = g.n_out / L;
      bool vec = aligned_to16(ibase) && L % V == 0 && run_stride % V == 0 && (!col_two || g.rin[1 - walk] % V == 0);
      for (int i = 0; vec && i < g.nk; i++)
        if (i != lane && g.kin[i] % V != 0) vec = false;
      const int v = vec ? V : 1;
      // long reduced runs: 4 row groups per block (see fold_col_kernel)
      const bool rg4 = run >= 64;
      const int64_t lanes = rg4 ? FOLD_THREADS / 4 : FOLD_THREADS;
      const int64_t lane_blocks = (L + lanes * v - 1) / (lanes * v);
      const int64_t blocks = lane_blocks * n_outer;
      if (blocks <= 0x7fffffffLL) {
        int nsplit = col_two ? (int)g.rshape[1 - walk] : pick_split(blocks, g.R, rg4 ? 64 : 16, cus);
        int64_t chunk = col_two ? run : (g.R + nsplit - 1) / nsplit;
        if (!col_two) {
          if (nsplit > 1) chunk = chunk_off_channel_stride(chunk, g.rin[0] * (int64_t)sizeof(S));
          nsplit = (int)((g.R + chunk - 1) / chunk);
        }
        a.split_stride = col_two ? g.rin[1 - walk] : chunk * run_stride;
        a.in = ibase;
        a.n_outer = (uint64_t)n_outer;
        a.L = (uint32_t)L;
        a.lane_blocks = (uint32_t)lane_blocks;
        a.out_lane_stride = g.kout[lane];
        a.R = g.R;
        a.r_stride = run_stride;
        a.chunk = chunk;
        a.nsplit = nsplit;
        if (nsplit > 1) {
          int rc = scratch.get(0, (size_t)nsplit * g.n_out * sizeof(C));
          if (rc) return rc;
          a.out = scratch.p[0];
        } else {
          a.out = obase;
        }
        dim3 grid((unsigned)blocks, (unsigned)nsplit);
        nxh_set_path(col_two ? "fold_col_outer" : nsplit > 1 ? "fold_col_split" : "fold_col");
        if (rg4) {
          if (vec) hipLaunchKernelGGL((fold_col_kernel<InS<DT>, CB, OutS<DT>, V, 4>), grid, dim3(FOLD_THREADS), 0, ctx->stream, a);
          else hipLaunchKernelGGL((fold_col_kernel<InS<DT>, CB, OutS<DT>, 1, 4>), grid, dim3(FOLD_THREADS), 0, ctx->stream, a);
        } else {
          if (vec) hipLaunchKernelGGL((fold_col_kernel<InS<DT>, CB, OutS<DT>, V, 1>), grid, dim3(FOLD_THREADS), 0, ctx->stream, a);
          else hipLaunchKernelGGL((fold_col_kernel<InS<DT>, CB, OutS<DT>, 1, 1>), grid, dim3(FOLD_THREADS), 0, ctx->stream, a);
        }
        NXH_HIP(op, hipGetLastError());
        if (nsplit > 1) {
          // the partial rows [nsplit][n_outer * L] are folded the same way
          ColArgs b = a;
          b.in = scratch.p[0];
          b.out = obase;
          dims_contig_in(&b.outer, L);
          b.R = nsplit;
          b.r_stride = g.n_out;
          b.chunk = nsplit;
          b.split_stride = 0;
          b.nsplit = 1;
          const bool vec2 = L % VC == 0;
          const int v2 = vec2 ? VC : 1;
          // 48 partial rows or more: sixteen row groups of four loads each, so that a lane's whole
          // share is in flight at once and four times as many blocks carry the launch (the second
          // pass is all latency: [64][8192] f32 partials, 2 MiB)
          const bool rg16b = nsplit >= 48;
          const bool rg4b = nsplit >= 16;
          const int64_t lanes2 = rg16b ? FOLD_THREADS / 16 : rg4b ? FOLD_THREADS / 4 : FOLD_THREADS;
          b.lane_blocks = (uint32_t)((L + lanes2 * v2 - 1) / (lanes2 * v2));
          dim3 grid2((unsigned)(b.lane_blocks * n_outer), 1);
          if (rg16b) {
            if (vec2) hipLaunchKernelGGL((fold_col_kernel<InC<C>, CB, OutS<DT>, VC, 16, 4>), grid2, dim3(FOLD_THREADS), 0, ctx->stream, b);
            else hipLaunchKernelGGL((fold_col_kernel<InC<C>, CB, OutS<DT>, 1, 16, 4>), grid2, dim3(FOLD_THREADS), 0, ctx->stream, b);
          } else if (rg4b) {
            if (vec2) hipLaunchKernelGGL((fold_col_kernel<InC<C>, CB, OutS<DT>, VC, 4>), grid2, dim3(FOLD_THREADS), 0, ctx->stream, b);
            else hipLaunchKernelGGL((fold_col_kernel<InC<C>, CB, OutS<DT>, 1, 4>), grid2, dim3(FOLD_THREADS), 0, ctx->stream, b);
          } else {
            if (vec2) hipLaunchKernelGGL((fold_col_kernel<InC<C>, CB, OutS<DT>, VC, 1>), grid2, dim3(FOLD_THREADS), 0, ctx->stream, b);
            else hipLaunchKernelGGL((fold_col_kernel<InC<C>, CB, OutS<DT>, 1, 1>), grid2, dim3(FOLD_THREADS), 0, ctx->stream, b);
          }
          NXH_HIP(op, hipGetLastError());
        }
        return NXH_OK;
      }
    }
  }

  // ---- fold_any ----
  AnyArgs a;
  if (!dims_fill(&a.kept, g.nk, g.kshape, g.kin, g.kout) || g.nr > FOLD_MAXD)
    return nxh_fail(NXH_FAILURE, op, "view has too many non-mergeable dimensions for one launch");
  a.in = ibase;
  a.out = obase;
  a.n_out = (uint64_t)g.n_out;
  a.nr = g.nr;
  a.R = (uint64_t)g.R;
  // the smallest-|stride| reduced dim runs innermost (nx_c_engine.c:1151-1164)
  int64_t rs[NXH_MAX_NDIM], rst[NXH_MAX_NDIM];
  for (int d = 0; d < g.nr; d++) {
    rs[d] = g.rshape[d];
    rst[d] = g.rin[d];
  }
  if (g.nr > 1) {
    int best = 0;
    for (int r = 1; r < g.nr; r++)
      if (std::llabs(rst[r]) < std::llabs(rst[best])) best = r;
    std::swap(rs[best], rs[g.nr - 1]);
    std::swap(rst[best], rst[g.nr - 1]);
  }
  for (int d = 0; d < g.nr; d++) {
    if (rs[d] > 0xffffffffLL) return nxh_fail(NXH_FAILURE, op, "reduced dimension too large");
    a.rshape[d] = (uint32_t)rs[d];
    a.rstride[d] = rst[d];
  }
  const uint64_t blocks = ((uint64_t)g.n_out + FOLD_THREADS - 1) / FOLD_THREADS;
  if (blocks > 0x7fffffffULL) return nxh_fail(NXH_FAILURE, op, "too many outputs for one launch");
  nxh_set_path("fold_any");
  hipLaunchKernelGGL((fold_any_kernel<InS<DT>, CB, OutS<DT>>), dim3((unsigned)blocks), dim3(FOLD_THREADS), 0, ctx->stream, a);
  NXH_HIP(op, hipGetLastError());
  return NXH_OK;
}

template <int OP>
struct FoldRow {
  fold_fn fn[NXH_DTYPE_COUNT] = {};
  template <int DT>
  void set() {
    if constexpr (fold_ok(OP, Tr<DT>::cat)) fn[DT] = &fold_launch<OP, DT>;
  }
  FoldRow() {
#define NXH_SET(DT) set<DT>();
    NXH_FOR_COMPUTE_DTYPES(NXH_SET)
#undef NXH_SET
  }
};

// The value 1 in each dtype's storage format, for prod over an empty extent.
static void storage_one(int dt, void *buf) {
  memset(buf, 0, 16);
  switch (dt) {
    case NXH_F16: *(uint16_t *)buf = 0x3c00; break;
    case NXH_BF16: *(uint16_t *)buf = 0x3f80; break;
    case NXH_F32: *(float *)buf = 1.0f; break;
    case NXH_F64: *(double *)buf = 1.0; break;
    case NXH_F8E4M3: *(uint8_t *)buf = 0x38; break;
    case NXH_F8E5M2: *(uint8_t *)buf = 0x3c; break;
    case NXH_C32: *(float *)buf = 1.0f; break;
    case NXH_C64: *(double *)buf = 1.0; break;
    default: *(uint8_t *)buf = 1; break;  // little-endian integers of any width
  }
}

static int reduce_entry(nxh_context *ctx, int op, const nxh_tensor *out, const nxh_tensor *x,
                        const int32_t *axes, int n_axes, bool fixed_scratch) {
  static const char *const names[NXH_REDUCE_COUNT] = {"reduce_sum", "reduce_prod", "reduce_max", "reduce_min"};
  if ((unsigned)op >= NXH_REDUCE_COUNT) return nxh_fail(NXH_INVALID_ARGUMENT, "reduce", "unknown op");
  const char *name = names[op];
  if (!ctx || !out || !x || (n_axes > 0 && !axes)) return nxh_fail(NXH_INVALID_ARGUMENT, name, "null argument");
  int rc = nxh_check_tensor(name, out);
  if (!rc) rc = nxh_check_tensor(name, x);
  if (rc) return rc;
  static const FoldRow<NXH_SUM> row_sum;
  static const FoldRow<NXH_PROD> row_prod;
  static const FoldRow<NXH_RMAX> row_max;
  static const FoldRow<NXH_RMIN> row_min;
  const fold_fn *rows[NXH_REDUCE_COUNT] = {row_sum.fn, row_prod.fn, row_max.fn, row_min.fn};
  const int dt = x->dtype;
  bool reduced[NXH_MAX_NDIM];
  nxh_tensor sq;
  rc = squeeze_out(name, x, out, axes, n_axes, reduced, &sq);
  if (rc) return rc;
  fold_fn fn = rows[op][dt];
  if (!fn) return nxh_fail(NXH_FAILURE, name, nxh_is_packed(dt) ? NXH_ERR_PACKED : NXH_ERR_UNSUPPORTED);
  if (out->dtype != dt) return nxh_fail(NXH_FAILURE, name, NXH_ERR_UNSUPPORTED);
  Geom g;
  geom_build(x, &sq, reduced, &g);
  g.fixed_scratch = fixed_scratch;
  if (g.n_out == 0) return NXH_OK;
  for (int j = 0; j < sq.ndim; j++)
    if (sq.shape[j] > 1 && sq.strides[j] == 0) return nxh_fail(NXH_INVALID_ARGUMENT, name, NXH_ERR_OUT_ALIASED);
  if (g.R == 0) {
    // max/min have no identity (nx_c_engine.c:1101-1105); sum/prod store 0/1
    if (op == NXH_RMAX || op == NXH_RMIN) return nxh_fail(NXH_INVALID_ARGUMENT, name, NXH_ERR_EMPTY_REDUCE);
    unsigned char one[16];
    if (op == NXH_PROD) storage_one(dt, one);
    else memset(one, 0, sizeof one);
    return nxh_fill(ctx, &sq, one);
  }
  std::lock_guard<std::mutex> guard(ctx->mu);
  NXH_HIP(name, hipSetDevice(ctx->device));
  if (!fixed_scratch) fold_note_access(ctx, x, &sq, g.n_out, g.R);  // (nxh_reduce_noalloc has noted it)
  return fn(ctx, name, x, &sq, g);
}

NXH_EXPORT int nxh_reduce(nxh_context *ctx, int op, const nxh_tensor *out, const nxh_tensor *x,
                          const int32_t *axes, int n_axes) {
  // what the eager call rejects at once is not recorded (the record would otherwise read a null axis list)
  const bool recordable = ctx && out && x && (unsigned)op < NXH_REDUCE_COUNT && n_axes >= 0 && n_axes <= NXH_MAX_NDIM &&
                          (n_axes == 0 || axes) && (unsigned)out->ndim <= NXH_MAX_NDIM && (unsigned)x->ndim <= NXH_MAX_NDIM &&
                          (unsigned)out->dtype < NXH_DTYPE_COUNT && (unsigned)x->dtype < NXH_DTYPE_COUNT;
  if (recordable) NXH_DEFER_RECORD(ctx, NXH_D_REDUCE, op, out, 1, axes, n_axes, nullptr, x);
  else NXH_DEFER_QUIET(ctx);
  return reduce_entry(ctx, op, out, x, axes, n_axes, false);
}

// The same reduction with the partial results of its split forms in the device's
// static workspace: no allocation, no free, the same kernels and the same split,
// so the result equals nxh_reduce's bit for bit. A split whose partials exceed
// the workspace is refused before anything is launched.
NXH_EXPORT int nxh_reduce_noalloc(nxh_context *ctx, int op, const nxh_tensor *out, const nxh_tensor *x,
                                  const int32_t *axes, int n_axes) {
  NXH_DEFER_TOUCH(ctx, 1, out, x);
  return reduce_entry(ctx, op, out, x, axes, n_axes, true);
}
