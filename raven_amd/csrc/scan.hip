// scan.hip — inclusive prefix scan along one axis (cumsum / cumprod / cummax /
// cummin).
//
// Semantics restate packages/nx/lib/backend_c/nx_c_fold.c:161-176 and the driver
// nx_c_engine.c:1257-1331: the running value lives in the dtype's compute type
// (f32 for f16/bf16/fp8, int64/uint64 modular for integers), a copy rounded to
// storage is written per element, the combine rules and NaN propagation are
// those of the reductions. Two launch forms:
//   scan_rows   the axis has unit stride on both sides: a wave64 per line walks
//               it in chunks of 64 x V elements (16-byte loads), each lane scans
//               its V elements, a 6-step shuffle scan combines the lane totals,
//               the chunk total is carried to the next chunk.
//   scan_lines  anything else (the unit-stride dim is a kept one, or strided
//               views): one lane per line walks the axis in order, 4 loads in
//               flight; adjacent lanes own adjacent lines, so accesses coalesce
//               whenever a kept dim is contiguous. When there are too few lines
//               to fill the chip the axis is cut into chunks (scan_chunks):
//               chunk totals, an exclusive scan of the totals per line, then
//               every chunk is scanned from its carry-in.
// Float sums and products are reassociated by scan_rows (tolerance-level
// differences, inside the reference contract's 6x arithmetic tolerance for
// scans); integer results are exact.

#include "fold_common.hpp"

struct ScanArgs {
  const void *in;
  void *out;
  FoldDims lines;  // the non-axis dims: line index -> offsets
  uint64_t n_lines;
  int64_t len;     // axis length
  int64_t in_step, out_step;
};

template <int DT, class CB>
__global__ __launch_bounds__(FOLD_THREADS) void scan_lines_kernel(ScanArgs a) {
  using TR = Tr<DT>;
  using S = typename TR::S;
  using C = typename TR::C;
  const uint64_t line = (uint64_t)blockIdx.x * FOLD_THREADS + threadIdx.x;
  if (line >= a.n_lines) return;
  int64_t in_off, out_off;
  fold_decode(a.lines, line, in_off, out_off);
  const S *p = (const S *)a.in + in_off;
  S *q = (S *)a.out + out_off;
  C s = CB::init();
  int64_t k = 0;
  for (; k + 4 <= a.len; k += 4) {
    S x[4];
#pragma unroll
    for (int j = 0; j < 4; j++) x[j] = p[(k + j) * a.in_step];
#pragma unroll
    for (int j = 0; j < 4; j++) {
      s = CB::apply(s, TR::ld(x[j]));
      q[(k + j) * a.out_step] = TR::st(s);
    }
  }
  for (; k < a.len; k++) {
    s = CB::apply(s, TR::ld(p[k * a.in_step]));
    q[k * a.out_step] = TR::st(s);
  }
}

// The chunked form: blockIdx.y is the chunk, `carry` is C[chunks][lines].
// PHASE 0 writes each chunk's total, PHASE 2 scans each chunk from its carry-in.
template <int DT, class CB, int PHASE>
__global__ __launch_bounds__(FOLD_THREADS) void scan_chunks_kernel(ScanArgs a, int64_t chunk, void *carry_v) {
  using TR = Tr<DT>;
  using S = typename TR::S;
  using C = typename TR::C;
  const uint64_t line = (uint64_t)blockIdx.x * FOLD_THREADS + threadIdx.x;
  if (line >= a.n_lines) return;
  int64_t in_off, out_off;
  fold_decode(a.lines, line, in_off, out_off);
  const int64_t k0 = (int64_t)blockIdx.y * chunk;
  const int64_t k1 = k0 + chunk < a.len ? k0 + chunk : a.len;
  const S *p = (const S *)a.in + in_off;
  S *q = (S *)a.out + out_off;
  C *carry = (C *)carry_v + (uint64_t)blockIdx.y * a.n_lines + line;
  C s = PHASE == 0 ? CB::init() : *carry;
  int64_t k = k0;
  for (; k + 4 <= k1; k += 4) {
    S x[4];
#pragma unroll
    for (int j = 0; j < 4; j++) x[j] = p[(k + j) * a.in_step];
#pragma unroll
    for (int j = 0; j < 4; j++) {
      s = CB::apply(s, TR::ld(x[j]));
      if (PHASE == 2) q[(k + j) * a.out_step] = TR::st(s);
    }
  }
  for (; k < k1; k++) {
    s = CB::apply(s, TR::ld(p[k * a.in_step]));
    if (PHASE == 2) q[k * a.out_step] = TR::st(s);
  }
  if (PHASE == 0) *carry = s;
}
// Turns the chunk totals of each line into carry-ins (an exclusive scan).
template <class C, class CB>
__global__ __launch_bounds__(FOLD_THREADS) void scan_carry_kernel(C *carry, uint64_t n_lines, int chunks) {
  const uint64_t line = (uint64_t)blockIdx.x * FOLD_THREADS + threadIdx.x;
  if (line >= n_lines) return;
  C run = CB::init();
  for (int c = 0; c < chunks; c++) {
    const C t = carry[(uint64_t)c * n_lines + line];
    carry[(uint64_t)c * n_lines + line] = run;
    run = CB::apply(run, t);
  }
}

template <class T>
__device__ __forceinline__ T shfl_up_any(T v, int delta) {
  constexpr int W = (sizeof(T) + 3) / 4;
  union {
    T t;
    uint32_t w[W];
  } u;
  u.w[W - 1] = 0;
  u.t = v;
#pragma unroll
  for (int i = 0; i < W; i++) u.w[i] = __shfl_up(u.w[i], delta, 64);
  return u.t;
}
template <class T>
__device__ __forceinline__ T shfl_any(T v, int src) {
  constexpr int W = (sizeof(T) + 3) / 4;
  union {
    T t;
    uint32_t w[W];
  } u;
  u.w[W - 1] = 0;
  u.t = v;
#pragma unroll
  for (int i = 0; i < W; i++) u.w[i] = __shfl(u.w[i], src, 64);
  return u.t;
}

// One wave per line (PHASE 1), or per chunk of a line (blockIdx.y; PHASE 0
// writes the chunk's total to `carry`, PHASE 2 scans the chunk from its
// carry-in). VEC: lines and chunks are 16-byte aligned.
template <int DT, class CB, int V, bool VEC, int PHASE>
__global__ __launch_bounds__(FOLD_THREADS) void scan_rows_kernel(ScanArgs a, int64_t chunk, void *carry_v) {
  using TR = Tr<DT>;
  using S = typename TR::S;
  using C = typename TR::C;
  const int lane = threadIdx.x & 63;
  const uint64_t line = (uint64_t)blockIdx.x * (FOLD_THREADS / 64) + (threadIdx.x >> 6);
  if (line >= a.n_lines) return;
  int64_t in_off, out_off;
  fold_decode(a.lines, line, in_off, out_off);
  const S *p = (const S *)a.in + in_off;
  S *q = (S *)a.out + out_off;
  const int64_t k0 = PHASE == 1 ? 0 : (int64_t)blockIdx.y * chunk;
  const int64_t k1 = PHASE == 1 ? a.len : (k0 + chunk < a.len ? k0 + chunk : a.len);
  C *slot = PHASE == 1 ? nullptr : (C *)carry_v + (uint64_t)blockIdx.y * a.n_lines + line;
  C carry = PHASE == 2 ? *slot : CB::init();
  for (int64_t base = k0; base < k1; base += 64 * V) {
    const int64_t e0 = base + (int64_t)lane * V;
    const int n = (int)(k1 - e0 < V ? (k1 - e0 < 0 ? 0 : k1 - e0) : V);  // this lane's live elements
    FVec<S, V> x;
    if (VEC && n == V) {
      x = *reinterpret_cast<const FVec<S, V> *>(p + e0);
    } else {
#pragma unroll
      for (int j = 0; j < V; j++)
        if (j < n) x.v[j] = p[e0 + j];
    }
    C r[V];
    C t = CB::init();
#pragma unroll
    for (int j = 0; j < V; j++) {
      if (j < n) t = CB::apply(t, TR::ld(x.v[j]));
      r[j] = t;
    }
    // inclusive scan of the lane totals across the wave
    C incl = t;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const C up = shfl_up_any(incl, d);
      if (lane >= d) incl = CB::apply(up, incl);
    }
    if constexpr (PHASE != 0) {
      C excl = shfl_up_any(incl, 1);
      excl = lane == 0 ? carry : CB::apply(carry, excl);
      FVec<S, V> y;
#pragma unroll
      for (int j = 0; j < V; j++) y.v[j] = TR::st(CB::apply(excl, r[j]));
      if (VEC && n == V) {
        *reinterpret_cast<FVec<S, V> *>(q + e0) = y;
      } else {
#pragma unroll
        for (int j = 0; j < V; j++)
          if (j < n) q[e0 + j] = y.v[j];
      }
    }
    carry = CB::apply(carry, shfl_any(incl, 63));
  }
  if (PHASE == 0 && lane == 0) *slot = carry;
}

template <int OP, int DT>
static int scan_launch(nxh_context *ctx, const char *op, const nxh_tensor *in, const nxh_tensor *out,
                       const Geom &g, int64_t out_axis_stride) {
  using TR = Tr<DT>;
  using S = typename TR::S;
  using CB = Combine<OP, typename TR::C, TR::cat>;
  constexpr int V = 16 / (int)sizeof(S) > 0 ? 16 / (int)sizeof(S) : 1;
  ScanArgs a;
  a.in = (const S *)in->data + in->offset;
  a.out = (S *)out->data + out->offset;
  if (!dims_fill(&a.lines, g.nk, g.kshape, g.kin, g.kout))
    return nxh_fail(NXH_FAILURE, op, "view has too many non-mergeable dimensions for one launch");
  a.n_lines = (uint64_t)g.n_out;
  a.len = g.R;
  a.in_step = g.nr ? g.rin[0] : 0;
  a.out_step = out_axis_stride;
  if (a.in_step == 1 && a.out_step == 1 && a.len >= 128) {
    const int64_t blocks = (g.n_out + 3) / 4;
    if (blocks > 0x7fffffffLL) return nxh_fail(NXH_FAILURE, op, "too many lines for one launch");
    bool vec = V > 1 && aligned_to16(a.in) && aligned_to16(a.out);
    for (int i = 0; vec && i < g.nk; i++)
      if (g.kin[i] % V != 0 || g.kout[i] % V != 0) vec = false;
    const int cus = ctx->compute_units > 0 ? ctx->compute_units : 256;
    // few long lines: a wave per chunk of 64 * V * k elements instead of per line
    int64_t chunks = std::min<int64_t>(((int64_t)cus * 16 + g.n_out - 1) / g.n_out, a.len / (64 * V * 4));
    if (chunks >= 2 && chunks <= 65535) {
      using C = typename TR::C;
      int64_t chunk = (a.len + chunks - 1) / chunks;
      chunk = (chunk + 64 * V - 1) / (64 * V) * (64 * V);  // whole wave steps: chunk starts stay aligned
      chunks = (a.len + chunk - 1) / chunk;
      Scratch scratch(ctx);
      int rc = scratch.get(0, (size_t)chunks * g.n_out * sizeof(C));
      if (rc) return rc;
      const dim3 grid((unsigned)blocks, (unsigned)chunks);
      nxh_set_path("scan_rows_chunks");
      if (vec) hipLaunchKernelGGL((scan_rows_kernel<DT, CB, V, true, 0>), grid, dim3(FOLD_THREADS), 0, ctx->stream, a, chunk, scratch.p[0]);
      else hipLaunchKernelGGL((scan_rows_kernel<DT, CB, V, false, 0>), grid, dim3(FOLD_THREADS), 0, ctx->stream, a, chunk, scratch.p[0]);
      hipLaunchKernelGGL((scan_carry_kernel<C, CB>), dim3((unsigned)((g.n_out + FOLD_THREADS - 1) / FOLD_THREADS)),
                         dim3(FOLD_THREADS), 0, ctx->stream, (C *)scratch.p[0], (uint64_t)g.n_out, (int)chunks);
      if (vec) hipLaunchKernelGGL((scan_rows_kernel<DT, CB, V, true, 2>), grid, dim3(FOLD_THREADS), 0, ctx->stream, a, chunk, scratch.p[0]);
      else hipLaunchKernelGGL((scan_rows_kernel<DT, CB, V, false, 2>), grid, dim3(FOLD_THREADS), 0, ctx->stream, a, chunk, scratch.p[0]);
    } else {
      nxh_set_path("scan_rows");
      if (vec) hipLaunchKernelGGL((scan_rows_kernel<DT, CB, V, true, 1>), dim3((unsigned)blocks), dim3(FOLD_THREADS), 0, ctx->stream, a, (int64_t)0, nullptr);
      else hipLaunchKernelGGL((scan_rows_kernel<DT, CB, V, false, 1>), dim3((unsigned)blocks), dim3(FOLD_THREADS), 0, ctx->stream, a, (int64_t)0, nullptr);
    }
  } else {
    const int64_t blocks = (g.n_out + FOLD_THREADS - 1) / FOLD_THREADS;
    if (blocks > 0x7fffffffLL) return nxh_fail(NXH_FAILURE, op, "too many lines for one launch");
    const int cus = ctx->compute_units > 0 ? ctx->compute_units : 256;
    // too few lines for one lane each to fill the chip: cut the axis into chunks
    int64_t chunks = std::min<int64_t>(((int64_t)cus * 1024 + g.n_out - 1) / g.n_out, a.len / 16);
    if (chunks >= 2 && chunks <= 65535) {
      using C = typename TR::C;
      int64_t chunk = (a.len + chunks - 1) / chunks;
      chunk = chunk_off_channel_stride(chunk, a.in_step * (int64_t)sizeof(S));
      chunks = (a.len + chunk - 1) / chunk;
      Scratch scratch(ctx);
      int rc = scratch.get(0, (size_t)chunks * g.n_out * sizeof(C));
      if (rc) return rc;
      const dim3 grid((unsigned)blocks, (unsigned)chunks);
      nxh_set_path("scan_chunks");
      hipLaunchKernelGGL((scan_chunks_kernel<DT, CB, 0>), grid, dim3(FOLD_THREADS), 0, ctx->stream, a, chunk, scratch.p[0]);
      hipLaunchKernelGGL((scan_carry_kernel<C, CB>), dim3((unsigned)blocks), dim3(FOLD_THREADS), 0, ctx->stream,
                         (C *)scratch.p[0], (uint64_t)g.n_out, (int)chunks);
      hipLaunchKernelGGL((scan_chunks_kernel<DT, CB, 2>), grid, dim3(FOLD_THREADS), 0, ctx->stream, a, chunk, scratch.p[0]);
    } else {
      nxh_set_path("scan_lines");
      hipLaunchKernelGGL((scan_lines_kernel<DT, CB>), dim3((unsigned)blocks), dim3(FOLD_THREADS), 0, ctx->stream, a);
    }
  }
  NXH_HIP(op, hipGetLastError());
  return NXH_OK;
}

typedef int (*scan_fn)(nxh_context *, const char *, const nxh_tensor *, const nxh_tensor *, const Geom &, int64_t);
template <int OP>
struct ScanRow {
  scan_fn fn[NXH_DTYPE_COUNT] = {};
  template <int DT>
  void set() {
    if constexpr (fold_ok(OP, Tr<DT>::cat)) fn[DT] = &scan_launch<OP, DT>;
  }
  ScanRow() {
#define NXH_SET(DT) set<DT>();
    NXH_FOR_COMPUTE_DTYPES(NXH_SET)
#undef NXH_SET
  }
};

NXH_EXPORT int nxh_scan(nxh_context *ctx, int op, const nxh_tensor *out, const nxh_tensor *x, int axis) {
  NXH_DEFER_BARRIER(ctx, out);
  static const char *const names[NXH_REDUCE_COUNT] = {"cumsum", "cumprod", "cummax", "cummin"};
  if ((unsigned)op >= NXH_REDUCE_COUNT) return nxh_fail(NXH_INVALID_ARGUMENT, "scan", "unknown op");
  const char *name = names[op];
  if (!ctx || !out || !x) return nxh_fail(NXH_INVALID_ARGUMENT, name, "null argument");
  int rc = nxh_check_tensor(name, out);
  if (!rc) rc = nxh_check_tensor(name, x);
  if (rc) return rc;
  static const ScanRow<NXH_SUM> row_sum;
  static const ScanRow<NXH_PROD> row_prod;
  static const ScanRow<NXH_RMAX> row_max;
  static const ScanRow<NXH_RMIN> row_min;
  const scan_fn *rows[NXH_REDUCE_COUNT] = {row_sum.fn, row_prod.fn, row_max.fn, row_min.fn};
  const int dt = x->dtype;
  scan_fn fn = rows[op][dt];
  if (!fn) return nxh_fail(NXH_FAILURE, name, nxh_is_packed(dt) ? NXH_ERR_PACKED : NXH_ERR_UNSUPPORTED);
  if (out->dtype != dt) return nxh_fail(NXH_FAILURE, name, NXH_ERR_UNSUPPORTED);
  if (axis < 0 || axis >= x->ndim) return nxh_fail(NXH_INVALID_ARGUMENT, name, NXH_ERR_AXIS);
  if (out->ndim != x->ndim) return nxh_fail(NXH_INVALID_ARGUMENT, name, NXH_ERR_OUT_RANK);
  for (int d = 0; d < x->ndim; d++)
    if (out->shape[d] != x->shape[d]) return nxh_fail(NXH_INVALID_ARGUMENT, name, NXH_ERR_SHAPE);
  // the lines are the "kept" dims of a reduction over `axis`
  bool reduced[NXH_MAX_NDIM];
  nxh_tensor sq = *out;
  sq.ndim = out->ndim - 1;
  for (int d = 0, j = 0; d < x->ndim; d++) {
    reduced[d] = d == axis;
    if (d == axis) continue;
    sq.shape[j] = out->shape[d];
    sq.strides[j] = out->strides[d];
    j++;
  }
  Geom g;
  geom_build(x, &sq, reduced, &g);
  if (g.n_out == 0 || x->shape[axis] == 0) return NXH_OK;
  for (int d = 0; d < out->ndim; d++)
    if (out->shape[d] > 1 && out->strides[d] == 0) return nxh_fail(NXH_INVALID_ARGUMENT, name, NXH_ERR_OUT_ALIASED);
  if (g.nr == 0) {  // axis of length 1
    g.nr = 1;
    g.rshape[0] = 1;
    g.rin[0] = 0;
    g.R = 1;
  }
  std::lock_guard<std::mutex> guard(ctx->mu);
  NXH_HIP(name, hipSetDevice(ctx->device));
  return fn(ctx, name, x, out, g, out->strides[axis]);
}
