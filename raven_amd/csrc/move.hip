// move.hip — gather, scatter, pad, cat (packages/nx/lib/backend_c/nx_c_move.c)
// and threefry (nx_c_random.c).
//
// gather (nx_c_move.c:342-458):
// out[c] = data[c with c[axis] <- indices[c]]; int32 indices, one negative wrap,
// then a bounds check whose failure is reported by the gather call itself, as
// in the reference: kernels raise a device flag and skip the access, the host
// reads the flag back after the launch. Bytes are moved untouched (any dtype).
//   gather_rows  axis 0 of a 2-D table with a column-broadcast index (the
//                embedding lookup): one wave64 copies one row with 16-byte
//                loads.
//   gather_any   one lane per output element, per-lane unravel.
//
// scatter (nx_c_move.c:460-586): the reference walks the index space serially in
// row-major order, so `Set keeps the last write and `Add accumulates in that
// order. All updates that can meet in one output element share their
// coordinates off the scatter axis and are visited in ascending axis order, so
// one lane per off-axis coordinate ("column") walking the axis in order
// reproduces the serial result exactly, with no atomics and no race: different
// columns touch disjoint outputs. When the index is the same for every column
// (indices broadcast off the axis) and the columns alone would not fill the
// chip, the targets are split over blocks as well (scatter_rows).
//
// pad / cat (nx_c_move.c:203-312) are, as in the reference, compositions of the
// copy and fill kernels over sub-views of the output: every output element is
// written once. With a contiguous output row, pad and cat of up to 8 members
// run as ONE kernel instead (each lane decides where its 16 bytes of output
// come from).
//
// threefry (nx_c_random.c:36-133): Threefry-2x32, 20 rounds, one lane per
// (key, counter) vector; normative bit for bit.

#include "nxh_common.hpp"
#include "stream_access.hpp"

struct alignas(16) G16 {
  uint64_t lo, hi;
};

struct GatherRowsArgs {
  const char *data;
  char *out;
  const int32_t *idx;
  int64_t idx_stride, data_row_stride, out_row_stride;  // elements
  int64_t rows, row_bytes, axis_len;
  int esize;
  int *fault;
};
template <class V>
__global__ __launch_bounds__(256) void gather_rows_kernel(GatherRowsArgs a) {
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= a.rows) return;
  int64_t index = a.idx[row * a.idx_stride];
  if (index < 0) index += a.axis_len;
  if (index < 0 || index >= a.axis_len) {
    if ((threadIdx.x & 63) == 0) atomicOr(a.fault, 1);
    return;
  }
  const V *src = reinterpret_cast<const V *>(a.data + index * a.data_row_stride * a.esize);
  V *dst = reinterpret_cast<V *>(a.out + row * a.out_row_stride * a.esize);
  const int64_t nv = a.row_bytes / (int64_t)sizeof(V);
  for (int64_t i = threadIdx.x & 63; i < nv; i += 64) dst[i] = src[i];
}

struct GatherAnyArgs {
  const char *data;
  char *out;
  const int32_t *idx;
  int ndim, axis;
  int64_t total, axis_len;
  int64_t shape[NXH_MAX_NDIM];
  int64_t dstride[NXH_MAX_NDIM], istride[NXH_MAX_NDIM], ostride[NXH_MAX_NDIM];
  int *fault;
};
// N: the type the element number is unravelled in (uint32_t when the output holds fewer than 2^32
// elements). With random indices the reads, not the arithmetic, are what costs: [8192,8192] f32 along
// axis 1 takes 448 us with either type, every lane of a wave on a cache line of its own.
template <class E, class N>
__global__ __launch_bounds__(256) void gather_any_kernel(GatherAnyArgs a) {
  const int64_t it = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (it >= a.total) return;
  N rem = (N)it;
  int64_t io = 0, oo = 0, doff = 0;
  for (int d = a.ndim - 1; d >= 0; d--) {
    const N extent = (N)a.shape[d];
    const N q = rem / extent;
    const int64_t c = (int64_t)(rem - q * extent);
    rem = q;
    io += c * a.istride[d];
    oo += c * a.ostride[d];
    if (d != a.axis) doff += c * a.dstride[d];
  }
  int64_t index = a.idx[io];
  if (index < 0) index += a.axis_len;
  if (index < 0 || index >= a.axis_len) {
    atomicOr(a.fault, 1);
    return;
  }
  doff += index * a.dstride[a.axis];
  reinterpret_cast<E *>(a.out)[oo] = reinterpret_cast<const E *>(a.data)[doff];
}

static bool contiguous_off0(const nxh_tensor *a) {
  if (a->offset != 0) return false;
  int64_t s = 1;
  for (int d = a->ndim - 1; d >= 0; d--) {
    if (a->shape[d] == 1) continue;
    if (a->strides[d] != s) return false;
    s *= a->shape[d];
  }
  return true;
}

template <class E>
static void launch_any_e(nxh_context *ctx, const GatherAnyArgs &a) {
  const dim3 grid((unsigned)((a.total + 255) / 256));
  if (a.total <= 0xffffffffLL) hipLaunchKernelGGL((gather_any_kernel<E, uint32_t>), grid, dim3(256), 0, ctx->stream, a);
  else hipLaunchKernelGGL((gather_any_kernel<E, int64_t>), grid, dim3(256), 0, ctx->stream, a);
}

NXH_EXPORT int nxh_gather(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *data,
                          const nxh_tensor *indices, int axis) {
  NXH_DEFER_TOUCH(ctx, 1, out, data, indices);
  const char *op = "gather";
  if (!ctx || !out || !data || !indices) return nxh_fail(NXH_INVALID_ARGUMENT, op, "null argument");
  int rc = nxh_check_tensor(op, out);
  if (!rc) rc = nxh_check_tensor(op, data);
  if (!rc) rc = nxh_check_tensor(op, indices);
  if (rc) return rc;
  const int dt = out->dtype;
  if (nxh_is_packed(dt)) return nxh_fail(NXH_FAILURE, op, NXH_ERR_PACKED);
  if (data->dtype != dt || indices->dtype != NXH_I32) return nxh_fail(NXH_FAILURE, op, NXH_ERR_UNSUPPORTED);
  if (axis < 0 || axis >= data->ndim) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_AXIS);
  if (data->ndim != indices->ndim || data->ndim != out->ndim) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
  for (int d = 0; d < out->ndim; d++)
    if (out->shape[d] != indices->shape[d]) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
  int64_t total = 1;
  for (int d = 0; d < out->ndim; d++) total *= out->shape[d];
  if (total == 0) return NXH_OK;
  const int es = (int)nxh_elem_size(dt);
  // Every coordinate off the gathered axis also indexes `data`, so it must be in
  // range there (the reference relies on the frontend for this; out-of-range
  // reads on a device would fault the GPU, so it is checked).
  for (int d = 0; d < out->ndim; d++)
    if (d != axis && out->shape[d] > data->shape[d]) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);

  std::lock_guard<std::mutex> guard(ctx->mu);
  NXH_HIP(op, hipSetDevice(ctx->device));
  if (int frc = nxh_settle_replay_faults(ctx, op)) return frc;
  const char *dbase = (const char *)data->data + data->offset * es;
  char *obase = (char *)out->data + out->offset * es;
  const int32_t *ibase = (const int32_t *)indices->data + indices->offset;

  // embedding-style fast path (nx_c_move.c:425-432)
  if (axis == 0 && data->ndim == 2 && indices->strides[1] == 0 && data->shape[1] == out->shape[1] &&
      contiguous_off0(data) && contiguous_off0(out)) {
    GatherRowsArgs a;
    a.data = dbase;
    a.out = obase;
    a.idx = ibase;
    a.idx_stride = indices->strides[0];
    a.data_row_stride = data->strides[0];
    a.out_row_stride = out->strides[0];
    a.rows = out->shape[0];
    a.row_bytes = out->shape[1] * es;
    a.axis_len = data->shape[0];
    a.esize = es;
    a.fault = ctx->fault_flag;
    if (out->shape[0] == 1) a.out_row_stride = 0;
    if (data->shape[0] == 1) a.data_row_stride = 0;
    const unsigned blocks = (unsigned)((a.rows + 3) / 4);
    nxh_set_path("gather_rows");
    const bool v16 = a.row_bytes % 16 == 0 && ((uintptr_t)dbase % 16) == 0 && ((uintptr_t)obase % 16) == 0 &&
                     (a.data_row_stride * es) % 16 == 0 && (a.out_row_stride * es) % 16 == 0;
    if (v16) hipLaunchKernelGGL((gather_rows_kernel<G16>), dim3(blocks), dim3(256), 0, ctx->stream, a);
    else if (es == 8 || es == 16) hipLaunchKernelGGL((gather_rows_kernel<uint64_t>), dim3(blocks), dim3(256), 0, ctx->stream, a);
    else if (es == 4) hipLaunchKernelGGL((gather_rows_kernel<uint32_t>), dim3(blocks), dim3(256), 0, ctx->stream, a);
    else if (es == 2) hipLaunchKernelGGL((gather_rows_kernel<uint16_t>), dim3(blocks), dim3(256), 0, ctx->stream, a);
    else hipLaunchKernelGGL((gather_rows_kernel<uint8_t>), dim3(blocks), dim3(256), 0, ctx->stream, a);
  } else {
    GatherAnyArgs a;
    a.data = dbase;
    a.out = obase;
    a.idx = ibase;
    a.ndim = out->ndim;
    a.axis = axis;
    a.total = total;
    a.axis_len = data->shape[axis];
    for (int d = 0; d < out->ndim; d++) {
      a.shape[d] = out->shape[d];
      a.dstride[d] = data->strides[d];
      a.istride[d] = indices->strides[d];
      a.ostride[d] = out->strides[d];
    }
    a.fault = ctx->fault_flag;
    if (total > 0x7fffffffLL * 256) return nxh_fail(NXH_FAILURE, op, "too many elements for one launch");
    nxh_set_path("gather_any");
    switch (es) {
      case 1: launch_any_e<uint8_t>(ctx, a); break;
      case 2: launch_any_e<uint16_t>(ctx, a); break;
      case 4: launch_any_e<uint32_t>(ctx, a); break;
      case 8: launch_any_e<uint64_t>(ctx, a); break;
      default: launch_any_e<G16>(ctx, a); break;
    }
  }
  NXH_HIP(op, hipGetLastError());
  // Data faults surface from this call (nx_c_move.c:448-458): read the flag back.
  return nxh_collect_index_fault(ctx, op);
}

// ── scatter ─────────────────────────────────────────────────────────────────
struct ScatterArgs {
  char *out;
  const int32_t *idx;
  const char *upd;
  int ncol_dims;  // off-axis dims
  int64_t columns, n_idx, axis_len;
  int64_t cshape[NXH_MAX_NDIM];
  int64_t c_ostride[NXH_MAX_NDIM], c_istride[NXH_MAX_NDIM], c_ustride[NXH_MAX_NDIM];
  int64_t a_ostride, a_istride, a_ustride;  // along the scatter axis
  int *fault;
};
// ADD: accumulate in the dtype's compute type; otherwise a byte-exact store.
template <int DT, bool ADD>
__global__ __launch_bounds__(256) void scatter_kernel(ScatterArgs a) {
  using TR = Tr<DT>;
  using S = typename TR::S;
  using C = typename TR::C;
  const int64_t col = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (col >= a.columns) return;
  int64_t rem = col, oo = 0, io = 0, uo = 0;
  for (int d = a.ncol_dims - 1; d >= 0; d--) {
    const int64_t c = rem % a.cshape[d];
    rem /= a.cshape[d];
    oo += c * a.c_ostride[d];
    io += c * a.c_istride[d];
    uo += c * a.c_ustride[d];
  }
  S *out = reinterpret_cast<S *>(a.out) + oo;
  const int32_t *idx = a.idx + io;
  const S *upd = reinterpret_cast<const S *>(a.upd) + uo;
  auto apply = [&](S *o, S u) {
    if constexpr (ADD) {
      const C x = TR::ld(*o), y = TR::ld(u);
      if constexpr (TR::cat == CAT_SINT) *o = TR::st((C)((uint64_t)x + (uint64_t)y));
      else *o = TR::st((C)(x + y));
    } else {
      *o = u;
    }
  };
  // Steps are taken eight at a time. When their targets are pairwise distinct
  // (the common case) the eight read-modify-writes are independent and their
  // memory round trips overlap; otherwise the batch is applied one by one, in
  // order, so duplicates still see each other.
  constexpr int B = 8;
  int64_t i = 0;
  for (; i + B <= a.n_idx; i += B) {
    int64_t t[B];
    S u[B];
    bool ok = true;
#pragma unroll
    for (int j = 0; j < B; j++) {
      int64_t index = idx[(i + j) * a.a_istride];
      if (index < 0) index += a.axis_len;
      ok &= index >= 0 && index < a.axis_len;
      t[j] = index;
      u[j] = upd[(i + j) * a.a_ustride];
    }
    if (!ok) {
      atomicOr(a.fault, 1);
      return;
    }
    bool distinct = true;
#pragma unroll
    for (int j = 1; j < B; j++)
#pragma unroll
      for (int k = 0; k < j; k++) distinct &= t[j] != t[k];
    if (distinct) {
      if constexpr (ADD) {
        S cur[B];
#pragma unroll
        for (int j = 0; j < B; j++) cur[j] = out[t[j] * a.a_ostride];
#pragma unroll
        for (int j = 0; j < B; j++) {
          const C x = TR::ld(cur[j]), y = TR::ld(u[j]);
          if constexpr (TR::cat == CAT_SINT) out[t[j] * a.a_ostride] = TR::st((C)((uint64_t)x + (uint64_t)y));
          else out[t[j] * a.a_ostride] = TR::st((C)(x + y));
        }
      } else {
#pragma unroll
        for (int j = 0; j < B; j++) out[t[j] * a.a_ostride] = u[j];
      }
    } else {
      for (int j = 0; j < B; j++) apply(out + t[j] * a.a_ostride, u[j]);
    }
  }
  for (; i < a.n_idx; i++) {
    int64_t index = idx[i * a.a_istride];
    if (index < 0) index += a.axis_len;
    if (index < 0 || index >= a.axis_len) {
      atomicOr(a.fault, 1);
      return;
    }
    apply(out + index * a.a_ostride, upd[i * a.a_ustride]);
  }
}
// The index depends on the axis position only (every stride of `indices` off
// the axis is 0: the embedding-gradient shape). One lane per column leaves most
// of the chip idle there, so the targets are cut into ranges of `range_rows`
// output rows as well: block (x, y) owns 256 columns and target range y. The
// block reads the index list SPAN positions at a time, each lane SCAN of them,
// and compacts the positions whose target falls in its range into an ordered
// list in LDS (ballots and popcounts keep the ascending position order). Every
// lane then applies the listed updates to its own column in that order, eight
// at a time when their targets are pairwise distinct. Outputs of different
// blocks are disjoint and each lane sees its column's updates in the serial
// order, so the result is the reference's.
// With V > 1 a lane owns V adjacent columns, moved as one 16-byte vector (the columns of `out`
// and `updates` are then contiguous and every row starts on a 16-byte boundary: checked on the
// host); a.columns counts lanes.
template <int DT, bool ADD, int V>
__global__ __launch_bounds__(256) void scatter_rows_kernel(ScatterArgs a, int64_t range_rows) {
  using TR = Tr<DT>;
  using E = typename TR::S;
  using C = typename TR::C;
  struct alignas(V > 1 ? 16 : alignof(E)) S {
    E v[V];
  };
  constexpr int SCAN = 8, SPAN = 256 * SCAN, B = 8;
  __shared__ int s_cnt[4 * SCAN];
  __shared__ int s_pos[SPAN], s_tgt[SPAN];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int64_t col = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const bool live = col < a.columns;
  if (!live) col = a.columns - 1;  // idle lanes still take part in ballots and barriers
  int64_t oo = 0, uo = 0;
  if constexpr (V > 1) {
    oo = uo = col * V;
  } else {
    int64_t rem = col;
    for (int d = a.ncol_dims - 1; d >= 0; d--) {
      const int64_t c = rem % a.cshape[d];
      rem /= a.cshape[d];
      oo += c * a.c_ostride[d];
      uo += c * a.c_ustride[d];
    }
  }
  // (the strides along the axis are multiples of V when V > 1, so S-sized steps stay whole)
  S *out = reinterpret_cast<S *>(reinterpret_cast<E *>(a.out) + oo);
  const S *upd = reinterpret_cast<const S *>(reinterpret_cast<const E *>(a.upd) + uo);
  const int64_t a_os = a.a_ostride / V, a_us = a.a_ustride / V;
  const int64_t lo = (int64_t)blockIdx.y * range_rows, hi = lo + range_rows;
  auto combine = [](S cur, S u) -> S {
    if constexpr (ADD) {
      S r;
#pragma unroll
      for (int e = 0; e < V; e++) {
        const C x = TR::ld(cur.v[e]), y = TR::ld(u.v[e]);
        if constexpr (TR::cat == CAT_SINT) r.v[e] = TR::st((C)((uint64_t)x + (uint64_t)y));
        else r.v[e] = TR::st((C)(x + y));
      }
      return r;
    } else {
      return u;
    }
  };
  for (int64_t base = 0; base < a.n_idx; base += SPAN) {
    int t[SCAN];  // targets index an axis of the output checked to fit 31 bits
    bool bad = false;
#pragma unroll
    for (int k = 0; k < SCAN; k++) {
      const int64_t i = base + (wave * SCAN + k) * 64 + lane;
      int64_t index = i < a.n_idx ? (int64_t)a.idx[i * a.a_istride] : 0;
      if (index < 0) index += a.axis_len;
      bad |= index < 0 || index >= a.axis_len;
      t[k] = (int)index;
    }
    // also separates this pass's LDS writes from the last pass's reads
    if (__syncthreads_or(bad)) {
      if (threadIdx.x == 0) atomicOr(a.fault, 1);
      return;
    }
    uint64_t hits[SCAN];
#pragma unroll
    for (int k = 0; k < SCAN; k++) {
      const int64_t i = base + (wave * SCAN + k) * 64 + lane;
      hits[k] = __ballot(t[k] >= lo && t[k] < hi && i < a.n_idx);
      if (lane == 0) s_cnt[wave * SCAN + k] = __popcll(hits[k]);
    }
    __syncthreads();
    int off = 0;
    for (int q = 0; q < wave * SCAN; q++) off += s_cnt[q];
#pragma unroll
    for (int k = 0; k < SCAN; k++) {
      if (hits[k] >> lane & 1) {
        const int r = off + __popcll(hits[k] & ((1ull << lane) - 1));
        s_pos[r] = (wave * SCAN + k) * 64 + lane;
        s_tgt[r] = t[k];
      }
      off += __popcll(hits[k]);
    }
    __syncthreads();
    int total = 0;
    for (int q = 0; q < 4 * SCAN; q++) total += s_cnt[q];
    if (!live) continue;  // barriers are reached at the top of the next round
    int m = 0;
    for (; m + B <= total; m += B) {
      int tg[B];
      S u[B];
#pragma unroll
      for (int j = 0; j < B; j++) {
        tg[j] = s_tgt[m + j];
        u[j] = upd[(base + s_pos[m + j]) * a_us];
      }
      bool distinct = true;
#pragma unroll
      for (int j = 1; j < B; j++)
#pragma unroll
        for (int k = 0; k < j; k++) distinct &= tg[j] != tg[k];
      if (distinct) {
        S cur[B];
        if constexpr (ADD) {
#pragma unroll
          for (int j = 0; j < B; j++) cur[j] = out[(int64_t)tg[j] * a_os];
        }
#pragma unroll
        for (int j = 0; j < B; j++) out[(int64_t)tg[j] * a_os] = combine(cur[j], u[j]);
      } else {
        for (int j = 0; j < B; j++) {
          S *o = out + (int64_t)tg[j] * a_os;
          *o = combine(*o, u[j]);
        }
      }
    }
    for (; m < total; m++) {
      S *o = out + (int64_t)s_tgt[m] * a_os;
      *o = combine(*o, upd[(base + s_pos[m]) * a_us]);
    }
  }
}
typedef void (*scatter_launch_fn)(nxh_context *, const ScatterArgs &, bool, int64_t, bool);
// range_rows > 0 selects the kernel that also splits the targets into ranges; `vec` its form
// with 16 bytes of columns per lane (a.columns then counts lanes).
template <int DT>
static void scatter_launch(nxh_context *ctx, const ScatterArgs &a, bool add, int64_t range_rows, bool vec) {
  const unsigned col_blocks = (unsigned)((a.columns + 255) / 256);
  if (range_rows > 0) {
    const dim3 grid(col_blocks, (unsigned)((a.axis_len + range_rows - 1) / range_rows));
    constexpr int V = 16 / (int)sizeof(typename Tr<DT>::S);
    if constexpr (V > 1) {
      if (vec) {
        if (add) hipLaunchKernelGGL((scatter_rows_kernel<DT, true, V>), grid, dim3(256), 0, ctx->stream, a, range_rows);
        else hipLaunchKernelGGL((scatter_rows_kernel<DT, false, V>), grid, dim3(256), 0, ctx->stream, a, range_rows);
        return;
      }
    }
    if (add) hipLaunchKernelGGL((scatter_rows_kernel<DT, true, 1>), grid, dim3(256), 0, ctx->stream, a, range_rows);
    else hipLaunchKernelGGL((scatter_rows_kernel<DT, false, 1>), grid, dim3(256), 0, ctx->stream, a, range_rows);
    return;
  }
  const dim3 grid(col_blocks);
  if (add) hipLaunchKernelGGL((scatter_kernel<DT, true>), grid, dim3(256), 0, ctx->stream, a);
  else hipLaunchKernelGGL((scatter_kernel<DT, false>), grid, dim3(256), 0, ctx->stream, a);
}

// ── scatter of one column (a vector's scatter: histograms, bin counts) ──────
// With a single column the kernels above have one lane per block to apply the updates with, and
// every block reads the whole index list (2^20 updates into 1000 bins: 2.1 ms). Here the updates
// are put in target order by a stable argsort of the (normalised) indices, and the first lane of
// every target's run applies the run in its order, which is index order: the serial result, no
// atomics. A lane's work is its target's number of updates.
__global__ __launch_bounds__(256) void scatter_keys_kernel(const int32_t *idx, int64_t stride, int64_t n, int64_t axis_len,
                                                           int32_t *key, int *fault) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  int64_t v = idx[i * stride];
  if (v < 0) v += axis_len;
  if (v < 0 || v >= axis_len) {
    atomicOr(fault, 1);
    v = -1;  // sorts first, applied by nobody
  }
  key[i] = (int32_t)v;
}
template <int DT, bool ADD>
__global__ __launch_bounds__(256) void scatter_sorted_kernel(const int32_t *key, const int32_t *perm, int64_t n, char *out_c,
                                                             int64_t os, const char *upd_c, int64_t us) {
  using TR = Tr<DT>;
  using S = typename TR::S;
  using C = typename TR::C;
  const int64_t p = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (p >= n) return;
  const int32_t k = key[perm[p]];
  if (k < 0 || (p > 0 && key[perm[p - 1]] == k)) return;  // out of range, or not the first of its target
  S *o = reinterpret_cast<S *>(out_c) + (int64_t)k * os;
  const S *upd = reinterpret_cast<const S *>(upd_c);
  S acc = *o;
  auto apply = [&](S u) {
    if constexpr (ADD) {
      const C x = TR::ld(acc), y = TR::ld(u);
      if constexpr (TR::cat == CAT_SINT) acc = TR::st((C)((uint64_t)x + (uint64_t)y));
      else acc = TR::st((C)(x + y));
    } else {
      acc = u;
    }
  };
  // eight positions at a time: their indices, targets and updates are fetched together, only the
  // additions wait for one another (a run of a thousand updates is a thousand dependent trips to
  // memory otherwise)
  constexpr int B = 8;
  int64_t q = p;
  bool more = true;
  while (more && q + B <= n) {
    int32_t i[B], t[B];
    S u[B];
#pragma unroll
    for (int j = 0; j < B; j++) i[j] = perm[q + j];
#pragma unroll
    for (int j = 0; j < B; j++) t[j] = key[i[j]];
#pragma unroll
    for (int j = 0; j < B; j++) u[j] = upd[(int64_t)i[j] * us];
#pragma unroll
    for (int j = 0; j < B; j++) {
      more = more && t[j] == k;
      if (more) apply(u[j]);
    }
    q += B;
  }
  for (; more && q < n; q++) {
    const int32_t i = perm[q];
    if (key[i] != k) break;
    apply(upd[(int64_t)i * us]);
  }
  *o = acc;
}
typedef void (*scatter_sorted_fn)(nxh_context *, const int32_t *, const int32_t *, const ScatterArgs &, bool);
template <int DT>
static void scatter_sorted_launch(nxh_context *ctx, const int32_t *key, const int32_t *perm, const ScatterArgs &a, bool add) {
  const dim3 grid((unsigned)((a.n_idx + 255) / 256));
  if (add) hipLaunchKernelGGL((scatter_sorted_kernel<DT, true>), grid, dim3(256), 0, ctx->stream, key, perm, a.n_idx, a.out,
                              a.a_ostride, a.upd, a.a_ustride);
  else hipLaunchKernelGGL((scatter_sorted_kernel<DT, false>), grid, dim3(256), 0, ctx->stream, key, perm, a.n_idx, a.out,
                          a.a_ostride, a.upd, a.a_ustride);
}
static int scatter_sorted(nxh_context *ctx, const char *op, const ScatterArgs &a, int dt, bool add) {
  struct Table {
    scatter_sorted_fn fn[NXH_DTYPE_COUNT] = {};
    Table() {
#define NXH_SC(DT) fn[DT] = &scatter_sorted_launch<DT>;
      NXH_FOR_COMPUTE_DTYPES(NXH_SC)
#undef NXH_SC
    }
  };
  static const Table table;
  if (!table.fn[dt]) return -1;
  // several calls in a row: no capture may begin between them (it would record the later launches
  // with blocks that are freed below)
  std::lock_guard<std::mutex> whole_call(ctx->call_mu);
  if (ctx->capture) return -1;
  void *key = nullptr, *perm = nullptr;
  const size_t bytes = (size_t)a.n_idx * sizeof(int32_t);
  int rc = nxh_alloc(ctx, bytes, &key);
  if (!rc) rc = nxh_alloc(ctx, bytes, &perm);
  if (!rc) {
    std::lock_guard<std::mutex> guard(ctx->mu);
    rc = nxh_settle_replay_faults(ctx, op);
    if (!rc) {
      hipLaunchKernelGGL(scatter_keys_kernel, dim3((unsigned)((a.n_idx + 255) / 256)), dim3(256), 0, ctx->stream, a.idx,
                         a.a_istride, a.n_idx, a.axis_len, (int32_t *)key, a.fault);
      if (hipGetLastError() != hipSuccess) rc = nxh_fail(NXH_FAILURE, op, "launch failed");
    }
  }
  if (!rc) {
    nxh_tensor kt{}, pt{};
    kt.data = key;
    pt.data = perm;
    kt.dtype = pt.dtype = NXH_I32;
    kt.ndim = pt.ndim = 1;
    kt.shape[0] = pt.shape[0] = a.n_idx;
    kt.strides[0] = pt.strides[0] = 1;
    rc = nxh_argsort(ctx, &pt, &kt, 0, 0);  // stable: equal targets stay in index order
  }
  if (!rc) {
    std::lock_guard<std::mutex> guard(ctx->mu);
    nxh_set_path("scatter_sorted");
    table.fn[dt](ctx, (const int32_t *)key, (const int32_t *)perm, a, add);
    if (hipGetLastError() != hipSuccess) rc = nxh_fail(NXH_FAILURE, op, "launch failed");
    else rc = nxh_collect_index_fault(ctx, op);
  }
  if (key) (void)nxh_free(ctx, key);
  if (perm) (void)nxh_free(ctx, perm);
  return rc;
}

NXH_EXPORT int nxh_scatter(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *indices,
                           const nxh_tensor *updates, int axis, int mode) {
  NXH_DEFER_TOUCH(ctx, 1, out, indices, updates);
  const char *op = "scatter";
  if (!ctx || !out || !indices || !updates) return nxh_fail(NXH_INVALID_ARGUMENT, op, "null argument");
  int rc = nxh_check_tensor(op, out);
  if (!rc) rc = nxh_check_tensor(op, indices);
  if (!rc) rc = nxh_check_tensor(op, updates);
  if (rc) return rc;
  const int dt = out->dtype;
  if (nxh_is_packed(dt)) return nxh_fail(NXH_FAILURE, op, NXH_ERR_PACKED);
  if (updates->dtype != dt || indices->dtype != NXH_I32) return nxh_fail(NXH_FAILURE, op, NXH_ERR_UNSUPPORTED);
  if (mode != 0 && mode != 1) return nxh_fail(NXH_INVALID_ARGUMENT, op, "mode must be 0 (set) or 1 (add)");
  if (axis < 0 || axis >= out->ndim) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_AXIS);
  if (out->ndim != indices->ndim || out->ndim != updates->ndim) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
  for (int d = 0; d < out->ndim; d++) {
    if (indices->shape[d] != updates->shape[d]) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
    if (d != axis && indices->shape[d] != out->shape[d]) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
  }
  for (int d = 0; d < out->ndim; d++)
    if (out->shape[d] > 1 && out->strides[d] == 0) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_OUT_ALIASED);
  ScatterArgs a;
  a.columns = 1;
  a.ncol_dims = 0;
  for (int d = 0; d < out->ndim; d++) {
    if (d == axis) continue;
    a.cshape[a.ncol_dims] = indices->shape[d];
    a.c_ostride[a.ncol_dims] = out->strides[d];
    a.c_istride[a.ncol_dims] = indices->strides[d];
    a.c_ustride[a.ncol_dims] = updates->strides[d];
    a.columns *= indices->shape[d];
    a.ncol_dims++;
  }
  a.n_idx = indices->shape[axis];
  if (a.columns == 0 || a.n_idx == 0) return NXH_OK;
  if (a.columns > 0x7fffffffLL * 256) return nxh_fail(NXH_FAILURE, op, "too many elements for one launch");
  const int64_t es = nxh_elem_size(dt);
  a.out = (char *)out->data + out->offset * es;
  a.idx = (const int32_t *)indices->data + indices->offset;
  a.upd = (const char *)updates->data + updates->offset * es;
  a.axis_len = out->shape[axis];
  a.a_ostride = out->strides[axis];
  a.a_istride = indices->strides[axis];
  a.a_ustride = updates->strides[axis];
  a.fault = ctx->fault_flag;
  struct Table {
    scatter_launch_fn fn[NXH_DTYPE_COUNT] = {};
    Table() {
#define NXH_SC(DT) fn[DT] = &scatter_launch<DT>;
      NXH_FOR_COMPUTE_DTYPES(NXH_SC)
#undef NXH_SC
    }
  };
  static const Table table_;
  const scatter_launch_fn *table = table_.fn;
  if (!table[dt]) return nxh_fail(NXH_FAILURE, op, NXH_ERR_UNSUPPORTED);
  if (a.columns == 1 && a.n_idx >= 4096 && a.n_idx <= 0x3fffffffLL && a.axis_len <= 0x7fffffffLL && !ctx->capture) {
    const int src = scatter_sorted(ctx, op, a, dt, mode == 1);
    if (src != -1) return src;
  }
  std::lock_guard<std::mutex> guard(ctx->mu);
  NXH_HIP(op, hipSetDevice(ctx->device));
  if (int frc = nxh_settle_replay_faults(ctx, op)) return frc;
  // Too few columns to fill the chip and one index per axis position: split the
  // targets over blocks too. The index list is read once per block, so this
  // pays only while the list is short next to the rows it spreads over.
  bool uniform_index = a.axis_len <= 0x7fffffffLL;
  for (int d = 0; d < a.ncol_dims; d++)
    if (a.cshape[d] > 1 && a.c_istride[d] != 0) uniform_index = false;
  // 16 bytes of columns per lane: the off-axis dims of `out` and `updates` are one contiguous
  // run, a whole number of vectors long, and every row of both starts on a 16-byte boundary
  // (embedding gradient [8192, 768] f32 into [50257, 768]: 38 -> 33 us)
  bool vec = uniform_index && es < 16 && a.columns % (16 / es) == 0 && a.a_ostride % (16 / es) == 0 &&
             a.a_ustride % (16 / es) == 0 && ((uintptr_t)a.out | (uintptr_t)a.upd) % 16 == 0;
  for (int64_t d = a.ncol_dims - 1, run = 1; d >= 0 && vec; d--) {
    if (a.cshape[d] > 1 && (a.c_ostride[d] != run || a.c_ustride[d] != run)) vec = false;
    run *= a.cshape[d];
  }
  int64_t range_rows = 0;
  const int64_t lanes = vec ? a.columns / (16 / es) : a.columns;
  const int64_t col_blocks = (lanes + 255) / 256;
  const int64_t want_blocks = (int64_t)ctx->compute_units * 3;  // measured best on the embedding-gradient shape
  if (uniform_index && a.n_idx >= 256 && col_blocks * 4 <= want_blocks) {
    int64_t ranges = want_blocks / col_blocks;
    if (ranges > a.axis_len) ranges = a.axis_len;
    if (ranges > 65535) ranges = 65535;
    if (ranges >= 2) range_rows = (a.axis_len + ranges - 1) / ranges;
  }
  vec = vec && range_rows > 0;
  if (vec) a.columns = lanes;
  nxh_set_path(vec ? "scatter_rows_16B" : range_rows > 0 ? "scatter_rows" : "scatter_columns");
  table[dt](ctx, a, mode == 1, range_rows, vec);
  NXH_HIP(op, hipGetLastError());
  return nxh_collect_index_fault(ctx, op);
}

// ── threefry2x32-20 ─────────────────────────────────────────────────────────
struct ThreefryArgs {
  const int32_t *key, *ctr;
  int32_t *out;
  int prefix_ndim;
  int64_t vectors;
  int64_t shape[NXH_MAX_NDIM];
  int64_t kstride[NXH_MAX_NDIM], cstride[NXH_MAX_NDIM], ostride[NXH_MAX_NDIM];
  int64_t key_last, ctr_last, out_last;  // stride of the 2-word axis
};
__device__ __forceinline__ uint32_t rotl32(uint32_t x, int r) { return (x << r) | (x >> (32 - r)); }
__global__ __launch_bounds__(256) void threefry_kernel(ThreefryArgs a) {
  const int64_t it = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (it >= a.vectors) return;
  int64_t rem = it, kb = 0, cb = 0, ob = 0;
  for (int d = a.prefix_ndim - 1; d >= 0; d--) {
    const int64_t c = rem % a.shape[d];
    rem /= a.shape[d];
    kb += c * a.kstride[d];
    cb += c * a.cstride[d];
    ob += c * a.ostride[d];
  }
  const uint32_t k0 = (uint32_t)a.key[kb], k1 = (uint32_t)a.key[kb + a.key_last];
  const uint32_t ks[3] = {k0, k1, 0x1BD11BDAu ^ k0 ^ k1};
  uint32_t x0 = (uint32_t)a.ctr[cb] + k0, x1 = (uint32_t)a.ctr[cb + a.ctr_last] + k1;
  constexpr int rots[8] = {13, 15, 26, 6, 17, 29, 16, 24};
#pragma unroll
  for (int r = 0; r < 20; r++) {
    x0 += x1;
    x1 = rotl32(x1, rots[r % 8]);
    x1 ^= x0;
    if ((r + 1) % 4 == 0) {
      const int s = (r + 1) / 4;
      x0 += ks[s % 3];
      x1 += ks[(s + 1) % 3] + (uint32_t)s;
    }
  }
  a.out[ob] = (int32_t)x0;
  a.out[ob + a.out_last] = (int32_t)x1;
}

// The dense form: counters and results are contiguous (vector, word) pairs, the keys one pair
// for all vectors or dense too. A lane takes two neighbouring vectors with one 16-byte load and
// one 16-byte store (two independent chains of rounds) and no division; a lane per vector with
// 4-byte accesses and a 64-bit division left the call at half the memory rate.
__device__ __forceinline__ void threefry_block(uint32_t k0, uint32_t k1, uint32_t &x0, uint32_t &x1) {
  const uint32_t ks[3] = {k0, k1, 0x1BD11BDAu ^ k0 ^ k1};
  x0 += k0;
  x1 += k1;
  constexpr int rots[8] = {13, 15, 26, 6, 17, 29, 16, 24};
#pragma unroll
  for (int r = 0; r < 20; r++) {
    x0 += x1;
    x1 = rotl32(x1, rots[r % 8]);
    x1 ^= x0;
    if ((r + 1) % 4 == 0) {
      const int s = (r + 1) / 4;
      x0 += ks[s % 3];
      x1 += ks[(s + 1) % 3] + (uint32_t)s;
    }
  }
}
__global__ __launch_bounds__(256) void threefry_dense_kernel(const int32_t *key, int64_t key_step, int64_t key_last,
                                                             const int32_t *ctr, int32_t *out, int64_t vectors) {
  typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
  const int64_t v = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 2;
  if (v >= vectors) return;
  const uint32_t ka0 = (uint32_t)key[v * key_step], ka1 = (uint32_t)key[v * key_step + key_last];
  if (v + 1 < vectors) {
    const uint32_t kb0 = (uint32_t)key[(v + 1) * key_step], kb1 = (uint32_t)key[(v + 1) * key_step + key_last];
    const u32x4 x = *reinterpret_cast<const u32x4 *>(ctr + 2 * v);
    uint32_t a0 = x[0], a1 = x[1], b0 = x[2], b1 = x[3];
    threefry_block(ka0, ka1, a0, a1);
    threefry_block(kb0, kb1, b0, b1);
    *reinterpret_cast<u32x4 *>(out + 2 * v) = u32x4{a0, a1, b0, b1};
  } else {
    uint32_t x0 = (uint32_t)ctr[2 * v], x1 = (uint32_t)ctr[2 * v + 1];
    threefry_block(ka0, ka1, x0, x1);
    out[2 * v] = (int32_t)x0;
    out[2 * v + 1] = (int32_t)x1;
  }
}

NXH_EXPORT int nxh_threefry(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *key,
                            const nxh_tensor *counter) {
  NXH_DEFER_TOUCH(ctx, 1, out, key, counter);
  const char *op = "threefry";
  if (!ctx || !out || !key || !counter) return nxh_fail(NXH_INVALID_ARGUMENT, op, "null argument");
  int rc = nxh_check_tensor(op, out);
  if (!rc) rc = nxh_check_tensor(op, key);
  if (!rc) rc = nxh_check_tensor(op, counter);
  if (rc) return rc;
  if (out->dtype != NXH_I32 || key->dtype != NXH_I32 || counter->dtype != NXH_I32)
    return nxh_fail(NXH_FAILURE, op, NXH_ERR_UNSUPPORTED);
  const char *bad = "threefry: last axis must have extent 2";
  if (key->ndim < 1 || key->ndim != counter->ndim || key->ndim != out->ndim) return nxh_fail(NXH_INVALID_ARGUMENT, op, bad);
  const int last = key->ndim - 1;
  for (int d = 0; d < key->ndim; d++)
    if (key->shape[d] != counter->shape[d] || key->shape[d] != out->shape[d]) return nxh_fail(NXH_INVALID_ARGUMENT, op, bad);
  if (key->shape[last] != 2) return nxh_fail(NXH_INVALID_ARGUMENT, op, bad);
  ThreefryArgs a;
  a.vectors = 1;
  a.prefix_ndim = last;
  for (int d = 0; d < last; d++) {
    a.shape[d] = key->shape[d];
    a.kstride[d] = key->strides[d];
    a.cstride[d] = counter->strides[d];
    a.ostride[d] = out->strides[d];
    a.vectors *= key->shape[d];
  }
  if (a.vectors == 0) return NXH_OK;
  if (a.vectors > 0x7fffffffLL * 256) return nxh_fail(NXH_FAILURE, op, "too many elements for one launch");
  a.key = (const int32_t *)key->data + key->offset;
  a.ctr = (const int32_t *)counter->data + counter->offset;
  a.out = (int32_t *)out->data + out->offset;
  a.key_last = key->strides[last];
  a.ctr_last = counter->strides[last];
  a.out_last = out->strides[last];
  std::lock_guard<std::mutex> guard(ctx->mu);
  NXH_HIP(op, hipSetDevice(ctx->device));
  // dense: every prefix dim composes with the next on all three operands, pairs are contiguous
  bool dense = last >= 1 && a.ctr_last == 1 && a.out_last == 1 && a.cstride[last - 1] == 2 && a.ostride[last - 1] == 2 &&
               ((uintptr_t)a.ctr % 16) == 0 && ((uintptr_t)a.out % 16) == 0;
  for (int d = last - 2; dense && d >= 0; d--)
    dense = a.cstride[d] == a.cstride[d + 1] * a.shape[d + 1] && a.ostride[d] == a.ostride[d + 1] * a.shape[d + 1] &&
            a.kstride[d] == a.kstride[d + 1] * a.shape[d + 1];
  if (dense) {
    nxh_set_path("threefry_dense");
    hipLaunchKernelGGL(threefry_dense_kernel, dim3((unsigned)((a.vectors + 511) / 512)), dim3(256), 0, ctx->stream, a.key,
                       a.kstride[last - 1], a.key_last, a.ctr, a.out, a.vectors);
    NXH_HIP(op, hipGetLastError());
    return NXH_OK;
  }
  nxh_set_path("threefry");
  hipLaunchKernelGGL(threefry_kernel, dim3((unsigned)((a.vectors + 255) / 256)), dim3(256), 0, ctx->stream, a);
  NXH_HIP(op, hipGetLastError());
  return NXH_OK;
}

// ── pad / cat: compositions of fill and copy over sub-views of the output ──
static bool has_zero_extent(const nxh_tensor *t) {
  for (int d = 0; d < t->ndim; d++)
    if (t->shape[d] == 0) return true;
  return false;
}

// The fused form: one lane per VP consecutive outputs of a row; each output is
// either the fill value or the input element `before` positions earlier. Used
// when rows are contiguous on both sides; the slab composition below covers the
// rest.
constexpr int PAD_MAXD = 8;
struct PadArgs {
  char *out;
  const char *in;
  int ndim;
  int64_t units;                 // lanes: outputs / VP
  uint32_t oshape[PAD_MAXD];     // out extents; the last one in units of VP elements
  int64_t ostride[PAD_MAXD], istride[PAD_MAXD];  // elements (outer dims)
  int64_t before[PAD_MAXD], ishape[PAD_MAXD];
  unsigned char fill[16];
  uint32_t stream_out;  // the stores go past the memory-side cache (decided per call, runtime.hip nxh_cache_hints)
};
template <class E, int VP>
__global__ __launch_bounds__(256) void pad_kernel(PadArgs a) {
  const int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (u >= a.units) return;
  int64_t rem = u, oo = 0, io = 0;
  bool inside = true;
  int64_t x0 = 0;
  for (int d = a.ndim - 1; d >= 0; d--) {
    const int64_t c = rem % a.oshape[d];
    rem /= a.oshape[d];
    if (d == a.ndim - 1) {
      x0 = c * VP;
      oo += x0;
    } else {
      oo += c * a.ostride[d];
      const int64_t ci = c - a.before[d];
      inside &= ci >= 0 && ci < a.ishape[d];
      io += ci * a.istride[d];
    }
  }
  const int last = a.ndim - 1;
  E fill;
  __builtin_memcpy(&fill, a.fill, sizeof(E));
  E v[VP];
  const int64_t xi = x0 - a.before[last];
  const E *src = reinterpret_cast<const E *>(a.in) + io + xi;
  if (inside && xi >= 0 && xi + VP <= a.ishape[last]) {
    // element-aligned only: the interior is shifted against the input by `before`
#pragma unroll
    for (int j = 0; j < VP; j++) v[j] = src[j];
  } else {
#pragma unroll
    for (int j = 0; j < VP; j++) v[j] = (inside && xi + j >= 0 && xi + j < a.ishape[last]) ? src[j] : fill;
  }
  struct alignas(sizeof(E) * VP >= 16 ? 16 : sizeof(E) * VP) Pack {
    E v[VP];
  } pk;
#pragma unroll
  for (int j = 0; j < VP; j++) pk.v[j] = v[j];
  Pack *dst = reinterpret_cast<Pack *>(reinterpret_cast<E *>(a.out) + oo);
  if (a.stream_out) store_stream(dst, pk);
  else *dst = pk;
}
template <class E>
static void pad_launch(nxh_context *ctx, const PadArgs &a, int vp) {
  const dim3 grid((unsigned)((a.units + 255) / 256));
  constexpr int VMAX = 16 / (int)sizeof(E) > 0 ? 16 / (int)sizeof(E) : 1;
  if (vp == VMAX && VMAX > 1) hipLaunchKernelGGL((pad_kernel<E, VMAX>), grid, dim3(256), 0, ctx->stream, a);
  else hipLaunchKernelGGL((pad_kernel<E, 1>), grid, dim3(256), 0, ctx->stream, a);
}
// Returns -1 when the call does not qualify for the fused kernel.
static int pad_fused(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x, const void *fill_value,
                     const int64_t *pad_before) {
  const int nd = out->ndim;
  if (nd < 1 || nd > PAD_MAXD) return -1;
  if (out->strides[nd - 1] != 1 || (x->strides[nd - 1] != 1 && x->shape[nd - 1] > 1)) return -1;
  const int es = (int)nxh_elem_size(out->dtype);
  int64_t total = 1;
  for (int d = 0; d < nd; d++) total *= out->shape[d];
  if (total == 0) return NXH_OK;
  for (int d = 0; d < nd; d++)
    if (out->shape[d] > 0xffffffffLL || (d < nd - 1 && out->strides[d] <= 0)) return -1;
  PadArgs a;
  a.out = (char *)out->data + out->offset * es;
  a.in = (const char *)x->data + x->offset * es;
  a.ndim = nd;
  const int vmax = 16 / es > 0 ? 16 / es : 1;
  bool vec = vmax > 1 && out->shape[nd - 1] % vmax == 0 && ((uintptr_t)a.out % 16) == 0;
  for (int d = 0; d < nd - 1 && vec; d++)
    if (out->shape[d] > 1 && out->strides[d] % vmax != 0) vec = false;
  const int vp = vec ? vmax : 1;
  for (int d = 0; d < nd; d++) {
    a.oshape[d] = (uint32_t)(d == nd - 1 ? out->shape[d] / vp : out->shape[d]);
    a.ostride[d] = out->strides[d];
    a.istride[d] = x->strides[d];
    a.before[d] = pad_before[d];
    a.ishape[d] = x->shape[d];
  }
  a.units = total / vp;
  if (a.units > 0x7fffffffLL * 256) return -1;
  memset(a.fill, 0, sizeof a.fill);
  memcpy(a.fill, fill_value, (size_t)es);
  std::lock_guard<std::mutex> guard(ctx->mu);
  NXH_HIP("pad", hipSetDevice(ctx->device));
  nxh_set_path("pad_fused");
  {
    uint64_t in_elems = 1;
    for (int d = 0; d < nd; d++)
      if (x->strides[d] != 0) in_elems *= (uint64_t)x->shape[d];
    const void *base[2] = {out->data, x->data};
    const uint64_t bytes[2] = {(uint64_t)total * (uint64_t)es, in_elems * (uint64_t)es};
    a.stream_out = nxh_cache_hints(ctx, 2, base, bytes, NXH_STREAM_OUT) & NXH_STREAM_OUT;
  }
  switch (es) {
    case 1: pad_launch<uint8_t>(ctx, a, vp); break;
    case 2: pad_launch<uint16_t>(ctx, a, vp); break;
    case 4: pad_launch<uint32_t>(ctx, a, vp); break;
    case 8: pad_launch<uint64_t>(ctx, a, vp); break;
    default: pad_launch<G16>(ctx, a, vp); break;
  }
  NXH_HIP("pad", hipGetLastError());
  return NXH_OK;
}

NXH_EXPORT int nxh_pad(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x, const void *fill_value,
                       const int64_t *pad_before) {
  NXH_DEFER_SETTLE(ctx, 1, out, x);  // (the fused kernel asks the cache policy itself; fills and copies do their own accounting)
  const char *op = "pad";
  if (!ctx || !out || !x || !fill_value || (out->ndim > 0 && !pad_before))
    return nxh_fail(NXH_INVALID_ARGUMENT, op, "null argument");
  int rc = nxh_check_tensor(op, out);
  if (!rc) rc = nxh_check_tensor(op, x);
  if (rc) return rc;
  if (out->ndim != x->ndim) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
  if (nxh_is_packed(out->dtype)) return nxh_fail(NXH_FAILURE, op, NXH_ERR_PACKED);
  if (out->dtype != x->dtype) return nxh_fail(NXH_FAILURE, op, NXH_ERR_UNSUPPORTED);
  for (int d = 0; d < out->ndim; d++)
    if (pad_before[d] < 0 || out->shape[d] - x->shape[d] - pad_before[d] < 0)
      return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
  for (int d = 0; d < out->ndim; d++)
    if (out->shape[d] > 1 && out->strides[d] == 0) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_OUT_ALIASED);
  rc = pad_fused(ctx, out, x, fill_value, pad_before);
  if (rc != -1) return rc;
  // `slab` narrows toward the interior: entering step d, axes < d carry the
  // interior extent and offset, axes >= d are still full (nx_c_move.c:246-268)
  nxh_tensor slab = *out;
  for (int d = 0; d < out->ndim; d++) {
    const int64_t before = pad_before[d];
    const int64_t after = out->shape[d] - x->shape[d] - before;
    if (before > 0) {
      slab.shape[d] = before;
      if (!has_zero_extent(&slab) && (rc = nxh_fill(ctx, &slab, fill_value))) return rc;
    }
    if (after > 0) {
      slab.shape[d] = after;
      slab.offset += (before + x->shape[d]) * out->strides[d];
      if (!has_zero_extent(&slab) && (rc = nxh_fill(ctx, &slab, fill_value))) return rc;
      slab.offset -= (before + x->shape[d]) * out->strides[d];
    }
    slab.shape[d] = x->shape[d];
    slab.offset += before * out->strides[d];
  }
  rc = nxh_copy(ctx, &slab, x);
  nxh_set_path("pad_slabs");
  return rc;
}

// The fused form of cat: one kernel for up to CAT_MAXM members; a lane owns VP
// consecutive outputs of a row, finds the member its axis coordinate falls in
// and reads that member through its own strides.
constexpr int CAT_MAXM = 8;
struct CatArgs {
  char *out;
  const char *in[CAT_MAXM];
  int ndim, axis, n;
  uint32_t whole;  // bit m: a lane's VP outputs inside member m are one aligned vector of it
  int64_t units;
  uint32_t oshape[PAD_MAXD];  // out extents; the last one in units of VP elements
  int64_t ostride[PAD_MAXD];
  int64_t istride[CAT_MAXM][PAD_MAXD];
  int64_t start[CAT_MAXM + 1];  // first axis coordinate of each member, and the end
  uint32_t stream_out;          // as in PadArgs
};
template <class E, int VP>
__global__ __launch_bounds__(256) void cat_kernel(CatArgs a) {
  const int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (u >= a.units) return;
  int64_t coord[PAD_MAXD], rem = u, oo = 0;
  const int last = a.ndim - 1;
  for (int d = last; d >= 0; d--) {
    const int64_t c = rem % a.oshape[d];
    rem /= a.oshape[d];
    coord[d] = d == last ? c * VP : c;
    oo += coord[d] * (d == last ? 1 : a.ostride[d]);
  }
  struct alignas(sizeof(E) * VP >= 16 ? 16 : sizeof(E) * VP) Pack {
    E v[VP];
  } pk;
  int m0 = 0;
  while (m0 + 1 < a.n && coord[a.axis] >= a.start[m0 + 1]) m0++;
  if (VP == 1 || (a.whole >> m0 & 1)) {
    // all VP outputs come from VP consecutive, aligned elements of member m0
    int64_t io = 0;
    for (int d = 0; d < a.ndim; d++) io += (coord[d] - (d == a.axis ? a.start[m0] : 0)) * a.istride[m0][d];
    pk = *reinterpret_cast<const Pack *>(reinterpret_cast<const E *>(a.in[m0]) + io);
  } else {
#pragma unroll
    for (int j = 0; j < VP; j++) {
      const int64_t ax = coord[a.axis] + (a.axis == last ? j : 0);
      int m = m0;
      while (m + 1 < a.n && ax >= a.start[m + 1]) m++;
      int64_t io = 0;
      for (int d = 0; d < a.ndim; d++) {
        int64_t c = coord[d] + (d == last ? j : 0);
        if (d == a.axis) c -= a.start[m];
        io += c * a.istride[m][d];
      }
      pk.v[j] = reinterpret_cast<const E *>(a.in[m])[io];
    }
  }
  Pack *dst = reinterpret_cast<Pack *>(reinterpret_cast<E *>(a.out) + oo);
  if (a.stream_out) store_stream(dst, pk);
  else *dst = pk;
}
template <class E>
static void cat_launch(nxh_context *ctx, const CatArgs &a, int vp) {
  const dim3 grid((unsigned)((a.units + 255) / 256));
  constexpr int VMAX = 16 / (int)sizeof(E) > 0 ? 16 / (int)sizeof(E) : 1;
  if (vp == VMAX && VMAX > 1) hipLaunchKernelGGL((cat_kernel<E, VMAX>), grid, dim3(256), 0, ctx->stream, a);
  else hipLaunchKernelGGL((cat_kernel<E, 1>), grid, dim3(256), 0, ctx->stream, a);
}
// Returns -1 when the call does not qualify (then the per-member copies run).
static int cat_fused(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *const *inputs, int n, int axis) {
  const int nd = out->ndim;
  if (n < 2 || n > CAT_MAXM || nd < 1 || nd > PAD_MAXD || out->strides[nd - 1] != 1) return -1;
  const int es = (int)nxh_elem_size(out->dtype);
  if (es == 0) return -1;
  int64_t total = 1;
  for (int d = 0; d < nd; d++) {
    if (out->shape[d] > 0xffffffffLL || (d < nd - 1 && out->shape[d] > 1 && out->strides[d] <= 0)) return -1;
    total *= out->shape[d];
  }
  if (total == 0) return NXH_OK;
  CatArgs a;
  a.out = (char *)out->data + out->offset * es;
  a.ndim = nd;
  a.axis = axis;
  a.n = n;
  int64_t pos = 0;
  for (int m = 0; m < n; m++) {
    a.in[m] = (const char *)inputs[m]->data + inputs[m]->offset * es;
    a.start[m] = pos;
    pos += inputs[m]->shape[axis];
    for (int d = 0; d < nd; d++) a.istride[m][d] = inputs[m]->strides[d];
  }
  a.start[n] = pos;
  if (pos != out->shape[axis]) return -1;
  const int vmax = 16 / es > 0 ? 16 / es : 1;
  bool vec = vmax > 1 && out->shape[nd - 1] % vmax == 0 && ((uintptr_t)a.out % 16) == 0;
  for (int d = 0; d < nd - 1 && vec; d++)
    if (out->shape[d] > 1 && out->strides[d] % vmax != 0) vec = false;
  const int vp = vec ? vmax : 1;
  for (int d = 0; d < nd; d++) {
    a.oshape[d] = (uint32_t)(d == nd - 1 ? out->shape[d] / vp : out->shape[d]);
    a.ostride[d] = out->strides[d];
  }
  a.units = total / vp;
  if (a.units > 0x7fffffffLL * 256) return -1;
  a.whole = 0;
  for (int m = 0; m < n && vp > 1; m++) {
    const nxh_tensor *in = inputs[m];
    bool ok = in->strides[nd - 1] == 1 && ((uintptr_t)a.in[m] % 16) == 0;
    for (int d = 0; d < nd - 1 && ok; d++)
      if (in->shape[d] > 1 && in->strides[d] % vp != 0) ok = false;
    // along the last axis a vector must not straddle two members
    if (axis == nd - 1 && (a.start[m] % vp != 0 || in->shape[axis] % vp != 0)) ok = false;
    if (ok) a.whole |= 1u << m;
  }
  std::lock_guard<std::mutex> guard(ctx->mu);
  NXH_HIP("cat", hipSetDevice(ctx->device));
  nxh_set_path("cat_fused");
  {
    const void *base[CAT_MAXM + 1] = {out->data};
    uint64_t bytes[CAT_MAXM + 1] = {(uint64_t)total * (uint64_t)es};
    for (int m = 0; m < n; m++) {
      uint64_t e = 1;
      for (int d = 0; d < nd; d++)
        if (inputs[m]->strides[d] != 0) e *= (uint64_t)inputs[m]->shape[d];
      base[m + 1] = inputs[m]->data;
      bytes[m + 1] = e * (uint64_t)es;
    }
    a.stream_out = nxh_cache_hints(ctx, n + 1, base, bytes, NXH_STREAM_OUT) & NXH_STREAM_OUT;
  }
  switch (es) {
    case 1: cat_launch<uint8_t>(ctx, a, vp); break;
    case 2: cat_launch<uint16_t>(ctx, a, vp); break;
    case 4: cat_launch<uint32_t>(ctx, a, vp); break;
    case 8: cat_launch<uint64_t>(ctx, a, vp); break;
    default: cat_launch<G16>(ctx, a, vp); break;
  }
  NXH_HIP("cat", hipGetLastError());
  return NXH_OK;
}

NXH_EXPORT int nxh_cat(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *const *inputs, int n_inputs,
                       int axis) {
  if (ctx && nxh_defer_active(ctx))
    if (int drc = nxh_defer_barrier(ctx, out)) return drc;
  const char *op = "cat";
  if (!ctx || !out || (n_inputs > 0 && !inputs)) return nxh_fail(NXH_INVALID_ARGUMENT, op, "null argument");
  int rc = nxh_check_tensor(op, out);
  if (rc) return rc;
  if (axis < 0 || axis >= out->ndim) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_AXIS);
  int64_t pos = 0;
  for (int m = 0; m < n_inputs; m++) {
    const nxh_tensor *in = inputs[m];
    if (!in) return nxh_fail(NXH_INVALID_ARGUMENT, op, "null argument");
    if ((rc = nxh_check_tensor(op, in))) return rc;
    if (in->ndim != out->ndim) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
    if (in->dtype != out->dtype) return nxh_fail(NXH_FAILURE, op, NXH_ERR_UNSUPPORTED);
    for (int d = 0; d < out->ndim; d++)
      if (d != axis && in->shape[d] != out->shape[d]) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
    pos += in->shape[axis];
    if (pos > out->shape[axis]) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
  }
  if (nxh_is_packed(out->dtype)) return nxh_fail(NXH_FAILURE, op, NXH_ERR_PACKED);
  for (int d = 0; d < out->ndim; d++)
    if (out->shape[d] > 1 && out->strides[d] == 0) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_OUT_ALIASED);
  rc = cat_fused(ctx, out, inputs, n_inputs, axis);  // (asks the cache policy with its operands' names)
  if (rc != -1) return rc;
  nxh_cache_opaque(ctx);
  pos = 0;
  for (int m = 0; m < n_inputs; m++) {
    const nxh_tensor *in = inputs[m];
    nxh_tensor slice = *out;
    slice.offset = out->offset + pos * out->strides[axis];
    for (int d = 0; d < out->ndim; d++) slice.shape[d] = in->shape[d];
    if (!has_zero_extent(&slice) && (rc = nxh_copy(ctx, &slice, in))) return rc;
    pos += in->shape[axis];
  }
  nxh_set_path("cat_slices");
  return NXH_OK;
}
