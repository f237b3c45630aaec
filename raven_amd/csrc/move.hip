// move.hip — gather (packages/nx/lib/backend_c/nx_c_move.c:342-458).
//
// out[c] = data[c with c[axis] <- indices[c]]; int32 indices, one negative wrap,
// then a bounds check whose failure is reported by the gather call itself, as
// in the reference: kernels raise a device flag and skip the access, the host
// reads the flag back after the launch. Bytes are moved untouched (any dtype).
//   gather_rows  axis 0 of a 2-D table with a column-broadcast index (the
//                embedding lookup): one wave64 copies one row with 16-byte
//                loads.
//   gather_any   one lane per output element, per-lane unravel.

#include "nxh_common.hpp"

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
template <class E>
__global__ __launch_bounds__(256) void gather_any_kernel(GatherAnyArgs a) {
  const int64_t it = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (it >= a.total) return;
  int64_t rem = it, io = 0, oo = 0, doff = 0;
  for (int d = a.ndim - 1; d >= 0; d--) {
    const int64_t c = rem % a.shape[d];
    rem /= a.shape[d];
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
  hipLaunchKernelGGL((gather_any_kernel<E>), dim3((unsigned)((a.total + 255) / 256)), dim3(256), 0, ctx->stream, a);
}

NXH_EXPORT int nxh_gather(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *data,
                          const nxh_tensor *indices, int axis) {
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
  NXH_HIP(op, hipMemcpyAsync(ctx->fault_flag_host, ctx->fault_flag, sizeof(int), hipMemcpyDeviceToHost, ctx->stream));
  NXH_HIP(op, hipStreamSynchronize(ctx->stream));
  if (*ctx->fault_flag_host != 0) {
    *ctx->fault_flag_host = 0;
    NXH_HIP(op, hipMemcpyAsync(ctx->fault_flag, ctx->fault_flag_host, sizeof(int), hipMemcpyHostToDevice, ctx->stream));
    NXH_HIP(op, hipStreamSynchronize(ctx->stream));
    return nxh_fail(NXH_FAILURE, op, NXH_ERR_INDEX_OOB);
  }
  return NXH_OK;
}
